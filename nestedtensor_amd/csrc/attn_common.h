// Pieces shared by the attention kernels (gfx950, wave64): operand fragment types
// of v_mfma_f32_32x32x16_{f16,bf16}, the packed conversions and dot products of
// the online softmax, and the cross-half maximum.
#pragma once
#include "nt_common.h"

namespace nt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float acc16 __attribute__((ext_vector_type(16)));

typedef float float2v __attribute__((ext_vector_type(2)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// max over the two lanes l and l ^ 32 without the LDS round trip of a shuffle:
// v_permlane32_swap exchanges the upper half of one register with the lower half
// of another, which leaves (lo, lo) in one and (hi, hi) in the other.  Written as
// inline asm: through the builtin, with the same value in both operands, the
// compiler keeps only the first result and drops the maximum (the kernel then
// sees the maximum of half of a row's keys).  The asm is opaque to the hazard
// recognizer, hence the wait states around the swap.
__device__ __forceinline__ float max_across_halves(float v) {
  float lo = v, hi = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
  return fmaxf(lo, hi);
}

template <typename T> struct AttnT;
template <> struct AttnT<_Float16> {
  typedef half8 Frag;
  typedef half4 Half;
  // two fp32 -> packed pair, round to nearest even (v_cvt_pk_f16_f32)
  static __device__ __forceinline__ uint32_t cvt2(float a, float b) {
    float2v x = {a, b};
    half2v h = __builtin_convertvector(x, half2v);
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
  }
  static constexpr uint32_t kOnePair = 0x3c003c00u;   // (1.0, 1.0)
  // acc + lo + hi of a packed pair, in fp32 (v_dot2c_f32_f16)
  static __device__ __forceinline__ float dot_ones(uint32_t pair, float acc) {
    half2v h, one = {(_Float16)1.0f, (_Float16)1.0f};
    __builtin_memcpy(&h, &pair, 4);
    return __builtin_amdgcn_fdot2(h, one, acc, false);
  }
  static __device__ __forceinline__ acc16 mma(Frag a, Frag b, acc16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct AttnT<__bf16> {
  typedef bf16x8 Frag;
  typedef bf16x4 Half;
  static __device__ __forceinline__ uint32_t cvt2(float a, float b) {
    float2v x = {a, b};
    bf16x2 h = __builtin_convertvector(x, bf16x2);
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
  }
  static constexpr uint32_t kOnePair = 0x3f803f80u;
  static __device__ __forceinline__ float dot_ones(uint32_t pair, float acc) {   // v_dot2c_f32_bf16
    bf16x2 h, one = {(__bf16)1.0f, (__bf16)1.0f};
    __builtin_memcpy(&h, &pair, 4);
    return __builtin_amdgcn_fdot2_f32_bf16(h, one, acc, false);
  }
  static __device__ __forceinline__ acc16 mma(Frag a, Frag b, acc16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// A query row's reference maximum moves only when a tile's maximum leaves this many
// powers of two around it (softmax is invariant to the reference; it only has to
// keep 2^(S - m_ref) inside the range of the storage type).
constexpr float kLazyMaxLog2 = 8.0f;

template <typename T> struct QScale;
template <> struct QScale<_Float16> {
  static __device__ __forceinline__ half8 run(half8 v, float s) {
    const _Float16 hs = (_Float16)s;
    return v * hs;   // v_pk_mul_f16
  }
};
template <> struct QScale<__bf16> {
  static __device__ __forceinline__ bf16x8 run(bf16x8 v, float s) {
    bf16x8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (__bf16)((float)v[j] * s);
    return r;
  }
};

}  // namespace nt
