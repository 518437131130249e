// Shared helpers of the nestedtensor_amd HIP library (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/nestedtensor_amd.h"

namespace nt {

constexpr int kWave = 64;

// Error text of the calling thread, returned by nt_last_error().
char* error_buffer();

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    return fail(NT_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  }
  return NT_OK;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 16-byte load from an address of any alignment (gfx950 runs with unaligned
// access mode; the compiler emits one global_load_dwordx4).
__device__ __forceinline__ u32x4 load16_unaligned(const char* p) {
  u32x4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}

__device__ __forceinline__ void store16(char* p, u32x4 v) {
  *reinterpret_cast<u32x4*>(p) = v;
}

__device__ __forceinline__ void store16_stream(char* p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// gelu(x) = x/2 (1 + erf(x / sqrt 2)) with erf from Abramowitz & Stegun 7.1.26
// (absolute error below 1.5e-7, i.e. below fp32 rounding of the result for |x| of
// order 1): one reciprocal, one 2^x and nine multiply-adds instead of the ~40
// instructions of erff, which made a fused epilogue slower than a second pass.
__device__ __forceinline__ float gelu_erf(float x) {
  const float z = fabsf(x) * 0.70710678118654752f;
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
  float p = 1.061405429f;
  p = fmaf(p, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  const float e = __builtin_amdgcn_exp2f(-z * z * 1.4426950408889634f);
  const float erf_abs = 1.0f - p * t * e;
  return 0.5f * x * (1.0f + copysignf(erf_abs, x));
}

// b with offsets[b] <= i < offsets[b + 1] (offsets non-decreasing, offsets[B] > i)
__device__ __forceinline__ int64_t find_segment(const int64_t* offsets, int64_t B, int64_t i) {
  int64_t lo = 0, hi = B;   // answer in [lo, hi)
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if (offsets[mid] <= i) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  return lo;
}

// Reductions over the 64 lanes of a wavefront on the vector ALU's data-parallel
// primitives: four shifted adds within each row of 16 lanes, then the row totals
// are passed on to rows 1 and 3 and to rows 2 and 3 (row_bcast:15, row_bcast:31);
// lane 63 holds the total and is read back as a scalar, so the result is uniform.
// Seven vector instructions, against six LDS-crossbar permutes and their address
// arithmetic for the same reduction written with __shfl_xor.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float src) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src),
                                                               CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float wave_reduce_sum(float v) {
  v += dpp_move<0x111, 0xf>(0.0f, v);   // row_shr:1
  v += dpp_move<0x112, 0xf>(0.0f, v);   // row_shr:2
  v += dpp_move<0x114, 0xf>(0.0f, v);   // row_shr:4
  v += dpp_move<0x118, 0xf>(0.0f, v);   // row_shr:8
  v += dpp_move<0x142, 0xa>(0.0f, v);   // row_bcast:15 into rows 1 and 3
  v += dpp_move<0x143, 0xc>(0.0f, v);   // row_bcast:31 into rows 2 and 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ int wave_reduce_sum(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);
  return __builtin_amdgcn_readlane(v, 63);
}
__device__ __forceinline__ float wave_reduce_max(float v) {
  const float lowest = -__builtin_inff();
  v = fmaxf(v, dpp_move<0x111, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<0x112, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<0x114, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<0x118, 0xf>(lowest, v));
  v = fmaxf(v, dpp_move<0x142, 0xa>(lowest, v));
  v = fmaxf(v, dpp_move<0x143, 0xc>(lowest, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

}  // namespace nt
