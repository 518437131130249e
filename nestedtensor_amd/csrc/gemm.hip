// Packed projection GEMM for nested multi-head attention (gfx950 MFMA).
//
//   C[M, N] = A[M, K] * W[N, K]^T + bias[N]
//
// A is the packed token buffer viewed as [T, E] (no padded rows exist), W is a
// torch Linear weight, so both operands are K-contiguous: every MFMA operand
// fragment is one 16-byte run of a row.  Workgroup tile 128 x 128, 256 threads
// as 2 x 2 wavefronts of 64 x 64 (2 x 2 MFMA 32x32 blocks each), K tiles of
// 128 bytes double-buffered in LDS with rows padded to 144 bytes so that the
// 128-bit fragment reads of 16 consecutive lanes fall into distinct banks.
// Global loads of tile k+1 are issued before the MFMAs of tile k.
// fp32 accumulation for all types; f16 / bf16 use v_mfma_f32_32x32x16_*,
// fp32 uses v_mfma_f32_32x32x2_f32.
#include "nt_common.h"

namespace nt {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float acc16 __attribute__((ext_vector_type(16)));

template <typename T> struct Mma;

template <> struct Mma<_Float16> {
  typedef half8 Frag;
  static constexpr int kK = 16;  // K per MFMA
  static __device__ __forceinline__ acc16 run(Frag a, Frag b, acc16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ _Float16 from_float(float x) { return (_Float16)x; }
  static __device__ __forceinline__ float to_float(_Float16 x) { return (float)x; }
};

template <> struct Mma<__bf16> {
  typedef bf16x8 Frag;
  static constexpr int kK = 16;
  static __device__ __forceinline__ acc16 run(Frag a, Frag b, acc16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ __bf16 from_float(float x) { return (__bf16)x; }
  static __device__ __forceinline__ float to_float(__bf16 x) { return (float)x; }
};

template <> struct Mma<float> {
  typedef float Frag;
  static constexpr int kK = 2;
  static __device__ __forceinline__ acc16 run(Frag a, Frag b, acc16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float from_float(float x) { return x; }
  static __device__ __forceinline__ float to_float(float x) { return x; }
};

constexpr int kBM = 128;
constexpr int kBN = 128;
constexpr int kRowBytes = 128;            // K-tile bytes per row
constexpr int kLdsRowBytes = 144;         // padded
constexpr int kTileLdsBytes = (kBM + kBN) * kLdsRowBytes;

// 16-byte piece `cc` (0..7) of row `row` of a K tile starting at element k0.
// Out-of-range rows / K tails read as zero.
template <typename T>
__device__ __forceinline__ u32x4 load_chunk(const T* base, int64_t ld, int64_t row, int64_t nrows,
                                            int64_t k, int64_t K) {
  constexpr int kPer = 16 / sizeof(T);
  u32x4 v = {0, 0, 0, 0};
  if (row < nrows) {
    const T* p = base + row * ld + k;
    if (k + kPer <= K) {
      v = load16_unaligned(reinterpret_cast<const char*>(p));
    } else {
      T tmp[kPer];
#pragma unroll
      for (int j = 0; j < kPer; ++j) tmp[j] = (k + j < K) ? p[j] : (T)0.0f;
      __builtin_memcpy(&v, tmp, 16);
    }
  }
  return v;
}

template <typename T>
__global__ __launch_bounds__(256) void linear_kernel(const T* __restrict__ A, int64_t lda,
                                                     const T* __restrict__ W,
                                                     const T* __restrict__ bias,
                                                     T* __restrict__ C, int64_t ldc, int64_t M,
                                                     int64_t N, int64_t K) {
  typedef Mma<T> MM;
  typedef typename MM::Frag Frag;
  constexpr int kPer = 16 / sizeof(T);          // elements per 16-byte chunk
  constexpr int kBK = kRowBytes / sizeof(T);    // elements per K tile
  constexpr int kSteps = kBK / MM::kK;          // MFMA steps per K tile
  constexpr int kFragBytes = (MM::kK / 2) * sizeof(T);

  extern __shared__ __align__(16) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1;   // wavefront row (0..1)
  const int wn = wave & 1;    // wavefront col (0..1)
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // Tiles of one column panel are adjacent in launch order, so workgroups that
  // run together share the same W panel in L2.
  const int64_t tiles_m = (M + kBM - 1) / kBM;
  const int64_t tile = blockIdx.x;
  const int64_t tm = tile % tiles_m;
  const int64_t tn = tile / tiles_m;
  const int64_t m0 = tm * kBM;
  const int64_t n0 = tn * kBN;

  acc16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int64_t nk = (K + kBK - 1) / kBK;
  u32x4 ra[4], rb[4];

  auto gload = [&](int64_t kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 3;
      const int cc = c & 7;
      const int64_t k = kt * kBK + cc * kPer;
      ra[i] = load_chunk<T>(A, lda, m0 + row, M, k, K);
      rb[i] = load_chunk<T>(W, K, n0 + row, N, k, K);
    }
  };
  auto lstore = [&](int buf) {
    char* base = lds + buf * kTileLdsBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + i * 256;
      const int row = c >> 3;
      const int cc = c & 7;
      store16(base + row * kLdsRowBytes + cc * 16, ra[i]);
      store16(base + (kBM + row) * kLdsRowBytes + cc * 16, rb[i]);
    }
  };

  gload(0);
  lstore(0);
  __syncthreads();

  for (int64_t kt = 0; kt < nk; ++kt) {
    const int buf = (int)(kt & 1);
    if (kt + 1 < nk) gload(kt + 1);
    const char* a_base = lds + buf * kTileLdsBytes + (wm * 64 + l32) * kLdsRowBytes;
    const char* b_base = lds + buf * kTileLdsBytes + (kBM + wn * 64 + l32) * kLdsRowBytes;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const int koff = s * MM::kK * (int)sizeof(T) + g * kFragBytes;
      Frag fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = *reinterpret_cast<const Frag*>(a_base + i * 32 * kLdsRowBytes + koff);
        fb[i] = *reinterpret_cast<const Frag*>(b_base + i * 32 * kLdsRowBytes + koff);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = MM::run(fa[i], fb[j], acc[i][j]);
    }
    if (kt + 1 < nk) lstore(buf ^ 1);
    __syncthreads();
  }

  // Epilogue: acc[i][j][e] is C[row, col] with
  //   row = m0 + wm*64 + i*32 + 8*(e/4) + 4*g + e%4,  col = n0 + wn*64 + j*32 + l32.
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t col = n0 + wn * 64 + j * 32 + l32;
    if (col >= N) continue;
    const float bv = bias ? MM::to_float(bias[col]) : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t row = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * g + (e & 3);
        if (row < M) C[row * ldc + col] = MM::from_float(acc[i][j][e] + bv);
      }
    }
  }
}

template <typename T>
static int launch_linear(const void* A, int64_t lda, const void* W, const void* bias, void* C,
                         int64_t ldc, int64_t M, int64_t N, int64_t K, hipStream_t stream) {
  const int64_t tiles = ((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN);
  if (tiles > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "linear: too many tiles");
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(linear_kernel<T>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       2 * kTileLdsBytes);
    if (e != hipSuccess) return fail(NT_ERR_HIP, "linear: %s", hipGetErrorString(e));
    attr_set = true;
  }
  hipLaunchKernelGGL((linear_kernel<T>), dim3((unsigned)tiles), dim3(256), 2 * kTileLdsBytes,
                     stream, static_cast<const T*>(A), lda, static_cast<const T*>(W),
                     static_cast<const T*>(bias), static_cast<T*>(C), ldc, M, N, K);
  return check_launch("linear_kernel");
}

}  // namespace nt

using namespace nt;

extern "C" int nt_linear(const void* A, int64_t lda, const void* W, const void* bias, void* C,
                         int64_t ldc, int64_t M, int64_t N, int64_t K, int dtype, void* stream) {
  if (M < 0 || N < 0 || K < 0 || lda < K || ldc < N) {
    return fail(NT_ERR_INVALID_ARGUMENT, "linear: bad shape M=%lld N=%lld K=%lld lda=%lld ldc=%lld",
                (long long)M, (long long)N, (long long)K, (long long)lda, (long long)ldc);
  }
  if (M == 0 || N == 0) return NT_OK;
  if (!A || !W || !C) return fail(NT_ERR_INVALID_ARGUMENT, "linear: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case NT_F32: return launch_linear<float>(A, lda, W, bias, C, ldc, M, N, K, s);
    case NT_F16: return launch_linear<_Float16>(A, lda, W, bias, C, ldc, M, N, K, s);
    case NT_BF16: return launch_linear<__bf16>(A, lda, W, bias, C, ldc, M, N, K, s);
    default: return fail(NT_ERR_INVALID_ARGUMENT, "linear: unknown dtype %d", dtype);
  }
}
