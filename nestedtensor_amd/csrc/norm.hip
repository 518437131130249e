// Row-wise ops on the packed token buffer of a nested tensor (gfx950): layer
// normalisation over the (regular) last dim, with an optional residual input, and
// the packed additions and multiplications of the reference (nested with nested
// of equal nested size, nested with a 1-D vector over the last dim, nested times
// a scalar).  A nested tensor [B, L_i, n] is
// one contiguous [T, n] matrix here, so none of these needs the nested size:
// they are the per-constituent at::layer_norm / at::add of the reference
// (nestedtensor/csrc/functions.cpp:65-112, BinaryOps.cpp:18-44, 97-107, 241-300) done in
// one launch over all constituents.  All are HBM-bound: every input element is
// read once and every output element written once.
//
// Layer norm: one wavefront per row (a workgroup per row for wide rows).  The
// row is read once into registers, 16 bytes per lane per piece; mean and variance
// are the exact two-pass sums in fp32 (as the reference's kernel,
// nestedtensor/csrc/cuda/transformer_kernels.cu:260-305), reduced with wave
// shuffles.  Rows beyond 16 KiB, or not made of aligned 16-byte pieces, re-read
// from cache instead of keeping the row in registers.  With a residual, the sum is rounded to the storage type before it
// is normalised: that is what the reference computes, as two separate ops.
#include "nt_common.h"

namespace nt {

constexpr int kNormRowsPerBlock = 4;   // one wavefront each

template <typename T>
__device__ __forceinline__ float wave_sum(float v) {
  return wave_reduce_sum(v);
}

// x (+ residual) of one 16-byte piece as floats
template <typename T>
__device__ __forceinline__ void piece_values(u32x4 raw, u32x4 raw_res, bool has_res, float* f) {
  constexpr int kPer = 16 / sizeof(T);
  T a[kPer], r[kPer];
  __builtin_memcpy(a, &raw, 16);
  __builtin_memcpy(r, &raw_res, 16);
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    f[j] = has_res ? (float)(T)((float)a[j] + (float)r[j]) : (float)a[j];
  }
}

// Rows of whole 16-byte pieces at 16-byte aligned addresses.  A row is handled by
// WAVES wavefronts (1: four rows per workgroup, 4: the workgroup shares one row and
// combines its partial sums through LDS); every lane keeps P pieces in registers,
// so a row has at most 64 * WAVES * P pieces.
template <typename T, int P, int WAVES>
__global__ __launch_bounds__(kWave * kNormRowsPerBlock) void layer_norm_rows_kernel(
    const T* __restrict__ x, const T* __restrict__ residual, const T* __restrict__ gamma,
    const T* __restrict__ beta, T* __restrict__ out, int64_t rows, int n, float eps) {
  constexpr int kPer = 16 / sizeof(T);
  constexpr int kTeam = kWave * WAVES;                    // threads per row
  constexpr int kRows = kNormRowsPerBlock / WAVES;        // rows per workgroup
  __shared__ float red_sum[kNormRowsPerBlock], red_sq[kNormRowsPerBlock];
  const int t = threadIdx.x % kTeam;
  const int64_t row = (int64_t)blockIdx.x * kRows + threadIdx.x / kTeam;
  if (row >= rows) return;   // WAVES == 4: the whole workgroup leaves together
  const int pieces = n / kPer;
  const char* xr = reinterpret_cast<const char*>(x + row * n);
  const char* rr = reinterpret_cast<const char*>(residual + row * n);
  const bool has_res = residual != nullptr;

  auto team_sum = [&](float v, float* red) -> float {
    v = wave_sum<T>(v);
    if (WAVES == 1) return v;
    if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = v;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += red[w];
    return total;
  };

  float f[P][kPer];
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int c = t + p * kTeam;
    if (c < pieces) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(xr + c * 16);
      u32x4 raw_res = raw;
      if (has_res) raw_res = *reinterpret_cast<const u32x4*>(rr + c * 16);
      piece_values<T>(raw, raw_res, has_res, f[p]);
    } else {
#pragma unroll
      for (int j = 0; j < kPer; ++j) f[p][j] = 0.0f;
    }
  }
  float sum = 0.0f;
#pragma unroll
  for (int p = 0; p < P; ++p)
#pragma unroll
    for (int j = 0; j < kPer; ++j) sum += f[p][j];
  const float mean = team_sum(sum, red_sum) / (float)n;
  float sq = 0.0f;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    if (t + p * kTeam < pieces) {
#pragma unroll
      for (int j = 0; j < kPer; ++j) sq += (f[p][j] - mean) * (f[p][j] - mean);
    }
  }
  const float rstd = 1.0f / sqrtf(team_sum(sq, red_sq) / (float)n + eps);
  char* orow = reinterpret_cast<char*>(out + row * n);
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int c = t + p * kTeam;
    if (c < pieces) {
      float g[kPer], b[kPer];
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        g[j] = 1.0f;
        b[j] = 0.0f;
      }
      if (gamma) {
        T tmp[kPer];
        const u32x4 raw = load16_unaligned(reinterpret_cast<const char*>(gamma + c * kPer));
        __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
        for (int j = 0; j < kPer; ++j) g[j] = (float)tmp[j];
      }
      if (beta) {
        T tmp[kPer];
        const u32x4 raw = load16_unaligned(reinterpret_cast<const char*>(beta + c * kPer));
        __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
        for (int j = 0; j < kPer; ++j) b[j] = (float)tmp[j];
      }
      T y[kPer];
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        float v = (f[p][j] - mean) * rstd;
        if (gamma) v = v * g[j];
        if (beta) v = v + b[j];
        y[j] = (T)v;
      }
      u32x4 o;
      __builtin_memcpy(&o, y, 16);
      store16_stream(orow + c * 16, o);
    }
  }
}

// Any n, any alignment: three passes over the row (the second and third hit the
// cache), one element per lane per step.
template <typename T>
__global__ __launch_bounds__(kWave * kNormRowsPerBlock) void layer_norm_rows_generic_kernel(
    const T* __restrict__ x, const T* __restrict__ residual, const T* __restrict__ gamma,
    const T* __restrict__ beta, T* __restrict__ out, int64_t rows, int64_t n, float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kNormRowsPerBlock + threadIdx.x / kWave;
  if (row >= rows) return;
  const T* xr = x + row * n;
  const T* rr = residual ? residual + row * n : nullptr;
  auto value = [&](int64_t i) -> float {
    return rr ? (float)(T)((float)xr[i] + (float)rr[i]) : (float)xr[i];
  };
  float sum = 0.0f;
  for (int64_t i = lane; i < n; i += kWave) sum += value(i);
  const float mean = wave_sum<T>(sum) / (float)n;
  float sq = 0.0f;
  for (int64_t i = lane; i < n; i += kWave) {
    const float d = value(i) - mean;
    sq += d * d;
  }
  const float rstd = 1.0f / sqrtf(wave_sum<T>(sq) / (float)n + eps);
  T* orow = out + row * n;
  for (int64_t i = lane; i < n; i += kWave) {
    float v = (value(i) - mean) * rstd;
    if (gamma) v = v * (float)gamma[i];
    if (beta) v = v + (float)beta[i];
    orow[i] = (T)v;
  }
}

template <typename T, int P, int WAVES>
static int launch_layer_norm_vec(const void* x, const void* residual, const void* gamma,
                                 const void* beta, void* out, int64_t rows, int64_t n, double eps,
                                 hipStream_t stream) {
  constexpr int kRows = kNormRowsPerBlock / WAVES;
  const int64_t blocks = (rows + kRows - 1) / kRows;
  if (blocks > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "layer_norm: too many rows");
  hipLaunchKernelGGL((layer_norm_rows_kernel<T, P, WAVES>), dim3((unsigned)blocks),
                     dim3(kWave * kNormRowsPerBlock), 0, stream, static_cast<const T*>(x),
                     static_cast<const T*>(residual), static_cast<const T*>(gamma),
                     static_cast<const T*>(beta), static_cast<T*>(out), rows, (int)n, (float)eps);
  return check_launch("layer_norm_rows_kernel");
}

template <typename T>
static int launch_layer_norm(const void* x, const void* residual, const void* gamma, const void* beta,
                             void* out, int64_t rows, int64_t n, double eps, hipStream_t stream) {
  constexpr int kPer = 16 / sizeof(T);
  const uintptr_t align = (uintptr_t)x | (uintptr_t)out | (uintptr_t)(residual ? residual : x);
  const int64_t pieces = n / kPer;
  if (n % kPer == 0 && align % 16 == 0 && pieces <= kWave * 4 * 4) {
    if (pieces <= 64) return launch_layer_norm_vec<T, 1, 1>(x, residual, gamma, beta, out, rows, n, eps, stream);
    if (pieces <= 128) return launch_layer_norm_vec<T, 2, 1>(x, residual, gamma, beta, out, rows, n, eps, stream);
    // up to 4 KiB a wavefront keeps the whole row (no barrier, no LDS): measured 4.7 against
    // 3.9 TB/s for 4 KiB rows shared by four wavefronts; at 8 KiB the shared row wins (4.8 : 3.6)
    if (pieces <= 256) return launch_layer_norm_vec<T, 4, 1>(x, residual, gamma, beta, out, rows, n, eps, stream);
    if (pieces <= 512) return launch_layer_norm_vec<T, 2, 4>(x, residual, gamma, beta, out, rows, n, eps, stream);
    return launch_layer_norm_vec<T, 4, 4>(x, residual, gamma, beta, out, rows, n, eps, stream);
  }
  const int64_t blocks = (rows + kNormRowsPerBlock - 1) / kNormRowsPerBlock;
  if (blocks > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "layer_norm: too many rows");
  hipLaunchKernelGGL((layer_norm_rows_generic_kernel<T>), dim3((unsigned)blocks),
                     dim3(kWave * kNormRowsPerBlock), 0, stream, static_cast<const T*>(x),
                     static_cast<const T*>(residual), static_cast<const T*>(gamma),
                     static_cast<const T*>(beta), static_cast<T*>(out), rows, n, (float)eps);
  return check_launch("layer_norm_rows_generic_kernel");
}

// Softmax (or log-softmax) over the last dim of every constituent.  Constituent b
// holds row_offsets[b + 1] - row_offsets[b] rows of equal length at element
// offset offsets[b]; the length differs between constituents when the last dim
// is ragged (the [H, L_i, L_i] score blocks of per-sequence attention).  One
// wavefront per row: it finds its constituent by binary search and keeps a row
// of up to 256 8-byte pieces (1024 16-bit or 512 32-bit elements) in registers;
// longer rows take three passes (maximum, sum of exponentials, result), the last
// two from cache.  fp32 arithmetic, one rounding, like at::softmax.
// exp(x) for x <= 0 through the hardware's 2^x: the argument's rounding adds a
// relative error of |x| * 1e-7 at most, and exp(x) is negligible long before that
// matters
__device__ __forceinline__ float fast_exp(float x) {
  return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
}

// one row of n elements, by one wavefront
template <typename T, bool LOG>
__device__ __forceinline__ void softmax_row(const T* __restrict__ src, T* __restrict__ dst, int64_t n,
                                            int lane) {
  constexpr int V = 8 / (int)sizeof(T);      // elements per 8-byte piece
  constexpr int kCache = 4;                  // pieces a lane keeps in registers
  const int64_t pieces = (n + V - 1) / V;
  if (pieces <= kWave * kCache) {
    // the row fits the wavefront's registers: one read, one write, 8 bytes per
    // lane and access at any alignment (rows of odd length start anywhere)
    float v[kCache][V];
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < kCache; ++k) {
      const int64_t i0 = (int64_t)(lane + k * kWave) * V;
      if ((int64_t)k * kWave * V >= n) {             // uniform: nobody has elements in this slot
#pragma unroll
        for (int j = 0; j < V; ++j) v[k][j] = -INFINITY;
        continue;
      }
      if (i0 + V <= n) {
        T t[V];
        __builtin_memcpy(t, src + i0, 8);
#pragma unroll
        for (int j = 0; j < V; ++j) v[k][j] = (float)t[j];
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) v[k][j] = i0 + j < n ? (float)src[i0 + j] : -INFINITY;
      }
#pragma unroll
      for (int j = 0; j < V; ++j) m = fmaxf(m, v[k][j]);
    }
    m = wave_reduce_max(m);
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < kCache; ++k) {
      if ((int64_t)k * kWave * V >= n) break;
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float e = fast_exp(v[k][j] - m);   // exp(-inf) = 0 for the slots past the row
        s += e;
        if (!LOG) v[k][j] = e;
      }
    }
    s = wave_reduce_sum(s);
    const float inv = 1.0f / s, ls = logf(s);
#pragma unroll
    for (int k = 0; k < kCache; ++k) {
      if ((int64_t)k * kWave * V >= n) break;
      const int64_t i0 = (int64_t)(lane + k * kWave) * V;
      T t[V];
#pragma unroll
      for (int j = 0; j < V; ++j) t[j] = (T)(LOG ? v[k][j] - m - ls : v[k][j] * inv);
      if (i0 + V <= n) {
        __builtin_memcpy(dst + i0, t, 8);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
          if (i0 + j < n) dst[i0 + j] = t[j];
      }
    }
    return;
  }
  // longer rows: three passes in 8-byte pieces, the second and third from cache
  const int64_t whole = n / V;                       // pieces without a tail
  float m = -INFINITY;
  for (int64_t p = lane; p < whole; p += kWave) {
    T t[V];
    __builtin_memcpy(t, src + p * V, 8);
#pragma unroll
    for (int j = 0; j < V; ++j) m = fmaxf(m, (float)t[j]);
  }
  for (int64_t i = whole * V + lane; i < n; i += kWave) m = fmaxf(m, (float)src[i]);
  m = wave_reduce_max(m);
  float s = 0.0f;
  for (int64_t p = lane; p < whole; p += kWave) {
    T t[V];
    __builtin_memcpy(t, src + p * V, 8);
#pragma unroll
    for (int j = 0; j < V; ++j) s += fast_exp((float)t[j] - m);
  }
  for (int64_t i = whole * V + lane; i < n; i += kWave) s += fast_exp((float)src[i] - m);
  s = wave_sum<T>(s);
  const float inv = 1.0f / s, ls = logf(s);
  for (int64_t p = lane; p < whole; p += kWave) {
    T t[V];
    __builtin_memcpy(t, src + p * V, 8);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float f = (float)t[j];
      t[j] = (T)(LOG ? f - m - ls : fast_exp(f - m) * inv);
    }
    __builtin_memcpy(dst + p * V, t, 8);
  }
  for (int64_t i = whole * V + lane; i < n; i += kWave) {
    const float f = (float)src[i];
    dst[i] = (T)(LOG ? f - m - ls : fast_exp(f - m) * inv);
  }
}

// One wavefront per row.  The two offset arrays are copied into LDS first when
// they fit (the search for the row's constituent is then a chain of LDS reads
// instead of global ones: the kernel is latency-bound on short rows).
constexpr int kSoftmaxMeta = 1024;

template <typename T, bool LOG>
__global__ __launch_bounds__(256) void softmax_rows_kernel(
    const T* __restrict__ x, T* __restrict__ out, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ row_offsets, int64_t B, int64_t total_rows) {
  __shared__ int64_t s_rows[kSoftmaxMeta], s_offs[kSoftmaxMeta];
  const int64_t* ro = row_offsets;
  const int64_t* eo = offsets;
  if (B + 1 <= kSoftmaxMeta) {                       // uniform over the grid
    for (int i = threadIdx.x; i <= B; i += 256) {
      s_rows[i] = row_offsets[i];
      s_offs[i] = offsets[i];
    }
    __syncthreads();
    ro = s_rows;
    eo = s_offs;
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = (int64_t)blockIdx.x * (256 / kWave) + (threadIdx.x / kWave);
  if (r >= total_rows) return;                       // after the only barrier
  const int64_t b = find_segment(ro, B, r);
  const int64_t first = ro[b], rows_b = ro[b + 1] - first;
  if (rows_b <= 0) return;                           // total_rows beyond row_offsets[B]: nothing to do
  const int64_t base = eo[b];
  const int64_t n = (eo[b + 1] - base) / rows_b;
  softmax_row<T, LOG>(x + base + (r - first) * n, out + base + (r - first) * n, n, lane);
}

template <typename T>
static int launch_softmax(const void* x, void* out, const int64_t* offsets, const int64_t* row_offsets,
                          int64_t B, int64_t total_rows, int log_softmax, hipStream_t stream) {
  const int64_t blocks = (total_rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "softmax_rows: too many rows");
  if (log_softmax) {
    hipLaunchKernelGGL((softmax_rows_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const T*>(x), static_cast<T*>(out), offsets, row_offsets, B, total_rows);
  } else {
    hipLaunchKernelGGL((softmax_rows_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const T*>(x), static_cast<T*>(out), offsets, row_offsets, B, total_rows);
  }
  return check_launch("softmax_rows_kernel");
}

// relu / gelu (erf) of every element of the packed buffer: the reference applies
// at::relu / at::gelu to the buffer (nestedtensor/csrc/activation.cpp:11-19, 34-46)
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void activation_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                         int64_t numel, int act) {
  constexpr int kPer = VEC ? 16 / sizeof(T) : 1;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x * kPer;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * kPer; i < numel; i += stride) {
    if (VEC) {
      const u32x4 raw = *reinterpret_cast<const u32x4*>(x + i);
      T v[kPer];
      __builtin_memcpy(v, &raw, 16);
#pragma unroll
      for (int j = 0; j < kPer; ++j) {
        const float f = (float)v[j];
        v[j] = (T)(act == 1 ? fmaxf(f, 0.0f) : gelu_erf(f));
      }
      u32x4 o;
      __builtin_memcpy(&o, v, 16);
      store16_stream(reinterpret_cast<char*>(out + i), o);
    } else {
      const float f = (float)x[i];
      out[i] = (T)(act == 1 ? fmaxf(f, 0.0f) : gelu_erf(f));
    }
  }
}

template <typename T>
static int launch_activation(const void* x, void* out, int64_t numel, int act, hipStream_t stream) {
  constexpr int kPer = 16 / sizeof(T);
  const bool vec = ((uintptr_t)x | (uintptr_t)out) % 16 == 0 && numel % kPer == 0;
  const int64_t per_thread = vec ? kPer : 1;
  int64_t blocks = (numel + 256 * per_thread - 1) / (256 * per_thread);
  if (blocks > (1 << 20)) blocks = 1 << 20;
  if (vec) {
    hipLaunchKernelGGL((activation_kernel<T, true>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const T*>(x), static_cast<T*>(out), numel, act);
  } else {
    hipLaunchKernelGGL((activation_kernel<T, false>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const T*>(x), static_cast<T*>(out), numel, act);
  }
  return check_launch("activation_kernel");
}

// OP 0: out[i] = a[i] + alpha * b[i % period]   (period == numel: plain packed add)
// OP 1: out[i] = alpha * a[i] * b[i % period], or alpha * a[i] when b is NULL
enum { kBinAdd = 0, kBinMul = 1 };

template <int OP>
__device__ __forceinline__ float bin_op(float a, float b, float alpha, bool has_b) {
  if (OP == kBinAdd) return a + alpha * b;
  return has_b ? alpha * (a * b) : alpha * a;
}

template <typename T, bool VEC, int OP>
__global__ __launch_bounds__(256) void add_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                  float alpha, T* __restrict__ out, int64_t numel,
                                                  int64_t period) {
  constexpr int kPer = VEC ? 16 / sizeof(T) : 1;
  const bool has_b = b != nullptr;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x * kPer;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * kPer; i < numel; i += stride) {
    if (VEC) {
      // period is a multiple of kPer here, so a piece never wraps
      const u32x4 ra = *reinterpret_cast<const u32x4*>(a + i);
      u32x4 rb = ra;
      if (has_b) rb = *reinterpret_cast<const u32x4*>(b + (period == numel ? i : i % period));
      T va[kPer], vb[kPer], vo[kPer];
      __builtin_memcpy(va, &ra, 16);
      __builtin_memcpy(vb, &rb, 16);
#pragma unroll
      for (int j = 0; j < kPer; ++j) vo[j] = (T)bin_op<OP>((float)va[j], (float)vb[j], alpha, has_b);
      u32x4 o;
      __builtin_memcpy(&o, vo, 16);
      store16_stream(reinterpret_cast<char*>(out + i), o);
    } else {
      const float fb = has_b ? (float)b[period == numel ? i : i % period] : 0.0f;
      out[i] = (T)bin_op<OP>((float)a[i], fb, alpha, has_b);
    }
  }
}

template <typename T, int OP>
static int launch_add(const void* a, const void* b, double alpha, void* out, int64_t numel,
                      int64_t period, hipStream_t stream) {
  constexpr int kPer = 16 / sizeof(T);
  const uintptr_t align = (uintptr_t)a | (uintptr_t)b | (uintptr_t)out;
  const bool vec = align % 16 == 0 && numel % kPer == 0 && period % kPer == 0;
  const int64_t per_thread = vec ? kPer : 1;
  int64_t blocks = (numel + 256 * per_thread - 1) / (256 * per_thread);
  if (blocks > (1 << 20)) blocks = 1 << 20;   // grid-stride beyond that
  const T* pa = static_cast<const T*>(a);
  const T* pb = static_cast<const T*>(b);
  T* po = static_cast<T*>(out);
  if (vec) {
    hipLaunchKernelGGL((add_kernel<T, true, OP>), dim3((unsigned)blocks), dim3(256), 0, stream, pa, pb,
                       (float)alpha, po, numel, period);
  } else {
    hipLaunchKernelGGL((add_kernel<T, false, OP>), dim3((unsigned)blocks), dim3(256), 0, stream, pa, pb,
                       (float)alpha, po, numel, period);
  }
  return check_launch("add_kernel");
}

}  // namespace nt

using namespace nt;

extern "C" int nt_layer_norm(const void* x, const void* residual, const void* gamma, const void* beta,
                             void* out, int64_t rows, int64_t n, double eps, int dtype, void* stream) {
  if (rows < 0 || n < 0) return fail(NT_ERR_INVALID_ARGUMENT, "layer_norm: negative extent");
  if (rows == 0 || n == 0) return NT_OK;
  if (!x || !out) return fail(NT_ERR_INVALID_ARGUMENT, "layer_norm: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case NT_F32: return launch_layer_norm<float>(x, residual, gamma, beta, out, rows, n, eps, s);
    case NT_F16: return launch_layer_norm<_Float16>(x, residual, gamma, beta, out, rows, n, eps, s);
    case NT_BF16: return launch_layer_norm<__bf16>(x, residual, gamma, beta, out, rows, n, eps, s);
    default: return fail(NT_ERR_UNSUPPORTED, "layer_norm: dtype %d is not f32, f16 or bf16", dtype);
  }
}

extern "C" int nt_softmax_rows(const void* x, void* out, const int64_t* offsets,
                               const int64_t* row_offsets, int64_t B, int64_t total_rows,
                               int log_softmax, int dtype, void* stream) {
  if (B < 0 || total_rows < 0) return fail(NT_ERR_INVALID_ARGUMENT, "softmax_rows: negative extent");
  if (B == 0 || total_rows == 0) return NT_OK;
  if (!x || !out || !offsets || !row_offsets) return fail(NT_ERR_INVALID_ARGUMENT, "softmax_rows: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case NT_F32: return launch_softmax<float>(x, out, offsets, row_offsets, B, total_rows, log_softmax, s);
    case NT_F16: return launch_softmax<_Float16>(x, out, offsets, row_offsets, B, total_rows, log_softmax, s);
    case NT_BF16: return launch_softmax<__bf16>(x, out, offsets, row_offsets, B, total_rows, log_softmax, s);
    default: return fail(NT_ERR_UNSUPPORTED, "softmax_rows: dtype %d is not f32, f16 or bf16", dtype);
  }
}

extern "C" int nt_add_packed(const void* a, const void* b, double alpha, void* out, int64_t numel,
                             int64_t period, int dtype, void* stream) {
  if (numel < 0 || period < 0) return fail(NT_ERR_INVALID_ARGUMENT, "add_packed: negative extent");
  if (numel == 0) return NT_OK;
  if (period == 0 || numel % period != 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "add_packed: numel %lld is not a multiple of the period %lld",
                (long long)numel, (long long)period);
  }
  if (!a || !b || !out) return fail(NT_ERR_INVALID_ARGUMENT, "add_packed: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case NT_F32: return launch_add<float, kBinAdd>(a, b, alpha, out, numel, period, s);
    case NT_F16: return launch_add<_Float16, kBinAdd>(a, b, alpha, out, numel, period, s);
    case NT_BF16: return launch_add<__bf16, kBinAdd>(a, b, alpha, out, numel, period, s);
    default: return fail(NT_ERR_UNSUPPORTED, "add_packed: dtype %d is not f32, f16 or bf16", dtype);
  }
}

extern "C" int nt_activation_packed(const void* x, void* out, int64_t numel, int act, int dtype,
                                    void* stream) {
  if (numel < 0) return fail(NT_ERR_INVALID_ARGUMENT, "activation_packed: negative extent");
  if (act != 1 && act != 2) return fail(NT_ERR_INVALID_ARGUMENT, "activation_packed: act %d is not 1 (relu) or 2 (gelu)", act);
  if (numel == 0) return NT_OK;
  if (!x || !out) return fail(NT_ERR_INVALID_ARGUMENT, "activation_packed: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case NT_F32: return launch_activation<float>(x, out, numel, act, s);
    case NT_F16: return launch_activation<_Float16>(x, out, numel, act, s);
    case NT_BF16: return launch_activation<__bf16>(x, out, numel, act, s);
    default: return fail(NT_ERR_UNSUPPORTED, "activation_packed: dtype %d is not f32, f16 or bf16", dtype);
  }
}

extern "C" int nt_mul_packed(const void* a, const void* b, double scale, void* out, int64_t numel,
                             int64_t period, int dtype, void* stream) {
  if (numel < 0 || period < 0) return fail(NT_ERR_INVALID_ARGUMENT, "mul_packed: negative extent");
  if (numel == 0) return NT_OK;
  if (!b) period = numel;
  if (period == 0 || numel % period != 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "mul_packed: numel %lld is not a multiple of the period %lld",
                (long long)numel, (long long)period);
  }
  if (!a || !out) return fail(NT_ERR_INVALID_ARGUMENT, "mul_packed: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case NT_F32: return launch_add<float, kBinMul>(a, b, scale, out, numel, period, s);
    case NT_F16: return launch_add<_Float16, kBinMul>(a, b, scale, out, numel, period, s);
    case NT_BF16: return launch_add<__bf16, kBinMul>(a, b, scale, out, numel, period, s);
    default: return fail(NT_ERR_UNSUPPORTED, "mul_packed: dtype %d is not f32, f16 or bf16", dtype);
  }
}
