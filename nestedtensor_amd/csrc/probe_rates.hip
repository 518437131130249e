// Instruction-rate probe for gfx950 (a measurement aid, not part of
// libnestedtensor_amd.so: it is built into libnt_probe.so and loaded only by
// `bench.py --mha-probe`).  The attention kernel's vector-ALU budget is set against
// the matrix pipe with these numbers: how long a wavefront-wide v_exp_f32 occupies
// a SIMD compared with a v_fma_f32, what a v_mfma_f32_32x32x16_f16 costs, and how
// much of the vector work runs beside the matrix instructions when both are in
// one instruction stream.
//
// Every kernel runs `waves_per_simd` wavefronts on each SIMD of the chip
// (workgroups of 256 threads, one per compute unit and wave slot) and repeats an
// unrolled body of independent instructions; the host reports nanoseconds per
// instruction and SIMD.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float acc16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

enum { kFma = 0, kExp32, kExp16, kCvtPk, kDot2, kMax3, kMfma, kLds128, kMfmaFma, kMfmaExp, kMfmaFmaExp, kMfmaV,
       kMfmaFmaExpV, kTileLike, kTileLikeLds, kTileLikeBarrier, kTileLikeLoads, kTileLikeRows, kTileLikeMaxFirst, kKinds };
constexpr int kAccInVgpr = 1000;   // OTHER code: no instruction of its own, the MFMA accumulators in VGPRs

// NM matrix instructions (four accumulators in turn), NV multiply-adds and NT
// exponentials per loop iteration, sixteen independent chains each.
template <int NM, int NV, int NT, int NOTHER, int OTHER>
__global__ __launch_bounds__(256) void rate_kernel(float* out, int iters) {
  __shared__ __align__(16) char lds[32768];
  float v[16], w[16];
  half2v h[16];
  for (int i = 0; i < 16; ++i) {
    v[i] = threadIdx.x * 0.01f + i * 0.1f - 0.5f;
    w[i] = -0.001f * i - threadIdx.x * 1e-5f;
    h[i][0] = (_Float16)(0.01f * i);
    h[i][1] = (_Float16)(0.02f * i + threadIdx.x * 1e-3f);
  }
  half8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (_Float16)(threadIdx.x * 0.001f + i);
    b[i] = (_Float16)(i * 0.5f - threadIdx.x * 0.002f);
  }
  acc16 acc[4];
  for (int n = 0; n < 4; ++n)
    for (int e = 0; e < 16; ++e) acc[n][e] = 0.0f;
  u32x4 ld[8];
  for (int i = 0; i < 8; ++i) ld[i] = (u32x4){0u, 0u, 0u, 0u};
  for (int i = threadIdx.x; i < 9216; i += 256) reinterpret_cast<uint32_t*>(lds)[i] = i;
  __syncthreads();
  const float c0 = out[0], c1 = out[1];
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < NM; ++n) {
      if (OTHER == kAccInVgpr) {
        // accumulators held in ordinary vector registers, as a kernel has them whose
        // vector instructions read the products (left to itself the compiler puts the
        // accumulators of this loop into the accumulation registers)
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc[n & 3]) : "v"(a), "v"(b));
      } else {
        acc[n & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[n & 3], 0, 0, 0);
      }
    }
#pragma unroll
    for (int n = 0; n < NV; ++n) v[n & 15] = __builtin_fmaf(v[n & 15], c0, c1);
#pragma unroll
    for (int n = 0; n < NT; ++n) w[n & 15] = __builtin_amdgcn_exp2f(w[n & 15]);
#pragma unroll
    for (int n = 0; n < NOTHER; ++n) {
      const int j = n & 15;
      if (OTHER == kExp16) {
        _Float16 r;
        asm volatile("v_exp_f16 %0, %1" : "=v"(r) : "v"(h[j][0]));
        h[j][0] = r;
      }
      if (OTHER == kCvtPk) {
        // (as an asm statement: the operands do not change in the loop, and the
        // compiler would hoist a plain conversion out of it)
        asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(h[j]) : "v"(v[j]), "v"(v[(j + 1) & 15]));
      }
      if (OTHER == kDot2) v[j] = __builtin_amdgcn_fdot2(h[j], h[(j + 1) & 15], v[j], false);
      if (OTHER == kMax3) v[j] = __builtin_fmaxf(__builtin_fmaxf(v[j], v[(j + 1) & 15]), v[(j + 2) & 15]);
      if (OTHER == kLds128) {
        ld[n & 7] ^= *reinterpret_cast<const u32x4*>(lds + ((threadIdx.x & 63) * 16 + (n & 31) * 1024 + (it & 1) * 16) % 32768);
      }
    }
  }
  float s = 0.0f;
  for (int n = 0; n < 4; ++n)
    for (int e = 0; e < 16; ++e) s += acc[n][e];
  for (int i = 0; i < 16; ++i) s += v[i] + w[i] + (float)h[i][0] + (float)h[i][1];
  for (int i = 0; i < 8; ++i) s += (float)(ld[i][0] + ld[i][1] + ld[i][2] + ld[i][3]);
  out[2 + (size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

// One key tile of the attention kernels as a wavefront sees it, without the rest
// of the kernel: eight matrix instructions for the scores of 64 keys (two chains
// of four), the row maximum, 32 exponentials, their packing and the row sums, then
// eight matrix instructions that take the packed probabilities as an operand.
// WITH_LDS: the sixteen operand fragments of the matrix instructions are read from
// LDS (16 bytes per lane each) instead of staying in registers.  No barrier, no
// global memory: what is left is the dependent chain scores -> maximum ->
// exponentials -> second product and whatever of it several wavefronts on a SIMD
// can overlap.
template <int MODE>
__global__ __launch_bounds__(256, 3) void tile_like_kernel(float* out, const uint32_t* __restrict__ src, int iters,
                                                           uint32_t noise) {
  constexpr bool WITH_LDS = MODE >= 1;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  __shared__ __align__(16) char lds[36864];
  // noise == 0: operands are small regular numbers (few bits change from one
  // instruction to the next).  Otherwise sign and mantissa of every fp16 operand
  // are pseudo-random (keys and values in +-[0.5, 1), queries in +-[1/8, 1/4)):
  // the same instruction stream with the switching activity of real data.
  const uint32_t keep = noise ? 0x83ff83ffu : 0x03ff03ffu;
  const uint32_t set = noise ? 0x38003800u : 0x2c002c00u;
  const long long cycles0 = clock64();
  const long long ticks0 = wall_clock64();
  for (int i = threadIdx.x; i < 9216; i += 256) {
    reinterpret_cast<uint32_t*>(lds)[i] =
        noise ? (mix32(noise + i * 2654435761u + blockIdx.x * 40503u) & keep) | set : 0x2c002c00u + (i & 255);
  }
  __syncthreads();
  half8 q[4], kf[8], vf[8];
  for (int s = 0; s < 8; ++s)
    for (int i = 0; i < 8; ++i) {
      kf[s][i] = (_Float16)(0.01f * (i + s) + threadIdx.x * 1e-4f);
      vf[s][i] = (_Float16)(0.02f * (i - s) - threadIdx.x * 1e-4f);
      if (s < 4) q[s][i] = (_Float16)(0.03f * i + 0.001f * s);
    }
  if (noise) {
    for (int s = 0; s < 4; ++s) {
      uint32_t w[4];
      for (int i = 0; i < 4; ++i) w[i] = (mix32(noise ^ (threadIdx.x * 16 + s * 4 + i + 77777u)) & 0x83ff83ffu) | 0x30003000u;
      __builtin_memcpy(&q[s], w, 16);
    }
  }
  acc16 negm, o[2];
  for (int e = 0; e < 16; ++e) {
    negm[e] = -1.0f;
    o[0][e] = 0.0f;
    o[1][e] = 0.0f;
  }
  float l_run = 0.0f, m_run = 0.0f;
  const char* base = lds + (threadIdx.x & 63) * 16;
  // MODE 4: rows of 144 bytes, a lane reads 16 bytes of row (lane % 32) at byte 16 (lane / 32)
  const char* rows = lds + (threadIdx.x & 31) * 144 + ((threadIdx.x >> 5) & 1) * 16;
  for (int it = 0; it < iters; ++it) {
    u32x4 stage[4];
    if (MODE >= 3) {
      // the next tile's 16 bytes per lane, four times, on their way from global memory
      const char* g = reinterpret_cast<const char*>(src) +
                      ((size_t)(blockIdx.x * 131 + it) % 128) * 16384 + threadIdx.x * 16;
#pragma unroll
      for (int i = 0; i < 4; ++i) stage[i] = *reinterpret_cast<const u32x4*>(g + i * 4096);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (WITH_LDS) {
#pragma unroll
      for (int s = 0; s < 8; ++s)
        kf[s] = *reinterpret_cast<const half8*>(
            MODE >= 4 ? rows + (it & 1) * 18432 + (s / 4) * 32 * 144 + (s % 4) * 32
                      : base + (MODE >= 2 ? (it & 1) * 16384 + (s & 7) * 1024 : ((it * 8 + s) & 15) * 1024));
    }
    acc16 sa0 = negm, sa1 = negm;
#pragma unroll
    for (int s = 0; s < 4; ++s) sa0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s], q[s], sa0, 0, 0, 0);
#pragma unroll
    for (int s = 0; s < 4; ++s) sa1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[4 + s], q[s], sa1, 0, 0, 0);
    if (WITH_LDS) {
#pragma unroll
      for (int s = 0; s < 8; ++s)
        vf[s] = *reinterpret_cast<const half8*>(
            MODE >= 4 ? rows + (it & 1) * 18432 + 9216 + (s % 2) * 32 * 144 + (s / 2) * 32
                      : base + (MODE >= 2 ? (it & 1) * 16384 + 8192 + (s & 7) * 1024
                                          : 16384 + ((it * 8 + s) & 15) * 1024));
    }
    float m = sa0[0];
#pragma unroll
    for (int e = 1; e < 16; ++e) m = __builtin_fmaxf(m, sa0[e]);
#pragma unroll
    for (int e = 0; e < 16; ++e) m = __builtin_fmaxf(m, sa1[e]);
    m_run = __builtin_fmaxf(m_run, m);
    if (MODE >= 5) {
      // the exponentials wait for the tile's maximum: a wavefront-uniform test (never
      // true on this data) that would move the reference maximum of the scores
      float lo = m, hi = m;
      asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(lo), "+v"(hi));
      m = __builtin_fmaxf(lo, hi);
      if (__any(m > 64.0f)) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          sa0[e] -= m;
          sa1[e] -= m;
          negm[e] -= m;
        }
      }
      asm volatile("" : "+v"(negm));
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      uint32_t pw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p0 = __builtin_amdgcn_exp2f(ks < 2 ? sa0[(ks & 1) * 8 + 2 * j] : sa1[(ks & 1) * 8 + 2 * j]);
        const float p1 = __builtin_amdgcn_exp2f(ks < 2 ? sa0[(ks & 1) * 8 + 2 * j + 1] : sa1[(ks & 1) * 8 + 2 * j + 1]);
        float2v x = {p0, p1};
        half2v hh = __builtin_convertvector(x, half2v);
        half2v one = {(_Float16)1.0f, (_Float16)1.0f};
        l_run = __builtin_amdgcn_fdot2(hh, one, l_run, false);
        __builtin_memcpy(&pw[j], &hh, 4);
      }
      half8 pf;
      __builtin_memcpy(&pf, pw, 16);
      o[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * ks], pf, o[0], 0, 0, 0);
      o[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * ks + 1], pf, o[1], 0, 0, 0);
    }
    if (MODE >= 2) {
      // the workgroup's next tile goes into the other LDS buffer, then everybody meets
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        u32x4 v = {0x2c002c00u + (uint32_t)it, 0x2c002c01u, 0x2c002c02u, 0x2c002c03u};
        if (MODE >= 3) v = (stage[i] & keep) | set;
        if (MODE >= 4) {
          *reinterpret_cast<u32x4*>(lds + ((it + 1) & 1) * 18432 + (i / 2) * 9216 +
                                    (threadIdx.x / 8 + (i % 2) * 32) * 144 + (threadIdx.x % 8) * 16) = v;
        } else {
          *reinterpret_cast<u32x4*>(lds + ((it + 1) & 1) * 16384 + i * 4096 + threadIdx.x * 16) = v;
        }
      }
      __syncthreads();
    }
  }
  float sum = l_run + m_run;
  for (int e = 0; e < 16; ++e) sum += o[0][e] + o[1][e];
  out[2 + (size_t)blockIdx.x * 256 + threadIdx.x] = sum;
  // the first workgroup's life on the shader clock and on the constant 100 MHz clock
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    out[0] = (float)(clock64() - cycles0);
    out[1] = (float)(wall_clock64() - ticks0);
  }
}

__global__ void noise_fill_kernel(uint32_t* p, size_t n, uint32_t seed) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    p[i] = mix32(seed + (uint32_t)i * 2654435761u);
  }
}

template <int MODE>
static int run_tile_like(int waves_per_simd, int iters, int cus, float* ms, uint32_t noise = 0,
                         float* clocks = nullptr) {
  float* out = nullptr;
  static uint32_t* src = nullptr;   // 2 MiB that the global loads of MODE 3 walk through
  static uint32_t src_noise = 0;
  constexpr size_t kSrcBytes = (size_t)132 * 16384;
  if (src == nullptr) {
    if (hipMalloc(&src, kSrcBytes) != hipSuccess) return 1;
    if (hipMemset(src, 0x11, kSrcBytes) != hipSuccess) return 1;
  }
  if (noise != src_noise) {
    if (noise) {
      hipLaunchKernelGGL(noise_fill_kernel, dim3(256), dim3(256), 0, 0, src, kSrcBytes / 4, noise);
    } else if (hipMemset(src, 0x11, kSrcBytes) != hipSuccess) {
      return 1;
    }
    src_noise = noise;
  }
  const int wgs = cus * waves_per_simd;
  if (hipMalloc(&out, (2 + (size_t)wgs * 256) * sizeof(float)) != hipSuccess) return 1;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return 1;
  hipLaunchKernelGGL(tile_like_kernel<MODE>, dim3(wgs), dim3(256), 0, 0, out, src, iters, noise);
  int rc = hipEventRecord(e0, 0) == hipSuccess ? 0 : 1;
  hipLaunchKernelGGL(tile_like_kernel<MODE>, dim3(wgs), dim3(256), 0, 0, out, src, iters, noise);
  if (hipEventRecord(e1, 0) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
      hipEventElapsedTime(ms, e0, e1) != hipSuccess) {
    rc = 1;
  }
  if (rc == 0 && clocks != nullptr && hipMemcpy(clocks, out, 8, hipMemcpyDeviceToHost) != hipSuccess) rc = 1;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(out);
  return rc;
}

template <int NM, int NV, int NT, int NOTHER, int OTHER>
static int run(int waves_per_simd, int iters, int cus, float* ms) {
  float* out = nullptr;
  const int wgs = cus * waves_per_simd;
  if (hipMalloc(&out, (2 + (size_t)wgs * 256) * sizeof(float)) != hipSuccess) return 1;
  if (hipMemset(out, 0, 8) != hipSuccess) return 1;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return 1;
  hipLaunchKernelGGL((rate_kernel<NM, NV, NT, NOTHER, OTHER>), dim3(wgs), dim3(256), 0, 0, out, iters);
  int rc = hipEventRecord(e0, 0) == hipSuccess ? 0 : 1;
  hipLaunchKernelGGL((rate_kernel<NM, NV, NT, NOTHER, OTHER>), dim3(wgs), dim3(256), 0, 0, out, iters);
  if (hipEventRecord(e1, 0) != hipSuccess || hipEventSynchronize(e1) != hipSuccess ||
      hipEventElapsedTime(ms, e0, e1) != hipSuccess) {
    rc = 1;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(out);
  return rc;
}

// Milliseconds of `iters` iterations of probe `kind` with `waves_per_simd` (1..3)
// wavefronts on every SIMD, and the instructions one iteration holds.
extern "C" int nt_probe_rate(int kind, int waves_per_simd, int iters, float* ms, int* per_iter) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
    return 1;
  }
  if (waves_per_simd < 1 || waves_per_simd > 3 || iters < 1) return 2;
  switch (kind) {
    case kFma: *per_iter = 64; return run<0, 64, 0, 0, 0>(waves_per_simd, iters, cus, ms);
    case kExp32: *per_iter = 64; return run<0, 0, 64, 0, 0>(waves_per_simd, iters, cus, ms);
    case kExp16: *per_iter = 64; return run<0, 0, 0, 64, kExp16>(waves_per_simd, iters, cus, ms);
    case kCvtPk: *per_iter = 64; return run<0, 0, 0, 64, kCvtPk>(waves_per_simd, iters, cus, ms);
    case kDot2: *per_iter = 64; return run<0, 0, 0, 64, kDot2>(waves_per_simd, iters, cus, ms);
    case kMax3: *per_iter = 64; return run<0, 0, 0, 64, kMax3>(waves_per_simd, iters, cus, ms);
    case kMfma: *per_iter = 16; return run<16, 0, 0, 0, 0>(waves_per_simd, iters, cus, ms);
    case kLds128: *per_iter = 32; return run<0, 0, 0, 32, kLds128>(waves_per_simd, iters, cus, ms);
    case kMfmaFma: *per_iter = 1; return run<16, 128, 0, 0, 0>(waves_per_simd, iters, cus, ms);
    case kMfmaExp: *per_iter = 1; return run<16, 0, 32, 0, 0>(waves_per_simd, iters, cus, ms);
    case kMfmaFmaExp: *per_iter = 1; return run<16, 128, 32, 0, 0>(waves_per_simd, iters, cus, ms);
    case kMfmaV: *per_iter = 16; return run<16, 0, 0, 0, kAccInVgpr>(waves_per_simd, iters, cus, ms);
    case kMfmaFmaExpV: *per_iter = 1; return run<16, 128, 32, 0, kAccInVgpr>(waves_per_simd, iters, cus, ms);
    case kTileLike: *per_iter = 1; return run_tile_like<0>(waves_per_simd, iters, cus, ms);
    case kTileLikeLds: *per_iter = 1; return run_tile_like<1>(waves_per_simd, iters, cus, ms);
    case kTileLikeBarrier: *per_iter = 1; return run_tile_like<2>(waves_per_simd, iters, cus, ms);
    case kTileLikeLoads: *per_iter = 1; return run_tile_like<3>(waves_per_simd, iters, cus, ms);
    case kTileLikeRows: *per_iter = 1; return run_tile_like<4>(waves_per_simd, iters, cus, ms);
    case kTileLikeMaxFirst: *per_iter = 1; return run_tile_like<5>(waves_per_simd, iters, cus, ms);
    default: return 2;
  }
}

// The key-tile stream in full (LDS rows, stores, barrier, global loads, maximum
// test) on regular operands (noise == 0) or on operands with pseudo-random signs
// and mantissas: milliseconds of `iters` tiles with `waves_per_simd` wavefronts on
// every SIMD, and what the first workgroup counted on the shader clock and on the
// constant 100 MHz clock meanwhile (their ratio is the shader frequency the chip
// held under that load).
extern "C" int nt_probe_tile_clock(unsigned noise, int waves_per_simd, int iters, float* ms, float* shader_cycles,
                                   float* ticks_100mhz) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
    return 1;
  }
  if (waves_per_simd < 1 || waves_per_simd > 3 || iters < 1) return 2;
  float clocks[2] = {0.0f, 0.0f};
  const int rc = run_tile_like<5>(waves_per_simd, iters, cus, ms, noise, clocks);
  *shader_cycles = clocks[0];
  *ticks_100mhz = clocks[1];
  return rc;
}
