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

enum { kFma = 0, kExp32, kExp16, kCvtPk, kDot2, kMax3, kMfma, kLds128, kMfmaFma, kMfmaExp, kMfmaFmaExp, kKinds };

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
  for (int i = threadIdx.x; i < 8192; i += 256) reinterpret_cast<uint32_t*>(lds)[i] = i;
  __syncthreads();
  const float c0 = out[0], c1 = out[1];
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int n = 0; n < NM; ++n) acc[n & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[n & 3], 0, 0, 0);
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
    default: return 2;
  }
}
