// Packed projection GEMM for nested multi-head attention (gfx950 MFMA).
//
//   C[M, N] = A[M, K] * W[N, K]^T + bias[N]
//
// A is the packed token buffer viewed as [T, E] (no padded rows exist), W is a
// torch Linear weight, so both operands are K-contiguous: every MFMA operand
// fragment is one 16-byte run of a row.  A workgroup owns a BM x BN tile of C,
// its wavefronts a WAVES_M x WAVES_N grid of (WM*32) x (WN*32) sub-tiles made of
// 32x32 MFMA blocks (fp32 accumulate; f16 / bf16: v_mfma_f32_32x32x16_*, fp32:
// v_mfma_f32_32x32x2_f32).  K is walked in tiles of 128 bytes per row.  When K
// is a whole number of tiles the K tiles go from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no ds_write), two to three
// tiles resident, in an unpadded layout whose 16-byte pieces are XOR-swizzled so
// that the 128-bit fragment reads of 16 consecutive lanes fall into distinct
// banks; any other K takes a register-staged loop with padded LDS rows and
// element-wise tails.
//
// Three tile shapes are compiled for problems that fill the chip (256x128,
// 256x192, 256x256, eight wavefronts each); the launcher picks per problem the
// one with the least rounds x tile cost over the CUs.  The bigger tiles read less
// LDS per MFMA and win once the grid is several rounds deep; the smaller ones
// quantise better on the projection shapes of one attention layer.  A problem
// with fewer 256x128 tiles than half the CUs (the query and output projections
// of cross-attention, a few thousand rows) takes 128x64 tiles of four
// wavefronts, or 128x128 when those would not fit in one round: its duration is
// one tile's life, and a quarter of a tile on four times as many CUs ends sooner
// (3200 x 512 x 512: 10.6 -> 6.3 us; the fused in-projection of a layer of a few
// hundred tokens: 16.0 -> 11.6 us).
//
// Epilogues:
//   plain  - C row-major + bias;
//   QKV    - the fused in-projection of self-attention: columns [0, n_split)
//            (Q and K) go row-major into C, columns [n_split, N) (V) are written
//            TRANSPOSED into Vt[n - n_split][m] so that the attention kernel
//            finds V^T tiles key-contiguous.
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
};

template <> struct Mma<__bf16> {
  typedef bf16x8 Frag;
  static constexpr int kK = 16;
  static __device__ __forceinline__ acc16 run(Frag a, Frag b, acc16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// fp32: v_mfma_f32_32x32x2_f32 contracts two k values per instruction, one per
// lane half.  Which two is free as long as both operands agree, so a fragment is
// the same 16-byte piece of a row as for the 16-bit types (lane half g holds
// k = 8 s + 4 g .. + 3 of step s) and is spent over four instructions: the LDS
// reads are the conflict-free 128-bit ones of the swizzled layout instead of
// 4-byte column reads (which collide four to eight ways in it).
typedef float f32x4 __attribute__((ext_vector_type(4)));
template <> struct Mma<float> {
  typedef f32x4 Frag;
  static constexpr int kK = 8;
  static __device__ __forceinline__ acc16 run(Frag a, Frag b, acc16 c) {
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], c, 0, 0, 0);
  }
};

template <int WAVES_M_, int WAVES_N_, int WM_, int WN_, int BKB_>
struct GemmCfg {
  static constexpr int kWavesM = WAVES_M_, kWavesN = WAVES_N_, kWM = WM_, kWN = WN_;
  static constexpr int kThreads = 64 * WAVES_M_ * WAVES_N_;
  static constexpr int kWavesPerSimd = kThreads >= 512 ? 2 : 1;   // the kernel is compiled for this occupancy
  static constexpr int kBM = WAVES_M_ * WM_ * 32;
  static constexpr int kBN = WAVES_N_ * WN_ * 32;
  static constexpr int kRowBytes = BKB_;              // K-tile bytes per row
  static constexpr int kLdsRow = BKB_ + 16;           // padded LDS row
  static constexpr int kChunksPerRow = BKB_ / 16;
  static constexpr int kChunks = (kBM + kBN) * kChunksPerRow;
  static constexpr int kPerA = kBM * kChunksPerRow / kThreads;   // A pieces per thread
  static constexpr int kPerB = kBN * kChunksPerRow / kThreads;   // W pieces per thread
  static constexpr int kPerThread = kPerA + kPerB;
  static constexpr int kBufBytes = (kBM + kBN) * kLdsRow;
  // direct global -> LDS loads: unpadded rows, the K tiles of A and of W in a ring
  // each, three tiles deep if that fits and two otherwise.  (A third tile for only
  // one of the operands, which fits beside two whole tiles of the 256x192 shape, was
  // measured for either operand: no change, the K loop is not waiting for latency.)
  static constexpr int kATileBytes = kBM * BKB_;
  static constexpr int kBTileBytes = kBN * BKB_;
  static constexpr int kLdsBudget = 160 * 1024 - 2048;
  static constexpr bool kThreeOfBoth = 3 * (kATileBytes + kBTileBytes) <= kLdsBudget;
  static constexpr int kBufsB = kThreeOfBoth ? 3 : 2;
  static constexpr int kBufsA = kThreeOfBoth ? 3 : 2;
  static constexpr int kRingBytes = kBufsA * kATileBytes + kBufsB * kBTileBytes;
  // tile buffers (kernels for a ragged K use two padded, register-staged buffers)
  static constexpr int kLdsBytes = kRingBytes > 2 * kBufBytes ? kRingBytes : 2 * kBufBytes;
  static_assert((kBM * kChunksPerRow) % kThreads == 0 && (kBN * kChunksPerRow) % kThreads == 0,
                "tile pieces must divide among the threads");
};

template <typename T>
struct GemmArgs {
  const T* A;
  int64_t lda;
  const T* W;
  const T* bias;
  T* C;
  int64_t ldc;
  int64_t M, N, K;
  T* Vt;            // QKV epilogue: transposed destination of columns >= n_split
  int64_t ldvt;
  int64_t n_split;
  int act;          // row-major tiles: 0 none, 1 relu, 2 gelu (erf) applied to A W^T + bias
};

// The activation of a feed-forward layer, applied in fp32 before the one rounding
// of the epilogue (wavefront-uniform switch; `act` is a kernel argument).
__device__ __forceinline__ float apply_act(float v, int act) {
  if (act == 1) return fmaxf(v, 0.0f);
  if (act == 2) return gelu_erf(v);
  return v;
}

// 16-byte piece of a row at element k.
// ALIGNED_K (K is a multiple of the K tile): branch-free and mask-free.
// Out-of-range rows are clamped to the last row -- they only feed accumulators
// that are never stored -- and the caller clamps the K tile index, so every
// address is valid and nothing has to be zeroed.  This matters: control flow
// around the loads, or a mask applied to the loaded value, makes the wavefront
// wait for the load right away and serialises the global-load / MFMA pipeline.
// Otherwise (any K): element-wise tail handling.
template <typename T, bool ALIGNED_K>
__device__ __forceinline__ u32x4 load_chunk(const T* base, int64_t ld, int64_t row, int64_t nrows,
                                            int64_t k, int64_t K) {
  constexpr int kPer = 16 / sizeof(T);
  if (ALIGNED_K) {
    const int64_t r = row < nrows ? row : nrows - 1;
    return load16_unaligned(reinterpret_cast<const char*>(base + r * ld + k));
  }
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

// kEpiAct: the plain epilogue with the activation of GemmArgs::act; a kernel of
// its own, because even a never-taken activation branch in the plain epilogue
// costs the projection GEMMs 10 % (measured)
enum { kEpiPlain = 0, kEpiQkv = 1, kEpiAct = 2 };

// One BM x BN tile.  VT_OUT marks a V tile of the fused QKV projection, whose
// result goes transposed into Vt.
//
// The accumulators of a 32x32 MFMA block hold, per lane, four runs of four
// consecutive rows of one column of D.  Both operand fragments have the same
// register layout, so exchanging them transposes D for free: a tile that goes
// row-major into C is computed as C^T (a lane then holds runs of four
// consecutive COLUMNS of one row of C), a V tile as C (runs of four consecutive
// tokens of one feature = consecutive elements of a Vt row).  The epilogue
// moves each 32-row strip through a private LDS region of the wavefront, 8 or
// 16 bytes per lane in, and back out as 16-byte pieces of whole rows, so the
// global stores are row-contiguous instead of 2 bytes per lane.
template <typename T, class Cfg, bool VT_OUT, bool ALIGNED_K, bool ACT = false>
__device__ __forceinline__ void gemm_tile(const GemmArgs<T>& a, int64_t m0, int64_t n0, char* lds) {
  typedef Mma<T> MM;
  typedef typename MM::Frag Frag;
  constexpr int kPer = 16 / sizeof(T);
  constexpr int kBK = Cfg::kRowBytes / sizeof(T);
  constexpr int kSteps = kBK / MM::kK;
  constexpr int kFragBytes = (MM::kK / 2) * sizeof(T);
  constexpr int WM = Cfg::kWM, WN = Cfg::kWN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / Cfg::kWavesN;
  const int wn = wave % Cfg::kWavesN;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  acc16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  const int64_t nk = (a.K + kBK - 1) / kBK;

  // bias of the tile's columns as fp32, behind the tile buffers (visible after
  // the first barrier below)
  if (tid < Cfg::kBN) {
    const int64_t col = n0 + tid;
    reinterpret_cast<float*>(lds + Cfg::kLdsBytes)[tid] =
        (a.bias && col < a.N) ? (float)a.bias[col] : 0.0f;
  }

  if (ALIGNED_K) {
    // K tiles travel global -> LDS directly (global_load_lds_dwordx4): no staging
    // registers, no ds_write instructions.  A wavefront-level load writes its 64
    // 16-byte pieces to 1 KiB of consecutive LDS, i.e. eight unpadded 128-byte rows,
    // so bank conflicts of the fragment reads are avoided by WHICH piece of the row a
    // lane fetches: slot p of row r holds piece p ^ ((r >> 1) & 7).  The compiler
    // does not see these loads (inline asm), so their completion is awaited by hand
    // before the barrier that publishes the tile.  The asm writes M0 (the LDS
    // destination).  M0 cannot be declared as a clobber: the compiler treats it as a
    // reserved register, warns and ignores the entry.  The s_mov and the load that
    // reads M0 sit in one asm statement, so the compiler cannot put anything
    // between them; in the other direction the rule for this file is that nothing
    // makes the compiler keep a value of its own in M0 across these statements (no
    // LDS-direct builtin, no dynamic register indexing, no sendmsg).
    static_assert(Cfg::kRowBytes == 128 && Cfg::kBM % 64 == 0 && Cfg::kBN % 64 == 0,
                  "1 KiB blocks of eight rows, a whole number of them per wavefront");
    constexpr int kWaves = Cfg::kThreads / 64;
    constexpr int kNA = Cfg::kBM / 8 / kWaves;      // 1 KiB blocks of an A tile per wavefront
    constexpr int kNW = Cfg::kBN / 8 / kWaves;      // ... of a W tile
    constexpr int kRA = Cfg::kBufsA, kRW = Cfg::kBufsB;
    static_assert(kRA >= 2 && kRW >= 2 && kRA - kRW <= 1 && kRW - kRA <= 1, "the wait below counts on the issue order");
    constexpr bool kWLast = kRW > kRA;              // the deeper ring is issued last in an iteration
    constexpr int kInFlight = (kRA - 2) * kNA + (kRW - 2) * kNW;   // loads that may be outstanding at a barrier
    static_assert(kInFlight <= 63, "vmcnt is a 6-bit counter");
    const char* aptr[kNA];
    const char* wptr[kNW];
#pragma unroll
    for (int i = 0; i < kNA; ++i) {
      const int r = (i * kWaves + wave) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      int64_t row = m0 + r;
      row = row < a.M ? row : a.M - 1;
      aptr[i] = reinterpret_cast<const char*>(a.A + row * a.lda + c * kPer);
    }
#pragma unroll
    for (int i = 0; i < kNW; ++i) {
      const int r = (i * kWaves + wave) * 8 + (lane >> 3);
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      int64_t row = n0 + r;
      row = row < a.N ? row : a.N - 1;
      wptr[i] = reinterpret_cast<const char*>(a.W + row * a.K + c * kPer);
    }
    const unsigned lds_base = (unsigned)reinterpret_cast<uintptr_t>(lds);
    constexpr int kWRing = kRA * Cfg::kATileBytes;          // the W ring lies behind the A ring
    auto dma_a = [&](int buf, int64_t kt_in) {
      const int64_t kt = kt_in >= nk ? nk - 1 : kt_in;    // past the end: re-read, never used
#pragma unroll
      for (int i = 0; i < kNA; ++i) {
        const unsigned dst = __builtin_amdgcn_readfirstlane(
            lds_base + (unsigned)(buf * Cfg::kATileBytes + (i * kWaves + wave) * 1024));
        const char* src = aptr[i] + kt * Cfg::kRowBytes;
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :: "v"(src), "s"(dst) : "memory");
      }
    };
    auto dma_w = [&](int buf, int64_t kt_in) {
      const int64_t kt = kt_in >= nk ? nk - 1 : kt_in;
#pragma unroll
      for (int i = 0; i < kNW; ++i) {
        const unsigned dst = __builtin_amdgcn_readfirstlane(
            lds_base + (unsigned)(kWRing + buf * Cfg::kBTileBytes + (i * kWaves + wave) * 1024));
        const char* src = wptr[i] + kt * Cfg::kRowBytes;
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :: "v"(src), "s"(dst) : "memory");
      }
    };
    const int sw = (l32 >> 1) & 7;
    auto read_frags = [&](Frag* fa, Frag* fb, int abuf, int wbuf, int s) {
      const char* a_base = lds + abuf * Cfg::kATileBytes + (wm * WM * 32 + l32) * 128;
      const char* b_base = lds + kWRing + wbuf * Cfg::kBTileBytes + (wn * WN * 32 + l32) * 128;
      const int off = s * MM::kK * (int)sizeof(T) + g * kFragBytes;   // byte offset in the row
      const int koff = ((((off >> 4) ^ sw)) << 4) | (off & 15);
#pragma unroll
      for (int i = 0; i < WM; ++i)
        fa[i] = *reinterpret_cast<const Frag*>(a_base + i * 32 * 128 + koff);
#pragma unroll
      for (int j = 0; j < WN; ++j)
        fb[j] = *reinterpret_cast<const Frag*>(b_base + j * 32 * 128 + koff);
    };
    // While K tile kt is multiplied, the tiles kt + 1 .. kt + kRA - 1 of A and
    // kt + 1 .. kt + kRW - 1 of W are resident or in flight.  Loads complete in the
    // order of issue and every iteration issues the tile of the deeper ring last,
    // so when at most kInFlight loads are outstanding, tile kt + 1 of both has landed.
    // Prologue: tiles in the order the loop would have issued them.
#pragma unroll
    for (int j = 0; j < (kRA > kRW ? kRA : kRW) - 1; ++j) {
      if (!kWLast && j < kRW - 1) dma_w(j, j);
      if (j < kRA - 1) dma_a(j, j);
      if (kWLast && j < kRW - 1) dma_w(j, j);
    }
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kInFlight) : "memory");
    __syncthreads();
    int abuf = 0, wbuf = 0;
    Frag fa[2][WM], fb[2][WN];
    for (int64_t kt = 0; kt < nk; ++kt) {
      // (kt + kR - 1) % kR: free since the last barrier
      // This iteration's loads (the tile of the shallower ring first) are not issued
      // in one burst: a DMA load occupies the issuing wavefront until the memory
      // path has taken its 64 addresses, so a burst keeps every wavefront of the
      // workgroup from its matrix instructions at the same time.  They are dealt out
      // behind the k-steps instead.
      const int a_new = abuf == 0 ? kRA - 1 : abuf - 1;     // (kt + kR - 1) % kR: free since the last barrier
      const int w_new = wbuf == 0 ? kRW - 1 : wbuf - 1;
      const int64_t a_kt = kt + kRA - 1 >= nk ? nk - 1 : kt + kRA - 1;   // past the end: re-read, never used
      const int64_t w_kt = kt + kRW - 1 >= nk ? nk - 1 : kt + kRW - 1;
      auto dma_one = [&](int idx) {
        const bool is_w = kWLast ? idx >= kNA : idx < kNW;
        const int i = kWLast ? (is_w ? idx - kNA : idx) : (is_w ? idx : idx - kNW);
        const unsigned off = is_w ? (unsigned)(kWRing + w_new * Cfg::kBTileBytes) : (unsigned)(a_new * Cfg::kATileBytes);
        const unsigned dst = __builtin_amdgcn_readfirstlane(lds_base + off + (unsigned)((i * kWaves + wave) * 1024));
        const char* src = is_w ? wptr[i] + w_kt * Cfg::kRowBytes : aptr[i] + a_kt * Cfg::kRowBytes;
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :: "v"(src), "s"(dst) : "memory");
      };
      constexpr int kLoads = kNA + kNW;
      read_frags(fa[0], fb[0], abuf, wbuf, 0);
#pragma unroll
      for (int s = 0; s < kSteps; ++s) {
        if (s + 1 < kSteps) read_frags(fa[(s + 1) & 1], fb[(s + 1) & 1], abuf, wbuf, s + 1);
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int jj = 0; jj < WN; ++jj) {
            if (VT_OUT) {
              acc[i][jj] = MM::run(fa[s & 1][i], fb[s & 1][jj], acc[i][jj]);
            } else {
              acc[i][jj] = MM::run(fb[s & 1][jj], fa[s & 1][i], acc[i][jj]);
            }
          }
#pragma unroll
        for (int idx = s * kLoads / kSteps; idx < (s + 1) * kLoads / kSteps; ++idx) dma_one(idx);
        __builtin_amdgcn_sched_barrier(0);
      }
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kInFlight) : "memory");
      __syncthreads();
      abuf = abuf + 1 == kRA ? 0 : abuf + 1;
      wbuf = wbuf + 1 == kRW ? 0 : wbuf + 1;
    }
    // The last iterations issued clamped re-reads of the last K tile; up to
    // kInFlight of them per lane may still be in flight, and their LDS destinations
    // overlap the strips of the epilogue.  Drain them, workgroup-wide.
    if (kInFlight > 0) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
  } else {
    // Any K: element-wise tails, one K tile in registers ahead of the MFMAs, two
    // padded LDS buffers.
    u32x4 stage[1][Cfg::kPerThread];
    auto gload = [&](int64_t kt) {
#pragma unroll
      for (int i = 0; i < Cfg::kPerA; ++i) {
        const int c = tid + i * Cfg::kThreads;
        stage[0][i] = load_chunk<T, false>(a.A, a.lda, m0 + c / Cfg::kChunksPerRow, a.M,
                                           kt * kBK + (c % Cfg::kChunksPerRow) * kPer, a.K);
      }
#pragma unroll
      for (int i = 0; i < Cfg::kPerB; ++i) {
        const int c = tid + i * Cfg::kThreads;
        stage[0][Cfg::kPerA + i] =
            load_chunk<T, false>(a.W, a.K, n0 + c / Cfg::kChunksPerRow, a.N,
                                 kt * kBK + (c % Cfg::kChunksPerRow) * kPer, a.K);
      }
    };
    auto lstore = [&](int buf) {
      char* base = lds + buf * Cfg::kBufBytes;
#pragma unroll
      for (int i = 0; i < Cfg::kPerThread; ++i) {
        const bool is_a = i < Cfg::kPerA;
        const int c = tid + (is_a ? i : i - Cfg::kPerA) * Cfg::kThreads;
        const int row = (is_a ? 0 : Cfg::kBM) + c / Cfg::kChunksPerRow;
        store16(base + row * Cfg::kLdsRow + (c % Cfg::kChunksPerRow) * 16, stage[0][i]);
      }
    };
    gload(0);
    lstore(0);
    __syncthreads();
    for (int64_t kt = 0; kt < nk; ++kt) {
      const int buf = (int)(kt & 1);
      if (kt + 1 < nk) gload(kt + 1);
      const char* a_base = lds + buf * Cfg::kBufBytes + (wm * WM * 32 + l32) * Cfg::kLdsRow;
      const char* b_base =
          lds + buf * Cfg::kBufBytes + (Cfg::kBM + wn * WN * 32 + l32) * Cfg::kLdsRow;
#pragma unroll
      for (int s = 0; s < kSteps; ++s) {
        const int koff = s * MM::kK * (int)sizeof(T) + g * kFragBytes;
        Frag fa[WM], fb[WN];
#pragma unroll
        for (int i = 0; i < WM; ++i)
          fa[i] = *reinterpret_cast<const Frag*>(a_base + i * 32 * Cfg::kLdsRow + koff);
#pragma unroll
        for (int j = 0; j < WN; ++j)
          fb[j] = *reinterpret_cast<const Frag*>(b_base + j * 32 * Cfg::kLdsRow + koff);
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j) {
            if (VT_OUT) {
              acc[i][j] = MM::run(fa[i], fb[j], acc[i][j]);
            } else {
              acc[i][j] = MM::run(fb[j], fa[i], acc[i][j]);
            }
          }
      }
      if (kt + 1 < nk) lstore(buf ^ 1);
      __syncthreads();
    }
  }

  // ---- epilogue ----------------------------------------------------------
  // (the K loop ended with a barrier and no load into LDS is outstanding: the tile
  // buffers are free)
  constexpr int kStripW = VT_OUT ? WM : WN;                    // 32-wide blocks per strip row
  constexpr int kStripRow = kStripW * 32 * (int)sizeof(T) + 16;
  constexpr int kCpr = kStripW * 32 * (int)sizeof(T) / 16;    // 16-byte pieces per strip row
  static_assert((Cfg::kThreads / 64) * 32 * kStripRow <= Cfg::kLdsBytes, "strips must fit");
  char* strip = lds + wave * (32 * kStripRow);
  const float* lds_bias = reinterpret_cast<const float*>(lds + Cfg::kLdsBytes);
  typedef T Quad __attribute__((ext_vector_type(4)));

  if (!VT_OUT) {
    // acc[i][j][e] = C[row, col], row = .. + i*32 + l32, col = .. + j*32 + 8*(e/4) + 4*g + e%4
    const bool row_vec_ok = (a.ldc * (int64_t)sizeof(T)) % 16 == 0 &&
                            reinterpret_cast<uintptr_t>(a.C) % 16 == 0;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
      for (int j = 0; j < WN; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int c0 = j * 32 + 8 * r + 4 * g;
          const float4 bv = *reinterpret_cast<const float4*>(lds_bias + wn * WN * 32 + c0);
          Quad q;
          if (!ACT) {
            q[0] = (T)(acc[i][j][4 * r + 0] + bv.x);
            q[1] = (T)(acc[i][j][4 * r + 1] + bv.y);
            q[2] = (T)(acc[i][j][4 * r + 2] + bv.z);
            q[3] = (T)(acc[i][j][4 * r + 3] + bv.w);
          } else {
            q[0] = (T)apply_act(acc[i][j][4 * r + 0] + bv.x, a.act);
            q[1] = (T)apply_act(acc[i][j][4 * r + 1] + bv.y, a.act);
            q[2] = (T)apply_act(acc[i][j][4 * r + 2] + bv.z, a.act);
            q[3] = (T)apply_act(acc[i][j][4 * r + 3] + bv.w, a.act);
          }
          *reinterpret_cast<Quad*>(strip + l32 * kStripRow + c0 * (int)sizeof(T)) = q;
        }
      }
      __builtin_amdgcn_wave_barrier();   // LDS serves a wavefront's accesses in order
#pragma unroll
      for (int it = 0; it < 32 * kCpr / 64; ++it) {
        const int idx = it * 64 + lane;
        const int r = idx / kCpr, c = idx % kCpr;
        const int64_t row = m0 + (wm * WM + i) * 32 + r;
        const int64_t col = n0 + wn * WN * 32 + c * kPer;
        const u32x4 v = *reinterpret_cast<const u32x4*>(strip + r * kStripRow + c * 16);
        if (row < a.M && col < a.N) {
          T* dst = a.C + row * a.ldc + col;
          if (row_vec_ok && col + kPer <= a.N) {
            store16(reinterpret_cast<char*>(dst), v);
          } else {
            T tmp[kPer];
            __builtin_memcpy(tmp, &v, 16);
#pragma unroll
            for (int e = 0; e < kPer; ++e)
              if (col + e < a.N) dst[e] = tmp[e];
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  } else {
    // acc[i][j][e] = C[row, col], row = .. + i*32 + 8*(e/4) + 4*g + e%4, col = .. + j*32 + l32
    const bool row_vec_ok = (a.ldvt * (int64_t)sizeof(T)) % 16 == 0 &&
                            reinterpret_cast<uintptr_t>(a.Vt) % 16 == 0;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const float bv = lds_bias[(wn * WN + j) * 32 + l32];
#pragma unroll
      for (int i = 0; i < WM; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          Quad q;
#pragma unroll
          for (int e = 0; e < 4; ++e) q[e] = (T)(acc[i][j][4 * r + e] + bv);
          *reinterpret_cast<Quad*>(strip + l32 * kStripRow +
                                   (i * 32 + 8 * r + 4 * g) * (int)sizeof(T)) = q;
        }
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int it = 0; it < 32 * kCpr / 64; ++it) {
        const int idx = it * 64 + lane;
        const int r = idx / kCpr, c = idx % kCpr;
        const int64_t col = n0 + (wn * WN + j) * 32 + r;           // feature
        const int64_t row = m0 + wm * WM * 32 + c * kPer;          // first token of the piece
        const u32x4 v = *reinterpret_cast<const u32x4*>(strip + r * kStripRow + c * 16);
        if (col < a.N && row < a.M) {
          T* dst = a.Vt + (col - a.n_split) * a.ldvt + row;
          if (row_vec_ok && row + kPer <= a.M) {
            store16(reinterpret_cast<char*>(dst), v);
          } else {
            T tmp[kPer];
            __builtin_memcpy(tmp, &v, 16);
#pragma unroll
            for (int e = 0; e < kPer; ++e)
              if (row + e < a.M) dst[e] = tmp[e];
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

// Workgroup i runs on XCD i % 8 and every XCD has its own L2.  The tile order
// gives XCD x the row tiles x, x + 8, x + 16, ... for every column panel, one
// column panel after the other: its share of A (an eighth of the rows) stays
// L2-resident while the W panels stream through, so A leaves HBM once instead
// of once per column panel.
// The second launch bound (wavefronts per SIMD the kernel is compiled for) is
// what lets the compiler keep a whole K tile of fragments in registers: left at
// its default it schedules for maximum occupancy, keeps three fragments live
// and waits for LDS in front of every MFMA.
template <typename T, class Cfg, int EPI, bool ALIGNED_K>
__global__ __launch_bounds__(Cfg::kThreads, Cfg::kWavesPerSimd) void linear_kernel(GemmArgs<T> a) {
  extern __shared__ __align__(16) char lds[];
  const int64_t tiles_m = (a.M + Cfg::kBM - 1) / Cfg::kBM;
  const int64_t per_xcd = (tiles_m + 7) / 8;
  const int64_t xcd = blockIdx.x & 7;
  const int64_t local = blockIdx.x >> 3;
  const int64_t tn = local / per_xcd;
  const int64_t tm = (local - tn * per_xcd) * 8 + xcd;
  if (tm >= tiles_m) return;
  const int64_t m0 = tm * Cfg::kBM;
  const int64_t n0 = tn * Cfg::kBN;
  if (EPI == kEpiQkv && n0 >= a.n_split) {
    gemm_tile<T, Cfg, true, ALIGNED_K>(a, m0, n0, lds);    // V tile: transposed into Vt
  } else {
    gemm_tile<T, Cfg, false, ALIGNED_K, EPI == kEpiAct>(a, m0, n0, lds);
  }
}

template <typename T, class Cfg, int EPI, bool ALIGNED_K>
static int launch_kernel(const GemmArgs<T>& a, hipStream_t stream) {
  const int64_t tiles_m = (a.M + Cfg::kBM - 1) / Cfg::kBM;
  const int64_t tiles_n = (a.N + Cfg::kBN - 1) / Cfg::kBN;
  const int64_t wgs = ((tiles_m + 7) / 8) * 8 * tiles_n;
  if (wgs > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "linear: too many tiles");
  const int lds_bytes = Cfg::kLdsBytes + Cfg::kBN * (int)sizeof(float);
  static bool attr_set = false;
  if (!attr_set && lds_bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(
        reinterpret_cast<const void*>(linear_kernel<T, Cfg, EPI, ALIGNED_K>),
        hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return fail(NT_ERR_HIP, "linear: %s", hipGetErrorString(e));
    attr_set = true;
  }
  hipLaunchKernelGGL((linear_kernel<T, Cfg, EPI, ALIGNED_K>), dim3((unsigned)wgs),
                     dim3(Cfg::kThreads), lds_bytes, stream, a);
  return check_launch("linear_kernel");
}

template <typename T, class Cfg, int EPI>
static int launch_cfg(const GemmArgs<T>& a, hipStream_t stream) {
  // the branch-free loads need whole K tiles
  const bool aligned = a.K > 0 && a.K % (Cfg::kRowBytes / (int64_t)sizeof(T)) == 0;
  if (aligned) return launch_kernel<T, Cfg, EPI, true>(a, stream);
  return launch_kernel<T, Cfg, EPI, false>(a, stream);
}

// WAVES_M, WAVES_N, WM, WN, K-tile bytes per row
typedef GemmCfg<4, 2, 2, 2, 128> Cfg128;   // 256 x 128
typedef GemmCfg<4, 2, 2, 3, 128> Cfg192;   // 256 x 192
typedef GemmCfg<4, 2, 2, 4, 128> Cfg256;   // 256 x 256
typedef GemmCfg<2, 2, 2, 1, 128> CfgSmall; // 128 x 64, four wavefronts: problems of fewer 256-row tiles than CUs
typedef GemmCfg<2, 2, 2, 2, 128> CfgMid;   // 128 x 128, four wavefronts

// Tile shape with the least estimated time.  A tile costs its area divided by the
// measured steady-state rate of its shape relative to 256x128 (wider wavefront
// tiles read less LDS and L2 per MFMA).  The number of tiles a CU runs one after
// the other is taken as the mean of the whole rounds (all tiles start together
// and take equally long) and of tiles / CUs (a partly filled last round runs
// faster, it shares the memory path with fewer workgroups); fitted on the
// projection shapes of the two attention benchmarks and on large square problems.
static int pick_cfg(int64_t M, int64_t N, int64_t n_split, int* which) {
  static int num_cus = 0;
  if (num_cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess ||
        prop.multiProcessorCount < 1) {
      return fail(NT_ERR_HIP, "linear: cannot query the device");
    }
    num_cus = prop.multiProcessorCount;
  }
  const int bn[3] = {Cfg128::kBN, Cfg192::kBN, Cfg256::kBN};
  const double eff[3] = {1.0, 1.08, 1.17};
  int best = -1;
  double best_cost = 0.0;
  for (int c = 0; c < 3; ++c) {
    if (n_split % bn[c] != 0) continue;          // a tile must not straddle the K | V boundary
    const int64_t tiles = ((M + 255) / 256) * ((N + bn[c] - 1) / bn[c]);
    const double whole = (double)((tiles + num_cus - 1) / num_cus);
    const double fluid = (double)tiles / num_cus;
    const double cost = 0.5 * (whole + fluid) * bn[c] / eff[c];
    if (best < 0 || cost < best_cost) {
      best = c;
      best_cost = cost;
    }
  }
  if (best < 0) {
    return fail(NT_ERR_UNSUPPORTED, "linear: QKV split %lld is not a multiple of a column tile",
                (long long)n_split);
  }
  // Fewer 256 x 128 tiles than half the CUs: the launch is one tile's life on a
  // fraction of the chip, and a quarter-size tile on four times as many CUs is shorter.
  if (((M + 255) / 256) * ((N + 127) / 128) * 2 <= num_cus) {
    const int small = ((M + 127) / 128) * ((N + 63) / 64) <= num_cus ? 3 : 4;
    const int64_t small_bn = small == 3 ? CfgSmall::kBN : CfgMid::kBN;
    if (n_split % small_bn == 0) best = small;   // (a tile must not straddle the K | V boundary)
  }
  *which = best;
  return NT_OK;
}

template <typename T, int EPI>
static int launch_epi(const GemmArgs<T>& a, hipStream_t stream) {
  int which = 0;
  // the fp32 path exists for parity checks; it is compiled for one shape only
  if constexpr (sizeof(T) == 4) {
    if (EPI == kEpiQkv && a.n_split % Cfg128::kBN != 0) {
      return fail(NT_ERR_UNSUPPORTED, "linear: QKV split %lld is not a multiple of the column tile",
                  (long long)a.n_split);
    }
    return launch_cfg<T, Cfg128, EPI>(a, stream);
  } else {
    const int rc = pick_cfg(a.M, a.N, EPI == kEpiQkv ? a.n_split : 0, &which);
    if (rc != NT_OK) return rc;
    if (which == 3) return launch_cfg<T, CfgSmall, EPI>(a, stream);
    if (which == 4) return launch_cfg<T, CfgMid, EPI>(a, stream);
    if (which == 1) return launch_cfg<T, Cfg192, EPI>(a, stream);
    if (which == 2) return launch_cfg<T, Cfg256, EPI>(a, stream);
    return launch_cfg<T, Cfg128, EPI>(a, stream);
  }
}

template <typename T>
static int launch_linear(GemmArgs<T> a, bool qkv, hipStream_t stream) {
  if (qkv) return launch_epi<T, kEpiQkv>(a, stream);
  if (a.act != 0) return launch_epi<T, kEpiAct>(a, stream);
  return launch_epi<T, kEpiPlain>(a, stream);
}

static int check_linear(const void* A, int64_t lda, const void* W, const void* C, int64_t ldc,
                        int64_t M, int64_t N, int64_t K) {
  if (M < 0 || N < 0 || K < 0 || lda < K || ldc < 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "linear: bad shape M=%lld N=%lld K=%lld lda=%lld ldc=%lld",
                (long long)M, (long long)N, (long long)K, (long long)lda, (long long)ldc);
  }
  if (M > 0 && N > 0 && (!A || !W || !C)) return fail(NT_ERR_INVALID_ARGUMENT, "linear: NULL pointer");
  return NT_OK;
}

template <typename T>
static GemmArgs<T> make_args(const void* A, int64_t lda, const void* W, const void* bias, void* C,
                             int64_t ldc, int64_t M, int64_t N, int64_t K) {
  GemmArgs<T> a;
  a.A = static_cast<const T*>(A);
  a.lda = lda;
  a.W = static_cast<const T*>(W);
  a.bias = static_cast<const T*>(bias);
  a.C = static_cast<T*>(C);
  a.ldc = ldc;
  a.M = M;
  a.N = N;
  a.K = K;
  a.Vt = nullptr;
  a.ldvt = 0;
  a.n_split = N;
  a.act = 0;
  return a;
}

}  // namespace nt

using namespace nt;

extern "C" int nt_linear_act(const void* A, int64_t lda, const void* W, const void* bias, void* C,
                             int64_t ldc, int64_t M, int64_t N, int64_t K, int act, int dtype,
                             void* stream) {
  int rc = check_linear(A, lda, W, C, ldc, M, N, K);
  if (rc != NT_OK) return rc;
  if (ldc < N) return fail(NT_ERR_INVALID_ARGUMENT, "linear: ldc %lld < N %lld", (long long)ldc, (long long)N);
  if (act < 0 || act > 2) return fail(NT_ERR_INVALID_ARGUMENT, "linear: activation %d is not 0, 1 or 2", act);
  if (M == 0 || N == 0) return NT_OK;
  hipStream_t s = (hipStream_t)stream;
#define NT_LIN_CASE(TYPE)                                                   \
  {                                                                         \
    GemmArgs<TYPE> a = make_args<TYPE>(A, lda, W, bias, C, ldc, M, N, K);   \
    a.act = act;                                                            \
    return launch_linear<TYPE>(a, false, s);                                \
  }
  switch (dtype) {
    case NT_F32: NT_LIN_CASE(float)
    case NT_F16: NT_LIN_CASE(_Float16)
    case NT_BF16: NT_LIN_CASE(__bf16)
    default: return fail(NT_ERR_INVALID_ARGUMENT, "linear: unknown dtype %d", dtype);
  }
#undef NT_LIN_CASE
}

extern "C" int nt_linear(const void* A, int64_t lda, const void* W, const void* bias, void* C,
                         int64_t ldc, int64_t M, int64_t N, int64_t K, int dtype, void* stream) {
  return nt_linear_act(A, lda, W, bias, C, ldc, M, N, K, 0, dtype, stream);
}

extern "C" int nt_linear_qkv(const void* A, int64_t lda, const void* W, const void* bias, void* QK,
                             int64_t ldqk, void* Vt, int64_t ldvt, int64_t M, int64_t E, int64_t K,
                             int dtype, void* stream) {
  int rc = check_linear(A, lda, W, QK, ldqk, M, 3 * E, K);
  if (rc != NT_OK) return rc;
  if (ldqk < 2 * E || ldvt < M) {
    return fail(NT_ERR_INVALID_ARGUMENT, "linear_qkv: ldqk %lld < 2E or ldvt %lld < M",
                (long long)ldqk, (long long)ldvt);
  }
  if (M == 0 || E == 0) return NT_OK;
  if (!Vt) return fail(NT_ERR_INVALID_ARGUMENT, "linear_qkv: Vt is NULL");
  hipStream_t s = (hipStream_t)stream;
#define NT_QKV_CASE(TYPE)                                                       \
  {                                                                             \
    GemmArgs<TYPE> a = make_args<TYPE>(A, lda, W, bias, QK, ldqk, M, 3 * E, K); \
    a.Vt = static_cast<TYPE*>(Vt);                                              \
    a.ldvt = ldvt;                                                              \
    a.n_split = 2 * E;                                                          \
    return launch_linear<TYPE>(a, true, s);                                     \
  }
  switch (dtype) {
    case NT_F32: NT_QKV_CASE(float)
    case NT_F16: NT_QKV_CASE(_Float16)
    case NT_BF16: NT_QKV_CASE(__bf16)
    default: return fail(NT_ERR_INVALID_ARGUMENT, "linear_qkv: unknown dtype %d", dtype);
  }
#undef NT_QKV_CASE
}

extern "C" int nt_linear_kv(const void* A, int64_t lda, const void* W, const void* bias, void* Kout,
                            int64_t ldk, void* Vt, int64_t ldvt, int64_t M, int64_t E, int64_t K, int dtype,
                            void* stream) {
  int rc = check_linear(A, lda, W, Kout, ldk, M, 2 * E, K);
  if (rc != NT_OK) return rc;
  if (ldk < E || ldvt < M) {
    return fail(NT_ERR_INVALID_ARGUMENT, "linear_kv: ldk %lld < E or ldvt %lld < M", (long long)ldk, (long long)ldvt);
  }
  if (M == 0 || E == 0) return NT_OK;
  if (!Vt) return fail(NT_ERR_INVALID_ARGUMENT, "linear_kv: Vt is NULL");
  hipStream_t s = (hipStream_t)stream;
  // the fused in-projection's kernel with the row-major | transposed boundary at column E
#define NT_KV_CASE(TYPE)                                                        \
  {                                                                             \
    GemmArgs<TYPE> a = make_args<TYPE>(A, lda, W, bias, Kout, ldk, M, 2 * E, K); \
    a.Vt = static_cast<TYPE*>(Vt);                                              \
    a.ldvt = ldvt;                                                              \
    a.n_split = E;                                                              \
    return launch_linear<TYPE>(a, true, s);                                     \
  }
  switch (dtype) {
    case NT_F32: NT_KV_CASE(float)
    case NT_F16: NT_KV_CASE(_Float16)
    case NT_BF16: NT_KV_CASE(__bf16)
    default: return fail(NT_ERR_INVALID_ARGUMENT, "linear_kv: unknown dtype %d", dtype);
  }
#undef NT_KV_CASE
}

extern "C" int nt_linear_transposed(const void* A, int64_t lda, const void* W, const void* bias,
                                    void* Ct, int64_t ldct, int64_t M, int64_t N, int64_t K, int dtype,
                                    void* stream) {
  int rc = check_linear(A, lda, W, Ct, ldct, M, N, K);
  if (rc != NT_OK) return rc;
  if (ldct < M) {
    return fail(NT_ERR_INVALID_ARGUMENT, "linear_transposed: ldct %lld < M %lld", (long long)ldct,
                (long long)M);
  }
  if (M == 0 || N == 0) return NT_OK;
  hipStream_t s = (hipStream_t)stream;
  // every tile is a transposed-output tile of the fused QKV kernel: split at column 0
#define NT_LT_CASE(TYPE)                                                     \
  {                                                                          \
    GemmArgs<TYPE> a = make_args<TYPE>(A, lda, W, bias, Ct, ldct, M, N, K);  \
    a.C = nullptr;                                                           \
    a.Vt = static_cast<TYPE*>(Ct);                                           \
    a.ldvt = ldct;                                                           \
    a.n_split = 0;                                                           \
    return launch_linear<TYPE>(a, true, s);                                  \
  }
  switch (dtype) {
    case NT_F32: NT_LT_CASE(float)
    case NT_F16: NT_LT_CASE(_Float16)
    case NT_BF16: NT_LT_CASE(__bf16)
    default: return fail(NT_ERR_INVALID_ARGUMENT, "linear_transposed: unknown dtype %d", dtype);
  }
#undef NT_LT_CASE
}
