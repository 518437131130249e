// Variable-length attention from a plan: persistent workgroups that stream the keys
// and values of a sequence through LDS in large segments (gfx950, head_dim 64,
// f16 / bf16).  An alternative structure to varlen_attention_vt_kernel
// (attention.hip) with the same results to rounding; measured on the attention
// benchmarks of this library it is the slower of the two (C3: 30 us against 27 us),
// so the host layer uses it only on request.
//
// The reference's chain is pad -> QK^T -> masked softmax -> PV -> un-pad over a
// [B, H, Lmax, Lmax] score tensor (csrc/cuda/mha.cpp:57-106, attention.cu:182-482).
// Here one workgroup per compute unit (twelve wavefronts, three per SIMD, 128 KiB
// of LDS) walks a list of STEPS that the host planned from the nested size.  A
// step brings up to four key tiles (64 keys each: a K tile and the matching V^T
// tile, 16 KiB) from global memory straight into one of two LDS segments
// (global_load_lds_dwordx4, no staging registers) while the previous step is
// being computed, and gives every wavefront one block of 32 query rows together
// with the range of tiles that holds its sequence's keys.  Long sequences: the
// wavefronts are up to twelve query blocks of ONE sequence and a chain of steps
// streams its keys, 256 per step, with the softmax state carried in registers; K
// and V^T are read once per 384 query rows and there is ONE barrier per 256 keys.
// Short sequences: a step holds several of them side by side (their tiles share
// the segment, each wavefront works on its own sequence), so no wavefront idles
// because a sequence has fewer than 384 rows.
//
// Per wavefront the arithmetic is that of varlen_attention_vt_kernel: S^T = K Q^T
// and O^T += V^T P^T on v_mfma_f32_32x32x16, one query row per lane, scores
// leaving the matrix pipe relative to a lazily moved reference maximum,
// denominators from the rounded probabilities.
//
// LDS layout of a tile: 64 rows of 128 bytes, unpadded (a wavefront-level DMA
// load fills 1 KiB = eight rows); the eight 16-byte pieces of row r are
// XOR-swizzled, slot p holds piece p ^ ((r >> 1) & 7), which makes the 128-bit
// fragment reads conflict-free.  LDS row rho of a K tile holds key perm(rho)
// (bits 2 and 3 of the index exchanged), the permutation that lets the score
// accumulators serve as the B operand of the second product as they stand.
//
// What the measurements say about this structure (traces and ablations of this
// kernel): a DMA load occupies the issuing wavefront until the memory path has
// taken its addresses, so a step's loads are dealt out behind the tiles; the
// descriptors are fetched with two wide scalar loads a step ahead; the code is
// kept to one instance of the tile body because a launch starts with a cold
// instruction cache.  With all of that a key tile still costs a SIMD about 770 ns
// of issue, whether two or three wavefronts share it: the vector and matrix
// instructions of a tile barely overlap on this part, and the work-list kernel,
// with three small workgroups per compute unit, hides its start-up better.
#include <algorithm>
#include <type_traits>
#include <vector>

#include "attn_common.h"

namespace nt {

constexpr int kChainWaves = 12;                // wavefronts per workgroup: three per SIMD
constexpr int kLoadWaves = 8;                  // the first eight move the tiles (eight 1 KiB blocks each)
constexpr int kSegSlots = 4;                   // key tiles per LDS segment
constexpr int kTileKeys = 64;
constexpr int kTileBytes = 8192;               // 64 rows x 128 bytes (head_dim 64)
constexpr int kSlotBytes = 2 * kTileBytes;     // K tile, then V^T tile
constexpr int kSegBytes = kSegSlots * kSlotBytes;
constexpr int kStepInts = 16 + 4 * kChainWaves; // 4 slots x 4 + 4 per wavefront
constexpr int kPlanHeader = 4;                 // {workgroups, offset of the steps (int32), steps, head_dim}

// Step descriptor (int32[kStepInts]):
//   slot s (4 ints at 4 s):   first key token of the tile, valid keys (0: slot unused),
//                             last key token of the sequence, head (slot 0 only)
//   wavefront w (16 + 4 w):   first query token of its block, query rows (0: idle),
//                             first slot | tiles << 4 | first-of-chain << 8 | last-of-chain << 9,
//                             valid keys of the last tile of its range (1..64)

template <typename T>
__global__ __launch_bounds__(64 * kChainWaves, kChainWaves / 4) void attention_chain_kernel(
    const T* __restrict__ Q, int64_t ldq, const T* __restrict__ K, int64_t ldk,
    const T* __restrict__ Vt, int64_t ldvt, T* __restrict__ O, int64_t ldo,
    const int32_t* __restrict__ plan, float scale_log2e) {
  typedef AttnT<T> AT;
  typedef typename AT::Frag Frag;
  constexpr int HD = 64, kQF = HD / 16, kDB = HD / 32;
  extern __shared__ __align__(16) char lds[];

  if ((int)blockIdx.x >= plan[0]) return;                   // uniform: launched wider than planned
  const int step_first = plan[kPlanHeader + blockIdx.x];
  const int step_end = plan[kPlanHeader + blockIdx.x + 1];
  if (step_first >= step_end) return;                       // uniform
  const int32_t* steps = plan + plan[1];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31;
  const int g = lane >> 5;
  const unsigned lds_base = (unsigned)reinterpret_cast<uintptr_t>(lds);

  // ---- global -> LDS: this wavefront moves rows 8 w .. 8 w + 7 of every K tile and
  // of every V^T tile of a step (one 1 KiB DMA load each)
  const int rho = 8 * wave + (lane >> 3);                               // LDS row of the tile
  const int piece = (lane & 7) ^ ((rho >> 1) & 7);                      // piece that lies in slot lane & 7
  const int key_of_row = (rho & ~12) | ((rho & 4) << 1) | ((rho & 8) >> 1);
  const int k_row_bytes = (int)(ldk * (int64_t)sizeof(T));               // the launcher checked that 64 rows fit 31 bits
  const int64_t v_lane_off = ((int64_t)rho * ldvt + piece * 8) * (int64_t)sizeof(T);
  // A step's descriptor as it is fetched: the four slots in one 64-byte scalar
  // load, this wavefront's entry in one of 16 bytes, both issued a step ahead of
  // their use so that no wavefront ever waits for a descriptor word by word.
  typedef int int16v __attribute__((ext_vector_type(16)));
  typedef int int4v __attribute__((ext_vector_type(4)));
  struct Desc {
    int16v d;       // slots
    int4v mine;     // this wavefront
  };
  auto load_desc = [&](int step) {
    const int32_t* p = steps + (int64_t)step * kStepInts;
    Desc r;
    r.d = *reinterpret_cast<const int16v*>(p);
    r.mine = *reinterpret_cast<const int4v*>(p + 16 + 4 * wave);
    return r;
  };
  // One slot of a step: two DMA loads per wavefront.  `s` is a run-time index; the
  // slot's words are picked with scalar selects (no register indexing: M0 belongs to
  // the DMA loads).  A load occupies the issuing wavefront until the memory path has
  // taken its 64 addresses, so the slots of the NEXT step are issued one by one
  // between the tiles of the current step, not all at once.
  auto issue_slot = [&](const Desc& ds, int buf, int s) {
    if (wave >= kLoadWaves) return;                                       // uniform per wavefront
    const int16v d = ds.d;
    const int tok0 = s == 0 ? d[0] : s == 1 ? d[4] : s == 2 ? d[8] : d[12];
    const int nv = s == 0 ? d[1] : s == 1 ? d[5] : s == 2 ? d[9] : d[13];
    const int last = s == 0 ? d[2] : s == 1 ? d[6] : s == 2 ? d[10] : d[14];
    if (nv == 0) return;                                                  // uniform
    const int h = d[3];
    // rows past the sequence's last key read that key again: valid memory, and a
    // copy of a valid key cannot raise the row maximum.  The tile's base address is
    // scalar arithmetic; a lane adds its row and piece.
    const int room = last - tok0;                                         // >= 0
    const int rel = key_of_row < room ? key_of_row : room;
    const char* kbase = reinterpret_cast<const char*>(K + (int64_t)tok0 * ldk + (int64_t)h * HD);
    const char* ksrc = kbase + (int64_t)(rel * k_row_bytes + piece * 16);
    const char* vbase = reinterpret_cast<const char*>(Vt + (int64_t)h * HD * ldvt + tok0);
    const char* vsrc = vbase + v_lane_off;
    const unsigned dst = lds_base + (unsigned)(buf * kSegBytes + s * kSlotBytes + wave * 1024);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(ksrc), "s"(dst) : "memory");
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(vsrc), "s"(dst + (unsigned)kTileBytes) : "memory");
  };
  // V^T columns of keys past the sequence's end are zeroed once the tile has
  // landed: their probabilities are zero, and 0 * x must not meet a NaN or an
  // infinity in whatever follows the sequence in memory.  A wavefront fixes the
  // rows it loaded itself, so its own wait for the loads is enough.
  auto sanitize = [&](const Desc& ds, int buf) {
    if (wave >= kLoadWaves) return;                                       // uniform per wavefront
    const int16v d = ds.d;
#pragma unroll
    for (int s = 0; s < kSegSlots; ++s) {
      const int nv = d[4 * s + 1];
      if (nv == 0 || nv >= kTileKeys) continue;                           // uniform
      int n = nv - piece * 8;
      n = n > 8 ? 8 : (n < 0 ? 0 : n);
      u32x4 m;
#pragma unroll
      for (int j = 0; j < 4; ++j) m[j] = n >= 2 * j + 2 ? 0xffffffffu : (n == 2 * j + 1 ? 0x0000ffffu : 0u);
      char* p = lds + buf * kSegBytes + s * kSlotBytes + kTileBytes + wave * 1024 + lane * 16;
      const u32x4 v = *reinterpret_cast<const u32x4*>(p);
      *reinterpret_cast<u32x4*>(p) = v & m;
    }
  };

  // ---- per-wavefront state of the chain ----
  Frag qf[kQF];
  u32x4 qn[kQF];                 // query fragments of the next chain, on their way
  acc16 o_acc[kDB];
  acc16 negm;                    // -m_ref in every element
  float l_run = 0.0f;
#pragma unroll
  for (int e = 0; e < 16; ++e) negm[e] = 0.0f;
#pragma unroll
  for (int i = 0; i < kDB; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
  auto fetch_q = [&](const Desc& ds) {
    const int nq = ds.mine[1];
    if (nq == 0 || !((ds.mine[2] >> 8) & 1)) return;                     // uniform per wavefront
    const int row = l32 < nq ? l32 : nq - 1;
    const T* qp = Q + ((int64_t)ds.mine[0] + row) * ldq + (int64_t)ds.d[3] * HD + g * 8;
#pragma unroll
    for (int s = 0; s < kQF; ++s) qn[s] = load16_unaligned(reinterpret_cast<const char*>(qp + s * 16));
  };

  // fragment addresses inside a tile: row l32 (+ 32 per block), piece 2 s + g
  const int sw = (l32 >> 1) & 7;
  int frag_off[kQF];
#pragma unroll
  for (int s = 0; s < kQF; ++s) frag_off[s] = l32 * 128 + (((2 * s + g) ^ sw) << 4);

#define NT_FENCE() __builtin_amdgcn_sched_barrier(0)
  // One key tile for this wavefront's 32 query rows; `slot_base` is the K tile,
  // the V^T tile follows it.  Same instruction order as varlen_attention_vt_kernel:
  // the exponentials of a k-step sit between the matrix instructions of the one
  // before it.  (One instance of this code only: a launch starts with a cold
  // instruction cache, and every copy of a path costs the workgroup its misses.)
  auto tile = [&](const char* slot_base, bool first, int n_last) {
    const bool partial = n_last < kTileKeys;
    Frag kf[2][kQF];
    auto read_k = [&](int kb, int s0, int s1) {
#pragma unroll
      for (int s = s0; s < s1; ++s)
        kf[kb][s] = *reinterpret_cast<const Frag*>(slot_base + kb * 4096 + frag_off[s]);
    };
    read_k(0, 0, kQF);
    read_k(1, 0, kQF / 2);
    NT_FENCE();
    acc16 sa[2];
#pragma unroll
    for (int s = 0; s < kQF; ++s) sa[0] = AT::mma(kf[0][s], qf[s], s == 0 ? negm : sa[0]);
    read_k(1, kQF / 2, kQF);
#pragma unroll
    for (int s = 0; s < kQF / 2; ++s) sa[1] = AT::mma(kf[1][s], qf[s], s == 0 ? negm : sa[1]);
    NT_FENCE();
    float m_tile = sa[0][0];
#pragma unroll
    for (int e = 1; e < 16; ++e) m_tile = fmaxf(m_tile, sa[0][e]);
    NT_FENCE();
#pragma unroll
    for (int s = kQF / 2; s < kQF; ++s) sa[1] = AT::mma(kf[1][s], qf[s], sa[1]);
    NT_FENCE();
    Frag vf[2][kDB];
    const char* vbase = slot_base + kTileBytes;
    auto read_v = [&](int ks) {
#pragma unroll
      for (int db = 0; db < kDB; ++db)
        vf[ks & 1][db] = *reinterpret_cast<const Frag*>(vbase + db * 4096 + frag_off[ks]);
    };
    read_v(0);
    NT_FENCE();
#pragma unroll
    for (int e = 0; e < 16; ++e) m_tile = fmaxf(m_tile, sa[1][e]);
    m_tile = max_across_halves(m_tile);
    // (last tile, fewer than 64 keys: the K rows past the last key are copies of it, so
    // they cannot have raised the maximum, and their V^T columns are zero; what they
    // add to the denominator is taken out below)
    if (__any(first ? fabsf(m_tile) > kLazyMaxLog2 : m_tile > kLazyMaxLog2)) {   // wavefront-uniform
      const float delta = first ? m_tile : fmaxf(m_tile, 0.0f);
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) sa[kb][e] -= delta;
#pragma unroll
      for (int e = 0; e < 16; ++e) negm[e] -= delta;
      if (!first) {
        const float alpha = __builtin_amdgcn_exp2f(-delta);
#pragma unroll
        for (int i = 0; i < kDB; ++i)
#pragma unroll
          for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;
        l_run *= alpha;
      }
    }
    // the compiler must not see that the elements of negm are equal: it would
    // rebuild the block from one register in front of every use
    asm volatile("" : "+v"(negm));
    float pr[8];
    uint32_t pw[4][4];
    auto exps = [&](int ks, int j0, int j1) {
#pragma unroll
      for (int j = j0; j < j1; ++j) pr[j] = __builtin_amdgcn_exp2f(sa[ks >> 1][(ks & 1) * 8 + j]);
    };
    auto cvts = [&](int ks) {
      // the denominator sums the rounded probabilities, the ones that meet V
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pw[ks][j] = AT::cvt2(pr[2 * j], pr[2 * j + 1]);
        l_run = AT::dot_ones(pw[ks][j], l_run);
      }
    };
    exps(0, 0, 8);
    cvts(0);
    NT_FENCE();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks < 3) read_v(ks + 1);
      Frag pf;
      __builtin_memcpy(&pf, pw[ks], 16);
      NT_FENCE();
#pragma unroll
      for (int m = 0; m < kDB; ++m) {
        o_acc[m] = AT::mma(vf[ks & 1][m], pf, o_acc[m]);
        NT_FENCE();
        if (ks < 3) {
          exps(ks + 1, 8 * m / kDB, 8 * (m + 1) / kDB);
          if (m == kDB - 1) cvts(ks + 1);
          NT_FENCE();
        }
      }
    }
    if (partial) {
      // every key past the end has exactly the probability of the last valid key
      // (its K row is a copy), and the highest key this lane half holds, 8 g + 55,
      // is one of them whenever the half holds any: the half holds keys
      // [8 g + 16 j, 8 g + 16 j + 8), j = 0..3
      int extra = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int over = 8 * g + 16 * j + 8 - n_last;
        over = over < 0 ? 0 : (over > 8 ? 8 : over);
        extra += over;
      }
      typename AT::Half last4;
      __builtin_memcpy(&last4, &pw[3][2], 8);
      l_run -= (float)extra * (float)last4[3];
    }
  };

  // ---- the walk over this workgroup's steps ----
  Desc cur = load_desc(step_first);
  Desc nxt = cur;
  fetch_q(cur);
  for (int sl = 0; sl < kSegSlots; ++sl) issue_slot(cur, 0, sl);
  for (int step = step_first; step < step_end; ++step) {
    const int buf = (step - step_first) & 1;
    const bool more = step + 1 < step_end;                  // uniform
    // the next step's descriptor starts travelling now; it is first needed after
    // this step's first tile
    if (more) nxt = load_desc(step + 1);
    // this wavefront's loads of the step have landed (and the query fragments, and
    // the result rows it stored before); then everybody's
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    sanitize(cur, buf);
    __syncthreads();
    // the other segment is free since that barrier: the next step travels while
    // this one is computed, one slot behind every tile
    const int q_tok = cur.mine[0], nq = cur.mine[1], bits = cur.mine[2], n_last = cur.mine[3];
    const int head = cur.d[3];
    const bool first = (bits >> 8) & 1, last = (bits >> 9) & 1;
    if (nq > 0 && first) {
#pragma unroll
      for (int s = 0; s < kQF; ++s) {
        Frag f;
        __builtin_memcpy(&f, &qn[s], 16);
        qf[s] = QScale<T>::run(f, scale_log2e);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) negm[e] = 0.0f;
#pragma unroll
      for (int i = 0; i < kDB; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
      l_run = 0.0f;
    }
    __builtin_amdgcn_sched_barrier(0);
    int sent = 0;
    if (nq > 0) {
      const int slot0 = bits & 15, nt_ = (bits >> 4) & 15;
      const char* seg = lds + buf * kSegBytes + slot0 * kSlotBytes;
      for (int t = 0; t < nt_; ++t) {
        tile(seg + t * kSlotBytes, first && t == 0, t == nt_ - 1 ? n_last : kTileKeys);
        if (more && sent < kSegSlots) issue_slot(nxt, buf ^ 1, sent++);
      }
    }
    // (a wavefront with fewer tiles than slots, or none, sends the rest now)
    for (; more && sent < kSegSlots; ++sent) issue_slot(nxt, buf ^ 1, sent);
    if (more) fetch_q(nxt);
    if (nq > 0) {
      if (last) {
        // lanes l and l ^ 32 hold the two halves of a row's keys
        const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
        if (l32 < nq) {
          const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
          T* op = O + ((int64_t)q_tok + l32) * ldo + (int64_t)head * HD;
#pragma unroll
          for (int db = 0; db < kDB; ++db) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const uint32_t w0 = AT::cvt2(o_acc[db][r * 4 + 0] * inv, o_acc[db][r * 4 + 1] * inv);
              const uint32_t w1 = AT::cvt2(o_acc[db][r * 4 + 2] * inv, o_acc[db][r * 4 + 3] * inv);
              const uint64_t bits64 = ((uint64_t)w1 << 32) | w0;
              __builtin_memcpy(reinterpret_cast<char*>(op + db * 32 + 8 * r + 4 * g), &bits64, 8);
            }
          }
        }
      }
    }
    cur = nxt;
  }
#undef NT_FENCE
}

// ---------------------------------------------------------------------------
// The planner (host).  Sequences are cut into chunks of at most eight blocks of
// 32 query rows (as even as possible).  A chunk whose keys fit one segment (four
// tiles) is packed with others into one step, first fit by decreasing size; a
// longer one becomes a chain of steps of its own.  Every chain is replicated per
// head, and the (chain, head) pairs are dealt to the workgroups longest first,
// each to the least loaded one.

struct Chunk {
  int64_t q_tok, k_tok;      // first query token of the chunk, first key token of the sequence
  int nq;                    // query rows of the chunk
  int lk;                    // keys of the sequence
  int blocks() const { return (nq + 31) / 32; }
  int tiles() const { return (lk + kTileKeys - 1) / kTileKeys; }
};

struct Chain {
  std::vector<int32_t> steps;   // n x 48, head left 0
  double cost = 0.0;
};

// Wavefronts w, w + 4, w + 8 share a SIMD: a step takes as long as its busiest SIMD.
static double step_cost(const int* tiles_of_wave) {
  int worst = 0;
  for (int i = 0; i < 4; ++i) {
    int sum = 0;
    for (int w = i; w < kChainWaves; w += 4) sum += tiles_of_wave[w];
    worst = std::max(worst, sum);
  }
  return 1.0 + worst;
}

static void put_slot(int32_t* d, int s, int64_t tok0, int nv, int64_t last) {
  d[4 * s] = (int32_t)tok0;
  d[4 * s + 1] = nv;
  d[4 * s + 2] = (int32_t)last;
  d[4 * s + 3] = 0;
}

static void put_wave(int32_t* d, int w, int64_t q_tok, int nq, int slot0, int nt, bool first, bool last, int n_last) {
  int32_t* m = d + 16 + 4 * w;
  m[0] = (int32_t)q_tok;
  m[1] = nq;
  m[2] = slot0 | (nt << 4) | ((first ? 1 : 0) << 8) | ((last ? 1 : 0) << 9);
  m[3] = n_last;
}

static int build_plan(const int64_t* q_lens, const int64_t* k_lens, int64_t B, int64_t H, int64_t n_wg,
                      std::vector<int32_t>* out) {
  std::vector<Chunk> small_chunks, long_chunks;
  int64_t q_tok = 0, k_tok = 0;
  for (int64_t b = 0; b < B; ++b) {
    const int64_t lq = q_lens[b], lk = k_lens[b];
    if (lq < 0 || lk < 0) return fail(NT_ERR_INVALID_ARGUMENT, "attention_plan: negative length");
    if (lq > 0 && lk == 0) {
      return fail(NT_ERR_UNSUPPORTED, "attention_plan: sequence %lld has queries but no keys", (long long)b);
    }
    if (lq > 0) {
      const int blocks = (int)((lq + 31) / 32);
      const int n_chunks = (blocks + kChainWaves - 1) / kChainWaves;
      const int per = (blocks + n_chunks - 1) / n_chunks;
      for (int c = 0; c < n_chunks; ++c) {
        const int64_t row0 = (int64_t)c * per * 32;
        if (row0 >= lq) break;
        Chunk ch;
        ch.q_tok = q_tok + row0;
        ch.k_tok = k_tok;
        ch.nq = (int)std::min<int64_t>((int64_t)per * 32, lq - row0);
        ch.lk = (int)lk;
        (ch.tiles() <= kSegSlots ? small_chunks : long_chunks).push_back(ch);
      }
    }
    q_tok += lq;
    k_tok += lk;
  }
  if (q_tok > 0x7fffffffLL - 64 || k_tok > 0x7fffffffLL - 64) {
    return fail(NT_ERR_UNSUPPORTED, "attention_plan: token indices are held as int32");
  }

  std::vector<Chain> chains;
  // long chunks: a chain of ceil(tiles / 4) steps, all wavefronts on one sequence
  for (const Chunk& ch : long_chunks) {
    Chain cn;
    const int tiles = ch.tiles(), n_steps = (tiles + kSegSlots - 1) / kSegSlots, blocks = ch.blocks();
    cn.steps.assign((size_t)n_steps * kStepInts, 0);
    for (int j = 0; j < n_steps; ++j) {
      int32_t* d = cn.steps.data() + (size_t)j * kStepInts;
      const int t0 = j * kSegSlots, nt = std::min(kSegSlots, tiles - t0);
      for (int s = 0; s < nt; ++s) {
        const int key0 = (t0 + s) * kTileKeys;
        put_slot(d, s, ch.k_tok + key0, std::min(kTileKeys, ch.lk - key0), ch.k_tok + ch.lk - 1);
      }
      const bool is_last = j == n_steps - 1;
      const int n_last = is_last ? ch.lk - (tiles - 1) * kTileKeys : kTileKeys;
      int tw[kChainWaves] = {0};
      for (int w = 0; w < blocks; ++w) {
        put_wave(d, w, ch.q_tok + 32 * w, std::min(32, ch.nq - 32 * w), 0, nt, j == 0, is_last, n_last);
        tw[w] = nt;
      }
      cn.cost += step_cost(tw);
    }
    chains.push_back(std::move(cn));
  }
  // short chunks: first fit by decreasing (tiles, blocks) into steps of 4 slots and 8 wavefronts
  std::sort(small_chunks.begin(), small_chunks.end(), [](const Chunk& a, const Chunk& b) {
    if (a.tiles() != b.tiles()) return a.tiles() > b.tiles();
    if (a.blocks() != b.blocks()) return a.blocks() > b.blocks();
    return a.q_tok < b.q_tok;
  });
  struct Bin {
    int slots = 0, waves = 0;
    std::vector<int> members;
  };
  std::vector<Bin> bins;
  for (size_t i = 0; i < small_chunks.size(); ++i) {
    const Chunk& ch = small_chunks[i];
    Bin* home = nullptr;
    for (Bin& b : bins) {
      if (b.slots + ch.tiles() <= kSegSlots && b.waves + ch.blocks() <= kChainWaves) {
        home = &b;
        break;
      }
    }
    if (!home) {
      bins.emplace_back();
      home = &bins.back();
    }
    home->slots += ch.tiles();
    home->waves += ch.blocks();
    home->members.push_back((int)i);
  }
  for (const Bin& b : bins) {
    Chain cn;
    cn.steps.assign(kStepInts, 0);
    int32_t* d = cn.steps.data();
    int slot = 0, w = 0;
    int tw[kChainWaves] = {0};
    for (int idx : b.members) {
      const Chunk& ch = small_chunks[idx];
      const int tiles = ch.tiles();
      for (int s = 0; s < tiles; ++s) {
        put_slot(d, slot + s, ch.k_tok + s * kTileKeys, std::min(kTileKeys, ch.lk - s * kTileKeys),
                 ch.k_tok + ch.lk - 1);
      }
      for (int j = 0; j < ch.blocks(); ++j, ++w) {
        put_wave(d, w, ch.q_tok + 32 * j, std::min(32, ch.nq - 32 * j), slot, tiles, true, true,
                 ch.lk - (tiles - 1) * kTileKeys);
        tw[w] = tiles;
      }
      slot += tiles;
    }
    cn.cost = step_cost(tw);
    chains.push_back(std::move(cn));
  }

  // (chain, head) pairs to workgroups: longest first, each to the least loaded
  std::vector<int> order(chains.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = (int)i;
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return chains[a].cost > chains[b].cost; });
  std::vector<double> load((size_t)n_wg, 0.0);
  std::vector<std::vector<std::pair<int, int>>> jobs((size_t)n_wg);
  // a heap of (load, workgroup)
  typedef std::pair<double, int> Slot;
  std::vector<Slot> heap;
  for (int i = 0; i < (int)n_wg; ++i) heap.push_back(Slot(0.0, i));
  auto cmp = [](const Slot& a, const Slot& b) { return a > b; };   // min-heap on load, then on index
  std::make_heap(heap.begin(), heap.end(), cmp);
  for (int c : order) {
    for (int h = 0; h < (int)H; ++h) {
      std::pop_heap(heap.begin(), heap.end(), cmp);
      Slot& s = heap.back();
      jobs[(size_t)s.second].push_back(std::make_pair(c, h));
      s.first += chains[c].cost;
      std::push_heap(heap.begin(), heap.end(), cmp);
    }
  }
  int64_t n_steps = 0;
  for (const Chain& c : chains) n_steps += (int64_t)(c.steps.size() / kStepInts) * H;
  const int64_t first_off = (kPlanHeader + n_wg + 1 + 3) / 4 * 4;
  const int64_t total = first_off + n_steps * kStepInts;
  if (total > 0x7fffffffLL || n_steps > 0x7fffffffLL / kStepInts) {
    return fail(NT_ERR_UNSUPPORTED, "attention_plan: too many steps");
  }
  out->assign((size_t)total, 0);
  int32_t* p = out->data();
  p[0] = (int32_t)n_wg;
  p[1] = (int32_t)first_off;
  p[2] = (int32_t)n_steps;
  p[3] = 64;
  int64_t at = 0;
  for (int64_t wg = 0; wg < n_wg; ++wg) {
    p[kPlanHeader + wg] = (int32_t)at;
    for (const auto& job : jobs[(size_t)wg]) {
      const Chain& c = chains[job.first];
      const size_t n = c.steps.size() / kStepInts;
      for (size_t j = 0; j < n; ++j) {
        int32_t* d = p + first_off + (at + (int64_t)j) * kStepInts;
        std::copy(c.steps.begin() + j * kStepInts, c.steps.begin() + (j + 1) * kStepInts, d);
        d[3] = job.second;
      }
      at += (int64_t)n;
    }
  }
  p[kPlanHeader + n_wg] = (int32_t)at;
  return NT_OK;
}

static int compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess ||
        prop.multiProcessorCount < 1) {
      (void)hipGetLastError();
      return -1;
    }
    n = prop.multiProcessorCount;
  }
  return n;
}

}  // namespace nt

using namespace nt;

extern "C" int64_t nt_attention_plan(const int64_t* q_lens, const int64_t* k_lens, int64_t B, int64_t num_heads,
                                     int64_t head_dim, int64_t n_workgroups, int32_t* plan, int64_t capacity) {
  if (B < 0 || num_heads < 1 || num_heads > 65535 || (B > 0 && (!q_lens || !k_lens))) {
    return -(int64_t)fail(NT_ERR_INVALID_ARGUMENT, "attention_plan: bad arguments");
  }
  if (head_dim != 64) {
    return -(int64_t)fail(NT_ERR_UNSUPPORTED, "attention_plan: head_dim %lld is not 64", (long long)head_dim);
  }
  if (n_workgroups <= 0) {
    n_workgroups = compute_units();
    if (n_workgroups < 1) return -(int64_t)fail(NT_ERR_HIP, "attention_plan: cannot query the device");
  }
  if (n_workgroups > 65535) return -(int64_t)fail(NT_ERR_INVALID_ARGUMENT, "attention_plan: too many workgroups");
  std::vector<int32_t> built;
  const int rc = build_plan(q_lens, k_lens, B, num_heads, n_workgroups, &built);
  if (rc != NT_OK) return -(int64_t)rc;
  if (plan && capacity >= (int64_t)built.size()) std::copy(built.begin(), built.end(), plan);
  return (int64_t)built.size();
}

extern "C" int nt_varlen_attention_planned(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* vt,
                                           int64_t ldvt, void* out, int64_t ldo, const int32_t* plan,
                                           int64_t n_workgroups, int64_t num_heads, int64_t head_dim,
                                           int64_t total_kv_tokens, float scale, int dtype, void* stream) {
  if (n_workgroups < 0 || num_heads < 1 || total_kv_tokens < 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "attention_planned: bad shape");
  }
  if (head_dim != 64) {
    return fail(NT_ERR_UNSUPPORTED, "attention_planned: head_dim %lld is not 64", (long long)head_dim);
  }
  if (dtype != NT_F16 && dtype != NT_BF16) {
    return fail(NT_ERR_UNSUPPORTED, "attention_planned: dtype must be f16 or bf16");
  }
  if (n_workgroups == 0) return NT_OK;
  if (!q || !k || !vt || !out || !plan) return fail(NT_ERR_INVALID_ARGUMENT, "attention_planned: NULL pointer");
  if (n_workgroups > 65535) return fail(NT_ERR_UNSUPPORTED, "attention_planned: too many workgroups");
  const int64_t E = num_heads * head_dim;
  if (ldq < E || ldk < E || ldo < E || ldvt < total_kv_tokens + 72) {
    return fail(NT_ERR_INVALID_ARGUMENT,
                "attention_planned: row strides too small (ldvt must be >= total_kv_tokens + 72)");
  }
  // the K rows travel as 16-byte DMA pieces; a tile's 64 rows are addressed with 32-bit offsets
  if (reinterpret_cast<uintptr_t>(k) % 16 != 0 || (ldk * 2) % 16 != 0 || ldk > (1 << 23)) {
    return fail(NT_ERR_UNSUPPORTED, "attention_planned: K rows must be 16-byte aligned and at most 2^23 elements apart");
  }
  hipStream_t s = (hipStream_t)stream;
  const int lds_bytes = 2 * kSegBytes;
  const float scale_log2e = scale * 1.4426950408889634f;
#define NT_CHAIN_LAUNCH(TYPE)                                                                              \
  {                                                                                                        \
    static bool attr_set = false;                                                                          \
    if (!attr_set) {                                                                                       \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_chain_kernel<TYPE>),      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);           \
      if (e != hipSuccess) return fail(NT_ERR_HIP, "attention_planned: %s", hipGetErrorString(e));         \
      attr_set = true;                                                                                     \
    }                                                                                                      \
    hipLaunchKernelGGL((attention_chain_kernel<TYPE>), dim3((unsigned)n_workgroups), dim3(64 * kChainWaves), \
                       lds_bytes, s, static_cast<const TYPE*>(q), ldq, static_cast<const TYPE*>(k), ldk,   \
                       static_cast<const TYPE*>(vt), ldvt, static_cast<TYPE*>(out), ldo, plan, scale_log2e); \
  }
  if (dtype == NT_F16) NT_CHAIN_LAUNCH(_Float16)
  else NT_CHAIN_LAUNCH(__bf16)
#undef NT_CHAIN_LAUNCH
  return check_launch("attention_chain_kernel");
}
