// Variable-length multi-head attention on the packed token layout (gfx950).
//
// The reference pads Q/K/V to [B, H, Lmax, hd], materialises [B, H, Lmax, Lmax]
// scores in HBM, masks and soft-maxes them and un-pads the result.  Here a
// workgroup owns (sequence b, head h, 128 query rows) and streams that
// sequence's own keys in tiles of 64: tiles beyond L_b are never issued, the
// scores never leave registers (online softmax), and Q/K/V are read straight
// out of the packed projection buffer [T, 3E] and O is written straight into
// the packed [T, E] layout (head split / merge are index arithmetic).
//
// MFMA formulation (v_mfma_f32_32x32x16_{f16,bf16}, fp32 accumulate), per
// wavefront (32 query rows):
//   S^T[key, q] = K[key, :] . Q[q, :]      A-operand = K rows (LDS), B = Q (regs)
//   O^T[d,  q] += V^T[d, key] P^T[key, q]  A-operand = V^T (LDS), B = P^T (regs)
// Working on the transposes puts one query row per lane (q = lane % 32), so
// the softmax row reductions are in-lane plus one cross-half shuffle, and the
// score accumulators are, as they stand, the B-operand of the second product.
//
// fp32 with head_dim 32 / 64 / 128 has a kernel of its own on the fp32 matrix
// instruction (further down).  Any other head_dim takes the generic kernel (one
// wavefront per query row, fp32 FMA); it is the parity path for shapes the MFMA
// kernels do not cover, not a performance path.
#include "attn_common.h"

namespace nt {

constexpr int kHd = 64;         // head_dim of the MFMA kernel
constexpr int kQTile = 128;     // query rows per workgroup (32 per wavefront)
constexpr int kKTile = 64;      // keys per step
constexpr int kKRow = 144;      // LDS bytes per K row (128 + 16 pad)
constexpr int kVRow = 144;      // LDS bytes per V^T row: 64 keys * 2 B + 16 pad
constexpr int kKBytes = kKTile * kKRow;
constexpr int kVBytes = kHd * kVRow;

template <typename T>
__global__ __launch_bounds__(256) void varlen_attention_kernel(
    const T* __restrict__ Q, int64_t ldq, const T* __restrict__ Kp, int64_t ldk,
    const T* __restrict__ Vp, int64_t ldv, T* __restrict__ O, int64_t ldo,
    const int64_t* __restrict__ q_offsets, const int64_t* __restrict__ kv_offsets, float scale_log2e) {
  typedef AttnT<T> AT;
  typedef typename AT::Frag Frag;

  __shared__ __align__(16) char lds_k[2][kKBytes];
  __shared__ __align__(16) char lds_v[2][kVBytes];

  const int b = blockIdx.z;
  const int h = blockIdx.y;
  const int64_t q_begin = q_offsets[b];
  const int64_t Lq = q_offsets[b + 1] - q_begin;
  const int64_t q0 = (int64_t)blockIdx.x * kQTile;
  if (q0 >= Lq) return;
  const int64_t kv_begin = kv_offsets[b];
  const int64_t Lk = kv_offsets[b + 1] - kv_begin;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  // Q fragments: B-operand of S^T = K Q^T.  Lane holds Q[q][16 s + 8 g .. +8].
  const int64_t q_row = q0 + wave * 32 + l32;
  const bool wave_active = (q0 + wave * 32) < Lq;
  Frag qf[4];
  {
    const bool ok = q_row < Lq;
    const T* qp = Q + (q_begin + (ok ? q_row : 0)) * ldq + h * kHd;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      u32x4 v = {0, 0, 0, 0};
      if (ok) v = load16_unaligned(reinterpret_cast<const char*>(qp + s * 16 + g * 8));
      __builtin_memcpy(&qf[s], &v, 16);
    }
  }

  acc16 o_acc[2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
  float m_run = -INFINITY;   // running row max (of raw scores), same in lanes l and l^32
  float l_run = 0.0f;        // this lane's share of the running row sum

  const int64_t ntiles = (Lk + kKTile - 1) / kKTile;
  const T* kbase = Kp + kv_begin * ldk + h * kHd;
  const T* vbase = Vp + kv_begin * ldv + h * kHd;

  // Each thread moves two 16-byte pieces of the K tile and two of the V tile.
  u32x4 rk[2], rv[2];
  auto gload = [&](int64_t t) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = tid + i * 256;       // 0..511
      const int key = c >> 3;            // 0..63
      const int cc = c & 7;
      const int64_t kr = t * kKTile + key;
      u32x4 zk = {0, 0, 0, 0}, zv = {0, 0, 0, 0};
      if (kr < Lk) {
        zk = load16_unaligned(reinterpret_cast<const char*>(kbase + kr * ldk + cc * 8));
        zv = load16_unaligned(reinterpret_cast<const char*>(vbase + kr * ldv + cc * 8));
      }
      rk[i] = zk;
      rv[i] = zv;
    }
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = tid + i * 256;
      const int key = c >> 3;
      const int cc = c & 7;
      store16(&lds_k[buf][key * kKRow + cc * 16], rk[i]);
      // V is stored transposed: lds_v[d][key]
      T tmp[8];
      __builtin_memcpy(tmp, &rv[i], 16);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        *reinterpret_cast<T*>(&lds_v[buf][(cc * 8 + j) * kVRow + key * 2]) = tmp[j];
      }
    }
  };

  gload(0);
  lstore(0);
  __syncthreads();

  for (int64_t t = 0; t < ntiles; ++t) {
    const int buf = (int)(t & 1);
    if (t + 1 < ntiles) gload(t + 1);

    if (wave_active) {
      // ---- S^T = K Q^T : two 32-key blocks ----
      acc16 s_acc[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int e = 0; e < 16; ++e) s_acc[kb][e] = 0.0f;
        const char* krow = &lds_k[buf][(kb * 32 + l32) * kKRow + g * 16];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          Frag kf = *reinterpret_cast<const Frag*>(krow + s * 32);
          s_acc[kb] = AT::mma(kf, qf[s], s_acc[kb]);
        }
      }
      // s_acc[kb][e] = score(key = t*64 + kb*32 + 8*(e/4) + 4*g + e%4, q = l32)
      const int64_t key_base = t * kKTile;
      const bool tail = key_base + kKTile > Lk;
      float m_tile = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          if (tail) {
            const int64_t key = key_base + kb * 32 + 8 * (e >> 2) + 4 * g + (e & 3);
            if (key >= Lk) s_acc[kb][e] = -INFINITY;
          }
          m_tile = fmaxf(m_tile, s_acc[kb][e]);
        }
      m_tile = max_across_halves(m_tile);
      const float m_new = fmaxf(m_run, m_tile);   // finite: every tile holds >= 1 valid key
      const float alpha = exp2f((m_run - m_new) * scale_log2e);
      const float m_scaled = m_new * scale_log2e;
      float l_tile = 0.0f;
      Frag pf[4];   // P^T as B-operand: k-step ks uses s_acc[ks/2][8*(ks%2) .. +8]
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          T tmp[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float p = exp2f(s_acc[kb][half * 8 + j] * scale_log2e - m_scaled);
            const T pt = (T)p;
            // sum what is actually multiplied with V, so rows are normalised
            // to the rounded probabilities
            l_tile += (float)pt;
            tmp[j] = pt;
          }
          __builtin_memcpy(&pf[kb * 2 + half], tmp, 16);
        }
      }
      l_run = l_run * alpha + l_tile;
      m_run = m_new;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;

      // ---- O^T += V^T P^T ----
      // k-step ks covers the keys the lane group holds in s_acc: slot j of
      // group g is key kb*32 + 16*half + 8*(j/4) + 4*g + j%4 (kb = ks/2, half = ks%2).
#pragma unroll
      for (int db = 0; db < 2; ++db) {
        const char* vrow = &lds_v[buf][(db * 32 + l32) * kVRow];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const int kb = ks >> 1, half = ks & 1;
          const int key_lo = kb * 32 + 16 * half + 4 * g;
          uint64_t lo = *reinterpret_cast<const uint64_t*>(vrow + key_lo * 2);
          uint64_t hi = *reinterpret_cast<const uint64_t*>(vrow + (key_lo + 8) * 2);
          uint64_t both[2] = {lo, hi};
          Frag vf;
          __builtin_memcpy(&vf, both, 16);
          o_acc[db] = AT::mma(vf, pf[ks], o_acc[db]);
        }
      }
    }

    if (t + 1 < ntiles) lstore(buf ^ 1);
    __syncthreads();
  }

  if (!wave_active || q_row >= Lq) return;
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  // (the shuffle above needs both half-waves; rows past Lq have already left,
  // but lanes l and l^32 share q_row, so they leave together)
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;   // no keys: zeros
  T* op = O + (q_begin + q_row) * ldo + h * kHd;
#pragma unroll
  for (int db = 0; db < 2; ++db) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      // d = db*32 + 8*r + 4*g + (0..3)
      T tmp[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) tmp[j] = (T)(o_acc[db][r * 4 + j] * inv);
      uint64_t bits;
      __builtin_memcpy(&bits, tmp, 8);
      __builtin_memcpy(reinterpret_cast<char*>(op + db * 32 + 8 * r + 4 * g), &bits, 8);
    }
  }
}

// ---------------------------------------------------------------------------
// Attention kernel of the fused layer: Q and K come row-major from the
// projection buffers, V comes TRANSPOSED (Vt[h*HD + d][token], written that way by
// the projection GEMM's epilogue), so a V^T tile is HD rows of 64 key-contiguous
// values and needs no transposition on its way into LDS.
//
// Work items {first query token, query length, first query row of the tile, 0,
// first key token, key length, 0, 0} come from a schedule the host builds from
// the nested size (longest sequences first, no item for a tile that does not
// exist), so every workgroup that is launched has work and the long sequences
// start first.  A workgroup is (item, head), head fastest: the items of ALL heads
// of the long sequences are dispatched before any short item.
//
// What keeps the vector ALU work per score low:
//
//  * Q is multiplied by scale * log2(e) once, when its fragments are loaded, so
//    the score accumulators are exponents of two as they stand;
//  * the reference maximum of a query row is not subtracted with an instruction
//    per score: the 32x32 blocks of S^T = K Q^T are accumulated onto a register
//    block that holds -m_ref (the third MFMA operand), so S - m_ref falls out
//    of the matrix pipe.  m_ref need not be the exact running maximum, softmax
//    is invariant to it; it only has to keep 2^(S - m_ref) inside the range of
//    the storage type.  It is set from the first tile and raised only when a
//    tile's maximum exceeds it by more than kLazyMaxLog2 (wavefront-uniform
//    branch, rare after the first tile), which is also the only place where the
//    output accumulators are rescaled;
//  * the denominators are sums of the ROUNDED probabilities (the ones that meet
//    V), two per v_dot2c instruction, accumulated in fp32;
//  * V^T tiles lie in LDS in key order (one 16-byte write per piece); the
//    permutation that the PV product needs (the eight keys a lane group holds in
//    its score accumulators must be one 16-byte run of a V^T row) is applied to
//    the ROW order of the K tile instead, where it is free: a thread simply
//    fetches another row.  LDS row rho = 16 ks + 8 a + 4 g + c of the K tile holds
//    key 16 ks + 8 g + 4 a + c;
//  * keys past L in the last tile: their K rows are copies of row L - 1 (valid
//    memory, cannot raise the maximum), their scores are set to -inf after the
//    maximum is taken and their V^T columns are zeroed on the way into LDS, so
//    nothing of what follows the sequence in memory can reach the result.
#ifndef NT_ATTN_WAVES_PER_EU
#define NT_ATTN_WAVES_PER_EU 3
#endif

template <typename T, int HD>
__global__ __launch_bounds__(256, (HD > 64 ? 2 : NT_ATTN_WAVES_PER_EU)) void varlen_attention_vt_kernel(
    const T* __restrict__ Q, int64_t ldq, const T* __restrict__ K, int64_t ldk,
    const T* __restrict__ Vt, int64_t ldvt, T* __restrict__ O, int64_t ldo,
    const int4* __restrict__ schedule, unsigned num_heads, float scale_log2e) {
  typedef AttnT<T> AT;
  typedef typename AT::Frag Frag;

  constexpr int kKR = HD * 2 + 16;
  constexpr int kQF = HD / 16;
  constexpr int kDB = HD / 32;
  constexpr int kKPieces = HD / 8;
  constexpr int kKRowsPerPass = 256 / kKPieces;
  constexpr int kKP = kKTile / kKRowsPerPass;
  constexpr int kVP = HD / 32;
  __shared__ __align__(16) char lds_k[2][kKTile * kKR];
  __shared__ __align__(16) char lds_v[2][HD * kVRow];

  // Every kernel argument is wanted in registers now, together with the work item,
  // not fetched piecemeal after the first branch: a workgroup of a short sequence is
  // a chain of dependent memory round trips, and each scalar fetch is one of them.
  asm volatile("" ::"s"(Q), "s"(K), "s"(Vt), "s"(O), "s"(ldq), "s"(ldk), "s"(ldvt), "s"(ldo));
  const int h = (int)(blockIdx.x % num_heads);
  // the whole work item in one 32-byte scalar load: everything below waits for it
  typedef int int8v __attribute__((ext_vector_type(8)));
  const int8v item = *reinterpret_cast<const int8v*>(schedule + 2 * (blockIdx.x / num_heads));
  const int64_t q_begin = item[0];
  const int Lq = item[1];
  const int q0 = item[2];
  const int64_t begin = item[4];
  const int L = item[5];
  if (L <= 0 || Lq <= 0) {   // uniform.  No keys: zeros, as in varlen_attention_kernel
    for (int i = threadIdx.x; i < kQTile * (HD / 8); i += 256) {
      const int row = q0 + i / (HD / 8);
      if (Lq > 0 && row < Lq) {
        const u32x4 z = {0, 0, 0, 0};
        __builtin_memcpy(reinterpret_cast<char*>(O + (q_begin + row) * ldo + h * HD + (i % (HD / 8)) * 8), &z, 16);
      }
    }
    return;
  }

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  const int q_row = q0 + wave * 32 + l32;
  const bool wave_active = (q0 + wave * 32) < Lq;
  Frag qf[kQF];
  {
    const int qr = q_row < Lq ? q_row : Lq - 1;
    const T* qp = Q + (q_begin + qr) * ldq + h * HD + g * 8;
#pragma unroll
    for (int s = 0; s < kQF; ++s) {
      u32x4 v = load16_unaligned(reinterpret_cast<const char*>(qp + s * 16));
      Frag f;
      __builtin_memcpy(&f, &v, 16);
      qf[s] = QScale<T>::run(f, scale_log2e);
    }
  }

  acc16 o_acc[kDB];
#pragma unroll
  for (int i = 0; i < kDB; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
  acc16 negm;           // -m_ref in every element
#pragma unroll
  for (int e = 0; e < 16; ++e) negm[e] = 0.0f;
  float l_run = 0.0f;   // this lane's share of the row's denominator

  const int ntiles = (L + kKTile - 1) / kKTile;
  // A workgroup's life is its number of key tiles, and three workgroups share a
  // SIMD: the launch ends when the longest sequences do.  Their wavefronts get the
  // higher issue priority, so they run near the speed of a SIMD of their own while
  // the short ones fill what is left.
  if (ntiles >= 7) {
    __builtin_amdgcn_s_setprio(3);
  } else if (ntiles >= 5) {
    __builtin_amdgcn_s_setprio(2);
  } else if (ntiles >= 3) {
    __builtin_amdgcn_s_setprio(1);
  }
  const T* kbase = K + begin * ldk + h * HD;
  const T* vbase = Vt + (int64_t)h * HD * ldvt + begin;

  const int r0 = tid >> 3;
  const int cc = tid & 7;
  const int kr0 = tid / kKPieces;
  const int kc = tid % kKPieces;
  // one tile of K and V^T pieces on its way from global memory to LDS
  struct Stage {
    u32x4 k[kKP], v[kVP];
  };
  Stage st;
  const char* k_last = reinterpret_cast<const char*>(kbase + (int64_t)(L - 1) * ldk + kc * 8);
  const int64_t k_step = (int64_t)kKTile * ldk * (int64_t)sizeof(T);
  const char* v_ptr[kVP];
#pragma unroll
  for (int i = 0; i < kVP; ++i) {
    v_ptr[i] = reinterpret_cast<const char*>(vbase + (int64_t)(r0 + i * 32) * ldvt + cc * 8);
  }
  auto gload = [&](Stage& sg, int t_in) {
    const int t = t_in < ntiles ? t_in : ntiles - 1;   // past the end: re-read, never used
    const char* tile = reinterpret_cast<const char*>(kbase + kc * 8) + t * k_step;
#pragma unroll
    for (int i = 0; i < kKP; ++i) {
      // LDS row `row` holds the key with bits 2 and 3 of the row index exchanged;
      // rows past L read row L - 1 (a valid key: it cannot raise the row maximum)
      const int row = kr0 + i * kKRowsPerPass;
      const int key = (row & ~12) | ((row & 4) << 1) | ((row & 8) >> 1);
      const int kr = t * kKTile + key;
      const char* src = tile + (int64_t)key * ldk * (int64_t)sizeof(T);
      sg.k[i] = load16_unaligned(kr < L ? src : k_last);
    }
    // V^T piece: keys 8 cc .. 8 cc + 7 of row d, read where it lies (the rows of Vt
    // are readable 72 elements past the last token)
#pragma unroll
    for (int i = 0; i < kVP; ++i) {
      sg.v[i] = load16_unaligned(v_ptr[i] + t * (kKTile * (int)sizeof(T)));
    }
  };
  // V^T columns of keys at or past L are zeroed in the last tile: their
  // probabilities are zero (below), and 0 * x must not meet a NaN or an infinity
  // in whatever follows the sequence in memory
  u32x4 vm;
  {
    int nv = L - ((ntiles - 1) * kKTile + cc * 8);
    nv = nv > 8 ? 8 : (nv < 0 ? 0 : nv);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      vm[j] = nv >= 2 * j + 2 ? 0xffffffffu : (nv == 2 * j + 1 ? 0x0000ffffu : 0u);
    }
  }
  auto lstore = [&](const Stage& sg, int buf, int t) {
#pragma unroll
    for (int i = 0; i < kKP; ++i) {
      store16(&lds_k[buf][(kr0 + i * kKRowsPerPass) * kKR + kc * 16], sg.k[i]);
    }
    if (t < ntiles - 1) {   // uniform: a full tile
#pragma unroll
      for (int i = 0; i < kVP; ++i) store16(&lds_v[buf][(r0 + i * 32) * kVRow + cc * 16], sg.v[i]);
      return;
    }
#pragma unroll
    for (int i = 0; i < kVP; ++i) store16(&lds_v[buf][(r0 + i * 32) * kVRow + cc * 16], sg.v[i] & vm);
  };
  const int n_last = L - (ntiles - 1) * kKTile;   // keys of the last tile, 1..64

  // The body of a tile is written in the order it should issue, and fenced so
  // that it does: matrix instructions execute in the background while the
  // wavefront goes on issuing vector instructions, but only if the two kinds
  // alternate in the instruction stream (the scheduler would otherwise group
  // all exponentials in front of all PV products).  NT_FENCE keeps the
  // scheduler from moving anything across it.
#define NT_FENCE() __builtin_amdgcn_sched_barrier(0)
  auto tile = [&](int buf, bool first, bool partial) {
    // S^T - m_ref: s[kb][e] belongs to LDS row 32 kb + 8 (e/4) + 4 g + e%4 of the K tile
    const char* krow = &lds_k[buf][l32 * kKR + g * 16];
    Frag kf[2][kQF];
    auto read_k = [&](int kb, int s0, int s1) {
#pragma unroll
      for (int s = s0; s < s1; ++s)
        kf[kb][s] = *reinterpret_cast<const Frag*>(krow + kb * 32 * kKR + s * 32);
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
    // the maximum of the first block while the second one is in the matrix pipe
    float m_tile = sa[0][0];
#pragma unroll
    for (int e = 1; e < 16; ++e) m_tile = fmaxf(m_tile, sa[0][e]);
    NT_FENCE();
#pragma unroll
    for (int s = kQF / 2; s < kQF; ++s) sa[1] = AT::mma(kf[1][s], qf[s], sa[1]);
    NT_FENCE();
    // V^T fragments of k-step 0 travel while the maximum is finished
    Frag vf[2][kDB];
    const char* vrow = &lds_v[buf][l32 * kVRow + g * 16];
    auto read_v = [&](int ks) {
#pragma unroll
      for (int db = 0; db < kDB; ++db)
        vf[ks & 1][db] = *reinterpret_cast<const Frag*>(vrow + db * 32 * kVRow + ks * 32);
    };
    read_v(0);
    NT_FENCE();
#pragma unroll
    for (int e = 0; e < 16; ++e) m_tile = fmaxf(m_tile, sa[1][e]);
    m_tile = max_across_halves(m_tile);
    // (last tile, fewer than 64 keys: the K rows past L are copies of row L - 1, so
    // they cannot have raised the maximum, and their V^T columns are zero, so they add
    // nothing to the output; what they add to the denominator is taken out below)
    //
    // The reference maximum starts at 0 and moves only when a tile's maximum leaves
    // [-2^3, 2^3] powers of two around it (first tile: either way, later only
    // upwards): for scores of ordinary size it never moves, and no tile pays the
    // 48 subtractions of a move.
    if (__any(first ? fabsf(m_tile) > kLazyMaxLog2 : m_tile > kLazyMaxLog2)) {   // wavefront-uniform
      // raise (first tile: set) the reference maximum of every row by delta
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
    // probabilities of k-step ks = 2 kb + half: sa[kb][8 half .. 8 half + 8)
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
          // the next k-step's eight exponentials, spread over this one's matrix instructions
          exps(ks + 1, 8 * m / kDB, 8 * (m + 1) / kDB);
          if (m == kDB - 1) cvts(ks + 1);
          NT_FENCE();
        }
      }
    }
    if (partial) {
      // The keys past L: their K rows are copies of row L - 1, so each of them has
      // exactly the probability of the last valid key, and the highest key this lane
      // half holds (8 g + 55, the last accumulator) is one of them whenever the half
      // holds any.  The lane half holds keys [8 g + 16 j, 8 g + 16 j + 8), j = 0..3.
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
  // Tile t + 1 travels global -> registers while tile t is computed, and goes
  // registers -> LDS (the other buffer) after the compute, before the barrier.
  // (Giving the loads two tiles of time to arrive, with a second register set,
  // was measured: no change.)
  gload(st, 0);
  lstore(st, 0, 0);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const int buf = t & 1;
    const bool more = t + 1 < ntiles;   // uniform
    if (more) gload(st, t + 1);
    // keep the loads above the MFMA / softmax work (the scheduler would sink them)
    __builtin_amdgcn_sched_barrier(0);
    if (wave_active) tile(buf, t == 0, t == ntiles - 1 && n_last < kKTile);
    // the last tile loads nothing and waits for nothing: a workgroup of a short
    // sequence is mostly its first loads and its last stores
    if (more) {
      lstore(st, buf ^ 1, t + 1);
      __syncthreads();
    }
  }

  if (!wave_active) return;
  // lanes l and l ^ 32 hold the two halves of a row's keys
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  if (q_row >= Lq) return;
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  T* op = O + (q_begin + q_row) * ldo + h * HD;
#pragma unroll
  for (int db = 0; db < kDB; ++db) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      uint32_t w0 = AT::cvt2(o_acc[db][r * 4 + 0] * inv, o_acc[db][r * 4 + 1] * inv);
      uint32_t w1 = AT::cvt2(o_acc[db][r * 4 + 2] * inv, o_acc[db][r * 4 + 3] * inv);
      uint64_t bits = ((uint64_t)w1 << 32) | w0;
      __builtin_memcpy(reinterpret_cast<char*>(op + db * 32 + 8 * r + 4 * g), &bits, 8);
    }
  }
}

// ---------------------------------------------------------------------------
// Generic kernel: any head_dim, any dtype, fp32 math.  One wavefront per
// (query row, head); keys in groups of 64 (one per lane), online softmax.

template <typename T> __device__ __forceinline__ float to_f(T x) { return (float)x; }

template <typename T>
__global__ __launch_bounds__(64) void attention_rows_kernel(
    const T* __restrict__ Q, int64_t ldq, const T* __restrict__ Kp, int64_t ldk,
    const T* __restrict__ Vp, int64_t ldv, T* __restrict__ O, int64_t ldo,
    const int64_t* __restrict__ q_offsets, const int64_t* __restrict__ kv_offsets, int head_dim,
    float scale) {
  const int b = blockIdx.z;
  const int h = blockIdx.y;
  const int64_t q_begin = q_offsets[b];
  const int64_t Lq = q_offsets[b + 1] - q_begin;
  const int64_t qi = blockIdx.x;
  if (qi >= Lq) return;
  const int64_t kv_begin = kv_offsets[b];
  const int64_t Lk = kv_offsets[b + 1] - kv_begin;
  const int lane = threadIdx.x;

  extern __shared__ float sm[];           // q[head_dim] then p[64]
  float* qs = sm;
  float* ps = sm + head_dim;
  const T* qp = Q + (q_begin + qi) * ldq + (int64_t)h * head_dim;
  for (int d = lane; d < head_dim; d += 64) qs[d] = to_f(qp[d]);
  __syncthreads();

  // each lane owns output dims lane, lane+64, ... (up to 8 => head_dim <= 512)
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;

  for (int64_t k0 = 0; k0 < Lk; k0 += 64) {
    const int64_t key = k0 + lane;
    float s = -INFINITY;
    if (key < Lk) {
      const T* kp = Kp + (kv_begin + key) * ldk + (int64_t)h * head_dim;
      float dot = 0.0f;
      for (int d = 0; d < head_dim; ++d) dot = fmaf(qs[d], to_f(kp[d]), dot);
      s = dot * scale;
    }
    float m_tile = s;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m_tile = fmaxf(m_tile, __shfl_xor(m_tile, off, 64));
    const float m_new = fmaxf(m_run, m_tile);
    const float alpha = __expf(m_run - m_new);
    const float p = (key < Lk) ? __expf(s - m_new) : 0.0f;
    float l_tile = p;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) l_tile += __shfl_xor(l_tile, off, 64);
    l_run = l_run * alpha + l_tile;
    m_run = m_new;
    __syncthreads();
    ps[lane] = p;
    __syncthreads();
    const int nk = (int)((Lk - k0) < 64 ? (Lk - k0) : 64);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int d = lane + i * 64;
      if (d < head_dim) {
        float a = acc[i] * alpha;
        const T* vp = Vp + (kv_begin + k0) * ldv + (int64_t)h * head_dim + d;
        for (int j = 0; j < nk; ++j) a = fmaf(ps[j], to_f(vp[j * ldv]), a);
        acc[i] = a;
      }
    }
  }
  T* op = O + (q_begin + qi) * ldo + (int64_t)h * head_dim;
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;   // no keys: zeros
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + i * 64;
    if (d < head_dim) op[d] = (T)(acc[i] * inv);
  }
}

// ---------------------------------------------------------------------------
// fp32 attention on the matrix pipe (v_mfma_f32_32x32x2_f32), head_dim 32 / 64 /
// 128.  Same transposed formulation as above: per wavefront 32 query rows, one
// per lane pair (q = lane % 32; the two lane halves hold different keys),
//   S^T[key, q] = K[key, :] . Q[q, :]      A = K rows (LDS), B = Q (registers)
//   O^T[d,  q] += V^T[d, key] P^T[key, q]  A = V as it lies row-major in LDS, B = P^T
// so the score accumulators are the B operand of the second product as they
// stand and V needs no transpose.  The k index of an MFMA step only has to mean
// the same thing in both operands: in the first product lane half g takes head
// dims 8t + 4g .. 8t + 4g + 3 over four consecutive steps (one 16-byte LDS read
// of the K row); in the second, step i contracts the key that accumulator i of
// that lane half holds, 8 (i / 4) + 4 g + i % 4.  Everything stays fp32
// (exp2 on scores prescaled by log2 e).  A workgroup owns 128 query rows of
// (sequence, head) and walks the sequence's keys in tiles of 32, the next tile's
// global loads in flight while the current one is multiplied, two LDS buffers.
template <int HD>
__device__ __forceinline__ void attention_f32_tile(
    const float* __restrict__ Q, int64_t ldq, const float* __restrict__ Kp, int64_t ldk,
    const float* __restrict__ Vp, int64_t ldv, float* __restrict__ O, int64_t ldo,
    const int64_t q_begin, const int64_t Lq, const int64_t q0, const int64_t kv_begin, const int64_t Lk,
    const int h, float scale_log2e, float* lds) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  constexpr int kKT = 32;                      // keys per tile
  constexpr int kKs = HD + 4;                  // K row stride in floats: 16-byte reads of 16 rows hit 16 bank groups
  constexpr int kVs = HD + 8;                  // V row stride: the two lane halves (keys 4 apart) use different banks
  constexpr int kBuf = kKT * (kKs + kVs);
  constexpr int kC4 = HD / 4;                  // 16-byte pieces per row
  constexpr int kPieces = kKT * kC4 / 256;     // pieces per thread and operand: 1, 2, 4
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, half = lane >> 5;

  // this lane's query row, prescaled: dims 8t + 4 half + u  ->  qf[4t + u]
  const int64_t qrow = q0 + wave * 32 + col;
  const bool q_ok = qrow < Lq;
  float qf[HD / 2];
  {
    const float* qp = Q + (q_begin + (q_ok ? qrow : q0)) * ldq + (int64_t)h * HD + 4 * half;
#pragma unroll
    for (int t = 0; t < HD / 8; ++t) {
      f32x4 v = *reinterpret_cast<const f32x4*>(qp + 8 * t);
#pragma unroll
      for (int u = 0; u < 4; ++u) qf[4 * t + u] = q_ok ? v[u] * scale_log2e : 0.0f;
    }
  }

  f32x4 kreg[kPieces], vreg[kPieces];
  const float* kbase = Kp + kv_begin * ldk + (int64_t)h * HD;
  const float* vbase = Vp + kv_begin * ldv + (int64_t)h * HD;
  auto gload = [&](int64_t k0) {
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int p = tid + 256 * i;
      const int row = p / kC4, c4 = p % kC4;
      const int64_t key = k0 + row;
      const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
      // rows past the last key are zero: 0 * V must not meet a NaN
      kreg[i] = key < Lk ? *reinterpret_cast<const f32x4*>(kbase + key * ldk + 4 * c4) : zero;
      vreg[i] = key < Lk ? *reinterpret_cast<const f32x4*>(vbase + key * ldv + 4 * c4) : zero;
    }
  };
  auto lstore = [&](float* buf) {
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int p = tid + 256 * i;
      const int row = p / kC4, c4 = p % kC4;
      *reinterpret_cast<f32x4*>(buf + row * kKs + 4 * c4) = kreg[i];
      *reinterpret_cast<f32x4*>(buf + kKT * kKs + row * kVs + 4 * c4) = vreg[i];
    }
  };

  acc16 o[HD / 32];
#pragma unroll
  for (int j = 0; j < HD / 32; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[j][i] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;       // l_run: this lane half's keys only

  const int64_t n_tiles = (Lk + kKT - 1) / kKT;
  if (n_tiles > 0) {
    gload(0);
    lstore(lds);
  }
  __syncthreads();
  for (int64_t t = 0; t < n_tiles; ++t) {
    float* cur = lds + (t & 1) * kBuf;
    const bool more = t + 1 < n_tiles;
    if (more) gload((t + 1) * kKT);
    const float* Ks = cur + col * kKs + 4 * half;
    const float* Vs = cur + kKT * kKs + 4 * half * kVs + col;

    acc16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.0f;
#pragma unroll
    for (int tt = 0; tt < HD / 8; ++tt) {
      const f32x4 kf = *reinterpret_cast<const f32x4*>(Ks + 8 * tt);
#pragma unroll
      for (int u = 0; u < 4; ++u) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[u], qf[4 * tt + u], s, 0, 0, 0);
    }
    // accumulator i: key 8 (i / 4) + 4 half + i % 4 of the tile, query col
    const int64_t left = Lk - t * kKT;
    if (left < kKT) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (8 * (i / 4) + 4 * half + (i % 4) >= left) s[i] = -INFINITY;
      }
    }
    float m_tile = s[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) m_tile = fmaxf(m_tile, s[i]);
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));      // finite: the tile holds a valid key
    const float m_new = fmaxf(m_run, m_tile);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float l_tile = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = __builtin_amdgcn_exp2f(s[i] - m_new);
      l_tile += s[i];
    }
    l_run = l_run * alpha + l_tile;
#pragma unroll
    for (int j = 0; j < HD / 32; ++j) {
#pragma unroll
      for (int i = 0; i < 16; ++i) o[j][i] *= alpha;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float* vrow = Vs + (8 * (i / 4) + (i % 4)) * kVs;
#pragma unroll
      for (int j = 0; j < HD / 32; ++j) {
        o[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * j], s[i], o[j], 0, 0, 0);
      }
    }
    if (more) lstore(lds + ((t + 1) & 1) * kBuf);
    __syncthreads();
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;     // no keys: zeros
  if (q_ok) {
    // accumulator i of block j: head dim 32 j + 8 (i / 4) + 4 half + i % 4
    float* op = O + (q_begin + qrow) * ldo + (int64_t)h * HD + 4 * half;
#pragma unroll
    for (int j = 0; j < HD / 32; ++j) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f32x4 v = {o[j][4 * g] * inv, o[j][4 * g + 1] * inv, o[j][4 * g + 2] * inv, o[j][4 * g + 3] * inv};
        *reinterpret_cast<f32x4*>(op + 32 * j + 8 * g) = v;
      }
    }
  }
}

// Workgroup = (128 query rows, head, sequence) on a padded grid: tiles past a
// sequence's last query row leave at once.
template <int HD>
__global__ __launch_bounds__(256) void varlen_attention_f32_kernel(
    const float* __restrict__ Q, int64_t ldq, const float* __restrict__ Kp, int64_t ldk,
    const float* __restrict__ Vp, int64_t ldv, float* __restrict__ O, int64_t ldo,
    const int64_t* __restrict__ q_offsets, const int64_t* __restrict__ kv_offsets,
    float scale_log2e) {
  __shared__ __align__(16) float lds[2 * 32 * (2 * HD + 12)];
  const int b = blockIdx.z, h = blockIdx.y;
  const int64_t q_begin = q_offsets[b];
  const int64_t Lq = q_offsets[b + 1] - q_begin;
  const int64_t q0 = (int64_t)blockIdx.x * 128;
  if (q0 >= Lq) return;                        // uniform
  const int64_t kv_begin = kv_offsets[b];
  attention_f32_tile<HD>(Q, ldq, Kp, ldk, Vp, ldv, O, ldo, q_begin, Lq, q0, kv_begin,
                         kv_offsets[b + 1] - kv_begin, h, scale_log2e, lds);
}

// The same tiles from a work list (the items of nt_varlen_attention_vt): only
// tiles that exist are launched, longest key sequences first, head fastest.
template <int HD>
__global__ __launch_bounds__(256) void varlen_attention_f32_sched_kernel(
    const float* __restrict__ Q, int64_t ldq, const float* __restrict__ Kp, int64_t ldk,
    const float* __restrict__ Vp, int64_t ldv, float* __restrict__ O, int64_t ldo,
    const int4* __restrict__ schedule, unsigned num_heads, float scale_log2e) {
  __shared__ __align__(16) float lds[2 * 32 * (2 * HD + 12)];
  const int h = (int)(blockIdx.x % num_heads);
  const int4 item = schedule[2 * (blockIdx.x / num_heads)];
  const int4 item_kv = schedule[2 * (blockIdx.x / num_heads) + 1];
  if (item.y <= 0 || item.z >= item.y) return;   // uniform: no query rows in this tile
  attention_f32_tile<HD>(Q, ldq, Kp, ldk, Vp, ldv, O, ldo, item.x, item.y, item.z, item_kv.x,
                         item_kv.y > 0 ? item_kv.y : 0, h, scale_log2e, lds);
}

template <int HD>
static int launch_f32(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                      int64_t ldv, void* out, int64_t ldo, const int64_t* qo, const int64_t* kvo,
                      int64_t B, int64_t H, int64_t max_q, float scale, hipStream_t s) {
  dim3 grid((unsigned)((max_q + 127) / 128), (unsigned)H, (unsigned)B);
  hipLaunchKernelGGL((varlen_attention_f32_kernel<HD>), grid, dim3(256), 0, s,
                     static_cast<const float*>(q), ldq, static_cast<const float*>(k), ldk,
                     static_cast<const float*>(v), ldv, static_cast<float*>(out), ldo, qo, kvo,
                     scale * 1.4426950408889634f);
  return check_launch("varlen_attention_f32_kernel");
}

template <typename T>
static int launch_generic(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                          int64_t ldv, void* out, int64_t ldo, const int64_t* qo,
                          const int64_t* kvo, int64_t B, int64_t H, int64_t hd, int64_t max_q,
                          float scale, hipStream_t s) {
  if (hd > 512) return fail(NT_ERR_UNSUPPORTED, "attention: head_dim %lld > 512", (long long)hd);
  dim3 grid((unsigned)max_q, (unsigned)H, (unsigned)B);
  const size_t lds = (size_t)(hd + 64) * sizeof(float);
  hipLaunchKernelGGL((attention_rows_kernel<T>), grid, dim3(64), lds, s,
                     static_cast<const T*>(q), ldq, static_cast<const T*>(k), ldk,
                     static_cast<const T*>(v), ldv, static_cast<T*>(out), ldo, qo, kvo, (int)hd,
                     scale);
  return check_launch("attention_rows_kernel");
}

template <typename T>
static int launch_mfma(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* v,
                       int64_t ldv, void* out, int64_t ldo, const int64_t* qo, const int64_t* kvo,
                       int64_t B, int64_t H, int64_t max_q, float scale, hipStream_t s) {
  dim3 grid((unsigned)((max_q + kQTile - 1) / kQTile), (unsigned)H, (unsigned)B);
  const float scale_log2e = scale * 1.4426950408889634f;
  hipLaunchKernelGGL((varlen_attention_kernel<T>), grid, dim3(256), 0, s,
                     static_cast<const T*>(q), ldq, static_cast<const T*>(k), ldk,
                     static_cast<const T*>(v), ldv, static_cast<T*>(out), ldo, qo, kvo,
                     scale_log2e);
  return check_launch("varlen_attention_kernel");
}

}  // namespace nt

using namespace nt;

extern "C" int nt_varlen_attention(const void* q, int64_t ldq, const void* k, int64_t ldk,
                                   const void* v, int64_t ldv, void* out, int64_t ldo,
                                   const int64_t* q_offsets, const int64_t* kv_offsets, int64_t B,
                                   int64_t num_heads, int64_t head_dim, int64_t max_q_len,
                                   float scale, int dtype, void* stream) {
  if (B < 0 || num_heads < 1 || head_dim < 1 || max_q_len < 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "attention: bad shape B=%lld H=%lld hd=%lld",
                (long long)B, (long long)num_heads, (long long)head_dim);
  }
  if (B == 0 || max_q_len == 0) return NT_OK;
  if (!q || !k || !v || !out || !q_offsets || !kv_offsets) {
    return fail(NT_ERR_INVALID_ARGUMENT, "attention: NULL pointer");
  }
  if (B > 65535 || num_heads > 65535) {
    return fail(NT_ERR_UNSUPPORTED, "attention: B and num_heads must be <= 65535");
  }
  const int64_t need = num_heads * head_dim;
  if (ldq < need || ldk < need || ldv < need || ldo < need) {
    return fail(NT_ERR_INVALID_ARGUMENT, "attention: row stride smaller than num_heads*head_dim");
  }
  hipStream_t s = (hipStream_t)stream;
  if (head_dim == kHd && dtype == NT_F16) {
    return launch_mfma<_Float16>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B,
                                 num_heads, max_q_len, scale, s);
  }
  if (head_dim == kHd && dtype == NT_BF16) {
    return launch_mfma<__bf16>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B,
                               num_heads, max_q_len, scale, s);
  }
  if (dtype == NT_F32 && (head_dim == 32 || head_dim == 64 || head_dim == 128) &&
      ((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16 == 0 &&
      (ldq | ldk | ldv | ldo) % 4 == 0) {
    // 16-byte row pieces: every row start must be 16-byte aligned
    if (head_dim == 32) {
      return launch_f32<32>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B, num_heads,
                            max_q_len, scale, s);
    }
    if (head_dim == 64) {
      return launch_f32<64>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B, num_heads,
                            max_q_len, scale, s);
    }
    return launch_f32<128>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B, num_heads,
                           max_q_len, scale, s);
  }
  switch (dtype) {
    case NT_F32:
      return launch_generic<float>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B,
                                   num_heads, head_dim, max_q_len, scale, s);
    case NT_F16:
      return launch_generic<_Float16>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B,
                                      num_heads, head_dim, max_q_len, scale, s);
    case NT_BF16:
      return launch_generic<__bf16>(q, ldq, k, ldk, v, ldv, out, ldo, q_offsets, kv_offsets, B,
                                    num_heads, head_dim, max_q_len, scale, s);
    default:
      return fail(NT_ERR_INVALID_ARGUMENT, "attention: unknown dtype %d", dtype);
  }
}

template <typename T, int HD>
static void launch_vt(dim3 grid, hipStream_t s, const void* q, int64_t ldq, const void* k, int64_t ldk,
                      const void* vt, int64_t ldvt, void* out, int64_t ldo, const int4* sched,
                      unsigned num_heads, float scale_log2e) {
  hipLaunchKernelGGL((varlen_attention_vt_kernel<T, HD>), grid, dim3(256), 0, s, static_cast<const T*>(q),
                     ldq, static_cast<const T*>(k), ldk, static_cast<const T*>(vt), ldvt,
                     static_cast<T*>(out), ldo, sched, num_heads, scale_log2e);
}

template <int HD>
static void launch_f32_sched(dim3 grid, hipStream_t s, const void* q, int64_t ldq, const void* k, int64_t ldk,
                             const void* v, int64_t ldv, void* out, int64_t ldo, const int4* sched,
                             unsigned num_heads, float scale_log2e) {
  hipLaunchKernelGGL((varlen_attention_f32_sched_kernel<HD>), grid, dim3(256), 0, s,
                     static_cast<const float*>(q), ldq, static_cast<const float*>(k), ldk,
                     static_cast<const float*>(v), ldv, static_cast<float*>(out), ldo, sched, num_heads,
                     scale_log2e);
}

extern "C" int nt_varlen_attention_scheduled(const void* q, int64_t ldq, const void* k, int64_t ldk,
                                             const void* v, int64_t ldv, void* out, int64_t ldo,
                                             const int32_t* schedule, int64_t n_work, int64_t num_heads,
                                             int64_t head_dim, float scale, int dtype, void* stream) {
  if (n_work < 0 || num_heads < 1) return fail(NT_ERR_INVALID_ARGUMENT, "attention_scheduled: bad shape");
  if (dtype != NT_F32 || (head_dim != 32 && head_dim != 64 && head_dim != 128)) {
    return fail(NT_ERR_UNSUPPORTED, "attention_scheduled: f32 with head_dim 32, 64 or 128 only (got dtype %d, "
                "head_dim %lld)", dtype, (long long)head_dim);
  }
  if (n_work == 0) return NT_OK;
  if (!q || !k || !v || !out || !schedule) {
    return fail(NT_ERR_INVALID_ARGUMENT, "attention_scheduled: NULL pointer");
  }
  const int64_t E = num_heads * head_dim;
  if (ldq < E || ldk < E || ldv < E || ldo < E) {
    return fail(NT_ERR_INVALID_ARGUMENT, "attention_scheduled: row stride smaller than num_heads*head_dim");
  }
  if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16 != 0 || (ldq | ldk | ldv | ldo) % 4 != 0) {
    return fail(NT_ERR_UNSUPPORTED, "attention_scheduled: rows must be 16-byte aligned");
  }
  if (num_heads > 65535 || n_work * num_heads > 0x7fffffffLL) {
    return fail(NT_ERR_UNSUPPORTED, "attention_scheduled: too many workgroups");
  }
  dim3 grid((unsigned)(n_work * num_heads), 1, 1);
  const float scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = (hipStream_t)stream;
  const int4* sched = reinterpret_cast<const int4*>(schedule);
  const unsigned nh = (unsigned)num_heads;
  if (head_dim == 32) launch_f32_sched<32>(grid, s, q, ldq, k, ldk, v, ldv, out, ldo, sched, nh, scale_log2e);
  else if (head_dim == 64) launch_f32_sched<64>(grid, s, q, ldq, k, ldk, v, ldv, out, ldo, sched, nh, scale_log2e);
  else launch_f32_sched<128>(grid, s, q, ldq, k, ldk, v, ldv, out, ldo, sched, nh, scale_log2e);
  return check_launch("varlen_attention_f32_sched_kernel");
}

extern "C" int nt_varlen_attention_vt(const void* q, int64_t ldq, const void* k, int64_t ldk,
                                      const void* vt, int64_t ldvt, void* out, int64_t ldo,
                                      const int32_t* schedule, int64_t n_work, int64_t num_heads,
                                      int64_t head_dim, int64_t total_kv_tokens, float scale, int dtype,
                                      void* stream) {
  if (n_work < 0 || num_heads < 1 || total_kv_tokens < 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "attention_vt: bad shape");
  }
  if (head_dim != 32 && head_dim != 64 && head_dim != 128) {
    return fail(NT_ERR_UNSUPPORTED, "attention_vt: head_dim %lld is not 32, 64 or 128", (long long)head_dim);
  }
  if (dtype != NT_F16 && dtype != NT_BF16) {
    return fail(NT_ERR_UNSUPPORTED, "attention_vt: dtype must be f16 or bf16");
  }
  if (n_work == 0) return NT_OK;
  if (!q || !k || !vt || !out || !schedule) return fail(NT_ERR_INVALID_ARGUMENT, "attention_vt: NULL pointer");
  if (n_work > 0x3fffffffLL || num_heads > 65535 || total_kv_tokens > 0x7fffffffLL) {
    return fail(NT_ERR_UNSUPPORTED, "attention_vt: too many work items, heads or tokens");
  }
  const int64_t E = num_heads * head_dim;
  if (ldq < E || ldk < E || ldo < E || ldvt < total_kv_tokens + 72) {
    return fail(NT_ERR_INVALID_ARGUMENT,
                "attention_vt: row strides too small (ldvt must be >= total_kv_tokens + 72)");
  }
  if (n_work * num_heads > 0x7fffffffLL) {
    return fail(NT_ERR_UNSUPPORTED, "attention_vt: too many workgroups");
  }
  dim3 grid((unsigned)(n_work * num_heads), 1, 1);
  const float scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = (hipStream_t)stream;
  const int4* sched = reinterpret_cast<const int4*>(schedule);
  const unsigned nh = (unsigned)num_heads;
#define NT_VT_ARGS grid, s, q, ldq, k, ldk, vt, ldvt, out, ldo, sched, nh, scale_log2e
  if (dtype == NT_F16) {
    if (head_dim == 32) launch_vt<_Float16, 32>(NT_VT_ARGS);
    else if (head_dim == 64) launch_vt<_Float16, 64>(NT_VT_ARGS);
    else launch_vt<_Float16, 128>(NT_VT_ARGS);
  } else {
    if (head_dim == 32) launch_vt<__bf16, 32>(NT_VT_ARGS);
    else if (head_dim == 64) launch_vt<__bf16, 64>(NT_VT_ARGS);
    else launch_vt<__bf16, 128>(NT_VT_ARGS);
  }
#undef NT_VT_ARGS
  return check_launch("varlen_attention_vt_kernel");
}
