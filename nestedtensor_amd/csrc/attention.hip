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
// Any head_dim / fp32 takes the generic kernel further down (one wavefront per
// query row, fp32 FMA); it is the parity path for shapes the MFMA kernel does
// not cover, not a performance path.
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
// of another, which leaves (lo, lo) in one and (hi, hi) in the other.
__device__ __forceinline__ float max_across_halves(float v) {
  const unsigned b = __builtin_bit_cast(unsigned, v);
  const auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
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
  static __device__ __forceinline__ acc16 mma(Frag a, Frag b, acc16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

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
// Self-attention kernel of the fused layer: Q and K come row-major from the
// [T, 2E] projection buffer, V comes TRANSPOSED (Vt[h*64 + d][token], written
// that way by the QKV GEMM epilogue), so a V^T tile is 64 rows of 64
// key-contiguous values and needs no transposition on its way into LDS.
//
// LDS layout of the V^T tile: within each group of 16 keys the positions are
// permuted (key = 8a + 4g + c  ->  position 8g + 4a + c) so that the eight keys a
// lane group needs for one MFMA k-step -- the keys whose probabilities it
// already holds in its score accumulators -- are one 16-byte read.

// Work items {first token, length, first query row, 0} come from a schedule the
// host builds from the nested size (longest sequences first, no item for a tile
// that does not exist), so every workgroup that is launched has work and the
// long sequences start first.
#ifndef NT_ATTN_WAVES_PER_EU
#define NT_ATTN_WAVES_PER_EU 3
#endif

// HD: head_dim, 32, 64 or 128.  Per key tile a workgroup stages 64 K rows of HD
// elements and HD V^T rows of 64 keys; a wavefront holds HD / 16 Q fragments and
// HD / 32 output accumulator blocks.  The benchmark shapes have HD = 64; 128 needs
// about 200 registers per lane, so two wavefronts per SIMD there.
template <typename T, int HD>
__global__ __launch_bounds__(256, (HD > 64 ? 2 : NT_ATTN_WAVES_PER_EU)) void varlen_attention_vt_kernel(
    const T* __restrict__ Q, int64_t ldq, const T* __restrict__ K, int64_t ldk,
    const T* __restrict__ Vt, int64_t ldvt, T* __restrict__ O, int64_t ldo,
    const int4* __restrict__ schedule, unsigned num_heads, float scale_log2e) {
  typedef AttnT<T> AT;
  typedef typename AT::Frag Frag;

  constexpr int kKR = HD * 2 + 16;          // LDS bytes per K row (16 pad: conflict-free fragment reads)
  constexpr int kQF = HD / 16;              // Q fragments = MFMA k-steps of the score product
  constexpr int kDB = HD / 32;              // 32-row blocks of O^T
  constexpr int kKPieces = HD / 8;          // 16-byte pieces per K row
  constexpr int kKRowsPerPass = 256 / kKPieces;
  constexpr int kKP = kKTile / kKRowsPerPass;   // K pieces per thread and tile
  constexpr int kVP = HD / 32;              // V^T pieces per thread and tile (8 per row, 32 rows a pass)
  __shared__ __align__(16) char lds_k[2][kKTile * kKR];
  __shared__ __align__(16) char lds_v[2][(HD + 1) * kVRow];   // row HD: ones (see below)

  // Head fastest: the schedule lists the longest sequences first, and this way
  // their items of ALL heads are dispatched before any short item (with the
  // item index fastest, the long items of the last heads would start last and
  // run alone at the end).
  const int h = (int)(blockIdx.x % num_heads);
  // item: {first query token, query length, first query row of this tile, 0,
  //        first key token, key length, 0, 0}; self-attention lists the same
  //        sequence twice, cross-attention the two sequences of the pair
  const int4 item = schedule[2 * (blockIdx.x / num_heads)];
  const int4 item_kv = schedule[2 * (blockIdx.x / num_heads) + 1];
  const int64_t q_begin = item.x;
  const int Lq = item.y;
  const int q0 = item.z;
  const int64_t begin = item_kv.x;   // of the keys
  const int L = item_kv.y;           // number of keys

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;

  const int q_row = q0 + wave * 32 + l32;
  const bool wave_active = (q0 + wave * 32) < Lq;
  Frag qf[kQF];
  {
    // rows past Lq read the last row; their results are never stored
    const int qr = q_row < Lq ? q_row : Lq - 1;
    const T* qp = Q + (q_begin + qr) * ldq + h * HD + g * 8;
#pragma unroll
    for (int s = 0; s < kQF; ++s) {
      u32x4 v = load16_unaligned(reinterpret_cast<const char*>(qp + s * 16));
      __builtin_memcpy(&qf[s], &v, 16);
    }
  }

  acc16 o_acc[kDB];
#pragma unroll
  for (int i = 0; i < kDB; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
  float m_run = -INFINITY;

  const int ntiles = (L + kKTile - 1) / kKTile;
  const T* kbase = K + begin * ldk + h * HD;
  const T* vbase = Vt + (int64_t)h * HD * ldvt + begin;

  // Each thread moves HD / 32 16-byte pieces of a K tile and as many of a V^T tile.
  // The loads are unconditional and unmasked (clamped addresses), so that the
  // wavefront only waits for them where the data is stored to LDS.  All per-thread
  // addressing is set up once; a step only advances pointers.
  const int r0 = tid >> 3;      // V^T: row of piece 0 (piece i: r0 + 32 i), keys 8 cc .. 8 cc + 7
  const int cc = tid & 7;
  const int kr0 = tid / kKPieces;   // K: row of piece 0 (piece i: kr0 + i * kKRowsPerPass)
  const int kc = tid % kKPieces;    //    elements 8 kc .. 8 kc + 7 of the row
  u32x4 rk[kKP], rv[kVP];
  const char* k_last = reinterpret_cast<const char*>(kbase + (int64_t)(L - 1) * ldk + kc * 8);
  const int64_t k_step = (int64_t)kKTile * ldk * (int64_t)sizeof(T);
  const char* v_ptr[kVP];
#pragma unroll
  for (int i = 0; i < kVP; ++i) {
    v_ptr[i] = reinterpret_cast<const char*>(vbase + (int64_t)(r0 + i * 32) * ldvt + cc * 8);
  }
  auto gload_k = [&](int t_in) {
    const int t = t_in < ntiles ? t_in : ntiles - 1;   // past the end: re-read, never used
    const char* tile = reinterpret_cast<const char*>(kbase + kc * 8) + t * k_step;
#pragma unroll
    for (int i = 0; i < kKP; ++i) {
      // rows past L read row L - 1 (a valid key: it cannot raise the row maximum)
      const int row = kr0 + i * kKRowsPerPass;
      const int kr = t * kKTile + row;
      const char* src = tile + (int64_t)row * ldk * (int64_t)sizeof(T);
      rk[i] = load16_unaligned(kr < L ? src : k_last);
    }
  };
  auto gload_v = [&](int t_in) {
    const int t = t_in < ntiles ? t_in : ntiles - 1;
    // V^T piece: keys key0 .. key0+7 of row d, read where it lies (the rows of Vt
    // are readable 72 elements past the last token)
#pragma unroll
    for (int i = 0; i < kVP; ++i) {
      rv[i] = load16_unaligned(v_ptr[i] + t * (kKTile * (int)sizeof(T)));
    }
  };
  auto lstore_k = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kKP; ++i) {
      store16(&lds_k[buf][(kr0 + i * kKRowsPerPass) * kKR + kc * 16], rk[i]);
    }
  };
  // piece cc = keys 8cc .. 8cc+7 = (ks = cc/2, a = cc%2); its low half (g = 0)
  // goes to position 16ks + 4a, its high half (g = 1) to 16ks + 8 + 4a.
  const int v_lo = (16 * (cc >> 1) + 4 * (cc & 1)) * 2;
  // keys at or past L are zeroed in the last tile: a probability must not meet
  // a NaN there, and the ones row must not count them
  uint32_t vm[4];
  {
    int nv = L - ((ntiles - 1) * kKTile + cc * 8);
    nv = nv > 8 ? 8 : (nv < 0 ? 0 : nv);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      vm[j] = nv >= 2 * j + 2 ? 0xffffffffu : (nv == 2 * j + 1 ? 0x0000ffffu : 0u);
    }
  }
  // Row 64 of a V^T buffer: 1 for every valid key.  Multiplied with P^T by the
  // matrix pipe it yields the softmax denominators, and because it is zero past L
  // (like the V^T columns) the keys of a partial tile need no masking of their
  // scores.  Full tiles share the all-ones row written here once; the last tile
  // writes its own masked row.
  if (r0 == 0) {
    const uint64_t ones = ((uint64_t)AT::kOnePair << 32) | AT::kOnePair;
#pragma unroll
    for (int b2 = 0; b2 < 2; ++b2) {
      char* row = &lds_v[b2][HD * kVRow + v_lo];
      *reinterpret_cast<uint64_t*>(row) = ones;
      *reinterpret_cast<uint64_t*>(row + 16) = ones;
    }
  }
  auto lstore_v = [&](int buf, int t) {
    if (t < ntiles - 1) {   // uniform: a full tile, nothing to mask
#pragma unroll
      for (int i = 0; i < kVP; ++i) {
        char* row = &lds_v[buf][(r0 + i * 32) * kVRow + v_lo];
        *reinterpret_cast<uint64_t*>(row) = ((uint64_t)rv[i].y << 32) | rv[i].x;
        *reinterpret_cast<uint64_t*>(row + 16) = ((uint64_t)rv[i].w << 32) | rv[i].z;
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < kVP; ++i) {
      char* row = &lds_v[buf][(r0 + i * 32) * kVRow + v_lo];
      const uint64_t lo = ((uint64_t)(rv[i].y & vm[1]) << 32) | (rv[i].x & vm[0]);
      const uint64_t hi = ((uint64_t)(rv[i].w & vm[3]) << 32) | (rv[i].z & vm[2]);
      *reinterpret_cast<uint64_t*>(row) = lo;
      *reinterpret_cast<uint64_t*>(row + 16) = hi;
    }
    if (r0 == 0) {
      char* row = &lds_v[buf][HD * kVRow + v_lo];
      const uint64_t lo = ((uint64_t)(AT::kOnePair & vm[1]) << 32) | (AT::kOnePair & vm[0]);
      const uint64_t hi = ((uint64_t)(AT::kOnePair & vm[3]) << 32) | (AT::kOnePair & vm[2]);
      *reinterpret_cast<uint64_t*>(row) = lo;
      *reinterpret_cast<uint64_t*>(row + 16) = hi;
    }
  };

  // S^T tile of K tile in lds_k[buf]:
  // s[kb][e] = score(key = 64 t + 32 kb + 8 (e/4) + 4 g + e%4, q = l32)
  auto scores = [&](acc16 (&sa)[2], int buf) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int e = 0; e < 16; ++e) sa[kb][e] = 0.0f;
      const char* krow = &lds_k[buf][(kb * 32 + l32) * kKR + g * 16];
#pragma unroll
      for (int s = 0; s < kQF; ++s) {
        Frag kf = *reinterpret_cast<const Frag*>(krow + s * 32);
        sa[kb] = AT::mma(kf, qf[s], sa[kb]);
      }
    }
  };

  // Online softmax of one tile's scores, then O^T += V^T P^T and the
  // denominators l += 1^T P^T from lds_v[vbuf].
  //
  // Keys past L in a partial tile: their K rows are copies of row L - 1, so they
  // cannot raise the row maximum; their V^T columns and their entries of the ones
  // row are zero, so they add nothing to O or l.  No score is ever masked.
  acc16 l_acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) l_acc[e] = 0.0f;
  auto softmax_pv = [&](acc16 (&sa)[2], int vbuf) {
    float m_tile = sa[0][0];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) m_tile = fmaxf(m_tile, sa[kb][e]);
    m_tile = max_across_halves(m_tile);
    const float m_new = fmaxf(m_run, m_tile);   // finite: every tile holds a valid key
    // raw v_exp_f32: arguments are <= 0, results in [0, 1]
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2e);
    const float m_scaled = m_new * scale_log2e;
    m_run = m_new;
    // the running maxima settle after the first tiles; then alpha is 1 in
    // every lane and the multiplications are skipped (wavefront-uniform)
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int i = 0; i < kDB; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;
      l_acc[0] *= alpha;   // every element of l_acc holds the same sum; [0] is the one read
    }
    Frag pf[4];   // P^T as B-operand: k-step ks = 2 kb + half uses sa[kb][8 half .. +8]
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float p0 =
              __builtin_amdgcn_exp2f(fmaf(sa[kb][half * 8 + 2 * j], scale_log2e, -m_scaled));
          const float p1 =
              __builtin_amdgcn_exp2f(fmaf(sa[kb][half * 8 + 2 * j + 1], scale_log2e, -m_scaled));
          w[j] = AT::cvt2(p0, p1);
        }
        __builtin_memcpy(&pf[kb * 2 + half], w, 16);
      }
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int db = 0; db < kDB; ++db) {
        const char* vrow = &lds_v[vbuf][(db * 32 + l32) * kVRow + g * 16];
        Frag vf = *reinterpret_cast<const Frag*>(vrow + ks * 32);
        o_acc[db] = AT::mma(vf, pf[ks], o_acc[db]);
      }
      // all 32 rows of this A-operand are the ones row: every lane gets l[q]
      Frag of = *reinterpret_cast<const Frag*>(&lds_v[vbuf][HD * kVRow + g * 16 + ks * 32]);
      l_acc = AT::mma(of, pf[ks], l_acc);
    }
  };

  // Tile t + 1 travels global -> registers while tile t is computed, and goes
  // registers -> LDS (the other buffer) after the compute, before the barrier.
  // Wavefronts of other workgroups on the SIMD (three fit) fill the matrix pipe
  // while this one runs its softmax, and the other way round.
  gload_k(0);
  gload_v(0);
  lstore_k(0);
  lstore_v(0, 0);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    const int buf = t & 1;
    gload_k(t + 1);   // past the end: re-reads the last tile
    gload_v(t + 1);
    // keep the loads above the MFMA / softmax work (the scheduler would sink them)
    __builtin_amdgcn_sched_barrier(0);
    if (wave_active) {
      acc16 sa[2];
      scores(sa, buf);
      softmax_pv(sa, buf);
    }
    lstore_k(buf ^ 1);          // past the end: harmless, the buffer is not read again
    lstore_v(buf ^ 1, t + 1);
    __syncthreads();
  }

  if (!wave_active || q_row >= Lq) return;
  const float l_tot = l_acc[0];
  const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
  T* op = O + (q_begin + q_row) * ldo + h * HD;
#pragma unroll
  for (int db = 0; db < kDB; ++db) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      // d = 32 db + 8 r + 4 g + (0..3)
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
