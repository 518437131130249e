// Mask -> nested size, and mask-driven compaction (gfx950, wave64).
//
// nested_tensor_from_tensor_mask keeps, in row-major order, the elements whose
// mask entry is true.  On the device that is a stream compaction per mask row:
//   1. nt_mask_row_counts: one wavefront per row, 64 mask bytes per step,
//      ballot + popcount -> keep-count per row;
//   2. an exclusive scan of the counts (scan.hip) -> output position of each row;
//   3. nt_compact_rows: one wavefront per row again; the rank of a kept entry
//      inside its 64-entry group is popcount(ballot & lanes-below), so kept
//      chunks land densely and in order.
// The host derives the nested size from the counts (extent = number of kept
// children per level) and checks that the selection is rectangular.
#include "nt_common.h"

namespace nt {

constexpr int kRowsPerBlock = 4;  // wavefronts per workgroup of the row kernels
constexpr int kBoxMaxDims = 6;    // row dims of a constituent that leading_box_kernel walks

// Predicates: a mask byte is kept if non-zero; a data element is kept if it
// differs from the padding value with the comparison of its type (so NaN != x is
// true and -0.0 != 0.0 is false, as for `tensor != padding` in torch).
struct NonZeroByte {
  typedef uint8_t type;
  __device__ __forceinline__ bool operator()(uint8_t x) const { return x != 0; }
};
template <typename T, typename C>
struct NotEqual {
  typedef T type;
  C pad;
  __device__ __forceinline__ bool operator()(T x) const { return (C)x != pad; }
};

// Bit j of the result: entry j of a lane's 16 bytes is kept.
template <typename P, int VEC>
__device__ __forceinline__ uint32_t lane_flags(const u32x4& raw, const P& pred) {
  typename P::type v[VEC];
  __builtin_memcpy(v, &raw, sizeof(v));   // 16 bytes wherever the vector path is taken
  uint32_t flags = 0;
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    if (pred(v[j])) flags |= 1u << j;
  }
  return flags;
}
// Sixteen mask bytes, four at a time in 32-bit arithmetic instead of sixteen
// compares and selects: bit 7 of every byte of t says "byte is non-zero" (the add
// carries into bit 7 exactly when one of the low seven bits is set), and the
// multiplication gathers the four bits, shifted down to bits 0 / 8 / 16 / 24, into
// bits 24..27 (the partial products land on ten different bit positions, so
// nothing carries).
template <>
__device__ __forceinline__ uint32_t lane_flags<NonZeroByte, 16>(const u32x4& raw, const NonZeroByte&) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  uint32_t flags = 0;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const uint32_t t = (((w[k] & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w[k]) & 0x80808080u;
    flags |= (((t >> 7) * 0x01020408u) >> 24) << (4 * k);
  }
  return flags;
}

// counts[r] = kept entries of row r; prefix[r] = 1 iff the kept entries are
// exactly the first counts[r] entries of the row.  A wavefront takes NR
// consecutive rows and walks them together, so that NR loads per lane are in
// flight at a time (NR = 4 for many rows of under 384 bytes, where one row per
// wavefront leaves the memory system idle; otherwise 1); a lane looks at VEC
// consecutive entries per step (16 bytes; one entry for short rows); ballots over
// the lanes' "full / non-empty / is a prefix" flags decide prefix-ness without
// any serial scan.  The results of a workgroup's 4 * NR rows leave through LDS as
// two contiguous stores: the destination may be pinned host memory.
template <typename P, int VEC, int NR>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void row_counts_kernel(
    const typename P::type* __restrict__ data, int64_t R, int64_t M, P pred,
    int32_t* __restrict__ counts, uint8_t* __restrict__ prefix) {
  typedef typename P::type T;
  __shared__ int32_t s_count[kRowsPerBlock * NR];
  __shared__ uint8_t s_prefix[kRowsPerBlock * NR];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t block_row0 = (int64_t)blockIdx.x * (kRowsPerBlock * NR);
  const int64_t row0 = block_row0 + wave * NR;
  int32_t count[NR];
  bool is_prefix[NR], ended[NR];   // ended: an entry that is not kept has been seen (wave-uniform)
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    count[r] = 0;
    is_prefix[r] = true;
    ended[r] = false;
  }
  for (int64_t base = 0; base < M; base += (int64_t)kWave * VEC) {
    const int64_t i0 = base + (int64_t)lane * VEC;
    // entries of this lane that exist (the last lanes of the last step hold fewer)
    const int64_t here = M - i0;
    const int exist = here >= VEC ? VEC : (here > 0 ? (int)here : 0);
    // A lane whose VEC entries run past the end of the row reads the LAST VEC
    // entries of the row instead (one whole 16-byte load like everyone else, no
    // element-wise tail) and drops the low VEC - exist flags: what is left are the
    // flags of entries i0 .. M - 1.  The vector path is only taken for M >= VEC.
    const int64_t ld = (VEC == 1 || here >= VEC) ? i0 : M - VEC;
    T v1[NR];         // VEC == 1
    u32x4 raw[NR];    // otherwise
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (row0 + r >= R) continue;
      const T* m = data + (row0 + r) * M;
      if (VEC == 1) {
        if (i0 < M) v1[r] = m[i0];
      } else {
        // any alignment: the part runs in unaligned-access mode
        raw[r] = load16_unaligned(reinterpret_cast<const char*>(m + ld));
      }
    }
    const uint64_t present = __ballot(exist > 0);
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (row0 + r >= R) continue;
      uint32_t flags = 0;
      if (VEC == 1) {
        if (exist > 0 && pred(v1[r])) flags = 1u;
      } else {
        flags = lane_flags<P, VEC>(raw[r], pred);
        flags = exist == VEC ? flags : (exist > 0 ? flags >> (VEC - exist) : 0u);
      }
      const int cnt = __popc(flags);
      count[r] += cnt;
      const uint64_t full = __ballot(cnt == exist && exist > 0);
      const uint64_t nonempty = __ballot(cnt > 0);
      const uint64_t lane_ok = __ballot(flags == ((1u << cnt) - 1u));
      const int q = __popcll(nonempty);
      const uint64_t low_q = q >= 64 ? ~0ull : ((1ull << q) - 1ull);
      const uint64_t low_qm1 = q == 0 ? 0ull : (low_q >> 1);
      bool ok = (lane_ok == ~0ull) && (nonempty == low_q) && ((full & low_qm1) == low_qm1);
      if (ended[r] && nonempty != 0) ok = false;
      is_prefix[r] = is_prefix[r] && ok;
      if (full != present) ended[r] = true;
    }
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int c = wave_reduce_sum(count[r]);
    if (lane == 0) {
      s_count[wave * NR + r] = c;
      s_prefix[wave * NR + r] = is_prefix[r] ? 1 : 0;
    }
  }
  __syncthreads();
  const int t = threadIdx.x;
  if (t < kRowsPerBlock * NR && block_row0 + t < R) {
    counts[block_row0 + t] = s_count[t];
    if (prefix) prefix[block_row0 + t] = s_prefix[t];
  }
}

template <typename P>
static int launch_row_counts(const void* data, int64_t R, int64_t M, P pred, int32_t* counts,
                             uint8_t* prefix, hipStream_t stream) {
  typedef typename P::type T;
  constexpr int kVec = 16 / sizeof(T);
  const T* d = static_cast<const T*>(data);
  // very short rows: one entry per lane keeps more lanes busy than 16 bytes per lane
  // (measured on 400 000 mask rows: 250 bytes 167 -> 64 us with 16-byte loads, 100
  // bytes 88 -> 61 us, 64 bytes 48 -> 57 us);
  const bool vec = M * (int64_t)sizeof(T) >= 96;
  // many short rows: four per wavefront, all of their loads in flight (400 000 rows
  // of 250 bytes: 64 against 72 us).  From a few hundred bytes per row one row per
  // wavefront is faster, the more the longer the rows: more wavefronts, each a short
  // chain (48 384 x 1015 bytes: 11.6 against 13.8 us; 8192 x 4096: 6.5 against 10.5).
  const int nr = (R >= 8192 && M * (int64_t)sizeof(T) < 384) ? 4 : 1;
  const int64_t blocks = (R + kRowsPerBlock * nr - 1) / (kRowsPerBlock * nr);
  if (blocks > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "row_counts: too many rows");
  dim3 grid((unsigned)blocks), block(kWave * kRowsPerBlock);
  if (vec && nr == 4) {
    hipLaunchKernelGGL((row_counts_kernel<P, kVec, 4>), grid, block, 0, stream, d, R, M, pred, counts, prefix);
  } else if (vec) {
    hipLaunchKernelGGL((row_counts_kernel<P, kVec, 1>), grid, block, 0, stream, d, R, M, pred, counts, prefix);
  } else if (nr == 4) {
    hipLaunchKernelGGL((row_counts_kernel<P, 1, 4>), grid, block, 0, stream, d, R, M, pred, counts, prefix);
  } else {
    hipLaunchKernelGGL((row_counts_kernel<P, 1, 1>), grid, block, 0, stream, d, R, M, pred, counts, prefix);
  }
  return check_launch("row_counts_kernel");
}

// UNIT: bytes moved per lane step in the cooperative path (1, 2, 4, 8 or 16).
template <int UNIT>
__device__ __forceinline__ void wave_copy_chunk(char* d, const char* s, int64_t bytes, int lane) {
  for (int64_t p = (int64_t)lane * UNIT; p < bytes; p += (int64_t)kWave * UNIT) {
    if (UNIT == 16) {
      *reinterpret_cast<u32x4*>(d + p) = *reinterpret_cast<const u32x4*>(s + p);
    } else if (UNIT == 8) {
      *reinterpret_cast<uint64_t*>(d + p) = *reinterpret_cast<const uint64_t*>(s + p);
    } else if (UNIT == 4) {
      *reinterpret_cast<uint32_t*>(d + p) = *reinterpret_cast<const uint32_t*>(s + p);
    } else if (UNIT == 2) {
      *reinterpret_cast<uint16_t*>(d + p) = *reinterpret_cast<const uint16_t*>(s + p);
    } else {
      d[p] = s[p];
    }
  }
}

// LANE_ELEM: chunk_bytes == UNIT and every lane moves its own chunk;
// otherwise the wavefront copies each kept chunk together.
template <int UNIT, bool LANE_ELEM>
__global__ __launch_bounds__(kWave * kRowsPerBlock) void compact_rows_kernel(
    const char* data, const uint8_t* mask, const int64_t* row_offsets, int64_t R, int64_t M,
    int64_t chunk_bytes, char* out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  if (row >= R) return;
  const uint8_t* m = mask + row * M;
  const char* src = data + row * M * chunk_bytes;
  char* dst = out + row_offsets[row] * chunk_bytes;
  int64_t kept = 0;
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (kWave - lane));
  for (int64_t base = 0; base < M; base += kWave) {
    const int64_t i = base + lane;
    const bool keep = (i < M) && (m[i] != 0);
    const uint64_t bal = __ballot(keep);
    if (LANE_ELEM) {
      if (keep) {
        const int64_t rank = kept + __popcll(bal & below);
        wave_copy_chunk<UNIT>(dst + rank * UNIT, src + i * UNIT, UNIT, 0);
      }
    } else {
      uint64_t bits = bal;
      int64_t rank = kept;
      while (bits) {  // uniform across the wavefront
        const int j = __ffsll((long long)bits) - 1;
        bits &= bits - 1;
        wave_copy_chunk<UNIT>(dst + rank * chunk_bytes, src + (base + j) * chunk_bytes,
                              chunk_bytes, lane);
        ++rank;
      }
    }
    kept += __popcll(bal);
  }
}

// Per constituent: do the row statistics describe a LEADING BOX (every row keeps
// the same leading w entries or nothing, and the rows that keep something are the
// rows whose index is below an extent in every row dim)?  That is what the mask
// of a padded tensor looks like, and then the nested size is (extents, w) and
// nothing else of the statistics has to leave the device.  One workgroup per
// constituent, one pass over its rows (the kernel is a chain of memory round
// trips; counting the extents along the axes first and comparing every row with
// the box in a second pass were three of them).
struct BoxDims {
  int64_t d[kBoxMaxDims];
};
constexpr int kBoxThreads = 1024;
__global__ __launch_bounds__(kBoxThreads) void leading_box_kernel(const int32_t* __restrict__ counts,
                                                                  const uint8_t* __restrict__ prefix,
                                                                  int64_t rows_per, BoxDims dims, int nd,
                                                                  int32_t* __restrict__ out, uint32_t* done,
                                                                  uint32_t done_value, uint32_t* arrivals,
                                                                  uint32_t stamp) {
  __shared__ int s_ext[kBoxMaxDims];
  __shared__ int s_bad;
  __shared__ unsigned s_kept, s_max_w, s_inv_min_w;
  const int64_t b = blockIdx.x;
  const int32_t* c = counts + b * rows_per;
  const uint8_t* pf = prefix + b * rows_per;
  const int t = threadIdx.x;
  if (t < kBoxMaxDims) s_ext[t] = 0;
  if (t == 0) {
    s_bad = 0;
    s_kept = 0;
    s_max_w = 0;
    s_inv_min_w = 0;
  }
  __syncthreads();
  // One pass over the rows (one memory round trip): the constituent keeps a leading
  // box iff no row fails the prefix test, every row that keeps anything keeps the
  // same number, and those rows are as many as their bounding box from the origin
  // holds (they all lie inside it, so then they fill it).
  // 32-bit index arithmetic (the host bounds rows_per): a 64-bit division per row and
  // dim made this kernel as long as the row counts themselves
  const int n_rows = (int)rows_per;
  int d[kBoxMaxDims];
#pragma unroll
  for (int k = 0; k < kBoxMaxDims; ++k) d[k] = (int)dims.d[k];
  int bad = 0, top[kBoxMaxDims];
  unsigned kept = 0, max_w = 0, inv_min_w = 0;
#pragma unroll
  for (int k = 0; k < kBoxMaxDims; ++k) top[k] = 0;
  for (int r = t; r < n_rows; r += kBoxThreads) {
    const int32_t count = c[r];
    bad |= pf[r] != 1;
    if (count == 0) continue;
    ++kept;
    max_w = (unsigned)count > max_w ? (unsigned)count : max_w;
    inv_min_w = ~(unsigned)count > inv_min_w ? ~(unsigned)count : inv_min_w;
    int rest = r;
#pragma unroll
    for (int k = kBoxMaxDims - 1; k >= 0; --k) {
      if (k < nd) {
        const int q = rest / d[k];
        const int i1 = rest - q * d[k] + 1;
        top[k] = i1 > top[k] ? i1 : top[k];
        rest = q;
      }
    }
  }
  if (bad) s_bad = 1;
  // folded over the wavefront first: a thousand lanes updating five LDS words one
  // after the other took longer than the rest of the kernel
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    kept += (unsigned)__shfl_xor((int)kept, off, kWave);
    const unsigned m1 = (unsigned)__shfl_xor((int)max_w, off, kWave);
    const unsigned m2 = (unsigned)__shfl_xor((int)inv_min_w, off, kWave);
    max_w = m1 > max_w ? m1 : max_w;
    inv_min_w = m2 > inv_min_w ? m2 : inv_min_w;
#pragma unroll
    for (int k = 0; k < kBoxMaxDims; ++k) {
      if (k < nd) {
        const int o = __shfl_xor(top[k], off, kWave);
        top[k] = o > top[k] ? o : top[k];
      }
    }
  }
  if ((t & (kWave - 1)) == 0 && kept) {
    atomicAdd(&s_kept, kept);
    atomicMax(&s_max_w, max_w);
    atomicMax(&s_inv_min_w, inv_min_w);
#pragma unroll
    for (int k = 0; k < kBoxMaxDims; ++k) {
      if (k < nd) atomicMax(&s_ext[k], top[k]);
    }
  }
  __syncthreads();
  if (t == 0) {
    unsigned long long volume = 1;
#pragma unroll
    for (int k = 0; k < kBoxMaxDims; ++k) {
      if (k < nd) volume *= (unsigned)s_ext[k];
    }
    if (s_kept != 0 && (s_max_w != ~s_inv_min_w || volume != s_kept)) s_bad = 1;
  }
  __syncthreads();
  // an empty box is described as all zeros (the extents are zero already when
  // nothing is kept)
  const int32_t w = (int32_t)s_max_w;
  if (stamp != 0) {
    // Every entry of the line travels with the call's stamp in the upper half of
    // one 8-byte word (a single store, atomic for whoever reads it): the host takes
    // an entry as soon as it carries the stamp, in any order, and the launch needs
    // no fence and no completion word, i.e. no round trip to host memory before it
    // can end.
    if (t < kBoxMaxDims + 2) {
      const int32_t v = t == 0 ? (s_bad ? 0 : 1) : (t == 1 ? w : (t - 2 < nd ? s_ext[t - 2] : 1));
      const uint64_t word = (uint64_t)(uint32_t)v | ((uint64_t)stamp << 32);
      __hip_atomic_store(reinterpret_cast<uint64_t*>(out) + b * (kBoxMaxDims + 2) + t, word, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_SYSTEM);
    }
    return;
  }
  if (t == 0) {
    // an empty box is described as all zeros (the rows' extents along the axes are
    // zero already when w is)
    out[b * (kBoxMaxDims + 2)] = s_bad ? 0 : 1;
    out[b * (kBoxMaxDims + 2) + 1] = w;
  }
  if (t < kBoxMaxDims) out[b * (kBoxMaxDims + 2) + 2 + t] = t < nd ? s_ext[t] : 1;
  if (done == nullptr) return;
  if (arrivals == nullptr) {
    // one completion word per constituent: every workgroup publishes its own line
    // (visible system-wide before the word) and nobody waits for anybody
    __threadfence_system();
    __syncthreads();
    if (t == 0) __hip_atomic_store(done + b, done_value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    return;
  }
  // The workgroup that arrives last tells the host (which polls `done`) that every
  // constituent's line is written: each workgroup makes its line visible system-wide
  // before it counts itself in, and the last one publishes after it has seen the
  // others' arrivals.  The counter is left at zero for the next launch.
  __threadfence_system();
  __syncthreads();
  if (t == 0) {
    const uint32_t before = atomicAdd(arrivals, 1u);
    if (before == gridDim.x - 1) {
      atomicExch(arrivals, 0u);
      __threadfence_system();
      __hip_atomic_store(done, done_value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

static int pick_unit(const void* a, const void* b, int64_t chunk_bytes) {
  uintptr_t x = (uintptr_t)a | (uintptr_t)b | (uintptr_t)chunk_bytes;
  if ((x & 15) == 0) return 16;
  if ((x & 7) == 0) return 8;
  if ((x & 3) == 0) return 4;
  if ((x & 1) == 0) return 2;
  return 1;
}

}  // namespace nt

using namespace nt;

extern "C" int nt_mask_row_counts(const uint8_t* mask, int64_t R, int64_t M, int32_t* counts,
                                  uint8_t* prefix, void* stream) {
  if (R < 0 || M < 0) return fail(NT_ERR_INVALID_ARGUMENT, "mask_row_counts: negative extent");
  if (R == 0) return NT_OK;
  if (!counts || (M > 0 && !mask)) return fail(NT_ERR_INVALID_ARGUMENT, "mask_row_counts: NULL pointer");
  return launch_row_counts(mask, R, M, NonZeroByte(), counts, prefix, (hipStream_t)stream);
}

extern "C" int64_t nt_leading_boxes_max_dims(void) { return kBoxMaxDims; }

static int leading_boxes(const int32_t* counts, const uint8_t* prefix, int64_t B, int64_t rows_per,
                         const int64_t* row_dims_host, int64_t nd, int32_t* boxes, uint32_t* done,
                         uint32_t done_value, uint32_t* arrivals, uint32_t stamp, void* stream) {
  if (B < 0 || rows_per < 1 || nd < 0 || nd > kBoxMaxDims || (nd > 0 && !row_dims_host)) {
    return fail(NT_ERR_INVALID_ARGUMENT, "leading_boxes: bad shape (B=%lld rows=%lld dims=%lld)", (long long)B,
                (long long)rows_per, (long long)nd);
  }
  if (B == 0) return NT_OK;
  if (B > 0x7fffffffLL || rows_per > 0x7fffffffLL) {
    return fail(NT_ERR_UNSUPPORTED, "leading_boxes: too many constituents or rows");
  }
  if (!counts || !prefix || !boxes) return fail(NT_ERR_INVALID_ARGUMENT, "leading_boxes: NULL pointer");
  BoxDims dims;
  int64_t prod = 1;
  for (int64_t k = 0; k < kBoxMaxDims; ++k) {
    dims.d[k] = k < nd ? row_dims_host[k] : 1;
    if (dims.d[k] < 1 || dims.d[k] > 0x7fffffffLL) return fail(NT_ERR_INVALID_ARGUMENT, "leading_boxes: bad row dim");
    prod *= dims.d[k];
  }
  if (prod != rows_per) return fail(NT_ERR_INVALID_ARGUMENT, "leading_boxes: row dims do not multiply to the rows");
  hipLaunchKernelGGL(leading_box_kernel, dim3((unsigned)B), dim3(kBoxThreads), 0, (hipStream_t)stream, counts, prefix,
                     rows_per, dims, (int)nd, boxes, done, done_value, arrivals, stamp);
  return check_launch("leading_box_kernel");
}

extern "C" int nt_leading_boxes(const int32_t* counts, const uint8_t* prefix, int64_t B, int64_t rows_per,
                                const int64_t* row_dims_host, int64_t nd, int32_t* boxes, uint32_t* done,
                                uint32_t done_value, uint32_t* arrivals, void* stream) {
  return leading_boxes(counts, prefix, B, rows_per, row_dims_host, nd, boxes, done, done_value, arrivals, 0, stream);
}

extern "C" int nt_leading_boxes_stamped(const int32_t* counts, const uint8_t* prefix, int64_t B, int64_t rows_per,
                                        const int64_t* row_dims_host, int64_t nd, uint64_t* lines, uint32_t stamp,
                                        void* stream) {
  if (stamp == 0) return fail(NT_ERR_INVALID_ARGUMENT, "leading_boxes_stamped: the stamp must not be 0");
  if ((uintptr_t)lines % 8 != 0) return fail(NT_ERR_INVALID_ARGUMENT, "leading_boxes_stamped: lines must be 8-byte aligned");
  return leading_boxes(counts, prefix, B, rows_per, row_dims_host, nd, reinterpret_cast<int32_t*>(lines), nullptr, 0,
                       nullptr, stamp, stream);
}

extern "C" int nt_value_row_counts(const void* data, int elem_type, double padding, int64_t R,
                                   int64_t M, int32_t* counts, uint8_t* prefix, void* stream) {
  if (R < 0 || M < 0) return fail(NT_ERR_INVALID_ARGUMENT, "value_row_counts: negative extent");
  if (R == 0) return NT_OK;
  if (!counts || (M > 0 && !data)) return fail(NT_ERR_INVALID_ARGUMENT, "value_row_counts: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  // `tensor != padding` as torch evaluates it: a floating tensor compares in its
  // own type, i.e. against the padding ROUNDED to that type (0.1 is not a half);
  // an integer tensor compares exactly against an integral padding, and in fp32
  // (torch's promotion of integer tensor and floating scalar) against any other.
  const bool integral = padding == (double)(int64_t)padding && padding >= -9.2e18 && padding <= 9.2e18;
  const int64_t ipad = integral ? (int64_t)padding : 0;
#define NT_INT_CASE(TYPE)                                                                          \
  if (integral) return launch_row_counts(data, R, M, NotEqual<TYPE, int64_t>{ipad}, counts, prefix, s); \
  return launch_row_counts(data, R, M, NotEqual<TYPE, float>{(float)padding}, counts, prefix, s);
  switch (elem_type) {
    case NT_F32: return launch_row_counts(data, R, M, NotEqual<float, float>{(float)padding}, counts, prefix, s);
    case NT_F16:
      return launch_row_counts(data, R, M, NotEqual<_Float16, float>{(float)(_Float16)padding}, counts, prefix, s);
    case NT_BF16:
      return launch_row_counts(data, R, M, NotEqual<__bf16, float>{(float)(__bf16)(float)padding}, counts, prefix, s);
    case NT_F64: return launch_row_counts(data, R, M, NotEqual<double, double>{padding}, counts, prefix, s);
    case NT_I8: NT_INT_CASE(int8_t)
    case NT_U8: NT_INT_CASE(uint8_t)
    case NT_I16: NT_INT_CASE(int16_t)
    case NT_I32: NT_INT_CASE(int32_t)
    case NT_I64: NT_INT_CASE(int64_t)
    default: return fail(NT_ERR_INVALID_ARGUMENT, "value_row_counts: unknown element type %d", elem_type);
  }
#undef NT_INT_CASE
}

extern "C" int nt_compact_rows(const void* data, const uint8_t* mask, const int64_t* row_offsets,
                               int64_t R, int64_t M, int64_t chunk_bytes, void* out,
                               void* stream) {
  if (R < 0 || M < 0 || chunk_bytes < 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "compact_rows: negative extent");
  }
  if (R == 0 || M == 0 || chunk_bytes == 0) return NT_OK;
  if (!data || !mask || !row_offsets || !out) {
    return fail(NT_ERR_INVALID_ARGUMENT, "compact_rows: NULL pointer");
  }
  const int64_t blocks = (R + kRowsPerBlock - 1) / kRowsPerBlock;
  if (blocks > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "compact_rows: too many rows");
  dim3 grid((unsigned)blocks), block(kWave * kRowsPerBlock);
  hipStream_t s = (hipStream_t)stream;
  const char* d = static_cast<const char*>(data);
  char* o = static_cast<char*>(out);
  const int unit = pick_unit(data, out, chunk_bytes);
#define NT_COMPACT(U, LE) \
  hipLaunchKernelGGL((compact_rows_kernel<U, LE>), grid, block, 0, s, d, mask, row_offsets, R, M, \
                     chunk_bytes, o)
  if (chunk_bytes == unit) {
    switch (unit) {
      case 16: NT_COMPACT(16, true); break;
      case 8: NT_COMPACT(8, true); break;
      case 4: NT_COMPACT(4, true); break;
      case 2: NT_COMPACT(2, true); break;
      default: NT_COMPACT(1, true); break;
    }
  } else {
    switch (unit) {
      case 16: NT_COMPACT(16, false); break;
      case 8: NT_COMPACT(8, false); break;
      case 4: NT_COMPACT(4, false); break;
      case 2: NT_COMPACT(2, false); break;
      default: NT_COMPACT(1, false); break;
    }
  }
#undef NT_COMPACT
  return check_launch("compact_rows_kernel");
}
