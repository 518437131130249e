// Consumers of the offsets array of a nested tensor (gfx950): row gather
// (embedding on packed indices, time-major re-ordering for a PackedSequence),
// per-constituent reduction of gathered rows (embedding_bag), and the column
// indices of the CSR view.  All are HBM-bound integer / copy work; the reference
// builds each of them on the host or with one ATen call per constituent
// (nestedtensor/csrc/functions.cpp:14-63, nestedtensor/nested/nested.py:43-118,
// 484-488, nestedtensor/csrc/nested_tensor_impl.h:326-349).
#include "nt_common.h"

namespace nt {

// dst row r = src row index[r]; rows are row_bytes long, moved in pieces of UNIT
// bytes (the largest power of two that divides row_bytes and both base
// addresses).  An index outside [0, src_rows) yields a zero row and is counted.
template <int UNIT>
__global__ __launch_bounds__(256) void gather_rows_kernel(
    const char* __restrict__ src, int64_t src_rows, int64_t row_bytes,
    const int64_t* __restrict__ index, char* __restrict__ dst, int64_t n_rows,
    int32_t* __restrict__ oob) {
  const int64_t pieces_per_row = row_bytes / UNIT;
  const int64_t total = n_rows * pieces_per_row;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; id < total; id += stride) {
    const int64_t r = id / pieces_per_row;
    const int64_t p = id - r * pieces_per_row;
    const int64_t s = index[r];
    const bool ok = s >= 0 && s < src_rows;
    if (!ok && p == 0 && oob) atomicAdd(oob, 1);
    char* d = dst + r * row_bytes + p * UNIT;
    const char* q = src + (ok ? s : 0) * row_bytes + p * UNIT;
    if (UNIT == 16) {
      u32x4 v = *reinterpret_cast<const u32x4*>(q);
      if (!ok) v = u32x4{0, 0, 0, 0};
      store16_stream(d, v);
    } else if (UNIT == 8) {
      *reinterpret_cast<uint64_t*>(d) = ok ? *reinterpret_cast<const uint64_t*>(q) : 0ull;
    } else if (UNIT == 4) {
      *reinterpret_cast<uint32_t*>(d) = ok ? *reinterpret_cast<const uint32_t*>(q) : 0u;
    } else if (UNIT == 2) {
      *reinterpret_cast<uint16_t*>(d) = ok ? *reinterpret_cast<const uint16_t*>(q) : (uint16_t)0;
    } else {
      *d = ok ? *q : (char)0;
    }
  }
}

// Time-major order of a PackedSequence: token t of the sequence at sorted
// position r goes to row step_starts[t] + r.  index_out[that row] = source row.
__global__ __launch_bounds__(256) void packed_sequence_index_kernel(
    const int64_t* __restrict__ offsets, const int64_t* __restrict__ rank,
    const int64_t* __restrict__ step_starts, int64_t B, int64_t T, int64_t* __restrict__ index_out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T) return;
  const int64_t b = find_segment(offsets, B, i);
  const int64_t t = i - offsets[b];
  index_out[step_starts[t] + rank[b]] = i;
}

// out[offsets[b] + j] = j
__global__ __launch_bounds__(256) void ragged_arange_kernel(const int64_t* __restrict__ offsets,
                                                            int64_t* __restrict__ out) {
  const int64_t b = blockIdx.x;
  const int64_t begin = offsets[b];
  const int64_t len = offsets[b + 1] - begin;
  const int64_t stride = (int64_t)gridDim.y * blockDim.x;
  for (int64_t j = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; j < len; j += stride) {
    out[begin + j] = j;
  }
}

enum { kBagSum = 0, kBagMean = 1, kBagMax = 2 };

// out[b, c] = reduce over the bag's tokens t of weight[indices[t], c], tokens in
// order (a thread owns a column, so sums are formed in token order like a
// sequential host loop).  Empty bags give 0 in every mode.
template <typename T>
__global__ __launch_bounds__(64) void embedding_bag_kernel(
    const T* __restrict__ weight, int64_t ldw, int64_t num_embeddings,
    const int64_t* __restrict__ indices, const int64_t* __restrict__ offsets, T* __restrict__ out,
    int64_t n, int mode, int32_t* __restrict__ oob) {
  constexpr int kAhead = 8;   // rows in flight per lane
  const int64_t b = blockIdx.x;
  const int64_t c = (int64_t)blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= n) return;
  const int64_t begin = offsets[b], end = offsets[b + 1];
  float acc = 0.0f;
  bool first = true;
  for (int64_t t0 = begin; t0 < end; t0 += kAhead) {
    float v[kAhead];
    bool use[kAhead];
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      const int64_t t = t0 + j;
      const int64_t row = t < end ? indices[t] : 0;
      const bool ok = row >= 0 && row < num_embeddings;
      if (t < end && !ok && c == 0 && oob) atomicAdd(oob, 1);
      use[j] = t < end && ok;
      v[j] = (float)weight[(use[j] ? row : 0) * ldw + c];
    }
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      if (use[j]) {
        if (mode == kBagMax) {
          acc = first ? v[j] : (v[j] > acc ? v[j] : acc);
        } else {
          acc += v[j];
        }
        first = false;
      }
    }
  }
  if (mode == kBagMean && end > begin) acc = acc / (float)(end - begin);
  out[b * n + c] = (T)acc;
}

// Rows of whole, aligned 16-byte pieces: a lane owns 8 (16-bit) or 4 (32-bit)
// consecutive columns, the kBagWaves wavefronts of a workgroup take blocks of
// kAhead tokens of the bag in turn, all kAhead rows in flight at once, and the
// partial results are combined through LDS in wavefront order (so sums are formed
// in a different order than a sequential loop, but always in the same one).  A
// bag is a chain of index -> row loads, so what it costs is the number of such
// rounds: 16 wavefronts x 8 rows cover a few hundred tokens in two or three; short
// bags get 4 wavefronts.
template <typename T, int kBagWaves>
__global__ __launch_bounds__(kBagWaves * 64) void embedding_bag_vec_kernel(
    const T* __restrict__ weight, int64_t ldw, int64_t num_embeddings,
    const int64_t* __restrict__ indices, const int64_t* __restrict__ offsets, T* __restrict__ out,
    int64_t n, int mode, int32_t* __restrict__ oob) {
  constexpr int kPer = 16 / sizeof(T);
  constexpr int kAhead = 8;
  __shared__ float part[kBagWaves][kWave][kPer];
  __shared__ int any_row[kBagWaves];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t b = blockIdx.x;
  const int64_t c0 = ((int64_t)blockIdx.y * kWave + lane) * kPer;   // first column of this lane
  const bool col_ok = c0 < n;                                       // n is a multiple of kPer
  const int64_t begin = offsets[b], end = offsets[b + 1];
  float acc[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) acc[j] = 0.0f;
  bool first = true;
  for (int64_t t0 = begin + wave * kAhead; t0 < end; t0 += kBagWaves * kAhead) {
    u32x4 raw[kAhead];
    bool use[kAhead];
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      const int64_t t = t0 + j;
      const int64_t row = t < end ? indices[t] : 0;
      const bool ok = row >= 0 && row < num_embeddings;
      if (t < end && !ok && lane == 0 && blockIdx.y == 0 && oob) atomicAdd(oob, 1);
      use[j] = t < end && ok;
      raw[j] = *reinterpret_cast<const u32x4*>(weight + (use[j] ? row : 0) * ldw + (col_ok ? c0 : 0));
    }
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      if (use[j]) {
        T v[kPer];
        __builtin_memcpy(v, &raw[j], 16);
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
          const float f = (float)v[e];
          if (mode == kBagMax) {
            acc[e] = first ? f : (f > acc[e] ? f : acc[e]);
          } else {
            acc[e] += f;
          }
        }
        first = false;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < kPer; ++e) part[wave][lane][e] = acc[e];
  if (lane == 0) any_row[wave] = first ? 0 : 1;
  __syncthreads();
  if (wave != 0 || !col_ok) return;
  float res[kPer];
  bool have = false;
#pragma unroll
  for (int e = 0; e < kPer; ++e) res[e] = 0.0f;
#pragma unroll
  for (int w = 0; w < kBagWaves; ++w) {
    if (!any_row[w]) continue;   // uniform
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
      const float f = part[w][lane][e];
      if (mode == kBagMax) {
        res[e] = have ? (f > res[e] ? f : res[e]) : f;
      } else {
        res[e] += f;
      }
    }
    have = true;
  }
  T o[kPer];
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    float f = res[e];
    if (mode == kBagMean && end > begin) f = f / (float)(end - begin);
    o[e] = (T)f;
  }
  u32x4 bits;
  __builtin_memcpy(&bits, o, 16);
  *reinterpret_cast<u32x4*>(out + b * n + c0) = bits;
}

static int pick_unit3(const void* a, const void* b, int64_t row_bytes) {
  const uintptr_t x = (uintptr_t)a | (uintptr_t)b | (uintptr_t)row_bytes;
  if ((x & 15) == 0) return 16;
  if ((x & 7) == 0) return 8;
  if ((x & 3) == 0) return 4;
  if ((x & 1) == 0) return 2;
  return 1;
}

template <int UNIT>
static void launch_gather(const void* src, int64_t src_rows, int64_t row_bytes, const int64_t* index,
                          void* dst, int64_t n_rows, int32_t* oob, hipStream_t stream) {
  const int64_t total = n_rows * (row_bytes / UNIT);
  int64_t blocks = (total + 255) / 256;
  if (blocks > (1 << 22)) blocks = 1 << 22;   // grid-stride beyond that
  hipLaunchKernelGGL((gather_rows_kernel<UNIT>), dim3((unsigned)blocks), dim3(256), 0, stream,
                     static_cast<const char*>(src), src_rows, row_bytes, index,
                     static_cast<char*>(dst), n_rows, oob);
}

}  // namespace nt

using namespace nt;

extern "C" int nt_gather_rows(const void* src, int64_t src_rows, int64_t row_bytes,
                              const int64_t* index, void* dst, int64_t n_rows, int32_t* oob_count,
                              void* stream) {
  if (src_rows < 0 || row_bytes < 0 || n_rows < 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "gather_rows: negative extent");
  }
  if (n_rows == 0 || row_bytes == 0) return NT_OK;
  if (!src || !index || !dst) return fail(NT_ERR_INVALID_ARGUMENT, "gather_rows: NULL pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (pick_unit3(src, dst, row_bytes)) {
    case 16: launch_gather<16>(src, src_rows, row_bytes, index, dst, n_rows, oob_count, s); break;
    case 8: launch_gather<8>(src, src_rows, row_bytes, index, dst, n_rows, oob_count, s); break;
    case 4: launch_gather<4>(src, src_rows, row_bytes, index, dst, n_rows, oob_count, s); break;
    case 2: launch_gather<2>(src, src_rows, row_bytes, index, dst, n_rows, oob_count, s); break;
    default: launch_gather<1>(src, src_rows, row_bytes, index, dst, n_rows, oob_count, s); break;
  }
  return check_launch("gather_rows_kernel");
}

extern "C" int nt_packed_sequence_index(const int64_t* offsets, const int64_t* rank,
                                        const int64_t* step_starts, int64_t B, int64_t total_rows,
                                        int64_t* index_out, void* stream) {
  if (B < 0 || total_rows < 0) return fail(NT_ERR_INVALID_ARGUMENT, "packed_sequence_index: negative extent");
  if (total_rows == 0) return NT_OK;
  if (B == 0 || !offsets || !rank || !step_starts || !index_out) {
    return fail(NT_ERR_INVALID_ARGUMENT, "packed_sequence_index: NULL pointer or no sequences");
  }
  const int64_t blocks = (total_rows + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "packed_sequence_index: too many rows");
  hipLaunchKernelGGL(packed_sequence_index_kernel, dim3((unsigned)blocks), dim3(256), 0,
                     (hipStream_t)stream, offsets, rank, step_starts, B, total_rows, index_out);
  return check_launch("packed_sequence_index_kernel");
}

extern "C" int nt_ragged_arange(const int64_t* offsets, int64_t B, int64_t max_len, int64_t* out,
                                void* stream) {
  if (B < 0 || max_len < 0) return fail(NT_ERR_INVALID_ARGUMENT, "ragged_arange: negative extent");
  if (B == 0 || max_len == 0) return NT_OK;
  if (!offsets || !out) return fail(NT_ERR_INVALID_ARGUMENT, "ragged_arange: NULL pointer");
  if (B > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "ragged_arange: too many rows");
  int64_t tiles = (max_len + 1023) / 1024;   // a block covers >= 4 elements per thread before looping
  if (tiles > 65535) tiles = 65535;
  hipLaunchKernelGGL(ragged_arange_kernel, dim3((unsigned)B, (unsigned)tiles), dim3(256), 0,
                     (hipStream_t)stream, offsets, out);
  return check_launch("ragged_arange_kernel");
}

extern "C" int nt_embedding_bag(const void* weight, int64_t ldw, int64_t num_embeddings,
                                const int64_t* indices, int64_t num_indices, const int64_t* offsets,
                                void* out, int64_t B, int64_t n, int mode, int dtype,
                                int32_t* oob_count, void* stream) {
  if (B < 0 || n < 0 || num_embeddings < 0 || ldw < n || num_indices < 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "embedding_bag: bad shape");
  }
  if (mode < 0 || mode > 2) return fail(NT_ERR_INVALID_ARGUMENT, "embedding_bag: mode %d", mode);
  if (B == 0 || n == 0) return NT_OK;
  if (!weight || !offsets || !out) return fail(NT_ERR_INVALID_ARGUMENT, "embedding_bag: NULL pointer");
  if (num_embeddings == 0) return fail(NT_ERR_INVALID_ARGUMENT, "embedding_bag: empty table");
  if (B > 0x7fffffffLL || (n + 63) / 64 > 65535) {
    return fail(NT_ERR_UNSUPPORTED, "embedding_bag: too many bags or columns");
  }
  hipStream_t s = (hipStream_t)stream;
  const int64_t elem = dtype == NT_F32 ? 4 : 2;
  const int64_t per = 16 / elem;
  const bool vec = n % per == 0 && ldw % per == 0 && (uintptr_t)weight % 16 == 0 && (uintptr_t)out % 16 == 0;
  dim3 grid((unsigned)B, (unsigned)(vec ? (n / per + 63) / 64 : (n + 63) / 64));
  const bool long_bags = num_indices >= 64 * B;     // 64 tokens per bag or more on average
#define NT_BAG_CASE(TYPE)                                                                         \
  if (vec) {                                                                                      \
    if (long_bags) {                                                                              \
      hipLaunchKernelGGL((embedding_bag_vec_kernel<TYPE, 16>), grid, dim3(16 * 64), 0, s,         \
                         static_cast<const TYPE*>(weight), ldw, num_embeddings, indices, offsets, \
                         static_cast<TYPE*>(out), n, mode, oob_count);                            \
    } else {                                                                                      \
      hipLaunchKernelGGL((embedding_bag_vec_kernel<TYPE, 4>), grid, dim3(4 * 64), 0, s,           \
                         static_cast<const TYPE*>(weight), ldw, num_embeddings, indices, offsets, \
                         static_cast<TYPE*>(out), n, mode, oob_count);                            \
    }                                                                                             \
  } else {                                                                                        \
    hipLaunchKernelGGL((embedding_bag_kernel<TYPE>), grid, dim3(64), 0, s,                        \
                       static_cast<const TYPE*>(weight), ldw, num_embeddings, indices, offsets,   \
                       static_cast<TYPE*>(out), n, mode, oob_count);                              \
  }                                                                                               \
  break;
  switch (dtype) {
    case NT_F32: NT_BAG_CASE(float)
    case NT_F16: NT_BAG_CASE(_Float16)
    case NT_BF16: NT_BAG_CASE(__bf16)
    default: return fail(NT_ERR_UNSUPPORTED, "embedding_bag: dtype %d is not f32, f16 or bf16", dtype);
  }
#undef NT_BAG_CASE
  return check_launch("embedding_bag_kernel");
}

// ---------------------------------------------------------------------------
// Per-constituent 2-D transpose on the packed buffer: constituent b is a
// row-major [rows[b], cols[b]] matrix at element offset offsets[b]; the result
// holds its [cols[b], rows[b]] transpose at the same offset.  With rows = C and
// cols = H_b * W_b this is NCHW -> NHWC of a batch of ragged images, and the
// other way round with the two exchanged (the reference's
// transpose_nchw_nhwc / transpose_nhwc_nchw, nestedtensor/csrc/transpose.cpp:87-204,
// kernels nestedtensor/csrc/cuda/transpose.cu).  One workgroup per TR x TC tile,
// through LDS, so that both the reads and the writes are contiguous per
// wavefront; tile_offsets[b] = number of tiles of all constituents before b, and
// a workgroup finds its constituent by binary search.  The caller picks the tile
// shape; 64 x 64 keeps the most workgroups in flight and is the fastest on image
// shapes, the taller and wider ones move longer contiguous pieces per tile row.
namespace nt {

constexpr int kTrMaxTileBytes = 32 * 1024;

template <typename U, int TR, int TC>
__global__ __launch_bounds__(256) void transpose_ragged_kernel(
    const U* __restrict__ in, U* __restrict__ out, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ rows, const int64_t* __restrict__ cols,
    const int64_t* __restrict__ tile_offsets, int64_t B) {
  // a lane moves V consecutive elements (8 bytes) per access on both sides
  constexpr int V = 8 / (int)sizeof(U);
  constexpr int kLanesIn = TC / V, kRowsPerPassIn = 256 / kLanesIn;
  constexpr int kLanesOut = TR / V, kRowsPerPassOut = 256 / kLanesOut;
  constexpr int kStride = TC + V;      // keeps every row of the tile 8-byte aligned
  static_assert(kLanesIn <= 256 && kLanesOut <= 256, "tile too wide for 256 lanes");
  __shared__ __align__(8) U tile[TR][kStride];
  // Workgroups are dealt to the 8 XCDs in turn; give each XCD a contiguous run of
  // tiles, so that neighbouring pieces of an output row meet in one L2.
  int64_t id = blockIdx.x;
  {
    const int64_t per_xcd = gridDim.x / 8;
    if (id < per_xcd * 8) id = (id % 8) * per_xcd + id / 8;
  }
  const int64_t b = find_segment(tile_offsets, B, id);
  const int64_t R = rows[b], C = cols[b];
  const int64_t tiles_c = (C + TC - 1) / TC;
  const int64_t local = id - tile_offsets[b];
  const int64_t r0 = (local / tiles_c) * TR;
  const int64_t c0 = (local % tiles_c) * TC;
  const U* src = in + offsets[b];
  U* dst = out + offsets[b];
  {
    const int lv = (threadIdx.x % kLanesIn) * V;   // first of this lane's V elements
    const int lr = threadIdx.x / kLanesIn;
    for (int r = lr; r < TR; r += kRowsPerPassIn) {
      if (r0 + r < R) {
        const U* p = src + (r0 + r) * C + c0 + lv;
        if (c0 + lv + V <= C) {
          uint64_t bits;
          __builtin_memcpy(&bits, p, 8);                // any alignment
          *reinterpret_cast<uint64_t*>(&tile[r][lv]) = bits;
        } else {
#pragma unroll
          for (int j = 0; j < V; ++j)
            if (c0 + lv + j < C) tile[r][lv + j] = p[j];
        }
      }
    }
  }
  __syncthreads();
  const int lv = (threadIdx.x % kLanesOut) * V;
  const int lr = threadIdx.x / kLanesOut;
  for (int c = lr; c < TC; c += kRowsPerPassOut) {
    if (c0 + c < C) {
      U v[V];
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = tile[lv + j][c];
      U* q = dst + (c0 + c) * R + r0 + lv;
      if (r0 + lv + V <= R) {
        uint64_t bits;
        __builtin_memcpy(&bits, v, 8);
        __builtin_memcpy(q, &bits, 8);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
          if (r0 + lv + j < R) q[j] = v[j];
      }
    }
  }
}

// 64 x 64 tiles of 2-byte elements (fp16 / bf16 images) with 16-byte global accesses
// on both sides.  The tile lies in LDS as dwords (two neighbouring columns each)
// with an odd row stride: a lane of the transposed read takes one dword of eight
// consecutive rows, which is conflict-free, and v_perm splits the eight dwords
// into the 16-byte pieces of two output rows.  Where every output row of the
// constituent is a whole number of 128-byte lines (rows % 64 == 0, e.g. NCHW ->
// NHWC of 64 or 256 channels, where a tile's output is one contiguous block) the
// stores are non-temporal: 4.9 -> 5.45 TB/s on 16 images [64, H, W].  Elsewhere a
// tile writes 128-byte pieces that straddle lines, which only the L2 can merge
// with the neighbouring tile's; non-temporal stores halve the rate there.
__global__ __launch_bounds__(256) void transpose_u16_kernel(
    const uint16_t* __restrict__ in, uint16_t* __restrict__ out, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ rows, const int64_t* __restrict__ cols,
    const int64_t* __restrict__ tile_offsets, int64_t B) {
  constexpr int TR = 64, TC = 64, S = TC / 2 + 1;
  __shared__ uint32_t tile[TR * S];
  int64_t id = blockIdx.x;
  {
    const int64_t per_xcd = gridDim.x / 8;
    if (id < per_xcd * 8) id = (id % 8) * per_xcd + id / 8;
  }
  const int64_t b = find_segment(tile_offsets, B, id);
  const int64_t R = rows[b], C = cols[b];
  const int64_t tiles_c = (C + TC - 1) / TC;
  const int64_t local = id - tile_offsets[b];
  const int64_t r0 = (local / tiles_c) * TR;
  const int64_t c0 = (local % tiles_c) * TC;
  const uint16_t* src = in + offsets[b];
  uint16_t* dst = out + offsets[b];
  {
    const int k = threadIdx.x & 7;
    const int lr = threadIdx.x >> 3;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int r = lr + 32 * pass;
      if (r0 + r < R) {
        const uint16_t* p = src + (r0 + r) * C + c0 + 8 * k;
        if (c0 + 8 * k + 8 <= C) {
          const u32x4 bits = load16_unaligned(reinterpret_cast<const char*>(p));
          uint32_t* t = &tile[r * S + 4 * k];
          t[0] = bits.x;
          t[1] = bits.y;
          t[2] = bits.z;
          t[3] = bits.w;
        } else {
          uint16_t* t16 = reinterpret_cast<uint16_t*>(&tile[r * S]) + 8 * k;
          for (int j = 0; j < 8; ++j) t16[j] = c0 + 8 * k + j < C ? p[j] : (uint16_t)0;
        }
      }
    }
  }
  __syncthreads();
  // lane = (eight rows, one pair of columns)
  const int lo = threadIdx.x & 7, cp = threadIdx.x >> 3;
  uint32_t x[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) x[j] = tile[(8 * lo + j) * S + cp];
  u32x4 even, odd;      // the pieces of output rows c and c + 1
  even.x = __builtin_amdgcn_perm(x[1], x[0], 0x05040100u);
  even.y = __builtin_amdgcn_perm(x[3], x[2], 0x05040100u);
  even.z = __builtin_amdgcn_perm(x[5], x[4], 0x05040100u);
  even.w = __builtin_amdgcn_perm(x[7], x[6], 0x05040100u);
  odd.x = __builtin_amdgcn_perm(x[1], x[0], 0x07060302u);
  odd.y = __builtin_amdgcn_perm(x[3], x[2], 0x07060302u);
  odd.z = __builtin_amdgcn_perm(x[5], x[4], 0x07060302u);
  odd.w = __builtin_amdgcn_perm(x[7], x[6], 0x07060302u);
  const int64_t c = c0 + 2 * cp;
  uint16_t* q = dst + c * R + r0 + 8 * lo;
  if (r0 + 8 * lo + 8 <= R) {
    // every piece is a whole aligned line when every output row starts on a line:
    // rows of a multiple of 64 elements in a constituent that starts on one
    const bool lines = (R & 63) == 0 && (reinterpret_cast<uintptr_t>(dst) & 127) == 0;
    if (lines) {
      if (c < C) __builtin_nontemporal_store(even, reinterpret_cast<u32x4*>(q));
      if (c + 1 < C) __builtin_nontemporal_store(odd, reinterpret_cast<u32x4*>(q + R));
    } else {
      if (c < C) __builtin_memcpy(q, &even, 16);
      if (c + 1 < C) __builtin_memcpy(q + R, &odd, 16);
    }
  } else {
    uint16_t ve[8], vo[8];
    __builtin_memcpy(ve, &even, 16);
    __builtin_memcpy(vo, &odd, 16);
    for (int j = 0; j < 8; ++j) {
      if (r0 + 8 * lo + j < R) {
        if (c < C) q[j] = ve[j];
        if (c + 1 < C) q[R + j] = vo[j];
      }
    }
  }
}

// The same transposition for output rows that do NOT begin on 128-byte lines
// (NHWC -> NCHW of images whose H x W is no multiple of 64: output row c begins R
// elements after row c - 1).  A 64-element piece of such a row covers two half
// lines, and half lines are stored at about half the rate of whole ones (the L2
// has to merge them with the neighbouring tile's).  So a tile here is not a
// rectangle: tile k of a 64-column block is, for every output row c of the block,
// the 64 elements of that row's k-th LINE.  The rows' lines begin up to 63 elements
// before element 64 k, so the workgroup loads the 128 input rows [64 k - 64, 64 k +
// 64) (each input row is read by two tiles; the second read hits the L2) and every
// output row takes its own aligned window out of LDS.  Eight lanes write one
// whole line, a store instruction eight of them; only a row's first and last
// line are partial.  A constituent has (ceil(R / 64) + 1) * ceil(C / 64) tiles.
__global__ __launch_bounds__(256) void transpose_u16_lines_kernel(
    const uint16_t* __restrict__ in, uint16_t* __restrict__ out, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ rows, const int64_t* __restrict__ cols,
    const int64_t* __restrict__ tile_offsets, int64_t B) {
  constexpr int S = 33;                       // dwords per LDS row: 64 columns and one of padding
  __shared__ uint32_t tile[128 * S];
  int64_t id = blockIdx.x;
  {
    const int64_t per_xcd = gridDim.x / 8;
    if (id < per_xcd * 8) id = (id % 8) * per_xcd + id / 8;
  }
  const int64_t b = find_segment(tile_offsets, B, id);
  const int64_t R = rows[b], C = cols[b];
  const int64_t tiles_c = (C + 63) / 64;
  const int64_t local = id - tile_offsets[b];
  const int64_t k64 = (local / tiles_c) * 64;      // 64 k
  const int64_t c0 = (local % tiles_c) * 64;
  const uint16_t* src = in + offsets[b];
  uint16_t* dst = out + offsets[b];
  {
    const int piece = threadIdx.x & 7, lr = threadIdx.x >> 3;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
      const int r = lr + 32 * pass;
      const int64_t row = k64 - 64 + r;            // input row, may lie outside [0, R)
      u32x4 bits = {0u, 0u, 0u, 0u};
      if (row >= 0 && row < R) {
        const uint16_t* p = src + row * C + c0 + 8 * piece;
        if (c0 + 8 * piece + 8 <= C) {
          bits = load16_unaligned(reinterpret_cast<const char*>(p));
        } else {
          uint16_t e[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) e[j] = c0 + 8 * piece + j < C ? p[j] : (uint16_t)0;
          __builtin_memcpy(&bits, e, 16);
        }
      }
      uint32_t* t = &tile[r * S + 4 * piece];
      t[0] = bits.x;
      t[1] = bits.y;
      t[2] = bits.z;
      t[3] = bits.w;
    }
  }
  __syncthreads();
  // lane = (output row c of the block, 16-byte piece j of its line)
  const int j = threadIdx.x & 7;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int cl = (threadIdx.x >> 3) + 32 * pass;
    const int64_t c = c0 + cl;
    if (c >= C) continue;
    const int64_t row_start = offsets[b] + c * R;          // element index of the output row in `out`
    const int ph = (int)(((reinterpret_cast<uintptr_t>(out) >> 1) + (uint64_t)row_start) & 63);
    const int first = 64 - ph + 8 * j;                     // first of this piece's eight rows of the tile
    const uint32_t sel = (cl & 1) ? 0x07060302u : 0x05040100u;
    const uint32_t* col = &tile[first * S + (cl >> 1)];
    uint32_t x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = col[i * S];
    u32x4 v;
    v.x = __builtin_amdgcn_perm(x[1], x[0], sel);
    v.y = __builtin_amdgcn_perm(x[3], x[2], sel);
    v.z = __builtin_amdgcn_perm(x[5], x[4], sel);
    v.w = __builtin_amdgcn_perm(x[7], x[6], sel);
    const int64_t r = k64 - ph + 8 * j;                    // first output element of the piece in its row
    uint16_t* q = out + row_start + r;
    if (r >= 0 && r + 8 <= R) {
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(q));       // 16-byte aligned by construction
    } else if (r + 8 > 0 && r < R) {
      uint16_t e[8];
      __builtin_memcpy(e, &v, 16);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (r + i >= 0 && r + i < R) q[i] = e[i];
    }
  }
  (void)dst;
}

// Matrices with at most kTrNarrow rows (or columns): images of a few channels.  A
// 64-wide tile would leave most of its lanes idle, so a workgroup takes a strip
// of 256 * V columns (rows) of the long side instead, with V = 8 / sizeof(U), and
// all the rows (columns) of the narrow side: the strip is contiguous in the
// output (input) and is moved with 8-byte accesses; on the other side every lane
// moves 8 contiguous bytes per row of the narrow side.  NARROW_ROWS: the input
// has few rows (NCHW -> NHWC of few channels); otherwise it has few columns.
constexpr int kTrNarrow = 16;

template <typename U, bool NARROW_ROWS>
__global__ __launch_bounds__(256) void transpose_narrow_kernel(
    const U* __restrict__ in, U* __restrict__ out, const int64_t* __restrict__ offsets,
    const int64_t* __restrict__ rows, const int64_t* __restrict__ cols,
    const int64_t* __restrict__ tile_offsets, int64_t B) {
  constexpr int V = 8 / (int)sizeof(U);
  constexpr int kStrip = 256 * V;
  __shared__ __align__(8) U tile[kStrip * kTrNarrow];
  const int64_t id = blockIdx.x;
  const int64_t b = find_segment(tile_offsets, B, id);
  const int64_t R = rows[b], C = cols[b];
  const int64_t s0 = (id - tile_offsets[b]) * kStrip;      // first index of the strip on the long side
  const U* src = in + offsets[b];
  U* dst = out + offsets[b];
  if ((NARROW_ROWS ? R : C) > kTrNarrow) return;   // not a strip matrix: the tile would not hold it
  const int narrow = (int)(NARROW_ROWS ? R : C);
  const int64_t long_n = NARROW_ROWS ? C : R;
  const int len = (int)(long_n - s0 < kStrip ? long_n - s0 : kStrip);   // strip length
  const int lv = threadIdx.x * V;
  // the contiguous side: len * narrow elements from s0 * narrow on
  const int n_lin = len * narrow;
  if (!NARROW_ROWS) {
    const U* p = src + s0 * narrow;
    for (int k = lv; k < n_lin; k += kStrip) {
      if (k + V <= n_lin) {
        uint64_t bits;
        __builtin_memcpy(&bits, p + k, 8);
        *reinterpret_cast<uint64_t*>(&tile[k]) = bits;
      } else {
        for (int j = 0; k + j < n_lin; ++j) tile[k + j] = p[k + j];
      }
    }
  } else {
    for (int r = 0; r < narrow; ++r) {
      const U* p = src + r * C + s0 + lv;
      if (lv + V <= len) {
        U v[V];
        __builtin_memcpy(v, p, 8);
#pragma unroll
        for (int j = 0; j < V; ++j) tile[(lv + j) * narrow + r] = v[j];
      } else {
        for (int j = 0; lv + j < len; ++j) tile[(lv + j) * narrow + r] = p[j];
      }
    }
  }
  __syncthreads();
  if (NARROW_ROWS) {
    U* q = dst + s0 * narrow;
    for (int k = lv; k < n_lin; k += kStrip) {
      if (k + V <= n_lin) {
        const uint64_t bits = *reinterpret_cast<const uint64_t*>(&tile[k]);
        __builtin_memcpy(q + k, &bits, 8);
      } else {
        for (int j = 0; k + j < n_lin; ++j) q[k + j] = tile[k + j];
      }
    }
  } else {
    for (int c = 0; c < narrow; ++c) {
      U* q = dst + c * R + s0 + lv;
      if (lv + V <= len) {
        U v[V];
#pragma unroll
        for (int j = 0; j < V; ++j) v[j] = tile[(lv + j) * narrow + c];
        __builtin_memcpy(q, v, 8);
      } else {
        for (int j = 0; lv + j < len; ++j) q[j] = tile[(lv + j) * narrow + c];
      }
    }
  }
}

template <typename U>
static int launch_transpose(const void* in, void* out, const int64_t* offsets, const int64_t* rows,
                            const int64_t* cols, const int64_t* tile_offsets, int64_t B,
                            int64_t total_tiles, int tile_rows, int tile_cols, hipStream_t stream) {
#define NT_TR_CASE(TR, TC)                                                                         \
  if (tile_rows == TR && tile_cols == TC) {                                                        \
    if constexpr ((size_t)TR * TC * sizeof(U) <= (size_t)kTrMaxTileBytes) {                        \
      hipLaunchKernelGGL((transpose_ragged_kernel<U, TR, TC>), dim3((unsigned)total_tiles),        \
                         dim3(256), 0, stream, static_cast<const U*>(in), static_cast<U*>(out),    \
                         offsets, rows, cols, tile_offsets, B);                                    \
      return check_launch("transpose_ragged_kernel");                                              \
    }                                                                                              \
  }
  constexpr int kStrip = 256 * 8 / (int)sizeof(U);
  if ((tile_rows == kTrNarrow && tile_cols == kStrip) || (tile_rows == kStrip && tile_cols == kTrNarrow)) {
    // the strip kernels; the caller guarantees rows[b] <= 16 (cols[b] <= 16) for every b
    if (tile_rows == kTrNarrow) {
      hipLaunchKernelGGL((transpose_narrow_kernel<U, true>), dim3((unsigned)total_tiles), dim3(256), 0,
                         stream, static_cast<const U*>(in), static_cast<U*>(out), offsets, rows, cols,
                         tile_offsets, B);
    } else {
      hipLaunchKernelGGL((transpose_narrow_kernel<U, false>), dim3((unsigned)total_tiles), dim3(256), 0,
                         stream, static_cast<const U*>(in), static_cast<U*>(out), offsets, rows, cols,
                         tile_offsets, B);
    }
    return check_launch("transpose_narrow_kernel");
  }
  if (sizeof(U) == 2 && tile_rows == 64 && tile_cols == 64) {
    hipLaunchKernelGGL(transpose_u16_kernel, dim3((unsigned)total_tiles), dim3(256), 0, stream,
                       static_cast<const uint16_t*>(in), static_cast<uint16_t*>(out), offsets, rows, cols,
                       tile_offsets, B);
    return check_launch("transpose_u16_kernel");
  }
  NT_TR_CASE(64, 64)
  NT_TR_CASE(64, 128)
  NT_TR_CASE(128, 64)
  NT_TR_CASE(128, 128)
  NT_TR_CASE(64, 256)
  NT_TR_CASE(256, 64)
#undef NT_TR_CASE
  return fail(NT_ERR_UNSUPPORTED,
              "transpose_ragged: tile %d x %d of %d-byte elements is not one of 64x64, 64x128, 128x64, "
              "128x128, 64x256, 256x64 within %d bytes, nor the 16 x %d / %d x 16 strip", tile_rows,
              tile_cols, (int)sizeof(U), kTrMaxTileBytes, kStrip, kStrip);
}

}  // namespace nt

extern "C" int nt_transpose_ragged_lines(const void* in, void* out, const int64_t* offsets, const int64_t* rows,
                                         const int64_t* cols, const int64_t* tile_offsets, int64_t B,
                                         int64_t total_tiles, int elem_bytes, void* stream) {
  if (B < 0 || total_tiles < 0) return nt::fail(NT_ERR_INVALID_ARGUMENT, "transpose_ragged_lines: negative extent");
  if (elem_bytes != 2) return nt::fail(NT_ERR_UNSUPPORTED, "transpose_ragged_lines: 2-byte elements only");
  if (B == 0 || total_tiles == 0) return NT_OK;
  if (!in || !out || !offsets || !rows || !cols || !tile_offsets) {
    return nt::fail(NT_ERR_INVALID_ARGUMENT, "transpose_ragged_lines: NULL pointer");
  }
  if (total_tiles > 0x7fffffffLL) return nt::fail(NT_ERR_UNSUPPORTED, "transpose_ragged_lines: too many tiles");
  hipLaunchKernelGGL(nt::transpose_u16_lines_kernel, dim3((unsigned)total_tiles), dim3(256), 0, (hipStream_t)stream,
                     static_cast<const uint16_t*>(in), static_cast<uint16_t*>(out), offsets, rows, cols,
                     tile_offsets, B);
  return nt::check_launch("transpose_u16_lines_kernel");
}

extern "C" int nt_transpose_ragged(const void* in, void* out, const int64_t* offsets,
                                   const int64_t* rows, const int64_t* cols,
                                   const int64_t* tile_offsets, int64_t B, int64_t total_tiles,
                                   int tile_rows, int tile_cols, int elem_bytes, void* stream) {
  if (B < 0 || total_tiles < 0) return nt::fail(NT_ERR_INVALID_ARGUMENT, "transpose_ragged: negative extent");
  if (B == 0 || total_tiles == 0) return NT_OK;
  if (!in || !out || !offsets || !rows || !cols || !tile_offsets) {
    return nt::fail(NT_ERR_INVALID_ARGUMENT, "transpose_ragged: NULL pointer");
  }
  if (total_tiles > 0x7fffffffLL) return nt::fail(NT_ERR_UNSUPPORTED, "transpose_ragged: too many tiles");
  hipStream_t s = (hipStream_t)stream;
  switch (elem_bytes) {
#define NT_TR_ARGS in, out, offsets, rows, cols, tile_offsets, B, total_tiles, tile_rows, tile_cols, s
    case 1: return nt::launch_transpose<uint8_t>(NT_TR_ARGS);
    case 2: return nt::launch_transpose<uint16_t>(NT_TR_ARGS);
    case 4: return nt::launch_transpose<uint32_t>(NT_TR_ARGS);
    case 8: return nt::launch_transpose<uint64_t>(NT_TR_ARGS);
#undef NT_TR_ARGS
    default: return nt::fail(NT_ERR_UNSUPPORTED, "transpose_ragged: element size %d", elem_bytes);
  }
}
