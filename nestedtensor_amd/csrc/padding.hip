// Packed <-> padded data movement and mask build for nested tensors (gfx950).
//
// One kernel family serves nt_add_padding, nt_remove_padding, nt_build_mask and
// nt_pack.  The unit of work is an output ROW: for a constituent with ragged
// dims (s_0 .. s_{j-1}) followed by `inner` regular elements, row (b, i_0 ..
// i_{j-2}) of the padded tensor is M_{j-1} * inner contiguous elements whose
// first s_{j-1} * inner elements are one contiguous run of the packed buffer
// (or nothing, if some i_k >= s_k) and whose remainder is padding.  Rows are
// decoded once per workgroup with scalar arithmetic; inside a row every lane
// moves 16-byte chunks: destination-aligned 128-bit stores, 128-bit loads of
// any alignment.  grid.x walks the 4 KiB tiles of a row, grid.y (and z) the rows,
// so workgroups that are dispatched together touch one compact, contiguous
// window of both buffers; measured on MI355X this ordering and one 16-byte
// chunk per lane (many small workgroups) give the highest HBM throughput, well
// above fewer workgroups with more chunks in flight per lane.
//
// All index math is int64: the largest configuration holds 1.7e10 elements.
#include "nt_common.h"

// Tuning knobs of the row kernels (compile-time).
#ifndef NT_ROW_UNROLL
#define NT_ROW_UNROLL 1          // 16-byte chunks in flight per lane
#endif
#ifndef NT_ROW_STREAM_STORE
#define NT_ROW_STREAM_STORE 1    // non-temporal stores for the output
#endif
#ifndef NT_ROW_TILE_FAST
#define NT_ROW_TILE_FAST 1       // 1: consecutive workgroups walk the tiles of one row
#endif
#ifndef NT_ROW_TARGET_WGS
#define NT_ROW_TARGET_WGS (1 << 24)
#endif
// Workgroups per row at most; longer rows are looped over.  Every tile of a
// padded row is written, so pad / mask take one workgroup per tile up to 16 MiB
// rows; un-pad and pack move only the valid prefix, and fewer, looping
// workgroups leave fewer of them without work on short rows.
#ifndef NT_ROW_MAX_TILES_PAD
#define NT_ROW_MAX_TILES_PAD 4096
#endif
#ifndef NT_ROW_MAX_TILES_UNPAD
#define NT_ROW_MAX_TILES_UNPAD 1024
#endif

namespace nt {

enum Mode { kPad = 0, kUnpad = 1, kOnes = 2, kPack = 3, kPadMask = 4 };

struct RowParams {
  const char* src;
  char* dst;
  const int64_t* offsets;
  const int64_t* sizes;
  const void* const* srcs;
  int64_t D;       // row stride of `sizes`
  int64_t nrag;    // ragged dims walked by the row decode, 1..3
  int64_t M0, M1, M2;
  int64_t inner;   // elements of the trailing regular dims
  int64_t nrows;
  u32x4 pad;       // padding value replicated to 16 bytes
  char* mask;      // kPadMask: one byte per element of dst, 1 where the element holds data
};

template <int EB> struct ElemT;
template <> struct ElemT<1> { typedef uint8_t type; };
template <> struct ElemT<2> { typedef uint16_t type; };
template <> struct ElemT<4> { typedef uint32_t type; };
template <> struct ElemT<8> { typedef uint64_t type; };

template <int EB, int MODE>
__device__ __forceinline__ void move_elem(char* d, const char* s, int64_t pos, int64_t valid,
                                          const u32x4& pad) {
  typedef typename ElemT<EB>::type T;
  T v;
  if (pos < valid) {
    if (MODE == kOnes) {
      v = (T)1;
    } else {
      v = *reinterpret_cast<const T*>(s + pos);
    }
  } else {
    if (EB == 8) {
      v = (T)(((uint64_t)pad.y << 32) | pad.x);
    } else {
      v = (T)pad.x;
    }
  }
  *reinterpret_cast<T*>(d + pos) = v;
}

// Which workgroups share a row: grid.y by default (consecutive workgroups walk
// different rows), grid.x when NT_ROW_TILE_FAST (consecutive workgroups walk the
// tiles of one row).
#if NT_ROW_TILE_FAST
__device__ __forceinline__ unsigned tile_index() { return blockIdx.x; }
__device__ __forceinline__ unsigned tile_count() { return gridDim.x; }
__device__ __forceinline__ int64_t row_index() { return (int64_t)blockIdx.y + (int64_t)blockIdx.z * 65535; }
#else
__device__ __forceinline__ unsigned tile_index() { return blockIdx.y; }
__device__ __forceinline__ unsigned tile_count() { return gridDim.y; }
__device__ __forceinline__ int64_t row_index() { return blockIdx.x; }
#endif

// Cooperative move of one row: bytes [0, valid) come from s, bytes [valid, total)
// are padding.  Called by every workgroup of the row's grid.y column.
template <int EB, int MODE, int kThreads>
__device__ __forceinline__ void move_row(char* d, const char* s, int64_t valid, int64_t total,
                                         const u32x4 pad) {
  constexpr int kUnroll = NT_ROW_UNROLL;
  const int tid = threadIdx.x & (kThreads - 1);   // 256: the workgroup, 64: one wavefront

  int64_t head = (int64_t)((0 - (uintptr_t)d) & 15);
  if (head > total) head = total;
  const int64_t nvec = (total - head) >> 4;
  const int64_t tail_start = head + (nvec << 4);

  if (tile_index() == 0) {
    // unaligned edges of the destination row: fewer than 32 bytes
    const int64_t nedge = (head + (total - tail_start)) / EB;
    for (int64_t e = tid; e < nedge; e += kThreads) {
      int64_t pos = e * EB;
      if (pos >= head) pos = tail_start + (pos - head);
      move_elem<EB, MODE>(d, s, pos, valid, pad);
    }
  }

  const int64_t tile_chunks = (int64_t)kThreads * kUnroll;
  for (int64_t c0 = (int64_t)tile_index() * tile_chunks; c0 < nvec;
       c0 += (int64_t)tile_count() * tile_chunks) {
    u32x4 v[kUnroll];
    int state[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t c = c0 + u * kThreads + tid;
      const int64_t pos = head + (c << 4);
      if (c >= nvec) {
        state[u] = 0;
      } else if (pos + 16 <= valid) {
        state[u] = 1;
        if (MODE == kOnes) {
          v[u] = u32x4{0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};
        } else {
          v[u] = load16_unaligned(s + pos);
        }
      } else if (pos >= valid) {
        state[u] = 1;
        v[u] = pad;
      } else {
        state[u] = 2;
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t c = c0 + u * kThreads + tid;
      const int64_t pos = head + (c << 4);
      if (state[u] == 1) {
#if NT_ROW_STREAM_STORE
        store16_stream(d + pos, v[u]);
#else
        store16(d + pos, v[u]);
#endif
      } else if (state[u] == 2) {
#pragma unroll
        for (int k = 0; k < 16; k += EB) {
          move_elem<EB, MODE>(d, s, pos + k, valid, pad);
        }
      }
    }
  }
}

// Every argument the row decode may touch, fetched in ONE batch of scalar loads at
// the top of a kernel.  Left to the compiler they are fetched piecemeal
// behind the decode's branches, each a round trip of its own, and a workgroup here
// lives for one 4 KiB tile (C5 pad: 2.4 % of the launch).  The statement depends on
// all of them and yields a zero the compiler cannot see through, which the caller
// adds to its row index so that the statement is kept.  It is neither volatile nor
// a memory clobber: behind a volatile statement the loads through offsets / sizes
// stop being scalar loads.
__device__ __forceinline__ int args_in_one_batch(const RowParams& p) {
  int zero;
  asm("s_mov_b32 %0, 0"
      : "=s"(zero)
      : "s"(p.src), "s"(p.dst), "s"(p.offsets), "s"(p.sizes), "s"(p.D), "s"(p.nrag), "s"(p.M0), "s"(p.M1),
        "s"(p.M2), "s"(p.inner), "s"(p.nrows));
  return __builtin_amdgcn_readfirstlane(zero);
}

// One row of work, decoded: bytes [0, valid) of d come from s, bytes [valid, total)
// are padding (kOnes: ones / zeros, s unused).
struct RowDesc {
  char* d;
  const char* s;
  int64_t valid, total;
};

// Decode row `row` (scalar arithmetic, uniform over the lanes that share the row).
// Returns false when the row has nothing to move.
// ONE_RAGGED: the launch has one ragged dim (a row is a whole constituent): a kernel
// of its own without the divisions of the other two cases, so that the decode is
// a few straight-line instructions from the kernel's entry.  A workgroup lives for
// one 4 KiB tile; with the general decode the one-ragged-dim path sat behind a far
// branch and cost the C5 pad launch 2.4 %.
template <int EB, int MODE, bool ONE_RAGGED>
__device__ __forceinline__ bool decode_row(const RowParams& p, int64_t row, RowDesc& r) {
  if (MODE == kPack) {
    const int64_t off = p.offsets[row];
    const int64_t n = (p.offsets[row + 1] - off) * EB;
    r.d = p.dst + off * EB;
    r.s = reinterpret_cast<const char*>(p.srcs[row]);
    r.valid = r.total = n;
    return n > 0;
  }
  int64_t b, src_off = 0, last;
  bool inside = true;
  if (ONE_RAGGED || p.nrag == 1) {
    b = row;
    last = p.sizes[b * p.D];
  } else if (p.nrag == 2) {
    b = row / p.M0;
    const int64_t i0 = row - b * p.M0;
    const int64_t* sz = p.sizes + b * p.D;
    inside = i0 < sz[0];
    last = sz[1];
    src_off = i0 * last;
  } else {
    const int64_t plane = p.M0 * p.M1;
    b = row / plane;
    const int64_t rr = row - b * plane;
    const int64_t i0 = rr / p.M1;
    const int64_t i1 = rr - i0 * p.M1;
    const int64_t* sz = p.sizes + b * p.D;
    inside = (i0 < sz[0]) && (i1 < sz[1]);
    last = sz[2];
    src_off = (i0 * sz[1] + i1) * last;
  }
  const int64_t Mlast = (ONE_RAGGED || p.nrag == 1) ? p.M0 : (p.nrag == 2 ? p.M1 : p.M2);
  const int64_t row_bytes = Mlast * p.inner * EB;
  const int64_t valid = inside ? last * p.inner * EB : 0;
  if (MODE == kOnes) {
    r.d = p.dst + row * row_bytes;
    r.s = nullptr;
    r.valid = valid;
    r.total = row_bytes;
    return true;
  }
  const int64_t packed_byte = (p.offsets[b] + src_off * p.inner) * EB;
  if (MODE == kPad || MODE == kPadMask) {
    r.d = p.dst + row * row_bytes;
    r.s = p.src + packed_byte;
    r.valid = valid;
    r.total = row_bytes;
    return true;
  }
  r.d = p.dst + packed_byte;      // kUnpad
  r.s = p.src + row * row_bytes;
  r.valid = r.total = valid;
  return valid > 0;
}

// WAVE_ROWS: rows of at most 1 KiB -- every wavefront of the workgroup takes a row
// of its own (4 rows per workgroup) instead of 192 lanes idling on one row.
template <int EB, int MODE, bool WAVE_ROWS, bool ONE_RAGGED>
__global__ __launch_bounds__(256) void row_kernel(RowParams p) {
  constexpr int kT = WAVE_ROWS ? 64 : 256;
  const int after_args = args_in_one_batch(p);
  const int64_t row = (WAVE_ROWS ? row_index() * 4 + (threadIdx.x >> 6) : row_index()) + after_args;
  if (row >= p.nrows) return;
  RowDesc r;
  if (!decode_row<EB, MODE, ONE_RAGGED>(p, row, r)) return;
  constexpr int kMove = MODE == kPack ? kUnpad : (MODE == kPadMask ? kPad : MODE);
  move_row<EB, kMove, kT>(r.d, r.s, r.valid, r.total, p.pad);
  if (MODE == kPadMask) {
    // the same workgroups write the row's mask bytes: ones over the valid prefix
    const u32x4 zero = {0u, 0u, 0u, 0u};
    move_row<1, kOnes, kT>(p.mask + (r.d - p.dst) / EB, nullptr, r.valid / EB, r.total / EB, zero);
  }
}

// NR short rows (one 16-byte chunk per lane covers a row) moved together by a
// lane group of kT lanes: the chunks of all of them are in flight at once.
template <int EB, int MODE, int kT, int NR>
__device__ __forceinline__ void move_rows(const RowDesc (&r)[NR], const bool (&on)[NR], const RowParams& p,
                                          const int tid) {
  constexpr int kMove = MODE == kPadMask ? kPad : MODE;
  // whole 16-byte chunks of the destination rows: all loads first, then all stores
  u32x4 v[NR];
  int state[NR];
  int64_t pos[NR], head[NR], tail_start[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    state[i] = 0;
    if (!on[i]) continue;
    int64_t h = (int64_t)((0 - (uintptr_t)r[i].d) & 15);
    if (h > r[i].total) h = r[i].total;
    const int64_t nvec = (r[i].total - h) >> 4;
    head[i] = h;
    tail_start[i] = h + (nvec << 4);
    pos[i] = h + ((int64_t)tid << 4);
    if (tid >= nvec) continue;
    if (pos[i] + 16 <= r[i].valid) {
      state[i] = 1;
      if (kMove == kOnes) {
        v[i] = u32x4{0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u};
      } else {
        v[i] = load16_unaligned(r[i].s + pos[i]);
      }
    } else if (pos[i] >= r[i].valid) {
      state[i] = 1;
      v[i] = p.pad;
    } else {
      state[i] = 2;
    }
  }
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    if (state[i] == 1) {
#if NT_ROW_STREAM_STORE
      store16_stream(r[i].d + pos[i], v[i]);
#else
      store16(r[i].d + pos[i], v[i]);
#endif
    } else if (state[i] == 2) {
      // the one chunk that straddles the valid / padding boundary
#pragma unroll
      for (int k = 0; k < 16; k += EB) move_elem<EB, kMove>(r[i].d, r[i].s, pos[i] + k, r[i].valid, p.pad);
    }
  }
  // unaligned edges of the destination rows: fewer than 32 bytes each
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    if (!on[i]) continue;
    const int64_t nedge = (head[i] + (r[i].total - tail_start[i])) / EB;
    if (tid < nedge) {
      int64_t e = (int64_t)tid * EB;
      if (e >= head[i]) e = tail_start[i] + (e - head[i]);
      move_elem<EB, kMove>(r[i].d, r[i].s, e, r[i].valid, p.pad);
    }
  }
  if (MODE == kPadMask) {
    // mask bytes of the same rows: ones over the valid prefix.  Rows here are at
    // most kT chunks of data, so a mask row is at most kT * 16 / EB bytes.
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      if (!on[i]) continue;
      char* m = p.mask + (r[i].d - p.dst) / EB;
      const int64_t mv = r[i].valid / EB, mt = r[i].total / EB;
      int64_t h = (int64_t)((0 - (uintptr_t)m) & 15);
      if (h > mt) h = mt;
      const int64_t nvec = (mt - h) >> 4;
      const int64_t ts = h + (nvec << 4);
      const int64_t mp = h + ((int64_t)tid << 4);
      if (tid < nvec) {
        if (mp + 16 <= mv) {
          store16_stream(m + mp, u32x4{0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u});
        } else if (mp >= mv) {
          store16_stream(m + mp, u32x4{0u, 0u, 0u, 0u});
        } else {
#pragma unroll
          for (int k = 0; k < 16; ++k) m[mp + k] = (mp + k) < mv ? 1 : 0;
        }
      }
      const int64_t nedge = h + (mt - ts);
      if (tid < nedge) {
        int64_t e = tid;
        if (e >= h) e = ts + (e - h);
        m[e] = e < mv ? 1 : 0;
      }
    }
  }
}

// Short rows, nrag == 1 (every row is a constituent of its own): a lane group --
// the workgroup, or one wavefront for rows of at most 1 KiB -- takes NR
// consecutive rows.  A row of a few KiB per workgroup leaves a CU with too few
// bytes in flight to cover the latency of the row decode (dependent scalar
// loads) and of the copy itself.
template <int EB, int MODE, int kT, int NR>
__global__ __launch_bounds__(256) void row_batch_kernel(RowParams p) {
  constexpr int kGroups = 256 / kT;
  const int after_args = args_in_one_batch(p);
  const int tid = threadIdx.x & (kT - 1);
  const int64_t group = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * kGroups + (threadIdx.x / kT);
  const int64_t row0 = group * NR + after_args;
  if (row0 >= p.nrows) return;
  // Row decode in three steps so that the size-table and offset loads of all NR
  // rows are in flight together (one memory round trip, not NR): coordinates of
  // the first row by division and of the others by increment, then every load,
  // then the arithmetic on what was loaded.
  int64_t cb[NR], c0[NR], c1[NR];
  {
    int64_t b, i0 = 0, i1 = 0;
    if (p.nrag == 1) {
      b = row0;
    } else if (p.nrag == 2) {
      b = row0 / p.M0;
      i0 = row0 - b * p.M0;
    } else {
      const int64_t plane = p.M0 * p.M1;
      b = row0 / plane;
      const int64_t rr = row0 - b * plane;
      i0 = rr / p.M1;
      i1 = rr - i0 * p.M1;
    }
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      cb[i] = b;
      c0[i] = i0;
      c1[i] = i1;
      if (p.nrag == 1) {
        ++b;
      } else if (p.nrag == 2) {
        if (++i0 == p.M0) { i0 = 0; ++b; }
      } else {
        if (++i1 == p.M1) {
          i1 = 0;
          if (++i0 == p.M0) { i0 = 0; ++b; }
        }
      }
    }
  }
  int64_t sz0[NR], sz1[NR], sz2[NR], off[NR];
  bool on[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    on[i] = row0 + i < p.nrows;
    const int64_t bb = on[i] ? cb[i] : 0;
    const int64_t* sz = p.sizes + bb * p.D;
    sz0[i] = sz[0];
    sz1[i] = p.nrag > 1 ? sz[1] : 0;
    sz2[i] = p.nrag > 2 ? sz[2] : 0;
    off[i] = MODE == kOnes ? 0 : p.offsets[bb];
  }
  const int64_t Mlast = p.nrag == 1 ? p.M0 : (p.nrag == 2 ? p.M1 : p.M2);
  const int64_t row_bytes = Mlast * p.inner * EB;
  RowDesc r[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    int64_t last, src_off = 0;
    bool inside = true;
    if (p.nrag == 1) {
      last = sz0[i];
    } else if (p.nrag == 2) {
      inside = c0[i] < sz0[i];
      last = sz1[i];
      src_off = c0[i] * last;
    } else {
      inside = (c0[i] < sz0[i]) && (c1[i] < sz1[i]);
      last = sz2[i];
      src_off = (c0[i] * sz1[i] + c1[i]) * last;
    }
    const int64_t valid = inside ? last * p.inner * EB : 0;
    const int64_t packed_byte = (off[i] + src_off * p.inner) * EB;
    const int64_t padded_byte = (row0 + i) * row_bytes;
    if (MODE == kUnpad) {
      r[i].d = p.dst + packed_byte;
      r[i].s = p.src + padded_byte;
      r[i].valid = r[i].total = valid;
      on[i] = on[i] && valid > 0;
    } else {
      r[i].d = p.dst + padded_byte;
      r[i].s = MODE == kOnes ? nullptr : p.src + packed_byte;
      r[i].valid = valid;
      r[i].total = row_bytes;
    }
  }
  move_rows<EB, MODE, kT, NR>(r, on, p, tid);
}

// Short rows, nrag >= 2: the rows of one constituent (and, with three ragged dims,
// of one index of the first) share their entry of the size table and their
// offset, so a lane group that walks `rows_per_group` consecutive rows decodes
// once (two divisions, one round trip to the tables) and then only adds strides;
// the rows are moved two at a time.  With one row per workgroup the decode was
// most of a workgroup's life: 4.4 TB/s on 16 fp32 images [3, H, W] against
// 5.9 TB/s this way.
template <int EB, int MODE, int kT>
__global__ __launch_bounds__(256) void row_group_kernel(RowParams p, int rows_per_group) {
  constexpr int kGroups = 256 / kT;
  const int after_args = args_in_one_batch(p);
  const int tid = threadIdx.x & (kT - 1);
  const int64_t group = ((int64_t)blockIdx.x + (int64_t)blockIdx.y * gridDim.x) * kGroups + (threadIdx.x / kT);
  const int64_t row0 = group * rows_per_group + after_args;
  if (row0 >= p.nrows) return;
  const int64_t count = p.nrows - row0 < rows_per_group ? p.nrows - row0 : rows_per_group;
  // coordinates of the first row: (b, i0) for two ragged dims, (b, i0, i1) for three
  int64_t b, i0, i1 = 0;
  if (p.nrag == 2) {
    b = row0 / p.M0;
    i0 = row0 - b * p.M0;
  } else {
    const int64_t plane = p.M0 * p.M1;
    b = row0 / plane;
    const int64_t rr = row0 - b * plane;
    i0 = rr / p.M1;
    i1 = rr - i0 * p.M1;
  }
  const int64_t Mlast = p.nrag == 2 ? p.M1 : p.M2;
  const int64_t row_bytes = Mlast * p.inner * EB;
  int64_t cur_b = -1, sz0 = 0, sz1 = 0, sz2 = 0, off = 0;
  for (int64_t j = 0; j < count; j += 2) {
    RowDesc r[2];
    bool on[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      on[u] = j + u < count;
      if (on[u] && b != cur_b) {   // uniform; once per constituent
        const int64_t* sz = p.sizes + b * p.D;
        sz0 = sz[0];
        sz1 = sz[1];
        sz2 = p.nrag > 2 ? sz[2] : 0;
        off = MODE == kOnes ? 0 : p.offsets[b];
        cur_b = b;
      }
      int64_t last, src_off;
      bool inside;
      if (p.nrag == 2) {
        inside = i0 < sz0;
        last = sz1;
        src_off = i0 * last;
      } else {
        inside = (i0 < sz0) && (i1 < sz1);
        last = sz2;
        src_off = (i0 * sz1 + i1) * last;
      }
      const int64_t valid = inside ? last * p.inner * EB : 0;
      const int64_t packed_byte = (off + src_off * p.inner) * EB;
      const int64_t padded_byte = (row0 + j + u) * row_bytes;
      if (MODE == kUnpad) {
        r[u].d = p.dst + packed_byte;
        r[u].s = p.src + padded_byte;
        r[u].valid = r[u].total = valid;
        on[u] = on[u] && valid > 0;
      } else {
        r[u].d = p.dst + padded_byte;
        r[u].s = MODE == kOnes ? nullptr : p.src + packed_byte;
        r[u].valid = valid;
        r[u].total = row_bytes;
      }
      // next row
      if (p.nrag == 2) {
        if (++i0 == p.M0) { i0 = 0; ++b; }
      } else if (++i1 == p.M1) {
        i1 = 0;
        if (++i0 == p.M0) { i0 = 0; ++b; }
      }
    }
    move_rows<EB, MODE, kT, 2>(r, on, p, tid);
  }
}

// Mask of a nested size without any row structure on the store side.  grid.y
// walks the planes -- one per constituent (two mask dims below the batch dim) or
// per (constituent, index of the first dim) (three) -- whose entry of the size
// table every lane of the workgroup shares; the lanes take the 16-byte chunks of
// the flat mask that overlap the plane, find the row of a chunk's first byte with
// one 32-bit division and set ones up to each row's length (a chunk may run over
// several rows).  The chunk that two planes share is written byte-wise by both,
// each its own bytes.  This runs at the speed of a plain fill; the row-by-row
// kernels spend more scalar work per row than a 1 KiB store is worth.
template <int PER>
__global__ __launch_bounds__(256) void mask_plane_kernel(char* mask, const int64_t* sizes, int64_t D, int K,
                                                         unsigned M0, unsigned rows, unsigned Mlast) {
  const int64_t plane = (int64_t)blockIdx.y + (int64_t)blockIdx.z * 65535;
  int64_t b = plane;
  bool inside0 = true;
  if (K == 3) {
    b = plane / M0;
    inside0 = (plane - b * M0) < sizes[b * D];
  }
  const int64_t* sz = sizes + b * D + (K - 2);
  const unsigned nrow = inside0 ? (unsigned)min((int64_t)rows, sz[0]) : 0u;   // rows that hold anything
  const unsigned len = (unsigned)min(sz[1], (int64_t)Mlast);
  const int64_t plane_bytes = (int64_t)rows * Mlast;
  const int64_t ps = plane * plane_bytes, pe = ps + plane_bytes;
  const int64_t g0 = ps >> 4;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int64_t g = g0 + (int64_t)blockIdx.x * (256 * PER) + k * 256 + threadIdx.x;
    const int64_t byte0 = g << 4;
    if (byte0 >= pe) break;
    const int64_t lo = byte0 > ps ? byte0 : ps;
    const int64_t hi = byte0 + 16 < pe ? byte0 + 16 : pe;
    const unsigned rel = (unsigned)(lo - ps);
    unsigned row = rel / Mlast;
    unsigned col = rel - row * Mlast;
    unsigned bits = 0;                       // bit j: byte byte0 + j is valid
    unsigned pos = (unsigned)(lo - byte0);
    const unsigned end = (unsigned)(hi - byte0);
    while (pos < end) {
      const unsigned n = min(end - pos, Mlast - col);
      if (row < nrow && col < len) {
        const unsigned v = min(len - col, n);
        bits |= ((1u << v) - 1u) << pos;
      }
      pos += n;
      ++row;
      col = 0;
    }
    if (end - (unsigned)(lo - byte0) == 16u) {
      u32x4 v;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const unsigned nib = (bits >> (4 * w)) & 0xfu;
        v[w] = (nib * 0x00204081u) & 0x01010101u;   // bit i of the nibble -> byte i
      }
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(mask + byte0));
    } else {
      for (unsigned j = (unsigned)(lo - byte0); j < end; ++j) mask[byte0 + j] = (bits >> j) & 1u;
    }
  }
}

// Launches mask_plane_kernel when its conditions hold; *done says whether it did.
static int try_mask_planes(char* mask, const int64_t* sizes, int64_t B, int64_t D, int64_t K,
                           const int64_t* ext, hipStream_t stream, bool* done) {
  *done = false;
  if (K < 2 || K > 3) return NT_OK;
  const int64_t Mlast = ext[K - 1], rows = ext[K - 2];
  const int64_t planes = K == 3 ? B * ext[0] : B;
  if (Mlast == 0 || rows == 0 || planes == 0 || reinterpret_cast<uintptr_t>(mask) % 16 != 0) return NT_OK;
  if (Mlast >= ((int64_t)1 << 31) || rows * Mlast >= ((int64_t)1 << 31) || planes > (int64_t)65535 * 65535 ||
      (K == 3 && ext[0] >= ((int64_t)1 << 31))) {
    return NT_OK;
  }
  if (planes * rows * Mlast < ((int64_t)1 << 20)) return NT_OK;   // tiny masks: the row kernels do
  constexpr int PER = 4;
  const int64_t chunks = (rows * Mlast + 15) / 16 + 1;     // a plane may start and end inside a chunk
  const int64_t gx = (chunks + 256 * PER - 1) / (256 * PER);
  dim3 grid((unsigned)gx, (unsigned)(planes < 65535 ? planes : 65535), (unsigned)((planes + 65534) / 65535));
  hipLaunchKernelGGL((mask_plane_kernel<PER>), grid, dim3(256), 0, stream, mask, sizes, D, (int)K,
                     (unsigned)(K == 3 ? ext[0] : 1), (unsigned)rows, (unsigned)Mlast);
  *done = true;
  return check_launch("mask_plane_kernel");
}

static u32x4 replicate_pad(int eb, uint64_t bits) {
  uint64_t v = bits;
  if (eb == 1) {
    v &= 0xffull;
    v |= v << 8;
    v |= v << 16;
    v |= v << 32;
  } else if (eb == 2) {
    v &= 0xffffull;
    v |= v << 16;
    v |= v << 32;
  } else if (eb == 4) {
    v &= 0xffffffffull;
    v |= v << 32;
  }
  u32x4 r;
  r.x = (uint32_t)v;
  r.y = (uint32_t)(v >> 32);
  r.z = r.x;
  r.w = r.y;
  return r;
}

template <int MODE, bool WAVE_ROWS>
static int launch_rows_t(int eb, const RowParams& p, int64_t max_row_bytes, hipStream_t stream) {
  const int64_t grid_rows = WAVE_ROWS ? (p.nrows + 3) / 4 : p.nrows;
  const int64_t tile_bytes = (WAVE_ROWS ? 64 : 256) * NT_ROW_UNROLL * 16;
  int64_t tiles = (max_row_bytes + tile_bytes - 1) / tile_bytes;
  // Enough workgroups to fill 256 CUs many times over, but very long rows are
  // walked by a bounded number of workgroups that each loop over tiles.
  int64_t y_cap = (int64_t)NT_ROW_TARGET_WGS / grid_rows;
  if (y_cap < 1) y_cap = 1;
  const int64_t max_tiles =
      (MODE == kPad || MODE == kOnes || MODE == kPadMask) ? NT_ROW_MAX_TILES_PAD : NT_ROW_MAX_TILES_UNPAD;
  if (y_cap > max_tiles) y_cap = max_tiles;
  int64_t gy = tiles < y_cap ? tiles : y_cap;
  if (gy < 1) gy = 1;
#if NT_ROW_TILE_FAST
  const int64_t gz = (grid_rows + 65534) / 65535;
  if (gz > 65535) return fail(NT_ERR_UNSUPPORTED, "row count %lld exceeds the grid limit", (long long)p.nrows);
  dim3 grid((unsigned)gy, (unsigned)(grid_rows < 65535 ? grid_rows : 65535), (unsigned)gz);
#else
  dim3 grid((unsigned)grid_rows, (unsigned)gy, 1);
#endif
  dim3 block(256, 1, 1);
#define NT_ROW_CASE(EB)                                                                               \
  if (p.nrag == 1 || MODE == kPack) {                                                                 \
    hipLaunchKernelGGL((row_kernel<EB, MODE, WAVE_ROWS, true>), grid, block, 0, stream, p);           \
  } else {                                                                                            \
    hipLaunchKernelGGL((row_kernel<EB, MODE, WAVE_ROWS, false>), grid, block, 0, stream, p);          \
  }                                                                                                   \
  break;
  switch (eb) {
    case 1: NT_ROW_CASE(1)
    case 2: NT_ROW_CASE(2)
    case 4: NT_ROW_CASE(4)
    case 8: NT_ROW_CASE(8)
    default: return fail(NT_ERR_INVALID_ARGUMENT, "elem_bytes must be 1, 2, 4 or 8, got %d", eb);
  }
#undef NT_ROW_CASE
  return check_launch("row_kernel");
}

#ifndef NT_ROW_GROUP
#define NT_ROW_GROUP 4           // rows per lane group of row_group_kernel (measured: 2 and 8 are 8-10 % slower)
#endif

// Short rows: see row_batch_kernel (nrag == 1) and row_group_kernel.
template <int MODE, int kT>
static int launch_batch(int eb, const RowParams& p, hipStream_t stream) {
  const int rpg = p.nrag == 1 ? 2 : NT_ROW_GROUP;
  const int64_t groups = (p.nrows + rpg - 1) / rpg;
  const int64_t wgs = (groups + (256 / kT) - 1) / (256 / kT);
  const int64_t gx = wgs < 65535 ? wgs : 65535;
  const int64_t gy = (wgs + gx - 1) / gx;
  if (gy > 65535) return fail(NT_ERR_UNSUPPORTED, "row count %lld exceeds the grid limit", (long long)p.nrows);
  dim3 grid((unsigned)gx, (unsigned)gy, 1), block(256, 1, 1);
#define NT_BATCH_CASE(EB)                                                                             \
  if (p.nrag == 1) {                                                                                  \
    hipLaunchKernelGGL((row_batch_kernel<EB, MODE, kT, 2>), grid, block, 0, stream, p);               \
  } else {                                                                                            \
    hipLaunchKernelGGL((row_group_kernel<EB, MODE, kT>), grid, block, 0, stream, p, rpg);             \
  }                                                                                                   \
  break;
  switch (eb) {
    case 1: NT_BATCH_CASE(1)
    case 2: NT_BATCH_CASE(2)
    case 4: NT_BATCH_CASE(4)
    case 8: NT_BATCH_CASE(8)
    default: return fail(NT_ERR_INVALID_ARGUMENT, "elem_bytes must be 1, 2, 4 or 8, got %d", eb);
  }
#undef NT_BATCH_CASE
  return check_launch("row_group_kernel");
}

template <int MODE>
static int launch_rows(int eb, const RowParams& p, int64_t max_row_bytes, hipStream_t stream) {
  if (p.nrows == 0 || max_row_bytes == 0) return NT_OK;
  if (p.nrows > 0x7fffffffLL) {
    return fail(NT_ERR_UNSUPPORTED, "row count %lld exceeds the grid limit", (long long)p.nrows);
  }
  if (MODE != kPack && p.nrows >= 4096) {
    // many short rows: several rows per lane group, all of their chunks in flight
    if (max_row_bytes <= 1024) return launch_batch<MODE, 64>(eb, p, stream);
    if (max_row_bytes <= 4096) return launch_batch<MODE, 256>(eb, p, stream);
  }
  if (max_row_bytes <= 1024 && MODE != kPack) return launch_rows_t<MODE, true>(eb, p, max_row_bytes, stream);
  return launch_rows_t<MODE, false>(eb, p, max_row_bytes, stream);
}

// Fills the geometry shared by pad / unpad / mask from the host-side extents.
static int fill_geometry(RowParams& p, int64_t B, int64_t D, int64_t nrag,
                         const int64_t* ext_host, int64_t n_ext, int64_t* max_row_elems) {
  if (B < 0 || D < 1 || nrag < 1 || nrag > 3 || nrag > D || n_ext < nrag) {
    return fail(NT_ERR_INVALID_ARGUMENT, "bad geometry: B=%lld D=%lld n_ragged=%lld",
                (long long)B, (long long)D, (long long)nrag);
  }
  if (ext_host == nullptr) return fail(NT_ERR_INVALID_ARGUMENT, "padded sizes are NULL");
  int64_t inner = 1;
  for (int64_t k = nrag; k < n_ext; ++k) inner *= ext_host[k];
  p.D = D;
  p.nrag = nrag;
  p.M0 = ext_host[0];
  p.M1 = nrag > 1 ? ext_host[1] : 1;
  p.M2 = nrag > 2 ? ext_host[2] : 1;
  p.inner = inner;
  int64_t rows = B;
  for (int64_t k = 0; k + 1 < nrag; ++k) rows *= ext_host[k];
  p.nrows = rows;
  *max_row_elems = ext_host[nrag - 1] * inner;
  for (int64_t k = 0; k < n_ext; ++k) {
    if (ext_host[k] < 0) return fail(NT_ERR_INVALID_ARGUMENT, "negative extent");
  }
  return NT_OK;
}

}  // namespace nt

using namespace nt;

extern "C" int nt_add_padding(const void* packed, void* padded, const int64_t* offsets,
                              const int64_t* sizes, int64_t B, int64_t D, int64_t n_ragged,
                              const int64_t* padded_sizes_host, int elem_bytes, uint64_t pad_bits,
                              void* stream) {
  RowParams p = {};
  int64_t max_row_elems = 0;
  int rc = fill_geometry(p, B, D, n_ragged, padded_sizes_host, D, &max_row_elems);
  if (rc != NT_OK) return rc;
  if (B == 0 || max_row_elems == 0) return NT_OK;
  if (!padded || !offsets || !sizes) return fail(NT_ERR_INVALID_ARGUMENT, "NULL pointer");
  p.src = static_cast<const char*>(packed);
  p.dst = static_cast<char*>(padded);
  p.offsets = offsets;
  p.sizes = sizes;
  p.pad = replicate_pad(elem_bytes, pad_bits);
  return launch_rows<kPad>(elem_bytes, p, max_row_elems * elem_bytes, (hipStream_t)stream);
}

extern "C" int nt_add_padding_mask(const void* packed, void* padded, uint8_t* mask,
                                   const int64_t* offsets, const int64_t* sizes, int64_t B, int64_t D,
                                   int64_t n_ragged, const int64_t* padded_sizes_host, int elem_bytes,
                                   uint64_t pad_bits, void* stream) {
  RowParams p = {};
  int64_t max_row_elems = 0;
  int rc = fill_geometry(p, B, D, n_ragged, padded_sizes_host, D, &max_row_elems);
  if (rc != NT_OK) return rc;
  if (B == 0 || max_row_elems == 0) return NT_OK;
  if (!padded || !mask || !offsets || !sizes) return fail(NT_ERR_INVALID_ARGUMENT, "NULL pointer");
  p.src = static_cast<const char*>(packed);
  p.dst = static_cast<char*>(padded);
  p.mask = reinterpret_cast<char*>(mask);
  p.offsets = offsets;
  p.sizes = sizes;
  p.pad = replicate_pad(elem_bytes, pad_bits);
  {
    // mask[b, i...] = all_k(i_k < sizes[b, k]) over every dim of the size table:
    // written at fill speed by a launch of its own where that kernel applies,
    // which beats carrying the mask along in the data kernel
    bool done = false;
    rc = try_mask_planes(p.mask, sizes, B, D, D, padded_sizes_host, (hipStream_t)stream, &done);
    if (rc != NT_OK) return rc;
    if (done) return launch_rows<kPad>(elem_bytes, p, max_row_elems * elem_bytes, (hipStream_t)stream);
  }
  return launch_rows<kPadMask>(elem_bytes, p, max_row_elems * elem_bytes, (hipStream_t)stream);
}

extern "C" int nt_remove_padding(const void* padded, void* packed, const int64_t* offsets,
                                 const int64_t* sizes, int64_t B, int64_t D, int64_t n_ragged,
                                 const int64_t* padded_sizes_host, int elem_bytes, void* stream) {
  RowParams p = {};
  int64_t max_row_elems = 0;
  int rc = fill_geometry(p, B, D, n_ragged, padded_sizes_host, D, &max_row_elems);
  if (rc != NT_OK) return rc;
  if (B == 0 || max_row_elems == 0) return NT_OK;
  if (!padded || !packed || !offsets || !sizes) return fail(NT_ERR_INVALID_ARGUMENT, "NULL pointer");
  p.src = static_cast<const char*>(padded);
  p.dst = static_cast<char*>(packed);
  p.offsets = offsets;
  p.sizes = sizes;
  p.pad = replicate_pad(elem_bytes, 0);
  return launch_rows<kUnpad>(elem_bytes, p, max_row_elems * elem_bytes, (hipStream_t)stream);
}

extern "C" int nt_build_mask(uint8_t* mask, const int64_t* sizes, int64_t B, int64_t D, int64_t K,
                             const int64_t* mask_sizes_host, void* stream) {
  RowParams p = {};
  int64_t max_row_elems = 0;
  if (K < 1 || K > 3 || K > D) {
    return fail(NT_ERR_INVALID_ARGUMENT, "mask dims K=%lld must be in 1..min(3, D)", (long long)K);
  }
  int rc = fill_geometry(p, B, D, K, mask_sizes_host, K, &max_row_elems);
  if (rc != NT_OK) return rc;
  if (B == 0 || max_row_elems == 0) return NT_OK;
  if (!mask || !sizes) return fail(NT_ERR_INVALID_ARGUMENT, "NULL pointer");
  bool done = false;
  rc = try_mask_planes(reinterpret_cast<char*>(mask), sizes, B, D, K, mask_sizes_host, (hipStream_t)stream, &done);
  if (rc != NT_OK || done) return rc;
  p.dst = reinterpret_cast<char*>(mask);
  p.sizes = sizes;
  p.pad = replicate_pad(1, 0);
  return launch_rows<kOnes>(1, p, max_row_elems, (hipStream_t)stream);
}

extern "C" int nt_pack(const void* const* srcs, void* packed, const int64_t* offsets, int64_t B,
                       int elem_bytes, void* stream) {
  if (B == 0) return NT_OK;
  if (B < 0 || !srcs || !packed || !offsets) return fail(NT_ERR_INVALID_ARGUMENT, "bad pack args");
  RowParams p = {};
  p.srcs = srcs;
  p.dst = static_cast<char*>(packed);
  p.offsets = offsets;
  p.nrows = B;
  p.nrag = 1;
  p.pad = replicate_pad(elem_bytes, 0);
  // Row lengths live on the device; size the grid for long rows and let short
  // rows finish early.
  return launch_rows<kPack>(elem_bytes, p, (int64_t)1 << 22, (hipStream_t)stream);
}

// nt_pack for a handful of constituents: the table (sizes, offsets, source
// pointers) travels in the kernel arguments, so nothing has to reach the device
// before the launch, and the kernel leaves a copy of the table in device memory
// for the operators that follow.
namespace nt {
constexpr int kPackTableMax = 384;     // int64 entries; with the other arguments well inside the 4 KiB of kernel arguments
struct PackTable {
  int64_t v[kPackTableMax];            // sizes[B * D], offsets[B + 1], source pointers[B]
};

template <int EB>
__global__ __launch_bounds__(256) void pack_table_kernel(PackTable t, char* dst, int64_t B, int64_t D,
                                                         int64_t* table_out) {
  const int64_t row = row_index();
  if (row >= B) return;
  if (row == 0 && tile_index() == 0 && table_out != nullptr) {
    const int64_t n = B * D + 2 * B + 1;
    for (int64_t i = threadIdx.x; i < n; i += 256) table_out[i] = t.v[i];
  }
  const int64_t off = t.v[B * D + row];
  const int64_t n = (t.v[B * D + row + 1] - off) * EB;
  if (n <= 0) return;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  move_row<EB, kUnpad, 256>(dst + off * EB, reinterpret_cast<const char*>(t.v[B * D + B + 1 + row]), n, n, zero);
}
// The first n entries of a table that travelled in the kernel arguments, written
// to device memory.
__global__ __launch_bounds__(256) void table_store_kernel(PackTable t, int n, int64_t* out) {
  for (int i = threadIdx.x; i < n; i += 256) out[i] = t.v[i];
}
}  // namespace nt

extern "C" int64_t nt_pack_table_max_entries(void) { return nt::kPackTableMax; }

extern "C" int nt_upload_table(const int64_t* table_host, int64_t n, int64_t* table_dev, void* stream) {
  if (n == 0) return NT_OK;
  if (n < 0 || !table_host || !table_dev) return fail(NT_ERR_INVALID_ARGUMENT, "bad upload_table args");
  if (n > nt::kPackTableMax) {
    return fail(NT_ERR_UNSUPPORTED, "table of %lld entries exceeds the %d that fit in kernel arguments",
                (long long)n, nt::kPackTableMax);
  }
  nt::PackTable t;
  for (int64_t i = 0; i < n; ++i) t.v[i] = table_host[i];
  for (int64_t i = n; i < nt::kPackTableMax; ++i) t.v[i] = 0;
  hipLaunchKernelGGL(nt::table_store_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, t, (int)n, table_dev);
  return check_launch("table_store_kernel");
}

extern "C" int nt_pack_table(const int64_t* table_host, int64_t B, int64_t D, void* packed,
                             int64_t* table_dev, int elem_bytes, void* stream) {
  if (B == 0) return NT_OK;
  const int64_t n = B * D + 2 * B + 1;
  if (B < 0 || D < 0 || !table_host) return fail(NT_ERR_INVALID_ARGUMENT, "bad pack args");
  if (n > nt::kPackTableMax) {
    return fail(NT_ERR_UNSUPPORTED, "pack table of %lld entries exceeds the %d that fit in kernel arguments",
                (long long)n, nt::kPackTableMax);
  }
  nt::PackTable t;
  int64_t longest = 0;
  for (int64_t i = 0; i < n; ++i) t.v[i] = table_host[i];
  for (int64_t i = n; i < nt::kPackTableMax; ++i) t.v[i] = 0;
  for (int64_t b = 0; b < B; ++b) {
    const int64_t len = t.v[B * D + b + 1] - t.v[B * D + b];
    if (len < 0) return fail(NT_ERR_INVALID_ARGUMENT, "pack offsets must not decrease");
    longest = len > longest ? len : longest;
  }
  if (longest == 0 && table_dev == nullptr) return NT_OK;
  if (longest > 0 && !packed) return fail(NT_ERR_INVALID_ARGUMENT, "bad pack args");
  // the grid of the row kernels for un-pad / pack: a bounded number of looping
  // workgroups per row, sized for the longest constituent
  const int64_t tile_bytes = 256 * NT_ROW_UNROLL * 16;
  int64_t tiles = (longest * elem_bytes + tile_bytes - 1) / tile_bytes;
  int64_t y_cap = (int64_t)NT_ROW_TARGET_WGS / B;
  if (y_cap < 1) y_cap = 1;
  if (y_cap > NT_ROW_MAX_TILES_UNPAD) y_cap = NT_ROW_MAX_TILES_UNPAD;
  int64_t gy = tiles < y_cap ? tiles : y_cap;
  if (gy < 1) gy = 1;
#if NT_ROW_TILE_FAST
  dim3 grid((unsigned)gy, (unsigned)B, 1);
#else
  dim3 grid((unsigned)B, (unsigned)gy, 1);
#endif
  hipStream_t s = (hipStream_t)stream;
  char* dst = static_cast<char*>(packed);
  switch (elem_bytes) {
    case 1: hipLaunchKernelGGL((nt::pack_table_kernel<1>), grid, dim3(256), 0, s, t, dst, B, D, table_dev); break;
    case 2: hipLaunchKernelGGL((nt::pack_table_kernel<2>), grid, dim3(256), 0, s, t, dst, B, D, table_dev); break;
    case 4: hipLaunchKernelGGL((nt::pack_table_kernel<4>), grid, dim3(256), 0, s, t, dst, B, D, table_dev); break;
    case 8: hipLaunchKernelGGL((nt::pack_table_kernel<8>), grid, dim3(256), 0, s, t, dst, B, D, table_dev); break;
    default: return fail(NT_ERR_INVALID_ARGUMENT, "elem_bytes must be 1, 2, 4 or 8, got %d", elem_bytes);
  }
  return check_launch("pack_table_kernel");
}
