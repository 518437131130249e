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

// WAVE_ROWS: rows of at most 1 KiB -- every wavefront of the workgroup takes a row
// of its own (4 rows per workgroup) instead of 192 lanes idling on one row.
template <int EB, int MODE, bool WAVE_ROWS>
__global__ __launch_bounds__(256) void row_kernel(RowParams p) {
  constexpr int kT = WAVE_ROWS ? 64 : 256;
  const int64_t row = WAVE_ROWS ? row_index() * 4 + (threadIdx.x >> 6) : row_index();
  if (row >= p.nrows) return;
  if (MODE == kPack) {
    const int64_t off = p.offsets[row];
    const int64_t n = (p.offsets[row + 1] - off) * EB;
    move_row<EB, kUnpad, kT>(p.dst + off * EB, reinterpret_cast<const char*>(p.srcs[row]), n, n,
                             p.pad);
    return;
  }
  int64_t b, src_off = 0, last;
  bool inside = true;
  if (p.nrag == 1) {
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
    const int64_t r = row - b * plane;
    const int64_t i0 = r / p.M1;
    const int64_t i1 = r - i0 * p.M1;
    const int64_t* sz = p.sizes + b * p.D;
    inside = (i0 < sz[0]) && (i1 < sz[1]);
    last = sz[2];
    src_off = (i0 * sz[1] + i1) * last;
  }
  const int64_t Mlast = p.nrag == 1 ? p.M0 : (p.nrag == 2 ? p.M1 : p.M2);
  const int64_t row_bytes = Mlast * p.inner * EB;
  const int64_t valid = inside ? last * p.inner * EB : 0;
  if (MODE == kOnes) {
    move_row<EB, kOnes, kT>(p.dst + row * row_bytes, nullptr, valid, row_bytes, p.pad);
  } else {
    const int64_t packed_byte = (p.offsets[b] + src_off * p.inner) * EB;
    if (MODE == kPad || MODE == kPadMask) {
      move_row<EB, kPad, kT>(p.dst + row * row_bytes, p.src + packed_byte, valid, row_bytes, p.pad);
      if (MODE == kPadMask) {
        // the same workgroups write the row's mask bytes: ones over the valid prefix
        const u32x4 zero = {0u, 0u, 0u, 0u};
        move_row<1, kOnes, kT>(p.mask + row * (row_bytes / EB), nullptr, valid / EB, row_bytes / EB, zero);
      }
    } else {
      if (valid > 0) {
        move_row<EB, kUnpad, kT>(p.dst + packed_byte, p.src + row * row_bytes, valid, valid, p.pad);
      }
    }
  }
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
  switch (eb) {
    case 1: hipLaunchKernelGGL((row_kernel<1, MODE, WAVE_ROWS>), grid, block, 0, stream, p); break;
    case 2: hipLaunchKernelGGL((row_kernel<2, MODE, WAVE_ROWS>), grid, block, 0, stream, p); break;
    case 4: hipLaunchKernelGGL((row_kernel<4, MODE, WAVE_ROWS>), grid, block, 0, stream, p); break;
    case 8: hipLaunchKernelGGL((row_kernel<8, MODE, WAVE_ROWS>), grid, block, 0, stream, p); break;
    default: return fail(NT_ERR_INVALID_ARGUMENT, "elem_bytes must be 1, 2, 4 or 8, got %d", eb);
  }
  return check_launch("row_kernel");
}

template <int MODE>
static int launch_rows(int eb, const RowParams& p, int64_t max_row_bytes, hipStream_t stream) {
  if (p.nrows == 0 || max_row_bytes == 0) return NT_OK;
  if (p.nrows > 0x7fffffffLL) {
    return fail(NT_ERR_UNSUPPORTED, "row count %lld exceeds the grid limit", (long long)p.nrows);
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
