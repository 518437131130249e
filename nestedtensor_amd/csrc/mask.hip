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

constexpr int kRowsPerBlock = 4;  // one wavefront per row, 4 rows per workgroup

__global__ __launch_bounds__(kWave * kRowsPerBlock) void mask_row_counts_kernel(
    const uint8_t* mask, int64_t R, int64_t M, int32_t* counts) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
  if (row >= R) return;
  const uint8_t* m = mask + row * M;
  int32_t count = 0;
  for (int64_t base = 0; base < M; base += kWave) {
    const int64_t i = base + lane;
    const bool keep = (i < M) && (m[i] != 0);
    count += __popcll(__ballot(keep));
  }
  if (lane == 0) counts[row] = count;
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
                                  void* stream) {
  if (R < 0 || M < 0) return fail(NT_ERR_INVALID_ARGUMENT, "mask_row_counts: negative extent");
  if (R == 0) return NT_OK;
  if (!counts || (M > 0 && !mask)) return fail(NT_ERR_INVALID_ARGUMENT, "mask_row_counts: NULL pointer");
  const int64_t blocks = (R + kRowsPerBlock - 1) / kRowsPerBlock;
  if (blocks > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "mask_row_counts: too many rows");
  hipLaunchKernelGGL(mask_row_counts_kernel, dim3((unsigned)blocks), dim3(kWave * kRowsPerBlock),
                     0, (hipStream_t)stream, mask, R, M, counts);
  return check_launch("mask_row_counts_kernel");
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
