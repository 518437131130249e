// Bias-free 1x1 convolution on the row-major (NCHW) packed buffer, without the two
// layout changes around the GEMM (gfx950, f16 / bf16).
//
// The reference turns a 1x1 convolution of a nested tensor of images into one
// matrix product over all pixels: transpose_nchw_nhwc, matmul with the [C_out,
// C_in] weight, transpose_nhwc_nchw (nestedtensor/csrc/conv2d.cpp:33-75).  The
// product itself is memory-bound at these depths (C_in = 64 -> C_out = 256: 128
// bytes in, 512 bytes out per pixel), so the two transposes triple its traffic.
// Here the product reads and writes the images as they lie: per image b,
//   Y_b[C_out, P_b] = W[C_out, C_in] X_b[C_in, P_b],
// with the pixels P_b = H_b W_b contiguous in both X_b and Y_b.
//
// Two things shape the kernel.
// (1) The matrix instruction wants eight consecutive K (input channels) of one
// pixel in a lane, while memory has consecutive pixels of one channel.  That
// transposition happens in LDS the way transpose_u16_kernel does it: a tile of X
// (C_in rows of 128 pixels) is stored as dwords (two neighbouring pixels) with an
// odd row stride, a lane reads the dword of its pixel pair in eight consecutive
// channel rows (conflict-free) and v_perm picks its pixel's half of each.  The
// pixels are the A operand (rows of the accumulator block) and the weight the B
// operand (lanes = output channels), so that a lane holds runs of four consecutive
// pixels of ONE output channel and the accumulators reach the output strip in LDS
// (rows = channels, elements = pixels) with 8-byte writes.
// (2) Output rows are P_b elements apart, so a 64-pixel piece of every row starts
// somewhere inside a 128-byte line, differently for every row, and a piece that
// covers two half lines is written at about half the rate of whole lines (measured:
// 2.5 TB/s of stores, which made a first version with plain 64-pixel tiles slower
// than the transposes it replaced).  So a tile is not a rectangle: tile k of an
// image is, for every output row, the 64 pixels of that row's k-th 128-byte LINE.
// The rows' lines begin up to 63 pixels before pixel 64 k, so the wavefront
// multiplies the 128 pixels [64 k - 64, 64 k + 64) (twice the matrix work, which
// is not what bounds the kernel) and every row then takes its own aligned
// 64-pixel window out of the strip: five dword reads and four v_alignbit per
// 16-byte piece when the window starts on an odd pixel.  Every store instruction
// of the wavefront then writes eight whole lines; only a row's first and last
// line are partial.
//
// Persistent workgroups (the weight is loaded into LDS once each) of WAVES
// wavefronts, and every wavefront works on tiles of its own with its own X tile
// and strip: no workgroup barrier after the weight is in place, the next tile's
// pixels are in flight in registers while the current tile is multiplied and
// stored, and the wavefronts of a compute unit drift apart so that their loads,
// products and stores overlap.
#include "attn_common.h"

namespace nt {

constexpr int kConvTile = 64;                 // pixels of a row that one tile writes
constexpr int kConvMaxIn = 128, kConvMaxOut = 512;

template <typename T, int WAVES, int LOADS>
__global__ __launch_bounds__(64 * WAVES) void conv1x1_nchw_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                  T* __restrict__ y,
                                                                  const int64_t* __restrict__ pix_offsets,
                                                                  const int64_t* __restrict__ tile_offsets, int64_t B,
                                                                  int64_t total_tiles, int c_in, int c_out) {
  typedef AttnT<T> AT;
  typedef typename AT::Frag Frag;
  constexpr int TW = 2 * kConvTile;             // pixels multiplied per tile
  constexpr int kPB = TW / 32;                  // 32-pixel blocks of those
  // LOADS: load instructions per tile and lane, each covering 4 channel rows of 128
  // pixels (a compile-time bound keeps the staged pieces in registers)
  constexpr int KS = LOADS / 4;                 // 16-channel steps of the product, at most
  constexpr int S = TW / 2 + 1;                 // dwords per row of the X tile (odd)
  constexpr int SSD = TW / 2 + 4;               // dwords per row of the output strip (8-byte aligned rows)
  extern __shared__ __align__(16) char lds[];
  const int SW = c_in + 8;                      // elements per row of the weight in LDS
  const int t = threadIdx.x, l = t & 63, wave = t >> 6;
  T* Wl = reinterpret_cast<T*>(lds);
  // The strip takes the place of the X tile: the tile is read into registers (pf) in full
  // before the first channel block is stored, and LDS operations of one wavefront
  // execute in order.
  const size_t x_bytes = (size_t)c_in * S * 4, strip_bytes = (size_t)32 * SSD * 4;
  char* mine = lds + (size_t)c_out * SW * sizeof(T) + (size_t)wave * (x_bytes > strip_bytes ? x_bytes : strip_bytes);
  uint32_t* Xl = reinterpret_cast<uint32_t*>(mine);
  uint32_t* strip = reinterpret_cast<uint32_t*>(mine);

  // the weight, once
  {
    const int per_row = c_in / 8;
    for (int i = t; i < c_out * per_row; i += 64 * WAVES) {
      const int row = i / per_row, ch = i - row * per_row;
      const u32x4 v = *reinterpret_cast<const u32x4*>(w + (size_t)row * c_in + ch * 8);
      *reinterpret_cast<u32x4*>(Wl + (size_t)row * SW + ch * 8) = v;
    }
  }
  __syncthreads();
  // tiles of this wavefront: first, first + G * WAVES, ... with G workgroups; the
  // workgroups of one XCD (ids congruent modulo 8) take a contiguous run
  const int64_t G = gridDim.x;
  int64_t wg = blockIdx.x;
  if (G % 8 == 0) wg = (int64_t)(blockIdx.x % 8) * (G / 8) + blockIdx.x / 8;
  const int64_t stride = G * WAVES;
  int64_t tile = wg * WAVES + wave;

  const int chunk = l & 15, row0 = l >> 4;      // this lane's 16-byte piece: 8 pixels of row row0 + 4 i
  u32x4 stage[LOADS];
  // pixels of the image, 64 k of the tile, image, its first pixel, and its tile range
  // (a wavefront's tiles are G * WAVES apart and an image has thousands: the range is
  // kept in registers and the search runs only when a tile leaves it)
  int64_t P = 0, k64 = 0, img = 0, pix0 = 0, t_lo = 0, t_hi = 0;
  auto locate = [&](int64_t id) {
    if (id >= t_hi) {
      img = find_segment(tile_offsets, B, id);
      t_lo = tile_offsets[img];
      t_hi = tile_offsets[img + 1];
      pix0 = pix_offsets[img];
      P = pix_offsets[img + 1] - pix0;
    }
    k64 = (id - t_lo) * kConvTile;
  };
  auto fetch = [&]() {
    const int64_t first = k64 - kConvTile + chunk * 8;      // first pixel of this piece, may lie outside [0, P)
    const T* xb = x + pix0 * c_in + first;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const T* p = xb + (int64_t)(row0 + 4 * i) * P;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row0 + 4 * i >= c_in) {
      } else if (first >= 0 && first + 8 <= P) {
        v = load16_unaligned(reinterpret_cast<const char*>(p));
      } else if (first + 8 > 0 && first < P) {
        T e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = (first + j >= 0 && first + j < P) ? p[j] : (T)0.0f;
        __builtin_memcpy(&v, e, 16);
      }
      stage[i] = v;
    }
  };
  if (tile < total_tiles) {
    locate(tile);
    fetch();
  }
  const int n = l & 31, g = l >> 5;
  const uint32_t sel = (n & 1) ? 0x07060302u : 0x05040100u;
  const int nob = c_out / 32;
  while (tile < total_tiles) {
    const int64_t cur_P = P, cur_k64 = k64, cur_pix0 = pix0;
    // registers -> this wavefront's X tile
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      if (row0 + 4 * i < c_in) {
        uint32_t* d = Xl + (row0 + 4 * i) * S + chunk * 4;
        d[0] = stage[i].x;
        d[1] = stage[i].y;
        d[2] = stage[i].z;
        d[3] = stage[i].w;
      }
    }
    __builtin_amdgcn_wave_barrier();
    const int64_t next = tile + stride;
    if (next < total_tiles) {
      locate(next);
      fetch();                                   // in flight during the products and stores below
    }
    // the pixel operands of the whole tile, once: pixel n of block pb, channels 16 ks + 8 g .. + 7
    Frag pf[KS][kPB];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (16 * ks < c_in) {
#pragma unroll
        for (int pb = 0; pb < kPB; ++pb) {
          const uint32_t* col = Xl + (16 * ks + 8 * g) * S + ((32 * pb + n) >> 1);
          uint32_t xv[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) xv[j] = col[j * S];
          u32x4 f;
          f.x = __builtin_amdgcn_perm(xv[1], xv[0], sel);
          f.y = __builtin_amdgcn_perm(xv[3], xv[2], sel);
          f.z = __builtin_amdgcn_perm(xv[5], xv[4], sel);
          f.w = __builtin_amdgcn_perm(xv[7], xv[6], sel);
          __builtin_memcpy(&pf[ks][pb], &f, 16);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();                          // the X tile is dead from here on
    const int64_t y_img = cur_pix0 * c_out;                  // first element of the image in y
    for (int ob = 0; ob < nob; ++ob) {
      acc16 acc[kPB];
#pragma unroll
      for (int pb = 0; pb < kPB; ++pb)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[pb][e] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (16 * ks < c_in) {
          const Frag wf = *reinterpret_cast<const Frag*>(Wl + (size_t)(ob * 32 + n) * SW + 16 * ks + 8 * g);
#pragma unroll
          for (int pb = 0; pb < kPB; ++pb) acc[pb] = AT::mma(pf[ks][pb], wf, acc[pb]);
        }
      }
      // accumulators (rows = pixels 8 q + 4 g + 0..3 of block pb, lane = channel n of the
      // block) -> strip row n, 8 bytes per run of four pixels
#pragma unroll
      for (int pb = 0; pb < kPB; ++pb)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint32_t two[2];
          two[0] = AT::cvt2(acc[pb][4 * q], acc[pb][4 * q + 1]);
          two[1] = AT::cvt2(acc[pb][4 * q + 2], acc[pb][4 * q + 3]);
          uint64_t v;
          __builtin_memcpy(&v, two, 8);
          *reinterpret_cast<uint64_t*>(strip + n * SSD + ((32 * pb + 8 * q + 4 * g) >> 1)) = v;
        }
      __builtin_amdgcn_wave_barrier();
      // every row takes the 64 pixels of its own line k out of the strip
#pragma unroll
      for (int ps = 0; ps < 4; ++ps) {
        const int r = ps * 8 + (l >> 3), j = l & 7;
        const int64_t row_start = y_img + (int64_t)(ob * 32 + r) * cur_P;     // element index in y
        const int ph = (int)(row_start & 63);
        const int col = kConvTile - ph + 8 * j;                              // first strip element of the piece
        const uint32_t* src = strip + r * SSD + (col >> 1);
        uint32_t d[5];
#pragma unroll
        for (int i = 0; i < 5; ++i) d[i] = src[i];
        u32x4 v;
        if (col & 1) {
          v.x = __builtin_amdgcn_alignbit(d[1], d[0], 16);
          v.y = __builtin_amdgcn_alignbit(d[2], d[1], 16);
          v.z = __builtin_amdgcn_alignbit(d[3], d[2], 16);
          v.w = __builtin_amdgcn_alignbit(d[4], d[3], 16);
        } else {
          v.x = d[0];
          v.y = d[1];
          v.z = d[2];
          v.w = d[3];
        }
        const int64_t pixel = cur_k64 - ph + 8 * j;                          // first pixel of the piece
        T* qd = y + row_start + pixel;
        if (pixel >= 0 && pixel + 8 <= cur_P) {
          *reinterpret_cast<u32x4*>(qd) = v;                                 // 16-byte aligned by construction
        } else if (pixel + 8 > 0 && pixel < cur_P) {
          T e[8];
          __builtin_memcpy(e, &v, 16);
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (pixel + i >= 0 && pixel + i < cur_P) qd[i] = e[i];
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    tile = next;
  }
}

static size_t conv_lds_bytes(int c_in, int c_out, int waves, size_t elem) {
  const size_t x_bytes = (size_t)c_in * (kConvTile + 1) * 4, strip_bytes = (size_t)32 * (kConvTile + 4) * 4;
  return (size_t)c_out * (c_in + 8) * elem + (size_t)waves * (x_bytes > strip_bytes ? x_bytes : strip_bytes);
}

template <typename T, int WAVES, int LOADS>
static int launch_conv(const void* x, const void* w, void* y, const int64_t* pix_offsets, const int64_t* tile_offsets,
                       int64_t B, int64_t total_tiles, int c_in, int c_out, int cus, hipStream_t stream) {
  const size_t lds = conv_lds_bytes(c_in, c_out, WAVES, sizeof(T));
  auto kernel = conv1x1_nchw_kernel<T, WAVES, LOADS>;
  static bool configured = false;      // one attribute call per instantiation (and process)
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024) != hipSuccess) {
      (void)hipGetLastError();
      return fail(NT_ERR_HIP, "conv1x1: cannot raise the dynamic LDS limit");
    }
    configured = true;
  }
  int64_t grid = cus;
  const int64_t needed = (total_tiles + WAVES - 1) / WAVES;
  if (grid > needed) grid = needed;
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(64 * WAVES), lds, stream, static_cast<const T*>(x),
                     static_cast<const T*>(w), static_cast<T*>(y), pix_offsets, tile_offsets, B, total_tiles, c_in,
                     c_out);
  return check_launch("conv1x1_nchw_kernel");
}

template <typename T, int WAVES>
static int launch_conv_w(const void* x, const void* w, void* y, const int64_t* pix_offsets,
                         const int64_t* tile_offsets, int64_t B, int64_t total_tiles, int c_in, int c_out, int cus,
                         hipStream_t stream) {
#define NT_CONV_ARGS x, w, y, pix_offsets, tile_offsets, B, total_tiles, c_in, c_out, cus, stream
  if (c_in <= 16) return launch_conv<T, WAVES, 4>(NT_CONV_ARGS);
  if (c_in <= 32) return launch_conv<T, WAVES, 8>(NT_CONV_ARGS);
  if (c_in <= 64) return launch_conv<T, WAVES, 16>(NT_CONV_ARGS);
  return launch_conv<T, WAVES, 32>(NT_CONV_ARGS);
#undef NT_CONV_ARGS
}

// The most wavefronts per workgroup (8, 7, 6, 4 or 2) whose tiles fit the LDS beside the weight; 0: none.
static int conv_waves(int c_in, int c_out, size_t elem) {
  const int choices[] = {8, 7, 6, 4, 2};
  for (int waves : choices) {
    if (conv_lds_bytes(c_in, c_out, waves, elem) <= 160 * 1024) return waves;
  }
  return 0;
}

template <typename T>
static int launch_conv_t(const void* x, const void* w, void* y, const int64_t* pix_offsets, const int64_t* tile_offsets,
                         int64_t B, int64_t total_tiles, int c_in, int c_out, int cus, hipStream_t stream) {
  switch (conv_waves(c_in, c_out, sizeof(T))) {
    case 8: return launch_conv_w<T, 8>(x, w, y, pix_offsets, tile_offsets, B, total_tiles, c_in, c_out, cus, stream);
    case 7: return launch_conv_w<T, 7>(x, w, y, pix_offsets, tile_offsets, B, total_tiles, c_in, c_out, cus, stream);
    case 6: return launch_conv_w<T, 6>(x, w, y, pix_offsets, tile_offsets, B, total_tiles, c_in, c_out, cus, stream);
    case 4: return launch_conv_w<T, 4>(x, w, y, pix_offsets, tile_offsets, B, total_tiles, c_in, c_out, cus, stream);
    case 2: return launch_conv_w<T, 2>(x, w, y, pix_offsets, tile_offsets, B, total_tiles, c_in, c_out, cus, stream);
    default: break;
  }
  return fail(NT_ERR_UNSUPPORTED, "conv1x1: %d -> %d channels do not fit the LDS (%zu bytes with two wavefronts)",
              c_in, c_out, conv_lds_bytes(c_in, c_out, 2, sizeof(T)));
}

}  // namespace nt

using namespace nt;

extern "C" int64_t nt_conv1x1_tile_pixels(void) { return kConvTile; }

extern "C" int nt_conv1x1_supported(int64_t c_in, int64_t c_out, int dtype) {
  if (dtype != NT_F16 && dtype != NT_BF16) return 0;
  if (c_in < 16 || c_in % 16 != 0 || c_in > kConvMaxIn || c_out < 32 || c_out % 32 != 0 || c_out > kConvMaxOut) return 0;
  return conv_waves((int)c_in, (int)c_out, 2) != 0;
}

extern "C" int nt_conv1x1_nchw(const void* x, const void* weight, void* y, const int64_t* pix_offsets,
                               const int64_t* tile_offsets, int64_t B, int64_t total_tiles, int64_t c_in,
                               int64_t c_out, int dtype, void* stream) {
  if (B < 0 || total_tiles < 0 || c_in < 1 || c_out < 1) {
    return fail(NT_ERR_INVALID_ARGUMENT, "conv1x1: bad shape");
  }
  if (c_in % 16 != 0 || c_in > kConvMaxIn || c_out % 32 != 0 || c_out > kConvMaxOut) {
    return fail(NT_ERR_UNSUPPORTED,
                "conv1x1: %lld -> %lld channels (input channels: a multiple of 16 up to %d; output channels: a "
                "multiple of 32 up to %d)", (long long)c_in, (long long)c_out, kConvMaxIn, kConvMaxOut);
  }
  if (dtype != NT_F16 && dtype != NT_BF16) return fail(NT_ERR_UNSUPPORTED, "conv1x1: dtype must be f16 or bf16");
  if (B == 0 || total_tiles == 0) return NT_OK;
  if (!x || !weight || !y || !pix_offsets || !tile_offsets) return fail(NT_ERR_INVALID_ARGUMENT, "conv1x1: NULL pointer");
  if ((reinterpret_cast<uintptr_t>(weight) & 15) != 0 || (reinterpret_cast<uintptr_t>(y) & 127) != 0) {
    return fail(NT_ERR_INVALID_ARGUMENT, "conv1x1: the weight must be 16-byte and the output 128-byte aligned");
  }
  if (total_tiles > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "conv1x1: too many tiles");
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
    (void)hipGetLastError();
    return fail(NT_ERR_HIP, "conv1x1: cannot query the device");
  }
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NT_F16) {
    return launch_conv_t<_Float16>(x, weight, y, pix_offsets, tile_offsets, B, total_tiles, (int)c_in, (int)c_out, cus, s);
  }
  return launch_conv_t<__bf16>(x, weight, y, pix_offsets, tile_offsets, B, total_tiles, (int)c_in, (int)c_out, cus, s);
}
