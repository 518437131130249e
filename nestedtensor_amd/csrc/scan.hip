// Device exclusive prefix scans (int64 results) for nested-tensor metadata.
//
// offsets[b] = sum_{c<b} prod_k sizes[c, k] is what turns a [B, D] size table
// into the element offsets of the packed buffer; the same scan over per-row
// keep-counts gives the output position of every row of a mask compaction.
// wave64 throughout: a wavefront scans 64 partial sums with __shfl_up, four
// wavefronts of a 256-thread workgroup are joined through LDS, and inputs
// larger than one 2048-item tile take three launches (tile sums, scan of the
// tile sums by one workgroup, rescan with carry).
#include "nt_common.h"

#include <atomic>

namespace nt {

constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanThreads * kScanItems;

struct SizesProd {
  const int64_t* sizes;
  int64_t D;
  __device__ __forceinline__ int64_t operator()(int64_t i) const {
    int64_t prod = 1;
    for (int64_t k = 0; k < D; ++k) prod *= sizes[i * D + k];
    return prod;
  }
};

struct LoadI32 {
  const int32_t* in;
  __device__ __forceinline__ int64_t operator()(int64_t i) const { return (int64_t)in[i]; }
};

struct LoadI64 {
  const int64_t* in;
  __device__ __forceinline__ int64_t operator()(int64_t i) const { return in[i]; }
};

__device__ __forceinline__ int64_t wave_inclusive_scan(int64_t v) {
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    int64_t up = __shfl_up(v, d, kWave);
    if (lane >= d) v += up;
  }
  return v;
}

// Exclusive scan of one int64 per thread across a 256-thread workgroup.
// Returns the exclusive prefix; *total receives the workgroup sum.
__device__ __forceinline__ int64_t block_exclusive_scan(int64_t v, int64_t* total) {
  __shared__ int64_t wave_sum[kScanThreads / kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t inc = wave_inclusive_scan(v);
  __syncthreads();  // protects wave_sum across repeated calls
  if (lane == kWave - 1) wave_sum[wave] = inc;
  __syncthreads();
  int64_t before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < kScanThreads / kWave; ++w) {
    const int64_t s = wave_sum[w];
    if (w < wave) before += s;
    all += s;
  }
  *total = all;
  return before + inc - v;
}

template <class Load>
__global__ __launch_bounds__(kScanThreads) void tile_sums_kernel(Load load, int64_t n,
                                                                 int64_t* tile_sums) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int64_t s = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    if (base + k < n) s += load(base + k);
  }
  int64_t total;
  block_exclusive_scan(s, &total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// In-place exclusive scan of m values by a single workgroup.
__global__ __launch_bounds__(kScanThreads) void scan_tile_sums_kernel(int64_t* v, int64_t m) {
  int64_t carry = 0;
  for (int64_t base = 0; base < m; base += kScanThreads) {
    const int64_t i = base + threadIdx.x;
    const int64_t x = i < m ? v[i] : 0;
    int64_t total;
    const int64_t ex = block_exclusive_scan(x, &total);
    if (i < m) v[i] = carry + ex;
    carry += total;
  }
}

// out[i] = carry(tile) + exclusive prefix inside the tile; the last tile also
// writes out[n] = grand total.
template <class Load>
__global__ __launch_bounds__(kScanThreads) void scan_tiles_kernel(Load load, int64_t n,
                                                                  const int64_t* tile_carry,
                                                                  int64_t* out) {
  const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanItems;
  int64_t x[kScanItems];
  int64_t s = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    x[k] = (base + k < n) ? load(base + k) : 0;
    s += x[k];
  }
  int64_t total;
  int64_t run = block_exclusive_scan(s, &total);
  run += tile_carry ? tile_carry[blockIdx.x] : 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    if (base + k < n) out[base + k] = run;
    run += x[k];
    if (base + k == n - 1) out[n] = run;
  }
}

__global__ void write_zero_kernel(int64_t* out) { out[0] = 0; }

template <class Load>
static int run_scan(Load load, int64_t n, int64_t* out, void* workspace, size_t workspace_bytes,
                    hipStream_t stream) {
  if (n < 0 || out == nullptr) return fail(NT_ERR_INVALID_ARGUMENT, "scan: bad arguments");
  if (n == 0) {
    hipLaunchKernelGGL(write_zero_kernel, dim3(1), dim3(1), 0, stream, out);
    return check_launch("write_zero_kernel");
  }
  const int64_t tiles = (n + kScanTile - 1) / kScanTile;
  if (tiles > 0x7fffffffLL) return fail(NT_ERR_UNSUPPORTED, "scan: input too large");
  if (tiles == 1) {
    hipLaunchKernelGGL((scan_tiles_kernel<Load>), dim3(1), dim3(kScanThreads), 0, stream, load, n,
                       (const int64_t*)nullptr, out);
    return check_launch("scan_tiles_kernel");
  }
  if (workspace == nullptr || workspace_bytes < (size_t)tiles * sizeof(int64_t)) {
    return fail(NT_ERR_WORKSPACE, "scan: workspace of %zu bytes needed, %zu given",
                (size_t)tiles * sizeof(int64_t), workspace_bytes);
  }
  int64_t* sums = static_cast<int64_t*>(workspace);
  hipLaunchKernelGGL((tile_sums_kernel<Load>), dim3((unsigned)tiles), dim3(kScanThreads), 0,
                     stream, load, n, sums);
  hipLaunchKernelGGL(scan_tile_sums_kernel, dim3(1), dim3(kScanThreads), 0, stream, sums, tiles);
  hipLaunchKernelGGL((scan_tiles_kernel<Load>), dim3((unsigned)tiles), dim3(kScanThreads), 0,
                     stream, load, n, (const int64_t*)sums, out);
  return check_launch("scan kernels");
}

// ---------------------------------------------------------------------------
// The allocation-free variant of nt_offsets_from_sizes keeps its tile sums in
// device memory that belongs to the library: a file-scope __device__ array.  In
// host code the array's name is only a handle for hipGetSymbolAddress; the
// address the kernels get is looked up once per device and cached here.  Every
// GPU holds its own copy of the array (kNoAllocMaxTiles * 8 bytes = 256 KiB)
// from the moment the code object is loaded there until the process ends.
constexpr int64_t kNoAllocMaxTiles = 32768;
constexpr int64_t kNoAllocMaxB = kNoAllocMaxTiles * kScanTile;   // 67 108 864 constituents
static __device__ __align__(256) int64_t scratch[kNoAllocMaxTiles];

constexpr int kMaxDevices = 64;
static std::atomic<int64_t*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, or nullptr with the error
// text set and its code in *rc.  The first call on a device asks the runtime; later calls read the
// cached pointer (threads that race on the first call store the same value).
static int64_t* scratch_on_current_device(int* rc) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    *rc = fail(NT_ERR_HIP, "offsets_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    return nullptr;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    *rc = fail(NT_ERR_UNSUPPORTED, "offsets_noalloc: device index %d is not in [0, %d)", dev, kMaxDevices);
    return nullptr;
  }
  int64_t* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p != nullptr) return p;
  void* addr = nullptr;
  e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || addr == nullptr) {
    *rc = fail(NT_ERR_HIP, "offsets_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    return nullptr;
  }
  p = static_cast<int64_t*>(addr);
  g_scratch_ptr[dev].store(p, std::memory_order_release);
  return p;
}

}  // namespace nt

using namespace nt;

extern "C" size_t nt_scan_workspace_bytes(int64_t n) {
  if (n <= kScanTile) return 0;
  return (size_t)((n + kScanTile - 1) / kScanTile) * sizeof(int64_t);
}

extern "C" size_t nt_offsets_workspace_bytes(int64_t B) { return nt_scan_workspace_bytes(B); }

extern "C" int nt_offsets_from_sizes(const int64_t* sizes, int64_t B, int64_t D, int64_t* offsets,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  if (D < 0) return fail(NT_ERR_INVALID_ARGUMENT, "offsets: D must be >= 0");
  if (B > 0 && D > 0 && sizes == nullptr) return fail(NT_ERR_INVALID_ARGUMENT, "offsets: sizes is NULL");
  SizesProd load{sizes, D};
  return run_scan(load, B, offsets, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int64_t nt_offsets_noalloc_max_count(void) { return kNoAllocMaxB; }

extern "C" int nt_offsets_from_sizes_noalloc(const int64_t* sizes, int64_t B, int64_t D,
                                             int64_t* offsets, void* stream) {
  if (D < 0) return fail(NT_ERR_INVALID_ARGUMENT, "offsets_noalloc: D must be >= 0");
  if (B > 0 && D > 0 && sizes == nullptr) {
    return fail(NT_ERR_INVALID_ARGUMENT, "offsets_noalloc: sizes is NULL");
  }
  if (B > kNoAllocMaxB) {
    return fail(NT_ERR_UNSUPPORTED,
                "offsets_noalloc: B = %lld exceeds the built-in scratch (at most %lld constituents); "
                "use nt_offsets_from_sizes with a caller-provided workspace",
                (long long)B, (long long)kNoAllocMaxB);
  }
  // Nothing in the scratch has to start at zero: the first launch writes the
  // sum of every tile before the second one reads it.
  int rc = NT_OK;
  int64_t* ws = scratch_on_current_device(&rc);
  if (ws == nullptr) return rc;
  SizesProd load{sizes, D};
  return run_scan(load, B, offsets, ws, (size_t)kNoAllocMaxTiles * sizeof(int64_t),
                  (hipStream_t)stream);
}

extern "C" int nt_exclusive_scan_i32(const int32_t* in, int64_t n, int64_t* out, void* workspace,
                                     size_t workspace_bytes, void* stream) {
  if (n > 0 && in == nullptr) return fail(NT_ERR_INVALID_ARGUMENT, "scan: input is NULL");
  LoadI32 load{in};
  return run_scan(load, n, out, workspace, workspace_bytes, (hipStream_t)stream);
}
