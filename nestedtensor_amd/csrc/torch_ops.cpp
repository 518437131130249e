// Operator layer of nestedtensor_amd as a C++ torch extension.
//
// The reference registers its operators from C++ with TORCH_LIBRARY_IMPL on its
// own dispatch key and a custom TensorImpl (nestedtensor/csrc/masking.cpp:652-675,
// csrc/mha.cpp:71-74, csrc/cuda/mha.cpp:109-113, csrc/py_init.cpp:132-216).  That
// key belongs to torch core now, so a nested tensor crosses the dispatcher in
// lowered form: (packed buffer, sizes[B, D], offsets[B + 1]).  This file
//
//   * defines the schemas of the reference's operators (same names, same argument
//     order; their `Tensor nt` argument is the Python wrapper, which
//     __torch_function__ lowers before the dispatcher sees it), and
//   * defines and implements, for the HIP device key, the lowered operators that
//     do the work: host code here only validates, sizes outputs, allocates them
//     from torch's caching allocator and calls the C ABI of
//     include/nestedtensor_amd.h on torch's current stream.
//
// Nothing here computes on the host except nested sizes (integers): converting a
// dense tensor + mask to a nested tensor needs the per-row keep-counts on the
// host to size its output, which is one device-to-host copy into pinned memory.
#include <ATen/ATen.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <algorithm>
#include <chrono>
#include <cstring>
#include <tuple>
#include <vector>

#include "../../include/nestedtensor_amd.h"

namespace {

using at::Tensor;

inline void check(int rc) {
  if (rc != NT_OK) {
    const char* msg = nt_last_error();
    TORCH_CHECK(false, "nestedtensor_amd: ", (msg && *msg) ? msg : "error", " (code ", rc, ")");
  }
}

inline void require_device(const Tensor& t, const char* what) {
  TORCH_CHECK(t.is_cuda(), "nestedtensor_amd: ", what, " runs on the HIP device only; got a tensor on ",
              t.device(), ". Move the nested tensor with .to('cuda') first.");
}

// Every pointer a kernel dereferences must be device memory of the input's
// device: a weight or bias left on the host would be read by the GPU as a stray
// address (a memory-access fault, not an exception).
inline void require_same_device(const Tensor& t, const Tensor& like, const char* what, const char* name) {
  TORCH_CHECK(!t.defined() || t.device() == like.device(), what, ": ", name, " is on ", t.device(),
              " but the input is on ", like.device(), ". Move the module with .to('cuda') first.");
}

inline void* stream_of(const Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

inline int elem_bytes(at::ScalarType st) {
  const int n = static_cast<int>(c10::elementSize(st));
  // masking.cpp:622 returns an uninitialised tensor for other dtypes; raise instead.
  TORCH_CHECK(n == 1 || n == 2 || n == 4 || n == 8, "Input datatype ", st, " is not supported.");
  return n;
}

inline int elem_type(at::ScalarType st) {
  switch (st) {
    case at::kFloat: return NT_F32;
    case at::kHalf: return NT_F16;
    case at::kBFloat16: return NT_BF16;
    case at::kDouble: return NT_F64;
    case at::kChar: return NT_I8;
    case at::kByte: return NT_U8;
    case at::kShort: return NT_I16;
    case at::kInt: return NT_I32;
    case at::kLong: return NT_I64;
    default: return -1;
  }
}

inline int dtype_code(at::ScalarType st) {
  switch (st) {
    case at::kFloat: return NT_F32;
    case at::kHalf: return NT_F16;
    case at::kBFloat16: return NT_BF16;
    default: TORCH_CHECK(false, "nestedtensor_amd: dtype ", st, " is not supported by this op");
  }
}

// The padding value converted the way the reference converts it, (T)(double)
// (masking.cpp:594,610), as raw bits in the low bytes.
uint64_t pad_bits(double padding, at::ScalarType st) {
  uint64_t bits = 0;
  switch (st) {
    case at::kFloat: { const float v = static_cast<float>(padding); std::memcpy(&bits, &v, 4); break; }
    case at::kDouble: std::memcpy(&bits, &padding, 8); break;
    case at::kHalf: { const c10::Half v(static_cast<float>(padding)); bits = v.x; break; }
    case at::kBFloat16: { const c10::BFloat16 v(static_cast<float>(padding)); bits = v.x; break; }
    case at::kBool: bits = padding != 0.0 ? 1 : 0; break;
    case at::kChar: case at::kByte: bits = static_cast<uint64_t>(static_cast<int64_t>(padding)) & 0xffu; break;
    case at::kShort: bits = static_cast<uint64_t>(static_cast<int64_t>(padding)) & 0xffffu; break;
    case at::kInt: bits = static_cast<uint64_t>(static_cast<int64_t>(padding)) & 0xffffffffu; break;
    case at::kLong: bits = static_cast<uint64_t>(static_cast<int64_t>(padding)); break;
    default: TORCH_CHECK(false, "Input datatype ", st, " is not supported.");
  }
  return bits;
}

// ---- metadata ---------------------------------------------------------------

// offsets[b] = sum_{c<b} prod_k sizes[c, k] on the device (nt_offsets_from_sizes).
Tensor offsets_from_sizes(const Tensor& sizes_dev) {
  require_device(sizes_dev, "device metadata");
  TORCH_CHECK(sizes_dev.scalar_type() == at::kLong && sizes_dev.dim() == 2 && sizes_dev.is_contiguous(),
              "offsets_from_sizes: sizes must be a contiguous int64 [B, D] tensor");
  const int64_t B = sizes_dev.size(0), D = sizes_dev.size(1);
  c10::hip::HIPGuard guard(sizes_dev.device().index());
  Tensor offsets = at::empty({B + 1}, sizes_dev.options());
  const size_t ws_bytes = nt_offsets_workspace_bytes(B);
  Tensor ws;
  if (ws_bytes) ws = at::empty({static_cast<int64_t>(ws_bytes)}, sizes_dev.options().dtype(at::kByte));
  check(nt_offsets_from_sizes(sizes_dev.const_data_ptr<int64_t>(), B, D, offsets.data_ptr<int64_t>(),
                              ws_bytes ? ws.data_ptr() : nullptr, ws_bytes, stream_of(sizes_dev)));
  return offsets;
}

// ---- packed <-> padded --------------------------------------------------------

struct PadArgs {
  int64_t B, D;
  std::vector<int64_t> out_shape;
};

PadArgs pad_args(const Tensor& buffer, const Tensor& sizes_dev, const Tensor& offsets_dev,
                 at::IntArrayRef padded_sizes, int64_t n_ragged, const char* what) {
  require_device(buffer, what);
  TORCH_CHECK(sizes_dev.dim() == 2 && sizes_dev.scalar_type() == at::kLong && sizes_dev.is_contiguous() &&
                  sizes_dev.device() == buffer.device(),
              what, ": sizes must be a contiguous int64 [B, D] tensor on the buffer's device");
  PadArgs a;
  a.B = sizes_dev.size(0);
  a.D = sizes_dev.size(1);
  TORCH_CHECK(offsets_dev.numel() == a.B + 1 && offsets_dev.scalar_type() == at::kLong &&
                  offsets_dev.is_contiguous() && offsets_dev.device() == buffer.device(),
              what, ": offsets must be a contiguous int64 [B + 1] tensor on the buffer's device");
  TORCH_CHECK(static_cast<int64_t>(padded_sizes.size()) == a.D, what, ": one padded extent per constituent dim");
  TORCH_CHECK(n_ragged >= 1 && n_ragged <= 3, what, " supports at most 3 irregular dimensions.");
  a.out_shape.reserve(a.D + 1);
  a.out_shape.push_back(a.B);
  for (int64_t v : padded_sizes) a.out_shape.push_back(v);
  return a;
}

// to_padded_tensor (masking.cpp:558-625) on the lowered form.
Tensor add_padding(const Tensor& buffer, const Tensor& sizes_dev, const Tensor& offsets_dev,
                   at::IntArrayRef padded_sizes, int64_t n_ragged, double padding) {
  const PadArgs a = pad_args(buffer, sizes_dev, offsets_dev, padded_sizes, n_ragged, "to_padded_tensor");
  c10::hip::HIPGuard guard(buffer.device().index());
  Tensor out = at::empty(a.out_shape, buffer.options());
  check(nt_add_padding(buffer.const_data_ptr(), out.data_ptr(), offsets_dev.const_data_ptr<int64_t>(),
                       sizes_dev.const_data_ptr<int64_t>(), a.B, a.D, n_ragged, padded_sizes.data(),
                       elem_bytes(buffer.scalar_type()), pad_bits(padding, buffer.scalar_type()),
                       stream_of(buffer)));
  return out;
}

// to_tensor_mask when the mask keeps every dim of the data, and pad_nt
// (masking.cpp:138-179, 251-296): data and mask in one launch.
std::tuple<Tensor, Tensor> add_padding_mask(const Tensor& buffer, const Tensor& sizes_dev,
                                            const Tensor& offsets_dev, at::IntArrayRef padded_sizes,
                                            int64_t n_ragged, double padding) {
  const PadArgs a = pad_args(buffer, sizes_dev, offsets_dev, padded_sizes, n_ragged, "to_tensor_mask");
  c10::hip::HIPGuard guard(buffer.device().index());
  Tensor out = at::empty(a.out_shape, buffer.options());
  Tensor mask = at::empty(a.out_shape, buffer.options().dtype(at::kBool));
  check(nt_add_padding_mask(buffer.const_data_ptr(), out.data_ptr(), static_cast<uint8_t*>(mask.data_ptr()),
                            offsets_dev.const_data_ptr<int64_t>(), sizes_dev.const_data_ptr<int64_t>(), a.B,
                            a.D, n_ragged, padded_sizes.data(), elem_bytes(buffer.scalar_type()),
                            pad_bits(padding, buffer.scalar_type()), stream_of(buffer)));
  return std::make_tuple(out, mask);
}

// from_padded_tensor (masking.cpp:459-509) on the lowered form: the entries of
// `padded` inside the nested size, packed.  total_numel = offsets[B] as the host knows it.
Tensor remove_padding(const Tensor& padded_in, const Tensor& sizes_dev, const Tensor& offsets_dev,
                      int64_t total_numel, int64_t n_ragged) {
  require_device(padded_in, "from_padded_tensor");
  const Tensor padded = padded_in.contiguous();
  const PadArgs a = pad_args(padded, sizes_dev, offsets_dev, padded.sizes().slice(1), n_ragged,
                             "from_padded_tensor");
  TORCH_CHECK(padded.size(0) == a.B, "Target size has a different batch size than the padded Tensor.");
  c10::hip::HIPGuard guard(padded.device().index());
  Tensor out = at::empty({total_numel}, padded.options());
  if (total_numel == 0) return out;
  const at::IntArrayRef ext = padded.sizes().slice(1);
  check(nt_remove_padding(padded.const_data_ptr(), out.data_ptr(), offsets_dev.const_data_ptr<int64_t>(),
                          sizes_dev.const_data_ptr<int64_t>(), a.B, a.D, n_ragged, ext.data(),
                          elem_bytes(padded.scalar_type()), stream_of(padded)));
  return out;
}

// Bool mask over [B, ext...] from the nested size (nt_build_mask): to_mask, and the
// collapsed mask of to_tensor_mask (masking.cpp:322-457).
Tensor build_mask(const Tensor& sizes_dev, at::IntArrayRef ext) {
  require_device(sizes_dev, "to_tensor_mask");
  TORCH_CHECK(sizes_dev.dim() == 2 && sizes_dev.scalar_type() == at::kLong && sizes_dev.is_contiguous(),
              "build_mask: sizes must be a contiguous int64 [B, D] tensor");
  const int64_t B = sizes_dev.size(0), D = sizes_dev.size(1), K = static_cast<int64_t>(ext.size());
  TORCH_CHECK(K >= 1 && K <= 3 && K <= D, "masks over more than 3 constituent dimensions are not supported.");
  std::vector<int64_t> shape;
  shape.push_back(B);
  for (int64_t v : ext) shape.push_back(v);
  c10::hip::HIPGuard guard(sizes_dev.device().index());
  Tensor mask = at::empty(shape, sizes_dev.options().dtype(at::kBool));
  check(nt_build_mask(static_cast<uint8_t*>(mask.data_ptr()), sizes_dev.const_data_ptr<int64_t>(), B, D, K,
                      ext.data(), stream_of(sizes_dev)));
  return mask;
}

// ---- list of device tensors -> packed -------------------------------------------

// impl::pack (Packed.h:75-98) with the checks of _verify_variables
// (creation.cpp:28-171) for constituents that already live on the device: one
// gather launch (nt_pack / nt_pack_table) instead of B copy_ calls.  The nested
// size, the element offsets computed from it and the table of source pointers
// reach the device in the launch's own arguments when they fit there, else in one
// copy from pinned memory.  Returns (buffer, sizes, sizes_dev, offsets_dev).
std::tuple<Tensor, Tensor, Tensor, Tensor> pack_device(at::TensorList tensors) {
  static const char* hint =
      "To form a valid NestedTensor all Tensor / NestedTensor constiuents of the given list must be "
      "of the same dimension, layout, device, scalar type and either all or none require gradients.";
  TORCH_CHECK(!tensors.empty(), "pack_device: empty list");
  const Tensor& first = tensors[0];
  require_device(first, "nested_tensor (device constituents)");
  const int64_t B = static_cast<int64_t>(tensors.size()), D = first.dim();
  for (const Tensor& t : tensors) {
    TORCH_CHECK(t.dim() == first.dim(), "Given Tensor / NestedTensor constiuent of dimension ", t.dim(),
                " doesn't match another constiuent of dimension ", first.dim(), ". ", hint);
    TORCH_CHECK(t.layout() == first.layout(), "Given Tensor / NestedTensor constiuent of layout ", t.layout(),
                " doesn't match another constiuent of layout ", first.layout(), ". ", hint);
    TORCH_CHECK(t.device() == first.device(), "Given Tensor / NestedTensor constiuent of device ", t.device(),
                " doesn't match another constiuent of device ", first.device(), ". ");
    TORCH_CHECK(t.scalar_type() == first.scalar_type(), "Given Tensor / NestedTensor constiuent of scalar type ",
                t.scalar_type(), " doesn't match another constiuent of scalar type ", first.scalar_type(), ". ");
    TORCH_CHECK(t.requires_grad() == first.requires_grad(),
                "Given Tensor / NestedTensor constiuent requires gradient in contrast to another constiuent. ", hint);
  }
  const int eb = elem_bytes(first.scalar_type());
  c10::hip::HIPGuard guard(first.device().index());
  std::vector<Tensor> keep;
  keep.reserve(B);
  for (const Tensor& t : tensors) keep.push_back(t.contiguous());
  Tensor sizes = at::empty({B, D}, at::kLong);
  int64_t* sp = sizes.data_ptr<int64_t>();
  const int64_t n = B * D + (B + 1) + B;
  // a small table goes to the device inside the kernel arguments of the pack
  // launch, which also writes the device copy; a large one is uploaded from pinned
  // memory first
  const bool in_args = n <= nt_pack_table_max_entries();
  Tensor host = in_args ? at::empty({n}, at::kLong)
                        : at::empty({n}, at::TensorOptions().dtype(at::kLong).pinned_memory(true));
  int64_t* h = host.data_ptr<int64_t>();
  int64_t* off = h + B * D;
  int64_t* ptrs = off + B + 1;
  int64_t acc = 0;
  for (int64_t b = 0; b < B; ++b) {
    const at::IntArrayRef shape = keep[b].sizes();
    for (int64_t k = 0; k < D; ++k) sp[b * D + k] = h[b * D + k] = shape[k];
    off[b] = acc;
    acc += keep[b].numel();
    ptrs[b] = reinterpret_cast<int64_t>(keep[b].const_data_ptr());
  }
  off[B] = acc;
  Tensor meta = at::empty({n}, first.options().dtype(at::kLong));
  Tensor sizes_dev = meta.narrow(0, 0, B * D).view({B, D});
  Tensor offsets_dev = meta.narrow(0, B * D, B + 1);
  Tensor buffer = at::empty({acc}, first.options());
  if (in_args) {
    check(nt_pack_table(h, B, D, buffer.data_ptr(), meta.data_ptr<int64_t>(), eb, stream_of(first)));
  } else {
    meta.copy_(host, /*non_blocking=*/true);
    if (acc > 0) {
      check(nt_pack(reinterpret_cast<const void* const*>(meta.const_data_ptr<int64_t>() + B * D + B + 1),
                    buffer.data_ptr(), offsets_dev.const_data_ptr<int64_t>(), B, eb, stream_of(first)));
    }
  }
  // `keep` may hold temporaries; torch's caching allocator reuses their blocks
  // only for later work on this same stream
  return std::make_tuple(buffer, sizes, sizes_dev, offsets_dev);
}

// ---- dense + mask -> nested ----------------------------------------------------

// Result of a dense -> nested conversion in lowered form.  sizes is a host int64
// [B, D] tensor (0-d for an empty nested tensor, EfficientSizeNode.h:8-12);
// sizes_dev / offsets_dev are its device mirror and the element offsets when the
// conversion had to build them anyway (undefined tensors otherwise).
struct Lowered {
  Tensor buffer, sizes, sizes_dev, offsets_dev;
};

Lowered empty_nt() {
  // nested_tensor([]): Packed.h:77-79, EfficientSizeNode.h:10-12
  return {at::ones({0}, at::kFloat), at::zeros({}, at::kLong), Tensor(), Tensor()};
}

Tensor sizes_from_shapes(const std::vector<std::vector<int64_t>>& shapes) {
  const int64_t n = static_cast<int64_t>(shapes.size());
  const int64_t d = static_cast<int64_t>(shapes[0].size());
  for (const auto& s : shapes) {
    TORCH_CHECK(static_cast<int64_t>(s.size()) == d, "Given Tensor / NestedTensor constiuent of dimension ",
                s.size(), " doesn't match another constiuent of dimension ", d, ". ");
  }
  Tensor sizes = at::empty({n, d}, at::kLong);
  int64_t* p = sizes.data_ptr<int64_t>();
  for (const auto& s : shapes)
    for (int64_t v : s) *p++ = v;
  return sizes;
}

// Every tensor[i] is a constituent, whole (masking.cpp:228-232).
Lowered keep_all(const Tensor& tensor) {
  const int64_t B = tensor.size(0);
  if (B == 0) return empty_nt();
  std::vector<int64_t> shape(tensor.sizes().begin() + 1, tensor.sizes().end());
  Tensor sizes = at::empty({B, static_cast<int64_t>(shape.size())}, at::kLong);
  int64_t* p = sizes.data_ptr<int64_t>();
  for (int64_t b = 0; b < B; ++b)
    for (int64_t v : shape) *p++ = v;
  return {tensor.contiguous().reshape({-1}).clone(), sizes, Tensor(), Tensor()};
}

Tensor as_byte_mask(const Tensor& mask) {
  if (mask.scalar_type() == at::kBool) return mask.contiguous().view(at::kByte);
  if (mask.scalar_type() == at::kByte) return mask.contiguous();
  return mask.ne(0).contiguous().view(at::kByte);
}

// Pinned staging memory for the one device-to-host copy of a conversion; grows,
// never shrinks, one per host thread.
Tensor& pinned_staging(int64_t bytes) {
  static thread_local Tensor buf;
  if (!buf.defined() || buf.numel() < bytes) {
    int64_t cap = 1 << 16;
    while (cap < bytes) cap <<= 1;
    buf = at::empty({cap}, at::TensorOptions().dtype(at::kByte).pinned_memory(true));
  }
  return buf;
}

// Wait until everything enqueued on `stream` so far has completed and its writes
// to pinned host memory are visible.  The stream itself writes a sequence number
// into a pinned word when it gets there (hipStreamWriteValue32) and the host
// polls that word: a few microseconds sooner than hipStreamSynchronize wakes up,
// which is most of what a small conversion costs.  Falls back to the blocking
// wait if the stream operation is not available or takes long.
void wait_for_stream(hipStream_t stream) {
  static thread_local Tensor flag_t;
  static thread_local uint32_t seq = 0;
  static thread_local bool usable = true;
  if (usable) {
    if (!flag_t.defined()) {
      flag_t = at::zeros({16}, at::TensorOptions().dtype(at::kInt).pinned_memory(true));
    }
    uint32_t* flag = reinterpret_cast<uint32_t*>(flag_t.data_ptr());
    const uint32_t want = ++seq;
    if (hipStreamWriteValue32(stream, flag, want, 0) == hipSuccess) {
      // Poll for at most 200 microseconds (an acquire load: the counts the kernel wrote
      // to pinned memory are read after it), then hand the wait to the runtime.  The
      // write-value operation follows the kernel in stream order; that the kernel's
      // own stores to host memory are visible by then is what the blocking
      // synchronise below guarantees in any case, and it runs whenever the flag
      // has not shown up in time.
      const auto t0 = std::chrono::steady_clock::now();
      for (int spin = 0;; ++spin) {
        if (__atomic_load_n(flag, __ATOMIC_ACQUIRE) == want) return;
        __builtin_ia32_pause();
        if ((spin & 255) == 255 &&
            std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(200)) break;
      }
    } else {
      (void)hipGetLastError();
      usable = false;
    }
  }
  C10_HIP_CHECK(hipStreamSynchronize(stream));
}

// The two words nt_leading_boxes signals its completion through: a pinned host
// word the last workgroup writes a sequence number into, and the device word its
// workgroups count their arrivals in (zero between launches; one per device, so
// conversions of one host thread must not overlap on a device, which the shared
// staging buffer rules out already).
struct BoxSignal {
  uint32_t* done;
  uint32_t* arrivals;   // nullptr: one completion word per constituent (`words` of them)
  uint32_t value;
  int64_t words;
};
constexpr int64_t kBoxWordsMax = 64;       // completion words in the pinned block
constexpr int64_t kBoxStampedMax = 1024;   // constituents up to which the host polls stamped lines
BoxSignal box_signal(const c10::Device& device, int64_t B) {
  static thread_local Tensor flag_t;
  static thread_local std::vector<Tensor> arrivals;
  static thread_local uint32_t seq = 0;
  if (!flag_t.defined()) flag_t = at::zeros({kBoxWordsMax}, at::TensorOptions().dtype(at::kInt).pinned_memory(true));
  // Up to kBoxStampedMax constituents the lines carry the call's stamp themselves
  // (nt_leading_boxes_stamped): no completion word, no counter (stamp 0 is never used).
  if (B <= kBoxStampedMax) {
    if (++seq == 0) ++seq;
    return {nullptr, nullptr, seq, 0};
  }
  const size_t idx = static_cast<size_t>(device.index());
  if (arrivals.size() <= idx) arrivals.resize(idx + 1);
  if (!arrivals[idx].defined()) {
    arrivals[idx] = at::zeros({16}, at::TensorOptions().dtype(at::kInt).device(device));
    C10_HIP_CHECK(hipStreamSynchronize(c10::hip::getCurrentHIPStream(device.index()).stream()));
  }
  return {reinterpret_cast<uint32_t*>(flag_t.data_ptr()), reinterpret_cast<uint32_t*>(arrivals[idx].data_ptr()), ++seq, 1};
}

// Polls the completion word for at most 200 microseconds (acquire: the lines the
// kernel wrote to pinned memory are read after it), then hands the wait to the
// runtime, after which the lines are visible in any case.
void wait_for_signal(const BoxSignal& sig, hipStream_t stream) {
  const auto t0 = std::chrono::steady_clock::now();
  for (int spin = 0;; ++spin) {
    int64_t seen = 0;
    while (seen < sig.words && __atomic_load_n(sig.done + seen, __ATOMIC_ACQUIRE) == sig.value) ++seen;
    if (seen == sig.words) return;
    __builtin_ia32_pause();
    if ((spin & 255) == 255 && std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(200)) break;
  }
  C10_HIP_CHECK(hipStreamSynchronize(stream));
}

// Scan the per-row keep-counts and move the kept chunks (nt_exclusive_scan_i32,
// nt_compact_rows).  Returns the packed 1-D buffer.
Tensor compact(const Tensor& data, const Tensor& bmask, int64_t R, int64_t M, int64_t chunk_elems,
               int64_t total_kept, const int32_t* counts_dev) {
  Tensor out = at::empty({total_kept * chunk_elems}, data.options());
  if (total_kept == 0 || chunk_elems == 0) return out;
  Tensor row_offsets = at::empty({R + 1}, data.options().dtype(at::kLong));
  const size_t ws_bytes = nt_scan_workspace_bytes(R);
  Tensor ws;
  if (ws_bytes) ws = at::empty({static_cast<int64_t>(ws_bytes)}, data.options().dtype(at::kByte));
  void* stream = stream_of(data);
  check(nt_exclusive_scan_i32(counts_dev, R, row_offsets.data_ptr<int64_t>(), ws_bytes ? ws.data_ptr() : nullptr,
                              ws_bytes, stream));
  check(nt_compact_rows(data.const_data_ptr(), static_cast<const uint8_t*>(bmask.const_data_ptr()),
                        row_offsets.const_data_ptr<int64_t>(), R, M,
                        chunk_elems * static_cast<int64_t>(data.element_size()), out.data_ptr(), stream));
  return out;
}

// Upload sizes[B, D] and the element offsets computed from them.  A table of up
// to nt_pack_table_max_entries() int64 rides in the arguments of a one-workgroup
// launch (nt_upload_table): no pinned block to find, no copy engine, and the
// launches behind it on the stream start a few microseconds earlier than behind
// a copy.  Larger tables go in one copy from torch's pinned-memory allocator,
// which keeps the block until the asynchronous copy has left it: no wait here.
void upload_meta(const Tensor& sizes, const Tensor& like, Tensor* sizes_dev, Tensor* offsets_dev, int64_t* total) {
  const int64_t B = sizes.size(0), D = sizes.size(1);
  const int64_t n = B * D + B + 1;
  static const int64_t kInArgs = nt_pack_table_max_entries();
  Tensor host;
  std::vector<int64_t> small;
  int64_t* h;
  if (n <= kInArgs) {
    small.resize(static_cast<size_t>(n));
    h = small.data();
  } else {
    host = at::empty({n}, at::TensorOptions().dtype(at::kLong).pinned_memory(true));
    h = host.data_ptr<int64_t>();
  }
  const int64_t* s = sizes.const_data_ptr<int64_t>();
  std::memcpy(h, s, static_cast<size_t>(B * D) * 8);
  int64_t* off = h + B * D;
  int64_t acc = 0;
  for (int64_t b = 0; b < B; ++b) {
    off[b] = acc;
    int64_t prod = 1;
    for (int64_t k = 0; k < D; ++k) prod *= s[b * D + k];
    acc += prod;
  }
  off[B] = acc;
  *total = acc;
  Tensor meta = at::empty({n}, like.options().dtype(at::kLong));
  if (n <= kInArgs) {
    check(nt_upload_table(h, n, meta.data_ptr<int64_t>(), stream_of(like)));
  } else {
    meta.copy_(host, /*non_blocking=*/true);
  }
  *sizes_dev = meta.narrow(0, 0, B * D).view({B, D});
  *offsets_dev = meta.narrow(0, B * D, B + 1);
}

// All n entries of p equal v (one block compare of the array against itself, shifted).
template <typename T>
bool all_equal(const T* p, int64_t n, T v) {
  if (n <= 0) return true;
  return p[0] == v && (n == 1 || std::memcmp(p, p + 1, static_cast<size_t>(n - 1) * sizeof(T)) == 0);
}

// Keep-counts c of one constituent, one per mask row, rows indexed by dims[0 .. nd)
// (row-major).  True iff they describe a leading box: c = w where every row index
// i_k < ext[k], 0 elsewhere, w > 0 (or everything 0).  Fills ext[0 .. nd] = (row
// extents, w).  Level by level from the innermost row dim: the children of the
// first parent are copies of the first child up to some extent and zero after it;
// the first parent then is the pattern for the level above.
bool leading_box(const int32_t* c, const int64_t* dims, int64_t nd, int64_t* ext) {
  int64_t n = 1;
  for (int64_t k = 0; k < nd; ++k) n *= dims[k];
  if (n == 0) return false;
  const int32_t w = c[0];
  if (w == 0) {
    for (int64_t k = 0; k <= nd; ++k) ext[k] = 0;
    return all_equal(c, n, int32_t(0));
  }
  int64_t block = 1;                       // entries of one child at the current level
  for (int64_t k = nd - 1; k >= 0; --k) {
    const int64_t d = dims[k];
    int64_t e = 1;
    while (e < d && std::memcmp(c, c + e * block, static_cast<size_t>(block) * 4) == 0) ++e;
    if (!all_equal(c + e * block, (d - e) * block, int32_t(0))) return false;
    ext[k] = e;
    block *= d;
  }
  ext[nd] = w;
  return true;
}

// General case of nt_from_tensor_mask (masking.cpp:203-222) for a mask over the
// first `mask_dims` dims of `tensor`.  Rows = everything but the last mask dim.
// `count_rows` fills device (counts, prefix flags); `byte_mask` materialises the
// mask, which only the non-prefix path needs.
template <class CountRows, class ByteMask>
Lowered from_rows(const Tensor& tensor, int64_t mask_dims, CountRows count_rows, ByteMask byte_mask) {
  // a mask row lives below the batch dim: the level tables below index [mask_dims - 2]
  TORCH_CHECK(mask_dims >= 2 && mask_dims <= tensor.dim(),
              "nested_tensor_from_tensor_mask: the mask needs a batch dim and at least one more (got ", mask_dims,
              " mask dims for a tensor of ", tensor.dim(), " dims)");
  const int64_t B = tensor.size(0);
  const at::IntArrayRef shape = tensor.sizes();
  const int64_t M = shape[mask_dims - 1];
  int64_t R = 1;
  for (int64_t k = 0; k + 1 < mask_dims; ++k) R *= shape[k];
  std::vector<int64_t> rest(shape.begin() + mask_dims, shape.end());
  int64_t chunk = 1;
  for (int64_t v : rest) chunk *= v;
  // count_shape = [B] + shape[1 : mask_dims - 1]; per constituent rows_per = R / B
  const int64_t levels = mask_dims - 1;            // mask dims below the batch dim
  const int64_t rows_per = B > 0 ? R / B : 0;

  TORCH_CHECK(R <= (int64_t(1) << 26), "nested_tensor_from_tensor_mask: ", R,
              " mask rows exceed what this conversion stages on the host (67 108 864)");
  c10::hip::HIPGuard guard(tensor.device().index());
  // The keep-counts (int32) and the "row keeps a prefix" flags (uint8) of the R
  // rows are what the nested size is derived from.  Whatever the host needs of
  // them is written by a kernel straight into pinned host memory (which the
  // device addresses), and the host waits for the stream.
  hipStream_t stream = c10::hip::getCurrentHIPStream(tensor.device().index()).stream();
  std::vector<int64_t> total(B, 0);
  std::vector<std::vector<int64_t>> extents(B, std::vector<int64_t>(levels, 0));   // outermost first
  static const int64_t kBoxDims = nt_leading_boxes_max_dims();
  const int64_t box_ints = kBoxDims + 2;
  // First the common case, a padded tensor's mask: every constituent keeps a
  // leading box.  The device decides that itself from the row statistics
  // (nt_leading_boxes) and only a few integers per constituent cross to the
  // host; reading the statistics of every row from pinned memory costs the host
  // more than the row-count kernel takes (29 us for the 38 400 rows of a batch of
  // sixteen 3 x 800-row images).
  bool boxes_ok = false;
  Tensor stats_dev;
  const bool try_boxes = R > 0 && rows_per > 0 && levels - 1 <= kBoxDims;
  Tensor& stage = pinned_staging(std::max<int64_t>(5 * R, try_boxes ? 8 * box_ints * B : 0) + 16);
  int32_t* counts = reinterpret_cast<int32_t*>(stage.data_ptr());
  uint8_t* prefix = static_cast<uint8_t*>(stage.data_ptr()) + 4 * R;
  if (try_boxes) {
    stats_dev = at::empty({5 * R + 16}, tensor.options().dtype(at::kByte));
    int32_t* counts_dev = reinterpret_cast<int32_t*>(stats_dev.data_ptr());
    uint8_t* prefix_dev = static_cast<uint8_t*>(stats_dev.data_ptr()) + 4 * R;
    count_rows(R, M, counts_dev, prefix_dev);
    int32_t* boxes = reinterpret_cast<int32_t*>(stage.data_ptr());
    const BoxSignal sig = box_signal(tensor.device(), B);
    std::vector<int32_t> unstamped;
    if (sig.done == nullptr) {
      // every entry arrives as {value, stamp} in one 8-byte word; poll until all carry
      // this call's stamp (bounded: then the stream is synchronised, after which they do)
      uint64_t* lines = reinterpret_cast<uint64_t*>(stage.data_ptr());
      check(nt_leading_boxes_stamped(counts_dev, prefix_dev, B, rows_per, shape.data() + 1, levels - 1, lines, sig.value,
                                     stream));
      const int64_t n_words = B * box_ints;
      const auto t0 = std::chrono::steady_clock::now();
      int64_t seen = 0;
      for (int spin = 0; seen < n_words; ++spin) {
        while (seen < n_words &&
               static_cast<uint32_t>(__atomic_load_n(lines + seen, __ATOMIC_ACQUIRE) >> 32) == sig.value) {
          ++seen;
        }
        if (seen == n_words) break;
        __builtin_ia32_pause();
        if ((spin & 255) == 255 && std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(200)) {
          C10_HIP_CHECK(hipStreamSynchronize(stream));
          break;
        }
      }
      unstamped.resize(static_cast<size_t>(n_words));
      for (int64_t i = 0; i < n_words; ++i) {
        const uint64_t word = __atomic_load_n(lines + i, __ATOMIC_ACQUIRE);
        TORCH_CHECK(static_cast<uint32_t>(word >> 32) == sig.value,
                    "nested_tensor_from_tensor_mask: the device did not deliver the nested size");
        unstamped[static_cast<size_t>(i)] = static_cast<int32_t>(static_cast<uint32_t>(word));
      }
      boxes = unstamped.data();
    } else {
      check(nt_leading_boxes(counts_dev, prefix_dev, B, rows_per, shape.data() + 1, levels - 1, boxes, sig.done, sig.value,
                             sig.arrivals, stream));
      wait_for_signal(sig, stream);
    }
    boxes_ok = true;
    for (int64_t b = 0; b < B && boxes_ok; ++b) boxes_ok = boxes[b * box_ints] == 1;
    if (boxes_ok) {
      for (int64_t b = 0; b < B; ++b) {
        const int32_t* bx = boxes + b * box_ints;
        int64_t prod = bx[1];
        for (int64_t k = 0; k + 1 < levels; ++k) {
          extents[b][k] = bx[1] == 0 ? 0 : bx[2 + k];
          prod *= extents[b][k];
        }
        extents[b][levels - 1] = bx[1];
        total[b] = prod;
      }
    } else {
      // some constituent keeps something else: the statistics of every row after all
      C10_HIP_CHECK(hipMemcpyAsync(counts, counts_dev, static_cast<size_t>(5 * R), hipMemcpyDeviceToHost, stream));
      C10_HIP_CHECK(hipStreamSynchronize(stream));
    }
  } else if (R > 0) {
    count_rows(R, M, counts, prefix);
    wait_for_stream(stream);
  }

  // Nested size from the counts: at every mask level the extent is the number of
  // children that keep anything (masking.cpp:203-222); the selection must be
  // rectangular or at::stack would have thrown.  `leading`: the kept children
  // come first at every level.
  bool leading = true;
  std::vector<uint8_t> alive, next;
  for (int64_t b = 0; b < B && !boxes_ok; ++b) {
    const int32_t* c = counts + b * rows_per;
    const uint8_t* pf = prefix + b * rows_per;
    // What a padded tensor's mask looks like: every row keeps the same leading w
    // entries or nothing, and the rows that keep something are a leading box of the
    // row dims.  Checked with block compares (each count is looked at about twice).
    if (rows_per > 0 && all_equal(pf, rows_per, uint8_t(1)) &&
        leading_box(c, shape.data() + 1, levels - 1, extents[b].data())) {
      int64_t prod = 1;
      for (int64_t v : extents[b]) prod *= v;
      total[b] = prod;
      continue;
    }
    // anything else: the walk over every row
    alive.resize(rows_per > 0 ? rows_per : 1);
    next.resize(rows_per > 0 ? rows_per : 1);
    int64_t sum = 0;
    int32_t mx = 0;
    uint8_t all_prefix = 1;
    for (int64_t r = 0; r < rows_per; ++r) {
      const int32_t v = c[r];
      sum += v;
      mx = v > mx ? v : mx;
      all_prefix &= pf[r];
      alive[r] = v > 0;
    }
    leading = leading && all_prefix != 0;
    total[b] = sum;
    extents[b][levels - 1] = mx;
    // walk the mask levels upwards: alive[i] = child i keeps anything
    int64_t n = rows_per;
    for (int64_t lev = levels - 2; lev >= 0; --lev) {
      const int64_t width = shape[lev + 1];      // children per parent at this level
      const int64_t parents = width > 0 ? n / width : 0;
      int64_t mxc = 0;
      for (int64_t p = 0; p < parents; ++p) {
        const uint8_t* a = alive.data() + p * width;
        int64_t cnt = a[0];
        uint8_t rises = 0;
        for (int64_t i = 1; i < width; ++i) {
          rises |= static_cast<uint8_t>(a[i] > a[i - 1]);
          cnt += a[i];
        }
        if (rises) leading = false;
        next[p] = cnt > 0;
        if (cnt > mxc) mxc = cnt;
      }
      extents[b][lev] = mxc;
      alive.swap(next);
      n = parents;
    }
  }
  std::vector<std::vector<int64_t>> shapes(B);
  int64_t kept_total = 0;
  for (int64_t b = 0; b < B; ++b) {
    int64_t prod = 1;
    for (int64_t v : extents[b]) prod *= v;
    TORCH_CHECK(prod == total[b], "stack expects each tensor to be equal size: the mask does not select "
                                  "a rectangular block in every constituent.");
    kept_total += total[b];
    if (total[b] != 0) {
      shapes[b] = extents[b];
      shapes[b].insert(shapes[b].end(), rest.begin(), rest.end());
    } else {
      shapes[b].assign(shape.begin() + 1, shape.begin() + mask_dims - 1);
      shapes[b].push_back(0);
    }
  }
  if (B == 0) return empty_nt();
  Tensor sizes = sizes_from_shapes(shapes);
  if (leading) {
    // Every constituent keeps a leading box: this is the length-based un-pad
    // (nt_remove_padding) with the nested size just derived.
    const int64_t D = sizes.size(1);
    TORCH_CHECK(D == tensor.dim() - 1, "Target size has different dimension as input padded Tensor.");
    Tensor sizes_dev, offsets_dev;
    int64_t numel = 0;
    upload_meta(sizes, tensor, &sizes_dev, &offsets_dev, &numel);
    // dims up to the last one that differs between constituents, or from the
    // padded extent, are walked as ragged
    int64_t n_ragged = 1;
    const int64_t* s = sizes.const_data_ptr<int64_t>();
    for (int64_t k = 0; k < D; ++k) {
      bool regular = true;
      for (int64_t b = 0; b < B && regular; ++b) regular = s[b * D + k] == shape[k + 1];
      if (!regular) n_ragged = k + 1;
    }
    TORCH_CHECK(n_ragged <= 3, "from_padded_tensor supports at most 3 irregular dimensions.");
    Tensor out = remove_padding(tensor, sizes_dev, offsets_dev, numel, n_ragged);
    return {out, sizes, sizes_dev, offsets_dev};
  }
  // rare: the selection is a box that does not start at the origin of every
  // constituent.  The compaction scans the counts on the device.
  Tensor counts_dev = at::empty({R}, tensor.options().dtype(at::kInt));
  C10_HIP_CHECK(hipMemcpyAsync(counts_dev.data_ptr(), counts, static_cast<size_t>(R) * 4, hipMemcpyHostToDevice, stream));
  C10_HIP_CHECK(hipStreamSynchronize(stream));   // the staging buffer is reused by the next conversion
  Tensor buf = compact(tensor, byte_mask(), R, M, chunk, kept_total, counts_dev.const_data_ptr<int32_t>());
  return {buf, sizes, Tensor(), Tensor()};
}

// nt_from_tensor_mask (masking.cpp:181-249) at nested_dim 1.
Lowered from_mask(const Tensor& tensor_in, const Tensor& mask_in, int64_t nested_dim) {
  TORCH_CHECK(nested_dim == 1, "Only nested_dim of 1 is currently supported.");
  // masking.cpp:228-234: an empty mask or a single true keeps everything, a single
  // false keeps nothing.
  if (mask_in.numel() == 0) return keep_all(tensor_in);
  if (mask_in.numel() == 1) {
    return mask_in.reshape({-1})[0].item<bool>() ? keep_all(tensor_in) : empty_nt();
  }
  TORCH_CHECK(tensor_in.device() == mask_in.device(), "tensor and mask must be on the same device.");
  require_device(tensor_in, "nested_tensor_from_tensor_mask");
  TORCH_CHECK(mask_in.dim() <= tensor_in.dim(), "Mask has more dimensions than the data tensor.");
  const int64_t B = tensor_in.size(0);
  TORCH_CHECK_INDEX(mask_in.size(0) >= B, "index ", mask_in.size(0), " is out of bounds for dimension 0 with size ", B);
  const Tensor mask = mask_in.narrow(0, 0, B);
  const Tensor tensor = tensor_in.contiguous();
  const Tensor bmask = as_byte_mask(mask);
  int64_t inner_numel = 1;
  for (int64_t k = 1; k < mask.dim(); ++k) inner_numel *= mask.size(k);
  c10::hip::HIPGuard guard(tensor.device().index());

  if (inner_numel == 1) {
    // One mask value per constituent (masking.cpp:186-201 on mask[i]): true keeps
    // tensor[i] whole; false drops it (0-d mask[i]) or leaves an empty constituent
    // of shape [1, .., 1, 0].
    const int64_t row_elems = B > 0 ? tensor[0].numel() : 0;
    Tensor keep_host = mask.reshape({B}).to(at::kBool).cpu();
    const bool* keep = keep_host.const_data_ptr<bool>();
    int64_t kept = 0;
    for (int64_t b = 0; b < B; ++b) kept += keep[b];
    Tensor stats = at::empty({8}, tensor.options().dtype(at::kInt));
    check(nt_mask_row_counts(static_cast<const uint8_t*>(bmask.const_data_ptr()), 1, B, stats.data_ptr<int32_t>(),
                             reinterpret_cast<uint8_t*>(stats.data_ptr<int32_t>() + 4), stream_of(tensor)));
    Tensor buf = compact(tensor, bmask, 1, B, row_elems, kept, stats.const_data_ptr<int32_t>());
    std::vector<int64_t> full(tensor.sizes().begin() + 1, tensor.sizes().end());
    if (mask.dim() == 1) {
      if (kept == 0) return empty_nt();
      std::vector<std::vector<int64_t>> shapes(kept, full);
      return {buf, sizes_from_shapes(shapes), Tensor(), Tensor()};
    }
    std::vector<int64_t> empty_shape(mask.dim() - 2, 1);
    empty_shape.push_back(0);
    std::vector<std::vector<int64_t>> shapes;
    for (int64_t b = 0; b < B; ++b) shapes.push_back(keep[b] ? full : empty_shape);
    if (shapes.empty()) return empty_nt();
    return {buf, sizes_from_shapes(shapes), Tensor(), Tensor()};
  }
  for (int64_t k = 1; k < mask.dim(); ++k) {
    TORCH_CHECK(tensor.size(k) == mask.size(k), "Mask of shape ", mask.sizes(),
                " does not match the leading dimensions of the data tensor ", tensor.sizes(), ".");
  }
  return from_rows(
      tensor, mask.dim(),
      [&](int64_t R, int64_t M, int32_t* counts, uint8_t* prefix) {
        check(nt_mask_row_counts(static_cast<const uint8_t*>(bmask.const_data_ptr()), R, M, counts, prefix,
                                 stream_of(tensor)));
      },
      [&]() { return bmask; });
}

// nested_tensor_from_padded_tensor (nested/masking.py:12-14) on the device: the
// mask `tensor != padding` has the dims of the data and is never materialised
// unless the selection is not a leading box.
Lowered from_value(const Tensor& tensor_in, double padding, int64_t nested_dim) {
  TORCH_CHECK(nested_dim == 1, "Only nested_dim of 1 is currently supported.");
  require_device(tensor_in, "nested_tensor_from_padded_tensor");
  const int et = elem_type(tensor_in.scalar_type());
  TORCH_CHECK(et >= 0, "Input datatype ", tensor_in.scalar_type(), " is not supported.");
  const Tensor tensor = tensor_in.contiguous();
  return from_rows(
      tensor, tensor.dim(),
      [&](int64_t R, int64_t M, int32_t* counts, uint8_t* prefix) {
        check(nt_value_row_counts(tensor.const_data_ptr(), et, padding, R, M, counts, prefix, stream_of(tensor)));
      },
      [&]() { return as_byte_mask(tensor.ne(padding)); });
}

std::tuple<Tensor, Tensor> nt_from_tensor_mask_op(const Tensor& tensor, const Tensor& mask, int64_t nested_dim) {
  Lowered r = from_mask(tensor, mask, nested_dim);
  return std::make_tuple(r.buffer, r.sizes);
}

std::tuple<Tensor, Tensor, Tensor, Tensor> from_tensor_mask_lowered(const Tensor& tensor, const Tensor& mask,
                                                                    int64_t nested_dim) {
  Lowered r = from_mask(tensor, mask, nested_dim);
  return std::make_tuple(r.buffer, r.sizes, r.sizes_dev.defined() ? r.sizes_dev : at::empty({0}, at::kLong),
                         r.offsets_dev.defined() ? r.offsets_dev : at::empty({0}, at::kLong));
}

std::tuple<Tensor, Tensor> nt_from_padded_tensor_op(const Tensor& tensor, double padding, int64_t nested_dim) {
  Lowered r = from_value(tensor, padding, nested_dim);
  return std::make_tuple(r.buffer, r.sizes);
}

std::tuple<Tensor, Tensor, Tensor, Tensor> from_padded_value_lowered(const Tensor& tensor, double padding,
                                                                     int64_t nested_dim) {
  Lowered r = from_value(tensor, padding, nested_dim);
  return std::make_tuple(r.buffer, r.sizes, r.sizes_dev.defined() ? r.sizes_dev : at::empty({0}, at::kLong),
                         r.offsets_dev.defined() ? r.offsets_dev : at::empty({0}, at::kLong));
}

// merge_tensor_mask (masking.cpp:12-43) on a dense (tensor, mask) pair, any
// device: the last mask dim is dropped while every one of its rows is all ones
// or all zeros; stops at mask_dim, and refuses a mask_dim it cannot reach.
std::tuple<Tensor, Tensor> merge_tensor_mask(const Tensor& tensor, const Tensor& mask_in,
                                             c10::optional<int64_t> mask_dim) {
  Tensor mask = mask_in;
  while (true) {
    if (mask_dim.has_value() && mask.dim() == *mask_dim) return std::make_tuple(tensor, mask);
    if (mask.dim() == 0) return std::make_tuple(tensor, mask);
    const int64_t last = mask.size(-1);
    Tensor collapsed = mask.sum(-1);
    const int64_t uniform = collapsed.eq(last).logical_or(collapsed.eq(0)).sum().item<int64_t>();
    if (uniform == collapsed.numel()) {
      mask = collapsed.to(at::kBool);
      continue;
    }
    TORCH_CHECK(!(mask_dim.has_value() && *mask_dim != mask.dim()),
                "Mask dimension is too small to represent data tensor.");
    return std::make_tuple(tensor.contiguous(), mask.contiguous());
  }
}

// ---- packed projections and nested multi-head attention -------------------------

// Weights and biases of an attention layer against the input x [T, E]: on x's
// device (a module left on the host would hand the kernels host pointers), biases
// of the length the kernels read (3 E for the in-projection, N for the output).
void check_mha_weights(const Tensor& x, int64_t E, const Tensor& W, const Tensor& b_in, const Tensor& Wo,
                       const Tensor& b_out) {
  require_same_device(W, x, "mha", "in_proj_weight");
  require_same_device(b_in, x, "mha", "in_proj_bias");
  require_same_device(Wo, x, "mha", "out_proj_weight");
  require_same_device(b_out, x, "mha", "out_proj_bias");
  TORCH_CHECK(!b_in.defined() || b_in.numel() == 3 * E, "in_proj_bias must have 3 * embed_dim = ", 3 * E,
              " elements, got ", b_in.defined() ? b_in.numel() : 0);
  TORCH_CHECK(!b_out.defined() || b_out.numel() == Wo.size(0), "out_proj_bias must have ", Wo.size(0),
              " elements, got ", b_out.defined() ? b_out.numel() : 0);
}

// y = act(x @ weight.T + bias) on a 2-D row-major view (nt_linear_act): the packed
// fast path of NestedTensor_matmul (matmul.cpp:13-41) with the packed bias add
// (BinaryOps.cpp:97-107) and, optionally, relu / gelu (activation.cpp:11-19, 34-46)
// in the GEMM epilogue.  act: 0 none, 1 relu, 2 gelu.
Tensor linear_packed(const Tensor& x, const Tensor& weight_in, const c10::optional<Tensor>& bias_in, int64_t act) {
  require_device(x, "linear");
  TORCH_CHECK(x.dim() == 2 && weight_in.dim() == 2 && x.stride(1) == 1, "linear: x must be a 2-D row-major view");
  TORCH_CHECK(act >= 0 && act <= 2, "linear: activation must be None, 'relu' or 'gelu'");
  const int64_t M = x.size(0), K = x.size(1), N = weight_in.size(0);
  TORCH_CHECK(weight_in.size(1) == K, "linear: weight of shape ", weight_in.sizes(),
              " does not match input feature size ", K);
  const Tensor weight = weight_in.contiguous();
  Tensor bias;
  if (bias_in.has_value() && bias_in->defined()) bias = bias_in->contiguous();
  TORCH_CHECK(weight.scalar_type() == x.scalar_type() && (!bias.defined() || bias.scalar_type() == x.scalar_type()),
              "linear: input, weight and bias must have the same dtype");
  require_same_device(weight, x, "linear", "weight");
  require_same_device(bias, x, "linear", "bias");
  TORCH_CHECK(!bias.defined() || bias.numel() == N, "linear: bias of ", bias.defined() ? bias.numel() : 0,
              " elements does not match the ", N, " output features");
  c10::hip::HIPGuard guard(x.device().index());
  Tensor out = at::empty({M, N}, x.options());
  check(nt_linear_act(x.const_data_ptr(), x.stride(0), weight.const_data_ptr(),
                      bias.defined() ? bias.const_data_ptr() : nullptr, out.data_ptr(), N, M, N, K,
                      static_cast<int>(act), dtype_code(x.scalar_type()), stream_of(x)));
  return out;
}

// The attention kernels that read V transposed.  A two-dimensional `schedule` is the
// work list of nt_varlen_attention_vt ([n_work, 8]); a one-dimensional one is the
// device copy of a plan of nt_attention_plan, for the kernel that streams the keys
// of a sequence through LDS (head_dim 64 only).
int compute_units_of(const c10::Device& device) {
  int n = 0;
  TORCH_CHECK(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device.index()) == hipSuccess && n > 0,
              "attention: cannot query the compute units of ", device);
  return n;
}

void check_attention_schedule(const Tensor& schedule, const Tensor& x) {
  TORCH_CHECK(schedule.scalar_type() == at::kInt && schedule.is_contiguous() && schedule.device() == x.device() &&
                  ((schedule.dim() == 2 && schedule.size(1) == 8) || (schedule.dim() == 1 && schedule.size(0) >= 4)),
              "mha: schedule must be a contiguous int32 [n_work, 8] work list or a one-dimensional plan on the "
              "input's device");
}

void launch_attention_vt(const void* q, int64_t ldq, const void* k, int64_t ldk, const Tensor& vt, int64_t ldvt,
                         Tensor& attn, int64_t E, const Tensor& schedule, int64_t num_heads, int64_t head_dim,
                         int64_t total_kv, double scaling, int dt, void* stream) {
  if (schedule.dim() == 1) {
    TORCH_CHECK(head_dim == 64, "mha: the planned attention kernel covers head_dim 64 only");
    // the plan was made for one workgroup per compute unit of this device (attention_plan
    // below); a workgroup beyond the plan's own count returns at once
    check(nt_varlen_attention_planned(q, ldq, k, ldk, vt.const_data_ptr(), ldvt, attn.data_ptr(), E,
                                      schedule.const_data_ptr<int32_t>(), compute_units_of(attn.device()), num_heads,
                                      head_dim, total_kv, static_cast<float>(scaling), dt, stream));
    return;
  }
  check(nt_varlen_attention_vt(q, ldq, k, ldk, vt.const_data_ptr(), ldvt, attn.data_ptr(), E,
                               schedule.const_data_ptr<int32_t>(), schedule.size(0), num_heads, head_dim, total_kv,
                               static_cast<float>(scaling), dt, stream));
}

// Plan of the planned attention kernel for sequences of the given query and key
// lengths (host int64 tensors), copied to `device`.
Tensor attention_plan(const Tensor& q_lens, const Tensor& k_lens, int64_t num_heads, int64_t head_dim,
                      c10::Device device) {
  TORCH_CHECK(q_lens.device().is_cpu() && k_lens.device().is_cpu() && q_lens.scalar_type() == at::kLong &&
                  k_lens.scalar_type() == at::kLong && q_lens.dim() == 1 && k_lens.dim() == 1 &&
                  q_lens.numel() == k_lens.numel(),
              "attention_plan: the lengths must be host int64 vectors of one size");
  TORCH_CHECK(device.is_cuda(), "attention_plan: the plan is for a GPU");
  const Tensor ql = q_lens.contiguous(), kl = k_lens.contiguous();
  const int64_t B = ql.numel();
  const int n_wg = compute_units_of(device);
  const int64_t n = nt_attention_plan(ql.const_data_ptr<int64_t>(), kl.const_data_ptr<int64_t>(), B, num_heads, head_dim,
                                      n_wg, nullptr, 0);
  TORCH_CHECK(n > 0, "attention_plan: ", nt_last_error());
  Tensor plan = at::empty({n}, at::TensorOptions().dtype(at::kInt));
  const int64_t m = nt_attention_plan(ql.const_data_ptr<int64_t>(), kl.const_data_ptr<int64_t>(), B, num_heads, head_dim,
                                      n_wg, plan.data_ptr<int32_t>(), n);
  TORCH_CHECK(m == n, "attention_plan: ", nt_last_error());
  return plan.to(device);
}

// Self-attention layer on the packed token buffer x [T, E] (min_mha, mha.cpp:18-69;
// bt_min_mha, cuda/mha.cpp:22-107, passes no out bias): fused QKV projection with V
// written transposed, attention over each sequence's own keys, output projection.
// `schedule` is the device work list of nt_varlen_attention_vt, or a plan (launch_attention_vt).
Tensor mha_self_packed(const Tensor& x, const Tensor& schedule, int64_t num_heads, int64_t head_dim,
                       const Tensor& in_proj_weight, const c10::optional<Tensor>& in_proj_bias, double scaling,
                       const Tensor& out_proj_weight, const c10::optional<Tensor>& out_proj_bias) {
  require_device(x, "multi-head attention");
  const int64_t E = num_heads * head_dim;
  TORCH_CHECK(x.dim() == 2 && x.size(1) == E && x.stride(1) == 1, "mha: x must be a [T, num_heads * head_dim] view");
  const at::ScalarType st = x.scalar_type();
  TORCH_CHECK(st == at::kHalf || st == at::kBFloat16, "mha_self_packed: dtype must be float16 or bfloat16");
  TORCH_CHECK(head_dim == 32 || head_dim == 64 || head_dim == 128, "mha_self_packed: head_dim must be 32, 64 or 128");
  const Tensor W = in_proj_weight.contiguous();
  TORCH_CHECK(W.dim() == 2 && W.size(0) == 3 * E && W.size(1) == E,
              "in_proj_weight must have shape [3 * embed_dim, embed_dim].");
  Tensor b_in, b_out;
  if (in_proj_bias.has_value() && in_proj_bias->defined()) b_in = in_proj_bias->contiguous();
  if (out_proj_bias.has_value() && out_proj_bias->defined()) b_out = out_proj_bias->contiguous();
  const Tensor Wo = out_proj_weight.contiguous();
  TORCH_CHECK(W.scalar_type() == st && Wo.scalar_type() == st && (!b_in.defined() || b_in.scalar_type() == st) &&
                  (!b_out.defined() || b_out.scalar_type() == st),
              "linear: input, weight and bias must have the same dtype");
  TORCH_CHECK(Wo.dim() == 2 && Wo.size(1) == E, "linear: weight of shape ", Wo.sizes(),
              " does not match input feature size ", E);
  check_mha_weights(x, E, W, b_in, Wo, b_out);
  check_attention_schedule(schedule, x);
  const int64_t T = x.size(0), N = Wo.size(0);
  const int64_t ldvt = (T + 72 + 63) / 64 * 64;   // rows readable 72 elements past the last token, 128-byte aligned
  c10::hip::HIPGuard guard(x.device().index());
  void* stream = stream_of(x);
  const int dt = dtype_code(st);
  Tensor qk = at::empty({T, 2 * E}, x.options());
  Tensor vt = at::empty({E, ldvt}, x.options());
  Tensor attn = at::empty({T, E}, x.options());
  Tensor out = at::empty({T, N}, x.options());
  if (T == 0) return out;
  check(nt_linear_qkv(x.const_data_ptr(), x.stride(0), W.const_data_ptr(), b_in.defined() ? b_in.const_data_ptr() : nullptr,
                      qk.data_ptr(), 2 * E, vt.data_ptr(), ldvt, T, E, E, dt, stream));
  const char* kptr = static_cast<const char*>(qk.const_data_ptr()) + E * static_cast<int64_t>(x.element_size());
  launch_attention_vt(qk.const_data_ptr(), 2 * E, kptr, 2 * E, vt, ldvt, attn, E, schedule, num_heads, head_dim, T,
                      scaling, dt, stream);
  check(nt_linear_act(attn.const_data_ptr(), E, Wo.const_data_ptr(), b_out.defined() ? b_out.const_data_ptr() : nullptr,
                      out.data_ptr(), N, T, N, E, 0, dt, stream));
  return out;
}

// ---- row-wise operators on the packed buffer ------------------------------------

const void* opt_ptr(const c10::optional<Tensor>& t) {
  return (t.has_value() && t->defined()) ? t->const_data_ptr() : nullptr;
}

// nt_layer_norm over the packed [rows, n] view of x; residual (same shape) is added
// first.  The caller has checked the nested sizes.
Tensor layer_norm_packed(const Tensor& x, const c10::optional<Tensor>& residual, const c10::optional<Tensor>& weight,
                         const c10::optional<Tensor>& bias, int64_t n, double eps) {
  require_device(x, "layer_norm");
  TORCH_CHECK(x.is_contiguous() && n > 0 && x.numel() % n == 0, "layer_norm: the buffer must hold whole rows of ", n);
  for (const auto* t : {&residual, &weight, &bias}) {
    TORCH_CHECK(!t->has_value() || !(*t)->defined() ||
                    ((*t)->scalar_type() == x.scalar_type() && (*t)->device() == x.device() && (*t)->is_contiguous()),
                "layer_norm: operands must be contiguous tensors of the input's dtype on the input's device");
  }
  TORCH_CHECK(!residual.has_value() || !residual->defined() || residual->numel() == x.numel(),
              "layer_norm: the residual must have the size of the input");
  for (const auto* t : {&weight, &bias}) {
    TORCH_CHECK(!t->has_value() || !(*t)->defined() || (*t)->numel() == n,
                "layer_norm: weight and bias must have ", n, " elements");
  }
  c10::hip::HIPGuard guard(x.device().index());
  Tensor out = at::empty_like(x);
  check(nt_layer_norm(x.const_data_ptr(), opt_ptr(residual), opt_ptr(weight), opt_ptr(bias), out.data_ptr(),
                      x.numel() / n, n, eps, dtype_code(x.scalar_type()), stream_of(x)));
  return out;
}

// mul == false: out[i] = a[i] + scale * b[i % period]; mul == true: out[i] = scale * a[i] * b[i % period]
// (b absent: scale * a[i]).
Tensor binary_packed(const Tensor& a, const c10::optional<Tensor>& b, double scale, int64_t period, bool mul) {
  require_device(a, mul ? "mul" : "add");
  const bool has_b = b.has_value() && b->defined();
  TORCH_CHECK(mul || has_b, "add: the second operand is missing");
  TORCH_CHECK(a.is_contiguous() && (!has_b || (b->is_contiguous() && b->scalar_type() == a.scalar_type() &&
                                               b->device() == a.device())),
              mul ? "mul" : "add", ": both operands must have the same dtype and device");
  TORCH_CHECK(!has_b || (period > 0 && b->numel() >= period), "packed binary op: operand shorter than its period");
  c10::hip::HIPGuard guard(a.device().index());
  Tensor out = at::empty_like(a);
  if (a.numel() == 0) return out;
  const int dt = dtype_code(a.scalar_type());
  if (mul) {
    check(nt_mul_packed(a.const_data_ptr(), opt_ptr(b), scale, out.data_ptr(), a.numel(), period, dt, stream_of(a)));
  } else {
    check(nt_add_packed(a.const_data_ptr(), b->const_data_ptr(), scale, out.data_ptr(), a.numel(), period, dt,
                        stream_of(a)));
  }
  return out;
}

Tensor softmax_rows(const Tensor& x, const Tensor& offsets, const Tensor& row_offsets, int64_t total_rows, bool log) {
  require_device(x, log ? "log_softmax" : "softmax");
  TORCH_CHECK(x.is_contiguous() && offsets.scalar_type() == at::kLong && row_offsets.scalar_type() == at::kLong &&
                  offsets.device() == x.device() && row_offsets.device() == x.device() &&
                  offsets.numel() == row_offsets.numel() && offsets.numel() >= 1,
              "softmax: offsets and row offsets must be int64 [B + 1] tensors on the buffer's device");
  c10::hip::HIPGuard guard(x.device().index());
  Tensor out = at::empty_like(x);
  if (x.numel() == 0) return out;
  check(nt_softmax_rows(x.const_data_ptr(), out.data_ptr(), offsets.const_data_ptr<int64_t>(),
                        row_offsets.const_data_ptr<int64_t>(), offsets.numel() - 1, total_rows, log ? 1 : 0,
                        dtype_code(x.scalar_type()), stream_of(x)));
  return out;
}

Tensor activation_packed(const Tensor& x, int64_t act) {
  require_device(x, "activation");
  TORCH_CHECK(x.is_contiguous() && (act == 1 || act == 2), "activation: relu (1) or gelu (2) of a contiguous buffer");
  c10::hip::HIPGuard guard(x.device().index());
  Tensor out = at::empty_like(x);
  if (x.numel() == 0) return out;
  check(nt_activation_packed(x.const_data_ptr(), out.data_ptr(), x.numel(), static_cast<int>(act),
                             dtype_code(x.scalar_type()), stream_of(x)));
  return out;
}

// ---- consumers of the offsets array ---------------------------------------------

// After a kernel that may have counted out-of-range indices: the running count
// goes to its pinned host mirror with an asynchronous copy on the same stream (a
// copy node when the stream is being captured).  Nothing waits for it here.
void mirror_counter(const c10::optional<Tensor>& counter, const c10::optional<Tensor>& mirror, void* stream) {
  if (!counter.has_value() || !counter->defined() || !mirror.has_value() || !mirror->defined()) return;
  TORCH_CHECK(mirror->is_pinned() && mirror->numel() >= 1 && mirror->scalar_type() == at::kInt,
              "index counter mirror must be a pinned int32 tensor");
  C10_HIP_CHECK(hipMemcpyAsync(mirror->data_ptr(), counter->const_data_ptr(), 4, hipMemcpyDeviceToHost,
                               static_cast<hipStream_t>(stream)));
}

int32_t* counter_ptr(const c10::optional<Tensor>& counter, const Tensor& like) {
  if (!counter.has_value() || !counter->defined()) return nullptr;
  TORCH_CHECK(counter->scalar_type() == at::kInt && counter->numel() >= 1 && counter->device() == like.device(),
              "index counter must be an int32 tensor on the device of the table");
  return counter->data_ptr<int32_t>();
}

// NestedTensor_embedding (functions.cpp:14-63) on the packed index buffer: one
// gather (nt_gather_rows), result [T, E].  Out-of-range indices give zero rows
// and are added to `counter` (device int32[1]) when one is passed.
Tensor embedding_packed(const Tensor& weight_in, const Tensor& indices, const c10::optional<Tensor>& counter,
                        const c10::optional<Tensor>& mirror) {
  require_device(indices, "embedding");
  TORCH_CHECK(weight_in.dim() == 2, "'weight' must be 2-D");
  TORCH_CHECK(indices.scalar_type() == at::kLong || indices.scalar_type() == at::kInt,
              "Expected tensor for argument #1 'indices' to have one of the following scalar types: Long, Int; "
              "but got ", indices.scalar_type(), " instead");
  TORCH_CHECK(weight_in.device() == indices.device(), "embedding: weight and indices must be on the same device");
  const Tensor weight = weight_in.contiguous();
  const Tensor idx = indices.scalar_type() == at::kLong ? indices.contiguous() : indices.to(at::kLong);
  const int64_t V = weight.size(0), E = weight.size(1), T = idx.numel();
  c10::hip::HIPGuard guard(weight.device().index());
  void* stream = stream_of(weight);
  Tensor out = at::empty({T, E}, weight.options());
  check(nt_gather_rows(weight.const_data_ptr(), V, E * static_cast<int64_t>(weight.element_size()),
                       idx.const_data_ptr<int64_t>(), out.data_ptr(), T, counter_ptr(counter, weight), stream));
  mirror_counter(counter, mirror, stream);
  return out;
}

// _nn_functional_embedding_bag (nested/nested.py:43-118): the bags are the
// constituents, `offsets` the nested tensor's device offsets.  mode: 0 sum, 1 mean, 2 max.
Tensor embedding_bag_packed(const Tensor& weight_in, const Tensor& indices, const Tensor& offsets, int64_t mode,
                            const c10::optional<Tensor>& counter, const c10::optional<Tensor>& mirror) {
  require_device(indices, "embedding_bag");
  TORCH_CHECK(weight_in.dim() == 2 && weight_in.device() == indices.device(),
              "embedding_bag: weight must be 2-D on the device of the indices");
  TORCH_CHECK(offsets.scalar_type() == at::kLong && offsets.numel() >= 1 && offsets.device() == indices.device() &&
                  offsets.is_contiguous(),
              "embedding_bag: offsets must be a contiguous int64 tensor on the device of the indices");
  const Tensor weight = weight_in.contiguous();
  const Tensor idx = indices.scalar_type() == at::kLong ? indices.contiguous() : indices.to(at::kLong);
  const int64_t V = weight.size(0), E = weight.size(1), B = offsets.numel() - 1;
  c10::hip::HIPGuard guard(weight.device().index());
  void* stream = stream_of(weight);
  Tensor out = at::empty({B, E}, weight.options());
  check(nt_embedding_bag(weight.const_data_ptr(), E, V, idx.const_data_ptr<int64_t>(), idx.numel(),
                         offsets.const_data_ptr<int64_t>(), out.data_ptr(), B, E, static_cast<int>(mode),
                         dtype_code(weight.scalar_type()), counter_ptr(counter, weight), stream));
  mirror_counter(counter, mirror, stream);
  return out;
}

// NestedTensor.to_packed_sequence (nested/nested.py:484-488) without the unbind:
// the order of torch.nn.utils.rnn.pack_sequence(..., enforce_sorted=False).
// lengths: host int64 [B] (all > 0); row_offsets: device token offsets [B + 1];
// buffer viewed as [T, row_elems].  The three small index arrays are derived here
// from the lengths (a sort of B numbers) and reach the device in one copy
// from pinned memory; the row order is then built on the device
// (nt_packed_sequence_index) and the rows moved by one gather.  Returns (data
// [T, row_elems], batch_sizes (host), sorted_indices, unsorted_indices (device)).
std::tuple<Tensor, Tensor, Tensor, Tensor> packed_sequence_lowered(const Tensor& buffer, const Tensor& lengths,
                                                                   const Tensor& row_offsets, int64_t row_elems) {
  require_device(buffer, "to_packed_sequence");
  TORCH_CHECK(lengths.device().is_cpu() && lengths.scalar_type() == at::kLong && lengths.dim() == 1 &&
                  lengths.is_contiguous(),
              "to_packed_sequence: lengths must be a contiguous host int64 vector");
  const int64_t B = lengths.numel();
  TORCH_CHECK(B > 0 && row_offsets.numel() == B + 1 && row_offsets.scalar_type() == at::kLong &&
                  row_offsets.device() == buffer.device() && row_offsets.is_contiguous(),
              "to_packed_sequence: row offsets must be a contiguous int64 [B + 1] tensor on the buffer's device");
  const int64_t* len = lengths.const_data_ptr<int64_t>();
  int64_t T = 0, Lmax = 0;
  for (int64_t b = 0; b < B; ++b) {
    TORCH_CHECK(len[b] > 0, "Length of all samples has to be greater than 0, but found an element in "
                            "'lengths' that is <= 0");
    T += len[b];
    Lmax = std::max(Lmax, len[b]);
  }
  TORCH_CHECK(buffer.numel() == T * row_elems, "to_packed_sequence: buffer does not hold ", T, " rows of ", row_elems);
  // decreasing length, ties as torch.sort leaves them: the same call that
  // torch.nn.utils.rnn.pack_padded_sequence(enforce_sorted=False) makes, so the
  // permutation is the reference's also where lengths repeat
  const Tensor order_t = std::get<1>(lengths.sort(/*dim=*/-1, /*descending=*/true)).contiguous();
  const int64_t* order = order_t.const_data_ptr<int64_t>();
  Tensor batch_sizes = at::empty({Lmax}, at::kLong);
  int64_t* bs = batch_sizes.data_ptr<int64_t>();
  const int64_t n = 2 * B + Lmax;
  Tensor host = at::empty({n}, at::TensorOptions().dtype(at::kLong).pinned_memory(true));
  int64_t* rank = host.data_ptr<int64_t>();
  int64_t* sorted = rank + B;
  int64_t* starts = sorted + B;
  for (int64_t r = 0; r < B; ++r) {
    sorted[r] = order[r];
    rank[order[r]] = r;
  }
  // batch_sizes[t] = number of sequences longer than t: walk the sorted lengths from the short end
  int64_t alive = B, acc = 0;
  for (int64_t t = 0; t < Lmax; ++t) {
    while (alive > 0 && len[order[alive - 1]] <= t) --alive;
    bs[t] = alive;
    starts[t] = acc;
    acc += alive;
  }
  c10::hip::HIPGuard guard(buffer.device().index());
  void* stream = stream_of(buffer);
  Tensor meta = at::empty({n}, buffer.options().dtype(at::kLong));
  meta.copy_(host, /*non_blocking=*/true);
  Tensor rank_dev = meta.narrow(0, 0, B), sorted_dev = meta.narrow(0, B, B), starts_dev = meta.narrow(0, 2 * B, Lmax);
  Tensor index = at::empty({T}, buffer.options().dtype(at::kLong));
  Tensor data = at::empty({T, row_elems}, buffer.options());
  check(nt_packed_sequence_index(row_offsets.const_data_ptr<int64_t>(), rank_dev.const_data_ptr<int64_t>(),
                                 starts_dev.const_data_ptr<int64_t>(), B, T, index.data_ptr<int64_t>(), stream));
  check(nt_gather_rows(buffer.const_data_ptr(), T, row_elems * static_cast<int64_t>(buffer.element_size()),
                       index.const_data_ptr<int64_t>(), data.data_ptr(), T, nullptr, stream));
  return std::make_tuple(data, batch_sizes, sorted_dev, rank_dev);
}

// One projection of the packed rows x [T, K] with rows [r0, r0 + n) of W and of the bias.
Tensor project_rows(const Tensor& x, const Tensor& W, const Tensor& bias, int64_t r0, int64_t n, void* stream) {
  const int64_t T = x.size(0), K = x.size(1);
  Tensor out = at::empty({T, n}, x.options());
  if (T == 0) return out;
  const char* w = static_cast<const char*>(W.const_data_ptr()) + r0 * K * static_cast<int64_t>(W.element_size());
  const char* b = bias.defined() ? static_cast<const char*>(bias.const_data_ptr()) + r0 * static_cast<int64_t>(bias.element_size())
                                 : nullptr;
  check(nt_linear_act(x.const_data_ptr(), x.stride(0), w, b, out.data_ptr(), n, T, n, K, 0, dtype_code(x.scalar_type()),
                      stream));
  return out;
}

void check_mha_operands(const Tensor& xq, const Tensor& xk, const Tensor& xv, int64_t E, const Tensor& W,
                        const Tensor& b_in, const Tensor& Wo, const Tensor& b_out) {
  const at::ScalarType st = xq.scalar_type();
  for (const Tensor* t : {&xq, &xk, &xv}) {
    TORCH_CHECK(t->dim() == 2 && t->size(1) == E && t->stride(1) == 1 && t->scalar_type() == st &&
                    t->device() == xq.device(),
                "mha: query, key and value must be [tokens, num_heads * head_dim] views of one dtype and device");
  }
  TORCH_CHECK(W.dim() == 2 && W.size(0) == 3 * E && W.size(1) == E,
              "in_proj_weight must have shape [3 * embed_dim, embed_dim].");
  TORCH_CHECK(W.scalar_type() == st && Wo.scalar_type() == st && (!b_in.defined() || b_in.scalar_type() == st) &&
                  (!b_out.defined() || b_out.scalar_type() == st),
              "linear: input, weight and bias must have the same dtype");
  TORCH_CHECK(Wo.dim() == 2 && Wo.size(1) == E, "linear: weight of shape ", Wo.sizes(),
              " does not match input feature size ", E);
  check_mha_weights(xq, E, W, b_in, Wo, b_out);
}

// Attention between different nested tensors (or with an embedding size the fused
// projection does not tile), f16 / bf16, head_dim 32 / 64 / 128 (min_mha,
// mha.cpp:42-65): three projections, the value one written transposed, the
// attention kernel with one key sequence per query sequence, output projection.
Tensor mha_cross_packed(const Tensor& xq, const Tensor& xk, const Tensor& xv, const Tensor& schedule, int64_t num_heads,
                        int64_t head_dim, const Tensor& in_proj_weight, const c10::optional<Tensor>& in_proj_bias,
                        double scaling, const Tensor& out_proj_weight, const c10::optional<Tensor>& out_proj_bias) {
  require_device(xq, "multi-head attention");
  const int64_t E = num_heads * head_dim;
  const Tensor W = in_proj_weight.contiguous(), Wo = out_proj_weight.contiguous();
  Tensor b_in, b_out;
  if (in_proj_bias.has_value() && in_proj_bias->defined()) b_in = in_proj_bias->contiguous();
  if (out_proj_bias.has_value() && out_proj_bias->defined()) b_out = out_proj_bias->contiguous();
  check_mha_operands(xq, xk, xv, E, W, b_in, Wo, b_out);
  check_attention_schedule(schedule, xq);
  const int64_t Tq = xq.size(0), Tk = xk.size(0), N = Wo.size(0);
  TORCH_CHECK(xv.size(0) == Tk, "key and value must have the same nested size.");
  c10::hip::HIPGuard guard(xq.device().index());
  void* stream = stream_of(xq);
  const int dt = dtype_code(xq.scalar_type());
  Tensor out = at::empty({Tq, N}, xq.options());
  if (Tq == 0) return out;
  Tensor q = project_rows(xq, W, b_in, 0, E, stream);
  const int64_t ldvt = (Tk + 72 + 63) / 64 * 64;
  Tensor vt = at::empty({E, ldvt}, xq.options());
  const int64_t es = static_cast<int64_t>(xq.element_size());
  Tensor k;
  if (xk.const_data_ptr() == xv.const_data_ptr() && xk.stride(0) == xv.stride(0) && E % 128 == 0) {
    // key and value are one buffer (the `memory` of a decoder layer): both
    // projections in one launch, the buffer read once
    k = at::empty({Tk, E}, xq.options());
    if (Tk > 0) {
      check(nt_linear_kv(xk.const_data_ptr(), xk.stride(0), static_cast<const char*>(W.const_data_ptr()) + E * E * es,
                         b_in.defined() ? static_cast<const char*>(b_in.const_data_ptr()) + E * es : nullptr,
                         k.data_ptr(), E, vt.data_ptr(), ldvt, Tk, E, E, dt, stream));
    }
  } else {
    k = project_rows(xk, W, b_in, E, E, stream);
    check(nt_linear_transposed(xv.const_data_ptr(), xv.stride(0),
                               static_cast<const char*>(W.const_data_ptr()) + 2 * E * E * es,
                               b_in.defined() ? static_cast<const char*>(b_in.const_data_ptr()) + 2 * E * es : nullptr,
                               vt.data_ptr(), ldvt, Tk, E, E, dt, stream));
  }
  Tensor attn = at::empty({Tq, E}, xq.options());
  launch_attention_vt(q.const_data_ptr(), E, k.const_data_ptr(), E, vt, ldvt, attn, E, schedule, num_heads, head_dim, Tk,
                      scaling, dt, stream);
  check(nt_linear_act(attn.const_data_ptr(), E, Wo.const_data_ptr(), b_out.defined() ? b_out.const_data_ptr() : nullptr,
                      out.data_ptr(), N, Tq, N, E, 0, dt, stream));
  return out;
}

// The same layer with V row-major: fp32 with head_dim 32 / 64 / 128 from the work
// list (`schedule`), anything else over the device row offsets on a padded grid.
// `same`: query, key and value are one nested tensor (one [T, 3E] projection).
Tensor mha_rowmajor_packed(const Tensor& xq, const Tensor& xk, const Tensor& xv, bool same,
                           const c10::optional<Tensor>& schedule, const Tensor& q_offsets, const Tensor& kv_offsets,
                           int64_t max_q, int64_t num_heads, int64_t head_dim, const Tensor& in_proj_weight,
                           const c10::optional<Tensor>& in_proj_bias, double scaling, const Tensor& out_proj_weight,
                           const c10::optional<Tensor>& out_proj_bias) {
  require_device(xq, "multi-head attention");
  const int64_t E = num_heads * head_dim;
  const Tensor W = in_proj_weight.contiguous(), Wo = out_proj_weight.contiguous();
  Tensor b_in, b_out;
  if (in_proj_bias.has_value() && in_proj_bias->defined()) b_in = in_proj_bias->contiguous();
  if (out_proj_bias.has_value() && out_proj_bias->defined()) b_out = out_proj_bias->contiguous();
  check_mha_operands(xq, xk, xv, E, W, b_in, Wo, b_out);
  const int64_t Tq = xq.size(0), N = Wo.size(0), B = q_offsets.numel() - 1;
  TORCH_CHECK(q_offsets.scalar_type() == at::kLong && kv_offsets.scalar_type() == at::kLong &&
                  kv_offsets.numel() == q_offsets.numel() && q_offsets.device() == xq.device() &&
                  kv_offsets.device() == xq.device(),
              "mha: row offsets must be int64 [B + 1] tensors on the input's device");
  c10::hip::HIPGuard guard(xq.device().index());
  void* stream = stream_of(xq);
  const int dt = dtype_code(xq.scalar_type());
  Tensor out = at::empty({Tq, N}, xq.options());
  if (Tq == 0) return out;
  Tensor q, k, v;
  int64_t qc = 0, kc = 0, vc = 0, ld = E;
  if (same) {
    q = project_rows(xq, W, b_in, 0, 3 * E, stream);     // [T, 3E]
    k = q;
    v = q;
    kc = E;
    vc = 2 * E;
    ld = 3 * E;
  } else {
    q = project_rows(xq, W, b_in, 0, E, stream);
    k = project_rows(xk, W, b_in, E, E, stream);
    v = project_rows(xv, W, b_in, 2 * E, E, stream);
  }
  const int64_t es = static_cast<int64_t>(xq.element_size());
  const char* qp = static_cast<const char*>(q.const_data_ptr()) + qc * es;
  const char* kp = static_cast<const char*>(k.const_data_ptr()) + kc * es;
  const char* vp = static_cast<const char*>(v.const_data_ptr()) + vc * es;
  Tensor attn = at::empty({Tq, E}, xq.options());
  const bool listed = schedule.has_value() && schedule->defined() && xq.scalar_type() == at::kFloat &&
                      (head_dim == 32 || head_dim == 64 || head_dim == 128);
  if (listed) {
    TORCH_CHECK(schedule->scalar_type() == at::kInt && schedule->dim() == 2 && schedule->size(1) == 8 &&
                    schedule->is_contiguous() && schedule->device() == xq.device(),
                "mha: schedule must be a contiguous int32 [n_work, 8] tensor on the input's device");
    check(nt_varlen_attention_scheduled(qp, ld, kp, ld, vp, ld, attn.data_ptr(), E, schedule->const_data_ptr<int32_t>(),
                                        schedule->size(0), num_heads, head_dim, static_cast<float>(scaling), dt, stream));
  } else {
    check(nt_varlen_attention(qp, ld, kp, ld, vp, ld, attn.data_ptr(), E, q_offsets.const_data_ptr<int64_t>(),
                              kv_offsets.const_data_ptr<int64_t>(), B, num_heads, head_dim, max_q,
                              static_cast<float>(scaling), dt, stream));
  }
  check(nt_linear_act(attn.const_data_ptr(), E, Wo.const_data_ptr(), b_out.defined() ? b_out.const_data_ptr() : nullptr,
                      out.data_ptr(), N, Tq, N, E, 0, dt, stream));
  return out;
}

}  // namespace

// Schemas.  The first block are the reference's operators, names and argument
// order as in nestedtensor/csrc/masking.cpp:652-675, csrc/mha.cpp:72,
// csrc/cuda/mha.cpp:110-111 and csrc/py_init.cpp:132-216; a `Tensor nt` argument
// is the Python NestedTensor wrapper, lowered by its __torch_function__.  The
// second block are the lowered operators implemented in this file.
TORCH_LIBRARY(nestedtensor, m) {
  m.def("to_padded_tensor(Tensor nt, float padding) -> Tensor");
  m.def("to_tensor_mask(Tensor nt, int? mask_dim) -> (Tensor, Tensor)");
  m.def("to_mask(Tensor nt, int? mask_dim) -> Tensor");
  m.def("nt_from_tensor_mask(Tensor tensor, Tensor mask, int nested_dim) -> (Tensor, Tensor)");
  m.def("get_max_size(Tensor nt) -> int[]");
  m.def("pad_nt(Tensor nt, int[] shape) -> (Tensor, Tensor)");
  m.def("merge_tensor_mask(Tensor tensor, Tensor mask, int? mask_dim=None) -> (Tensor, Tensor)");
  m.def("min_mha(int num_heads, int head_dim, float dropout_p, bool training, Tensor query, "
        "Tensor key, Tensor value, Tensor in_proje_weight, Tensor? in_proj_bias, float scaling, "
        "Tensor out_proj_weight, Tensor out_proj_bias) -> Tensor");
  m.def("bt_min_mha(int num_heads, int head_dim, float dropout_p, bool training, Tensor query, "
        "Tensor key, Tensor value, Tensor attr_kernel, Tensor attr_bias, float scaling, "
        "Tensor out_proj_weight, Tensor out_proj_bias) -> Tensor");
  m.def("is_nested_tensor_impl(Tensor tensor) -> bool");
  m.def("nested_dim(Tensor tensor) -> int");
  m.def("to_nested_tensor(Tensor tensor, int? dim) -> Tensor");
  m.def("sizes(Tensor tensor) -> int?[]");
  m.def("len(Tensor self) -> int");
  m.def("get_dim(Tensor self) -> int");
  m.def("get_numel(Tensor self) -> int");
  m.def("get_is_contiguous(Tensor self, MemoryFormat memory_format) -> bool");
  m.def("make_contiguous(Tensor self) -> Tensor");
  m.def("to_tensor_list(Tensor tensor) -> Tensor[]");
  m.def("transpose_nhwc_nchw(Tensor self) -> Tensor");
  m.def("transpose_nchw_nhwc(Tensor self) -> Tensor");
  m.def("to_sparse_csr(Tensor tensor) -> Tensor");
  // no counterpart among the reference's ops (it builds the mask in Python,
  // nestedtensor/nested/masking.py:12-14); same lowered return convention as
  // nt_from_tensor_mask: (packed buffer, sizes[B, D]), sizes 0-d for an empty result
  m.def("nt_from_padded_tensor(Tensor tensor, float padding, int nested_dim) -> (Tensor, Tensor)");

  m.def("offsets_from_sizes(Tensor sizes) -> Tensor");
  m.def("pack_device(Tensor[] tensors) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def("add_padding(Tensor buffer, Tensor sizes, Tensor offsets, int[] padded_sizes, int n_ragged, "
        "float padding) -> Tensor");
  m.def("add_padding_mask(Tensor buffer, Tensor sizes, Tensor offsets, int[] padded_sizes, int n_ragged, "
        "float padding) -> (Tensor, Tensor)");
  m.def("remove_padding(Tensor padded, Tensor sizes, Tensor offsets, int total_numel, int n_ragged) -> Tensor");
  m.def("build_mask(Tensor sizes, int[] extents) -> Tensor");
  m.def("from_tensor_mask_lowered(Tensor tensor, Tensor mask, int nested_dim) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def("from_padded_value_lowered(Tensor tensor, float padding, int nested_dim) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def("embedding_packed(Tensor weight, Tensor indices, Tensor? counter, Tensor? mirror) -> Tensor");
  m.def("embedding_bag_packed(Tensor weight, Tensor indices, Tensor offsets, int mode, Tensor? counter, "
        "Tensor? mirror) -> Tensor");
  m.def("packed_sequence_lowered(Tensor buffer, Tensor lengths, Tensor row_offsets, int row_elems) -> "
        "(Tensor, Tensor, Tensor, Tensor)");
  m.def("layer_norm_packed(Tensor x, Tensor? residual, Tensor? weight, Tensor? bias, int n, float eps) -> Tensor");
  m.def("binary_packed(Tensor a, Tensor? b, float scale, int period, bool mul) -> Tensor");
  m.def("softmax_rows(Tensor x, Tensor offsets, Tensor row_offsets, int total_rows, bool log) -> Tensor");
  m.def("activation_packed(Tensor x, int act) -> Tensor");
  m.def("linear_packed(Tensor x, Tensor weight, Tensor? bias, int act) -> Tensor");
  m.def("attention_plan(Tensor q_lens, Tensor k_lens, int num_heads, int head_dim, Device device) -> Tensor");
  m.def("mha_self_packed(Tensor x, Tensor schedule, int num_heads, int head_dim, Tensor in_proj_weight, "
        "Tensor? in_proj_bias, float scaling, Tensor out_proj_weight, Tensor? out_proj_bias) -> Tensor");
  m.def("mha_cross_packed(Tensor xq, Tensor xk, Tensor xv, Tensor schedule, int num_heads, int head_dim, "
        "Tensor in_proj_weight, Tensor? in_proj_bias, float scaling, Tensor out_proj_weight, "
        "Tensor? out_proj_bias) -> Tensor");
  m.def("mha_rowmajor_packed(Tensor xq, Tensor xk, Tensor xv, bool same, Tensor? schedule, Tensor q_offsets, "
        "Tensor kv_offsets, int max_q, int num_heads, int head_dim, Tensor in_proj_weight, Tensor? in_proj_bias, "
        "float scaling, Tensor out_proj_weight, Tensor? out_proj_bias) -> Tensor");
}

// "CUDA" is the dispatch key of the HIP device on PyTorch-ROCm.
TORCH_LIBRARY_IMPL(nestedtensor, CUDA, m) {
  m.impl("offsets_from_sizes", offsets_from_sizes);
  m.impl("pack_device", pack_device);
  m.impl("add_padding", add_padding);
  m.impl("add_padding_mask", add_padding_mask);
  m.impl("remove_padding", remove_padding);
  m.impl("build_mask", build_mask);
  m.impl("from_padded_value_lowered", from_padded_value_lowered);
  m.impl("nt_from_padded_tensor", nt_from_padded_tensor_op);
  m.impl("linear_packed", linear_packed);
  m.impl("mha_self_packed", mha_self_packed);
  m.impl("mha_cross_packed", mha_cross_packed);
  m.impl("mha_rowmajor_packed", mha_rowmajor_packed);
  m.impl("layer_norm_packed", layer_norm_packed);
  m.impl("binary_packed", binary_packed);
  m.impl("softmax_rows", softmax_rows);
  m.impl("activation_packed", activation_packed);
  m.impl("embedding_packed", embedding_packed);
  m.impl("embedding_bag_packed", embedding_bag_packed);
  m.impl("packed_sequence_lowered", packed_sequence_lowered);
}

// Operators on plain tensors of any device: merge_tensor_mask is host logic over
// torch reductions; nt_from_tensor_mask answers the trivial masks (empty, one
// element) for any device and raises for host tensors otherwise.
TORCH_LIBRARY_IMPL(nestedtensor, CompositeExplicitAutograd, m) {
  m.impl("merge_tensor_mask", merge_tensor_mask);
  m.impl("attention_plan", attention_plan);   // host lengths in, device plan out
  m.impl("nt_from_tensor_mask", nt_from_tensor_mask_op);
  m.impl("from_tensor_mask_lowered", from_tensor_mask_lowered);
}
