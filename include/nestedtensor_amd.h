/*
 * nestedtensor_amd -- C ABI of the MI355X (gfx950) ragged hot path.
 *
 * The reference (pytorch/nestedtensor) has no C ABI: its device code is reached
 * through C++ templates `*_kernelLauncher<T>(ptrs, int metadata..., cudaStream_t)`
 * (nestedtensor/csrc/cuda/padding.h:12-45, cuda/attention.h:25-51) called from
 * the operator layer (nestedtensor/csrc/masking.cpp, csrc/cuda/mha.cpp).  The
 * entry points below are the plain-C surface those call sites would bind
 * instead.  Each one cites the reference interface it replaces.
 *
 * Conventions
 *  - all pointers are device pointers unless a parameter is named `*_host`;
 *  - a nested tensor of nested_dim 1 is (packed buffer, sizes[B, D] int64,
 *    offsets[B + 1] int64); offsets are ELEMENT offsets into the packed buffer;
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *  - functions enqueue work on `stream` and return; they never allocate device
 *    memory, never synchronise and never throw.  Scratch memory, where needed,
 *    is passed in as `workspace` with the size the matching `*_workspace_bytes`
 *    function reports;
 *  - return value: NT_OK or an NT_ERR_* code; nt_last_error() gives the text
 *    for the calling thread.
 */
#ifndef NESTEDTENSOR_AMD_H
#define NESTEDTENSOR_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NT_ABI_VERSION 1

enum {
  NT_OK = 0,
  NT_ERR_INVALID_ARGUMENT = 1,
  NT_ERR_UNSUPPORTED = 2,
  NT_ERR_HIP = 3,
  NT_ERR_WORKSPACE = 4
};

/* element types: the first three are the types of the attention path */
enum {
  NT_F32 = 0, NT_F16 = 1, NT_BF16 = 2,
  NT_F64 = 3, NT_I8 = 4, NT_U8 = 5, NT_I16 = 6, NT_I32 = 7, NT_I64 = 8
};

/* No reference counterpart: ABI handshake and error text. */
int nt_abi_version(void);
const char* nt_last_error(void);

/* ---- metadata: device prefix scan ------------------------------------- */

/* offsets[0] = 0, offsets[b + 1] = offsets[b] + prod_k sizes[b, k] for b < B.
 * Replaces the host loop batch_offsets_from_efficient_size
 * (nestedtensor/csrc/masking.cpp:110-125) and the unused int32 Blelloch scan
 * exclusiveScan_kernelLauncher (nestedtensor/csrc/cuda/cuda_kernels.cu:271-517).
 * D == 0 gives prod = 1 (0-d constituents). */
size_t nt_offsets_workspace_bytes(int64_t B);
int nt_offsets_from_sizes(const int64_t* sizes, int64_t B, int64_t D,
                          int64_t* offsets, void* workspace, size_t workspace_bytes,
                          void* stream);

/* nt_offsets_from_sizes without a workspace argument and without any allocation.
 * No counterpart in the reference: it exists for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  The tile sums of the scan live in a 256 KiB array in
 * the library's own device data segment (one copy per GPU, held until the
 * process ends), which bounds B at nt_offsets_noalloc_max_count() = 67 108 864;
 * larger B returns NT_ERR_UNSUPPORTED.  Results are bit-identical to
 * nt_offsets_from_sizes.  All calls on one GPU share that array: calls that
 * overlap on one GPU (different streams or threads) race on it; calls on one
 * stream are ordered.  The first call on a device resolves the array's address
 * (hipGetSymbolAddress) and should be made outside stream capture. */
int64_t nt_offsets_noalloc_max_count(void);
int nt_offsets_from_sizes_noalloc(const int64_t* sizes, int64_t B, int64_t D, int64_t* offsets,
                                  void* stream);

/* ---- packed <-> padded ------------------------------------------------- */

/* padded[b, i_1..i_D] = inside(sizes[b]) ? packed[offsets[b] + lin(i)] : pad
 * with padded of shape [B, padded_sizes_host[0..D)] (the batch maxima).
 * `n_ragged` (1..3) leading constituent dims may differ between constituents;
 * the trailing D - n_ragged dims must equal padded_sizes_host[k] for every b.
 * `elem_bytes` in {1, 2, 4, 8}; `pad_bits` is the padding value already
 * converted to the element type, in the low elem_bytes bytes.
 * Replaces add_padding_kernelLauncher<T> (nestedtensor/csrc/cuda/padding.h:12-23,
 * kernels padding.cu:10-193) as called by to_padded_tensor
 * (nestedtensor/csrc/masking.cpp:558-625). */
int nt_add_padding(const void* packed, void* padded, const int64_t* offsets,
                   const int64_t* sizes, int64_t B, int64_t D, int64_t n_ragged,
                   const int64_t* padded_sizes_host, int elem_bytes, uint64_t pad_bits,
                   void* stream);

/* nt_add_padding plus the mask of the same shape in one launch: mask[b, i...] = 1
 * where padded[b, i...] holds data and 0 where it holds padding, one byte per
 * element of padded (a bool tensor).  Replaces add_padding_mask_kernelLauncher
 * (nestedtensor/csrc/cuda/padding.cu:217-262, called from to_tensor_mask,
 * nestedtensor/csrc/masking.cpp:251-296), which covers 3-d nested tensors with a
 * [B, L] mask only; this one covers the case where the mask keeps every dim of
 * the data (no trailing regular dim to collapse, e.g. ragged images), the only
 * case where the mask is large enough to matter.  Arguments as nt_add_padding. */
int nt_add_padding_mask(const void* packed, void* padded, uint8_t* mask, const int64_t* offsets,
                        const int64_t* sizes, int64_t B, int64_t D, int64_t n_ragged,
                        const int64_t* padded_sizes_host, int elem_bytes, uint64_t pad_bits,
                        void* stream);

/* packed[offsets[b] + lin(i)] = padded[b, i] for i inside sizes[b]: the
 * length-based inverse of nt_add_padding.  Replaces
 * remove_padding_kernelLauncher<T> (nestedtensor/csrc/cuda/padding.h:36-45,
 * kernels padding.cu:286-394) as called by from_padded_tensor
 * (nestedtensor/csrc/masking.cpp:459-509). */
int nt_remove_padding(const void* padded, void* packed, const int64_t* offsets,
                      const int64_t* sizes, int64_t B, int64_t D, int64_t n_ragged,
                      const int64_t* padded_sizes_host, int elem_bytes, void* stream);

/* mask[b, i_1..i_K] = all_k(i_k < sizes[b, k]) as bytes 0/1, shape
 * [B, mask_sizes_host[0..K)], K <= D, K in 1..3.  Together with nt_add_padding
 * (pad 0) this is to_tensor_mask; alone it is to_mask.  Replaces
 * add_padding_mask_kernelLauncher<T> (nestedtensor/csrc/cuda/padding.h:25-34,
 * kernel padding.cu:217-262: one thread per batch entry) and the host fill
 * loops of to_mask (nestedtensor/csrc/masking.cpp:436-451, 353-406). */
int nt_build_mask(uint8_t* mask, const int64_t* sizes, int64_t B, int64_t D, int64_t K,
                  const int64_t* mask_sizes_host, void* stream);

/* Gather B contiguous device tensors into one packed buffer:
 * packed[offsets[b] .. offsets[b+1]) = *srcs[b].  `srcs` is a device array of
 * B device pointers.  Replaces the per-constituent copy_ loop of impl::pack
 * (nestedtensor/csrc/storage/Packed.h:75-98). */
int nt_pack(const void* const* srcs, void* packed, const int64_t* offsets, int64_t B,
            int elem_bytes, void* stream);

/* nt_pack for a handful of constituents, without anything on the device before
 * the launch: table_host (host memory) holds sizes[B * D], then offsets[B + 1]
 * (element offsets), then the B source pointers, B * D + 2 B + 1 int64 entries in
 * all, at most nt_pack_table_max_entries().  The table travels in the kernel
 * arguments; if table_dev is not NULL the kernel also leaves a copy of it there
 * (device int64, same layout), which is the device metadata the pad / mask
 * operators take.  Same reference code as nt_pack (impl::pack,
 * nestedtensor/csrc/storage/Packed.h:75-98). */
int64_t nt_pack_table_max_entries(void);
int nt_pack_table(const int64_t* table_host, int64_t B, int64_t D, void* packed, int64_t* table_dev,
                  int elem_bytes, void* stream);

/* A small table of host int64 (a nested size and its offsets, at most
 * nt_pack_table_max_entries() entries) to device memory, carried by the kernel
 * arguments of a one-workgroup launch: ordered on `stream` like any kernel, no
 * staging buffer, no copy engine.  Replaces the metadata upload the reference
 * does with Tensor::to(kCUDA, ..., non_blocking) before its padding kernels
 * (nestedtensor/csrc/masking.cpp:471-472, 578-579). */
int nt_upload_table(const int64_t* table_host, int64_t n, int64_t* table_dev, void* stream);

/* ---- mask -> nested size, compaction ----------------------------------- */

/* Row statistics of a byte mask viewed as [R, M] (nonzero = true):
 * counts[r] = number of true entries in row r (int32); prefix[r] (may be NULL)
 * = 1 iff those are exactly the first counts[r] entries of the row.  One
 * wavefront per row, 16 mask bytes per lane and step, ballot + popcount.  The
 * reference has no device counterpart: it reads every mask element with
 * .item<bool>() on the host (nestedtensor/csrc/masking.cpp:190-201). */
int nt_mask_row_counts(const uint8_t* mask, int64_t R, int64_t M, int32_t* counts,
                       uint8_t* prefix, void* stream);

/* The nested size straight from the row statistics, when the mask is that of a
 * padded tensor.  counts / prefix (device) are the statistics of B constituents
 * of rows_per rows each, the rows of a constituent indexed row-major by the nd
 * row dims `row_dims_host` (host int64, their product is rows_per; nd <=
 * nt_leading_boxes_max_dims()).  boxes (device or device-visible host memory)
 * receives max_dims + 2 int32 per constituent: {ok, w, extent[0 .. max_dims)}:
 * ok = 1 iff every row keeps exactly its first w entries or nothing, and the rows
 * that keep something are those whose index is below extent[k] in every row dim
 * k; the constituent's size is then (extent[0 .. nd), w), as the reference's walk
 * over the mask finds it (nestedtensor/csrc/masking.cpp:203-222).  ok = 0: the
 * caller has to look at the statistics itself.
 * done (may be NULL): a word in device-visible host memory that receives
 * done_value, with system-wide release, once every line of boxes is written, so
 * that a host thread polling it (acquire) can read boxes from host memory without
 * a stream synchronisation.  arrivals: a device word that is zero when the launch
 * starts and is left zero; launches that share it must not overlap.  With done
 * and WITHOUT arrivals (NULL), done is an array of B words and word b receives
 * done_value as soon as line b is written (nothing is counted, nobody waits for
 * the last line: the host polls the B words). */
int64_t nt_leading_boxes_max_dims(void);
int nt_leading_boxes(const int32_t* counts, const uint8_t* prefix, int64_t B, int64_t rows_per,
                     const int64_t* row_dims_host, int64_t nd, int32_t* boxes, uint32_t* done,
                     uint32_t done_value, uint32_t* arrivals, void* stream);

/* nt_leading_boxes for a host that polls: lines (device-visible host memory, 8-byte
 * aligned) receives max_dims + 2 uint64 per constituent, entry i of a line =
 * (uint32) entry i of nt_leading_boxes' line in the low half and `stamp` (not 0)
 * in the high half, each written with one 8-byte store.  An entry is valid for the
 * host the moment its high half reads `stamp` (use a stamp the buffer has not held
 * before, e.g. a call counter); no fence and no completion word are involved, so
 * the launch ends without a round trip to host memory. */
int nt_leading_boxes_stamped(const int32_t* counts, const uint8_t* prefix, int64_t B, int64_t rows_per,
                             const int64_t* row_dims_host, int64_t nd, uint64_t* lines, uint32_t stamp,
                             void* stream);

/* The same statistics for the mask `data != padding` of a dense tensor viewed as
 * [R, M] elements of type elem_type, without materialising the mask; the
 * comparison is the one of the element type (NaN != x is true, -0.0 != 0.0 is
 * false).  Replaces `mask = (tensor != padding)` followed by the host walk in
 * nested_tensor_from_padded_tensor (nestedtensor/nested/masking.py:12-14). */
int nt_value_row_counts(const void* data, int elem_type, double padding, int64_t R, int64_t M,
                        int32_t* counts, uint8_t* prefix, void* stream);

/* Compaction of the rows of `data` viewed as [R, M, chunk_bytes]: the kept
 * chunks of row r (mask[r, m] != 0) are written, in order, starting at byte
 * out + row_offsets[r] * chunk_bytes, where row_offsets is the exclusive scan
 * of counts (nt_exclusive_scan_i32).  Replaces the recursive host walk of
 * nt_from_tensor_mask (nestedtensor/csrc/masking.cpp:181-249). */
int nt_compact_rows(const void* data, const uint8_t* mask, const int64_t* row_offsets,
                    int64_t R, int64_t M, int64_t chunk_bytes, void* out, void* stream);

/* out[0] = 0, out[i + 1] = out[i] + in[i] (int32 in, int64 out, n + 1 outputs). */
size_t nt_scan_workspace_bytes(int64_t n);
int nt_exclusive_scan_i32(const int32_t* in, int64_t n, int64_t* out, void* workspace,
                          size_t workspace_bytes, void* stream);

/* ---- nested multi-head attention --------------------------------------- */

/* C[M, N] = A[M, K] * W[N, K]^T + bias[N] (bias may be NULL); row-major, A with
 * row stride lda, C with row stride ldc (elements).  fp32 accumulation.
 * This is the packed projection of the reference: NestedTensor_matmul's
 * single GEMM on buffer.reshape(-1, E) (nestedtensor/csrc/matmul.cpp:13-41)
 * plus the packed bias add (nestedtensor/csrc/BinaryOps.cpp:97-107); call sites
 * nestedtensor/csrc/mha.cpp:42-54,66-67 and csrc/cuda/mha.cpp:57,106. */
int nt_linear(const void* A, int64_t lda, const void* W, const void* bias, void* C,
              int64_t ldc, int64_t M, int64_t N, int64_t K, int dtype, void* stream);

/* nt_linear with an activation applied to A W^T + bias in fp32 before the one
 * rounding: act 0 none, 1 relu, 2 gelu (erf form, torch's default).  The first
 * feed-forward projection of an encoder layer in one launch; the reference has
 * the pieces unfused: the packed matmul (nestedtensor/csrc/matmul.cpp:13-41), the
 * packed bias add (nestedtensor/csrc/BinaryOps.cpp:97-107) and at::gelu / at::relu
 * on the buffer (nestedtensor/csrc/activation.cpp:11-19, 34-46), plus an unwired
 * add_bias_act kernel (nestedtensor/csrc/cuda/cuda_kernels.cu:73-107). */
int nt_linear_act(const void* A, int64_t lda, const void* W, const void* bias, void* C,
                  int64_t ldc, int64_t M, int64_t N, int64_t K, int act, int dtype, void* stream);

/* Self/cross attention on packed projections, one softmax per (sequence, head)
 * over that sequence's own keys only:
 *   out[q_off[b] + i, h*hd + d] = sum_j softmax_j(scale * q_i . k_j) v_j[d]
 * q rows are q[(q_off[b] + i) * ldq + h*hd ...], k/v likewise with kv_off.
 * f16 / bf16 with head_dim 64 and f32 with head_dim 32, 64 or 128 (rows 16-byte
 * aligned) run on the matrix pipe; anything else takes a scalar kernel (one
 * wavefront per query row and head), which is a parity path, not a fast one.
 * Replaces the padded chain of bt_min_mha
 * (nestedtensor/csrc/cuda/mha.cpp:59-105: to_padded_tensor, batched QK^T,
 * softmax_kernel_kernelLauncher of cuda/attention.h:25-33, PV,
 * from_padded_tensor) and the unwired add_QKV_bias_padding /
 * transpose_rm_padding kernels (nestedtensor/csrc/cuda/attention.cu:107-174,
 * 488-538); semantics are those of the per-sequence loop of min_mha
 * (nestedtensor/csrc/mha.cpp:58-65). */
int nt_varlen_attention(const void* q, int64_t ldq, const void* k, int64_t ldk,
                        const void* v, int64_t ldv, void* out, int64_t ldo,
                        const int64_t* q_offsets, const int64_t* kv_offsets, int64_t B,
                        int64_t num_heads, int64_t head_dim, int64_t max_q_len,
                        float scale, int dtype, void* stream);

/* The fused in-projection of self-attention: [Q | K | V] = A * W^T + bias with
 * W [3E, K]; Q and K are written row-major into QK[M, 2E] (row stride ldqk), V is
 * written transposed, Vt[e][m] (row stride ldvt >= M; nt_varlen_attention_vt
 * wants ldvt >= M + 72), which is the layout nt_varlen_attention_vt reads.  Replaces the packed in-projection
 * at::matmul(query, attr_kernel.t()) + attr_bias of bt_min_mha
 * (nestedtensor/csrc/cuda/mha.cpp:57) together with the chunk / reshape /
 * transpose views that follow it (:60-69), and stands where the unwired
 * add_QKV_bias_padding kernel (nestedtensor/csrc/cuda/attention.cu:107-174)
 * was meant to go. */
int nt_linear_qkv(const void* A, int64_t lda, const void* W, const void* bias, void* QK,
                  int64_t ldqk, void* Vt, int64_t ldvt, int64_t M, int64_t E, int64_t K,
                  int dtype, void* stream);

/* The key and value projections of cross-attention in one launch, for keys and
 * values that are the same tensor (the usual `memory` of a decoder layer):
 * [Kp | V] = A * W^T + bias with W [2E, K] (rows [E, 3E) of an in-projection
 * weight); Kp is written row-major into Kout[M, E] (row stride ldk), V transposed
 * into Vt[e][m] (row stride ldvt >= M; nt_varlen_attention_vt wants >= M + 72).
 * E must be a multiple of 128.  Replaces the `k` and `v` matmuls and bias adds of
 * min_mha (nestedtensor/csrc/mha.cpp:45-54) when key and value are one buffer: A
 * is read once instead of twice. */
int nt_linear_kv(const void* A, int64_t lda, const void* W, const void* bias, void* Kout, int64_t ldk,
                 void* Vt, int64_t ldvt, int64_t M, int64_t E, int64_t K, int dtype, void* stream);

/* Ct[n][m] = (A[M, K] * W[N, K]^T + bias[N])[m][n]: nt_linear with the result
 * written transposed (row stride ldct >= M).  The value projection of
 * cross-attention (nestedtensor/csrc/mha.cpp:48-54, the `v` matmul and bias add)
 * in the layout nt_varlen_attention_vt reads; it wants ldct >= M + 72. */
int nt_linear_transposed(const void* A, int64_t lda, const void* W, const void* bias, void* Ct,
                         int64_t ldct, int64_t M, int64_t N, int64_t K, int dtype, void* stream);

/* Attention on projections in the layout the GEMMs above write: Q rows at
 * q[token * ldq + h*hd], K rows at k[token * ldk + h*hd], V transposed in
 * Vt[(h*hd + d) * ldvt + token]; head_dim hd is 32, 64 or 128, dtype f16 or bf16.  For
 * self-attention on the output of nt_linear_qkv, q = QK, k = QK + E, ldq = ldk =
 * ldqk.  `schedule` is a device array of n_work int32[8] work items {first query
 * token, query length, first query row of the tile (multiple of 128), 0, first
 * key token, key length, 0, 0}: one per 128-query tile of every sequence
 * (for cross-attention: of every query sequence, with the key sequence it
 * attends to), in the order they should start (longest key sequences first); a
 * workgroup is launched per (item, head), so no padded tile is ever issued.  The
 * rows of Vt must be readable up to 72 elements past the last key token
 * (ldvt >= total_kv_tokens + 72); what is stored there is ignored.  An item
 * with key length 0 writes zeros to its query rows, one with query length 0 does
 * nothing; first tokens and lengths are int32 (at most 2^31 - 1 tokens in total)
 * and must describe rows inside the buffers, the kernel cannot check them.
 * Output and semantics as nt_varlen_attention. */
int nt_varlen_attention_vt(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* vt,
                           int64_t ldvt, void* out, int64_t ldo, const int32_t* schedule,
                           int64_t n_work, int64_t num_heads, int64_t head_dim,
                           int64_t total_kv_tokens, float scale, int dtype, void* stream);

/* The same attention from a PLAN instead of a work list (head_dim 64, f16 / bf16):
 * persistent workgroups, one per compute unit, twelve wavefronts each, that bring a
 * sequence's K and V^T tiles into LDS with direct global -> LDS loads, 256 keys per
 * step, and give every wavefront one block of 32 query rows: K / V^T are read once
 * per 384 query rows, there is one barrier per 256 keys, and short sequences share
 * a workgroup.  An alternative to nt_varlen_attention_vt with the same results to
 * rounding; on the attention benchmarks of this library it is the slower of the two
 * (the host layer uses it only on request).  Replaces the same reference chain as
 * nt_varlen_attention_vt (nestedtensor/csrc/cuda/mha.cpp:59-105, the masked softmax
 * of nestedtensor/csrc/cuda/attention.cu:182-482), with the semantics of the
 * per-sequence loop of min_mha (nestedtensor/csrc/mha.cpp:58-65).
 *
 * nt_attention_plan builds the plan on the HOST from the query and key lengths
 * of the B sequences (host int64 arrays; a sequence with queries must have
 * keys) for `num_heads` heads and `n_workgroups` workgroups (<= 0: the compute
 * units of the current device).  It returns the number of int32 the plan holds,
 * or minus an NT_ERR_* code, and writes the plan when `plan` is not NULL and
 * `capacity` (in int32) suffices: call it once with NULL to size the buffer.
 * plan[0] is the number of workgroups to launch.  The caller copies the plan to
 * device memory; it depends on the lengths, the head count and the workgroup
 * count only, so it can be kept for as long as the nested size lives. */
int64_t nt_attention_plan(const int64_t* q_lens, const int64_t* k_lens, int64_t B, int64_t num_heads,
                          int64_t head_dim, int64_t n_workgroups, int32_t* plan, int64_t capacity);

/* Operands as nt_varlen_attention_vt (Q, K row-major with 16-byte aligned K rows,
 * V transposed with ldvt >= total_kv_tokens + 72); `plan` is the DEVICE copy of
 * what nt_attention_plan built for these sequences and head count, n_workgroups
 * its plan[0].  The kernel cannot check the plan against the buffers. */
int nt_varlen_attention_planned(const void* q, int64_t ldq, const void* k, int64_t ldk, const void* vt,
                                int64_t ldvt, void* out, int64_t ldo, const int32_t* plan,
                                int64_t n_workgroups, int64_t num_heads, int64_t head_dim,
                                int64_t total_kv_tokens, float scale, int dtype, void* stream);

/* nt_varlen_attention (V row-major) driven by the work list of
 * nt_varlen_attention_vt instead of a padded grid: one workgroup per (item,
 * head), so only query tiles that exist are launched and the long sequences
 * start first.  f32 with head_dim 32, 64 or 128; every row 16-byte aligned
 * (pointers and row strides).  The reference runs f32 bt_min_mha through the same
 * padded chain as the other types (nestedtensor/csrc/cuda/mha.cpp:59-105). */
int nt_varlen_attention_scheduled(const void* q, int64_t ldq, const void* k, int64_t ldk,
                                  const void* v, int64_t ldv, void* out, int64_t ldo,
                                  const int32_t* schedule, int64_t n_work, int64_t num_heads,
                                  int64_t head_dim, float scale, int dtype, void* stream);

/* ---- row-wise ops on the packed buffer (the steps either side of attention
 *      in an encoder layer) ------------------------------------------------ */

/* out[r, :] = layer_norm(x[r, :] (+ residual[r, :])) * gamma + beta over the last
 * dim of the packed [rows, n] view of a nested tensor whose last dim is regular;
 * residual, gamma and beta may be NULL.  Mean and variance are two-pass fp32 sums
 * (biased variance), rstd = 1 / sqrt(var + eps); with a residual the sum is first
 * rounded to the storage type, as the reference's separate add does.  Replaces
 * NestedTensor_layer_norm (nestedtensor/csrc/functions.cpp:65-112), whose device
 * fast path is nestedtensor/csrc/cuda/layernorm.cpp:14-76 with the kernel of
 * nestedtensor/csrc/cuda/transformer_kernels.cu:260-335, preceded by the packed
 * residual add NestedTensor_add_Tensor (nestedtensor/csrc/BinaryOps.cpp:18-44). */
int nt_layer_norm(const void* x, const void* residual, const void* gamma, const void* beta,
                  void* out, int64_t rows, int64_t n, double eps, int dtype, void* stream);

/* out[i] = a[i] + alpha * b[i % period], fp32 math, rounded to the storage type.
 * period == numel: the sum of two nested tensors of equal nested size, done on
 * their packed buffers (nestedtensor/csrc/BinaryOps.cpp:18-44).  period == n: a
 * nested tensor with regular last dim n plus a 1-D tensor of n elements
 * (nestedtensor/csrc/BinaryOps.cpp:97-107).  numel must be a multiple of period. */
int nt_add_packed(const void* a, const void* b, double alpha, void* out, int64_t numel,
                  int64_t period, int dtype, void* stream);

/* Softmax (log_softmax != 0: log-softmax) over the last dim of every constituent
 * of a nested tensor, on the packed buffer: constituent b has row_offsets[b + 1]
 * - row_offsets[b] rows of (offsets[b + 1] - offsets[b]) / rows elements each at
 * element offset offsets[b]; the row length may differ between constituents (a
 * ragged last dim, the [H, L_i, L_i] scores of per-sequence attention).  fp32
 * arithmetic, one rounding.  One launch for the per-constituent at::softmax of
 * NestedTensor_softmax / NestedTensor_log_softmax
 * (nestedtensor/csrc/SoftMax.cpp:12-46, call site nestedtensor/csrc/mha.cpp:58);
 * it is also the masked row softmax of the reference's GPU path
 * (nestedtensor/csrc/cuda/attention.cu:229-304) without the padding.  offsets and
 * row_offsets are int64[B + 1] on the device; total_rows = row_offsets[B]. */
int nt_softmax_rows(const void* x, void* out, const int64_t* offsets, const int64_t* row_offsets,
                    int64_t B, int64_t total_rows, int log_softmax, int dtype, void* stream);

/* out[i] = relu(x[i]) (act 1) or gelu(x[i]) (act 2, erf form), fp32 arithmetic, one
 * rounding: at::relu / at::gelu on the packed buffer, as NestedTensor_relu /
 * NestedTensor_gelu do (nestedtensor/csrc/activation.cpp:11-19, 34-46). */
int nt_activation_packed(const void* x, void* out, int64_t numel, int act, int dtype, void* stream);

/* out[i] = scale * a[i] * b[i % period] in fp32, rounded once; b == NULL gives
 * out[i] = scale * a[i] (period is then ignored).  period == numel: nested *
 * nested of equal nested size; period == last-dim size: nested * 1-D vector;
 * b == NULL: nested * scalar, the q * scaling step of min_mha.  Replaces the
 * per-constituent at::mul of NestedTensor_mul_Tensor
 * (nestedtensor/csrc/BinaryOps.cpp:241-300, call site nestedtensor/csrc/mha.cpp:46)
 * by one launch over the packed buffer. */
int nt_mul_packed(const void* a, const void* b, double scale, void* out, int64_t numel,
                  int64_t period, int dtype, void* stream);

/* ---- consumers of the offsets array (interop formats) ------------------- */

/* dst row r = src row index[r]; rows of row_bytes bytes, src has src_rows rows.
 * An index outside [0, src_rows) gives a zero row and, if oob_count is not NULL,
 * increments *oob_count (device int32).  With src = an embedding table and index
 * = the packed index buffer of a nested tensor this is the reference's packed
 * embedding (NestedTensor_embedding, nestedtensor/csrc/functions.cpp:27-55: one
 * at::embedding over the buffer); with the index built by
 * nt_packed_sequence_index it re-orders token rows for a PackedSequence. */
int nt_gather_rows(const void* src, int64_t src_rows, int64_t row_bytes, const int64_t* index,
                   void* dst, int64_t n_rows, int32_t* oob_count, void* stream);

/* Row order of torch.nn.utils.rnn.PackedSequence for the sequences of a nested
 * tensor [B, L_i, *]: index_out[step_starts[t] + rank[b]] = offsets[b] + t for
 * every token t of every sequence b.  offsets int64[B + 1] are token offsets,
 * rank[b] is the position of sequence b in the order of decreasing length,
 * step_starts[t] the number of rows of all time steps before t (exclusive prefix
 * sum of batch_sizes; at least max L_i entries).  All device arrays.  Replaces
 * the unbind + torch.nn.utils.rnn.pack_sequence of NestedTensor.to_packed_sequence
 * (nestedtensor/nested/nested.py:484-488). */
int nt_packed_sequence_index(const int64_t* offsets, const int64_t* rank, const int64_t* step_starts,
                             int64_t B, int64_t total_rows, int64_t* index_out, void* stream);

/* out[offsets[b] + j] = j for 0 <= j < offsets[b+1] - offsets[b]: the column
 * indices of the CSR view of a nested tensor of 1-D constituents, whose
 * crow_indices are offsets themselves (NestedTensor_to_sparse_csr,
 * nestedtensor/csrc/nested_tensor_impl.h:326-349, which concatenates one
 * torch::arange per constituent on the host).  max_len >= the longest row. */
int nt_ragged_arange(const int64_t* offsets, int64_t B, int64_t max_len, int64_t* out, void* stream);

/* out[b, :] = sum (mode 0), mean (1) or max (2) over t in [offsets[b], offsets[b+1])
 * of weight[indices[t], :]; weight [num_embeddings, n] with row stride ldw, fp32
 * accumulation in token order, empty bags give 0.  The bags are the constituents
 * of a nested tensor of 1-D index tensors and offsets is its offsets array: the
 * reference builds the same offsets in a host loop and calls torch.embedding_bag
 * (nestedtensor/nested/nested.py:43-118).  Indices out of range are skipped and
 * counted in *oob_count if it is not NULL.  num_indices = offsets[B], the length
 * of indices, as the host knows it: it only sizes the workgroups (bags of 64
 * indices or more on average get 16 wavefronts each instead of 4). */
int nt_embedding_bag(const void* weight, int64_t ldw, int64_t num_embeddings, const int64_t* indices,
                     int64_t num_indices, const int64_t* offsets, void* out, int64_t B, int64_t n,
                     int mode, int dtype, int32_t* oob_count, void* stream);

/* Per-constituent 2-D transpose on the packed buffer: constituent b, a row-major
 * [rows[b], cols[b]] matrix at element offset offsets[b], is written as its
 * [cols[b], rows[b]] transpose at the same offset of out.  rows = C, cols =
 * H_b * W_b is the reference's transpose_nchw_nhwc, the two exchanged its
 * transpose_nhwc_nchw (nestedtensor/csrc/transpose.cpp:87-204 with the
 * launchers of nestedtensor/csrc/cuda/transpose.h:11-31).  A workgroup moves one
 * tile_rows x tile_cols tile of one constituent; the caller chooses the shape
 * among 64x64, 64x128, 128x64, 128x128, 64x256, 256x64 with tile_rows *
 * tile_cols * elem_bytes <= 32768 (taller tiles write longer contiguous pieces
 * of the output rows), or, with S = 2048 / elem_bytes, the strips 16 x S when
 * every rows[b] <= 16 and S x 16 when every cols[b] <= 16 (a constituent that
 * breaks that promise is left unwritten).  tile_offsets int64[B + 1]: tile_offsets[b] = sum over c < b of
 * ceil(rows[c] / tile_rows) * ceil(cols[c] / tile_cols) (nt_offsets_from_sizes
 * over a [B, 2] array of the two tile counts builds it); total_tiles =
 * tile_offsets[B].  All arrays on the device. */
int nt_transpose_ragged(const void* in, void* out, const int64_t* offsets, const int64_t* rows,
                        const int64_t* cols, const int64_t* tile_offsets, int64_t B,
                        int64_t total_tiles, int tile_rows, int tile_cols, int elem_bytes,
                        void* stream);

/* nt_transpose_ragged for 2-byte elements when the OUTPUT rows do not begin on
 * 128-byte lines (NHWC -> NCHW of images whose H x W is no multiple of 64): every
 * output row is written as whole lines from its own aligned window of the input
 * rows.  Same operands; the tiles are counted differently: constituent b has
 * (ceil(rows[b] / 64) + 1) * ceil(cols[b] / 64) tiles.  Same reference code
 * (nestedtensor/csrc/transpose.cpp:183-204, cuda/transpose.cu). */
int nt_transpose_ragged_lines(const void* in, void* out, const int64_t* offsets, const int64_t* rows,
                              const int64_t* cols, const int64_t* tile_offsets, int64_t B,
                              int64_t total_tiles, int elem_bytes, void* stream);

/* Bias-free 1x1 convolution of B row-major images straight on the packed buffer:
 * image b is x + pix_offsets[b] * c_in, a [c_in, P_b] matrix with the P_b = H_b W_b
 * pixels contiguous, and the result y + pix_offsets[b] * c_out = weight[c_out,
 * c_in] times it, [c_out, P_b].  pix_offsets (device int64 [B + 1]) are the
 * cumulative pixel counts; tile_offsets (device int64 [B + 1]) the cumulative tile
 * counts with ceil(P_b / t) + 1 tiles for image b, t = nt_conv1x1_tile_pixels()
 * (a tile is one 128-byte line of every output row, and the rows' lines begin up
 * to t - 1 pixels before a multiple of t); total_tiles their sum.  y must be
 * 128-byte aligned.  f16 / bf16, fp32 accumulation; nt_conv1x1_supported() says
 * whether a pair of depths is covered (c_in a multiple of 16 up to 128, c_out a
 * multiple of 32 up to 512, and the weight plus two wavefronts' tiles must fit the
 * 160 KiB of LDS), otherwise NT_ERR_UNSUPPORTED.  Replaces transpose_nchw_nhwc +
 * matmul + transpose_nhwc_nchw of the reference's 1x1 path
 * (nestedtensor/csrc/conv2d.cpp:33-75) by one launch that reads and writes every
 * element once. */
int nt_conv1x1_supported(int64_t c_in, int64_t c_out, int dtype);
int64_t nt_conv1x1_tile_pixels(void);
int nt_conv1x1_nchw(const void* x, const void* weight, void* y, const int64_t* pix_offsets,
                    const int64_t* tile_offsets, int64_t B, int64_t total_tiles, int64_t c_in,
                    int64_t c_out, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NESTEDTENSOR_AMD_H */
