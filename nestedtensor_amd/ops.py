"""Operator layer: the reference's ``torch.ops.nestedtensor.*`` surface for the
ragged hot path, lowered to the C ABI.

The reference registers these ops on ``DispatchKey::NestedTensor`` with a custom
TensorImpl (nestedtensor/csrc/masking.cpp:652-675, csrc/mha.cpp:71-74,
csrc/cuda/mha.cpp:109-113, csrc/py_init.cpp:132-216).  That dispatch key belongs
to torch core now, so here the ``Tensor nt`` argument is the Python
``NestedTensor`` wrapper: ``NestedTensor.__torch_function__`` intercepts the op
call and routes it to the functions below, which work on
``(buffer, sizes, offsets)``.  Schemas (names, argument order) are the
reference's.  Host code in this file only validates, sizes outputs from the
host copy of the nested size and launches; all data movement and arithmetic is
in the HIP library.
"""

import torch

from . import _C
from .impl import NestedTensorImpl

# The schemas (same names and argument order as the reference) and the lowered
# operators that do the work live in the C++ extension csrc/torch_ops.cpp
# (TORCH_LIBRARY(nestedtensor, ...)), loaded by _C.  Overloads are resolved once.
_add_padding = _C.ops.add_padding.default
_add_padding_mask = _C.ops.add_padding_mask.default
_remove_padding = _C.ops.remove_padding.default
_build_mask = _C.ops.build_mask.default
_linear_packed = _C.ops.linear_packed.default
_mha_self_packed = _C.ops.mha_self_packed.default
_mha_cross_packed = _C.ops.mha_cross_packed.default
_mha_rowmajor_packed = _C.ops.mha_rowmajor_packed.default
_layer_norm_packed = _C.ops.layer_norm_packed.default
_binary_packed = _C.ops.binary_packed.default
_softmax_rows = _C.ops.softmax_rows.default
_activation_packed = _C.ops.activation_packed.default
_embedding_packed = _C.ops.embedding_packed.default
_embedding_bag_packed = _C.ops.embedding_bag_packed.default
_packed_sequence_lowered = _C.ops.packed_sequence_lowered.default


_ELEM_BYTES = {}


def _elem_bytes(dtype):
    n = _ELEM_BYTES.get(dtype)
    if n is None:
        n = _ELEM_BYTES[dtype] = torch.empty((), dtype=dtype).element_size()
    if n not in (1, 2, 4, 8):
        # masking.cpp:622 returns an uninitialised tensor for other dtypes; raise instead.
        raise RuntimeError("Input datatype %s is not supported." % dtype)
    return n


def _n_ragged(impl):
    """Number of leading constituent dims the row decode must walk: up to and
    including the last irregular dim.  Trailing regular dims are one contiguous
    run (the generalisation of _collapse_two_dims_3, masking.cpp:535-556)."""
    opt = impl.opt_sizes()[1:]
    n = 1
    for k, v in enumerate(opt):
        if v is None:
            n = k + 1
    return n


def _check_no_empty(impl):
    if impl.has_empty_constituent():
        # masking.cpp:140-142, 640-642
        raise RuntimeError("Empty tensors are not yet supported.")


# ---------------------------------------------------------------------------
# host nested tensors
#
# The reference serves nested tensors in host memory with CPU loops
# (masking.cpp:297-319, 511-532, 627-649).  Here the conversions exist on the
# device only; a nested tensor whose buffer lies in host memory is staged: the
# packed buffer goes to the current device, the device path runs, and the dense
# results come back to the host.  Same results, two extra copies.


def _to_host(result):
    if isinstance(result, tuple):
        return tuple(_to_host(r) for r in result)
    return result.cpu() if torch.is_tensor(result) else result


def _stage(impl, what, with_data=True):
    """Device twin of a host nested tensor: the packed buffer copied to the
    current device (or, when only the nested size is needed, an empty buffer)."""
    dev = _C.staging_device(what)
    buf = impl.buffer.to(dev) if with_data else torch.empty(0, dtype=impl.buffer.dtype, device=dev)
    return impl.with_buffer(buf)


# ---------------------------------------------------------------------------
# packed -> padded


def add_padding(impl, padding, with_mask=False, shape=None):
    """Launch nt_add_padding: [B, max_1..max_D] from the packed buffer (or
    [B] + shape for a caller-given shape that holds every constituent).  With
    with_mask, nt_add_padding_mask writes the bool mask of the same shape in the
    same launch and (padded, mask) is returned."""
    if not impl.buffer.is_cuda:
        return _to_host(add_padding(_stage(impl, "to_padded_tensor"), padding, with_mask, shape))
    B, D = impl.B, impl.D
    max_size = impl.max_sizes()
    nrag = _n_ragged(impl)
    if shape is not None:
        shape = [int(v) for v in shape]
        if len(shape) != D or any(s < m for s, m in zip(shape, max_size)):
            raise RuntimeError("pad_nt: shape %s does not hold constituents of up to %s" % (shape, max_size))
        # a dim that is regular but shorter than the requested extent is walked as ragged
        for k in range(D):
            if shape[k] != max_size[k]:
                nrag = max(nrag, k + 1)
        max_size = shape
    if nrag > 3:
        raise RuntimeError("to_padded_tensor supports at most 3 irregular dimensions.")
    _elem_bytes(impl.buffer.dtype)
    if with_mask:
        return _add_padding_mask(impl.buffer, impl.sizes_dev(), impl.offsets_dev(), max_size, nrag,
                                 float(padding))
    return _add_padding(impl.buffer, impl.sizes_dev(), impl.offsets_dev(), max_size, nrag, float(padding))


def pad_nt(impl, shape):
    """pad_nt (masking.cpp:138-179): every constituent padded with 0 to `shape`,
    stacked, and the mask of the same shape (bool here, uint8 in the reference)."""
    if impl.B == 0:
        return torch.tensor([0]), torch.tensor([False])          # masking.cpp:164-167
    _check_no_empty(impl)
    if impl.D == 0:
        return impl.buffer.clone(), torch.ones(impl.B, dtype=torch.bool, device=impl.buffer.device)
    return add_padding(impl, 0, with_mask=True, shape=shape)


def merge_tensor_mask(tensor, mask, mask_dim=None):
    """merge_tensor_mask (masking.cpp:12-43) on a dense (tensor, mask) pair: the
    last mask dim is dropped while every one of its rows is all ones or all
    zeros; stops at mask_dim, and refuses a mask_dim it cannot reach."""
    while True:
        if mask_dim is not None and mask.dim() == mask_dim:
            return tensor, mask
        if mask.dim() == 0:
            return tensor, mask
        last = mask.size(-1)
        collapsed = mask.sum(-1)
        uniform = int(((collapsed == last) | (collapsed == 0)).sum())
        if uniform == collapsed.numel():
            mask = collapsed.to(torch.bool)
            continue
        if mask_dim is not None and mask_dim != mask.dim():
            raise RuntimeError("Mask dimension is too small to represent data tensor.")
        return tensor.contiguous(), mask.contiguous()


def to_padded_tensor(impl, padding):
    """to_padded_tensor (masking.cpp:558-650)."""
    opt = impl.opt_sizes()
    if len(opt) == 1 and opt[0] == 1:
        return impl.buffer                       # masking.cpp:628-631 (alias)
    if impl.B == 0:
        return torch.tensor([float(padding)])     # masking.cpp:634-636
    if impl.D == 0:
        # B scalars: the stack of the constituents.  (The reference pushes every
        # 0-d constituent twice, masking.cpp:644-647; not followed.)
        return impl.buffer.clone()
    _check_no_empty(impl)
    return add_padding(impl, padding)


# ---------------------------------------------------------------------------
# masks


def _collapsed_mask_dims(impl, mask_dim):
    """Closed form of merge_tensor_mask (masking.cpp:12-43) on the mask of a
    nested tensor without empty constituents: starting from [B, max_1..max_D],
    the last dim collapses iff it is regular; if every dim is regular the batch
    dim collapses too and the mask is the scalar True.  Collapsing stops at
    mask_dim.  Returns the number of mask dims kept (0 = scalar)."""
    opt = impl.opt_sizes()
    cur = impl.dim()
    while True:
        if mask_dim is not None and cur == mask_dim:
            return cur
        if cur == 0:
            return 0
        # last mask dim is index cur-1 of opt_sizes; the batch dim (index 0)
        # collapses when everything after it did.
        if cur == 1 or opt[cur - 1] is not None:
            cur -= 1
            continue
        if mask_dim is not None and mask_dim != cur:
            raise RuntimeError("Mask dimension is too small to represent data tensor.")
        return cur


def build_mask(impl, kept_dims):
    """Bool mask over [B, max_1..max_{kept_dims-1}] (nt_build_mask)."""
    dev = impl.buffer.device
    if kept_dims == 0:
        return torch.tensor(True, device=dev)
    if kept_dims == 1:
        return torch.ones(impl.B, dtype=torch.bool, device=dev)
    if not impl.buffer.is_cuda:
        return _to_host(build_mask(_stage(impl, "to_mask", with_data=False), kept_dims))
    K = kept_dims - 1
    if K > 3:
        raise RuntimeError("masks over more than 3 constituent dimensions are not supported.")
    return _build_mask(impl.sizes_dev(), impl.max_sizes()[:K])


def _check_mask_dim(impl, mask_dim):
    if mask_dim is not None and mask_dim > impl.dim():
        raise RuntimeError(
            "Requested mask dimension %d is bigger than dimension %d of given NestedTensor."
            % (mask_dim, impl.dim()))


def to_tensor_mask(impl, mask_dim=None):
    """to_tensor_mask (masking.cpp:251-320).  The mask is always bool (the
    reference's device path returns bool, its host path uint8 when nothing
    collapsed)."""
    _check_mask_dim(impl, mask_dim)
    opt = impl.opt_sizes()
    dev = impl.buffer.device
    if len(opt) == 1 and opt[0] == 1:
        # masking.cpp:305-313
        mask = torch.tensor(True, device=dev) if (mask_dim is None or mask_dim == 0) \
            else torch.tensor([True], device=dev)
        return impl.buffer.reshape(-1), mask
    if impl.B == 0:
        # masking.cpp:164-167 then merge_tensor_mask
        if mask_dim == 1:
            return torch.tensor([0]), torch.tensor([False])
        return torch.tensor([0]), torch.tensor(False)
    if impl.D == 0:
        # masking.cpp:91
        raise RuntimeError("Internal error: Expected sizes_size_1 to be greater than 0.")
    _check_no_empty(impl)
    kept = _collapsed_mask_dims(impl, mask_dim)
    if kept == impl.dim() and _n_ragged(impl) <= 3:
        # nothing collapsed: the mask has the shape of the data and is written by
        # the same launch (the fused kernel of padding.cu:217-262, generalised)
        return add_padding(impl, 0, with_mask=True)
    data = add_padding(impl, 0)
    return data, build_mask(impl, kept)


def to_mask(impl, mask_dim=None):
    """to_mask (masking.cpp:408-457)."""
    _check_mask_dim(impl, mask_dim)
    opt = impl.opt_sizes()
    dev = impl.buffer.device
    if len(opt) == 1 and opt[0] == 1:
        return torch.tensor(True, device=dev) if (mask_dim is None or mask_dim == 0) \
            else torch.tensor([True], device=dev)
    if impl.B == 0:
        raise RuntimeError("to_mask of an empty NestedTensor is not defined.")
    if impl.dim() > 1 and mask_dim is not None and mask_dim > 1:
        # masking.cpp:428-453: the first mask_dim - 1 constituent dims, no merge
        K = mask_dim - 1
        if impl.has_empty_constituent() and bool((impl.sizes[:, :K] == 0).any()):
            raise RuntimeError("Empty tensors are not yet supported.")
        return build_mask(impl, mask_dim)
    if impl.D == 0:
        raise RuntimeError("Internal error: Expected sizes_size_1 to be greater than 0.")
    _check_no_empty(impl)
    return build_mask(impl, _collapsed_mask_dims(impl, mask_dim))


# ---------------------------------------------------------------------------
# padded -> packed (length based)


def from_padded_tensor(padded, target):
    """from_padded_tensor (masking.cpp:459-533): gather the entries inside
    ``target``'s nested size out of ``padded``.  ``target`` is a NestedTensorImpl
    whose nested size the result takes."""
    if padded.dim() != target.dim():
        raise RuntimeError("Target size has different dimension as input padded Tensor.")
    if not padded.is_cuda:
        # a host tensor: staged through the device, the packed result comes back
        res = from_padded_tensor(padded.to(_C.staging_device("from_padded_tensor")), target)
        return res.with_buffer(res.buffer.cpu())
    padded = padded.contiguous()
    B, D = target.B, target.D
    if padded.size(0) != B:
        raise RuntimeError("Target size has a different batch size than the padded Tensor.")
    ext = list(padded.shape[1:])
    mx = target.max_sizes()
    for k in range(D):
        if mx[k] > ext[k]:
            raise RuntimeError("Target size exceeds the padded Tensor in dimension %d." % (k + 1))
    nrag = _n_ragged(target)
    # a dim that is regular in `target` but shorter than the padded extent must
    # be walked as ragged
    opt = target.opt_sizes()[1:]
    for k in range(D):
        if opt[k] is not None and opt[k] != ext[k]:
            nrag = max(nrag, k + 1)
    if nrag > 3:
        raise RuntimeError("from_padded_tensor supports at most 3 irregular dimensions.")
    _elem_bytes(padded.dtype)
    total = target.numel()
    if total == 0:
        return target.with_buffer(torch.empty(0, dtype=padded.dtype, device=padded.device))
    if target.buffer.device != padded.device:
        target = target.with_buffer(torch.empty(0, dtype=padded.dtype, device=padded.device))
    out = _remove_padding(padded, target.sizes_dev(), target.offsets_dev(), total, nrag)
    return target.with_buffer(out)


# ---------------------------------------------------------------------------
# nested multi-head attention


_ACTS = {None: 0, "none": 0, "relu": 1, "gelu": 2}


def linear(x, weight, bias, activation=None):
    """y = act(x @ weight.T + bias) on a 2-D row-major view (nt_linear_act).  This
    is the packed fast path of NestedTensor_matmul (matmul.cpp:13-41) with the
    packed bias add (BinaryOps.cpp:97-107) and, optionally, relu / gelu
    (activation.cpp:11-19, 34-46) fused into the GEMM epilogue."""
    _C.require_device(x, "linear")
    assert x.dim() == 2 and weight.dim() == 2 and x.stride(1) == 1
    if activation not in _ACTS:
        raise RuntimeError("linear: activation must be None, 'relu' or 'gelu', got %r" % (activation,))
    M, K = x.shape
    N = weight.size(0)
    if weight.size(1) != K:
        raise RuntimeError("linear: weight of shape %s does not match input feature size %d"
                           % (tuple(weight.shape), K))
    return _linear_packed(x, weight, bias, _ACTS[activation])


def linear_nt(impl, weight, bias=None, activation=None):
    """F.linear on a NestedTensor [B, L_i, K] (nested.py:17-28): one GEMM on the
    packed [T, K] view, with an optional fused activation."""
    opt = impl.opt_sizes()
    if impl.dim() != 3 or opt[2] is None:
        raise NotImplementedError("linear on a NestedTensor needs dim 3 and a regular last dim.")
    out = linear(impl.buffer.reshape(-1, opt[2]), weight, bias, activation)
    sizes = impl.sizes.clone()
    sizes[:, 1] = weight.size(0)
    return NestedTensorImpl(out.reshape(-1), sizes)


def activation(impl, kind):
    """relu / gelu of a NestedTensor: one launch over the packed buffer
    (NestedTensor_relu / NestedTensor_gelu, activation.cpp:11-19, 34-46); the
    storage layout does not matter."""
    buf = impl.buffer
    _C.require_device(buf, kind)
    return impl.with_buffer(_activation_packed(buf, _ACTS[kind]))


_attention_kernel = "work_list"


def set_attention_kernel(kind):
    """Which kernel runs f16 / bf16 attention with head_dim 64: "work_list" (the
    default: one small workgroup per 128 query rows of a head, the faster one on every
    measured batch) or "planned" (persistent workgroups that stream a sequence's
    keys through LDS from a host-made plan).  Same results to rounding; other head
    dims always take the work list.  Returns the previous setting."""
    global _attention_kernel
    if kind not in ("work_list", "planned"):
        raise ValueError("attention kernel must be 'work_list' or 'planned', not %r" % (kind,))
    previous, _attention_kernel = _attention_kernel, kind
    return previous


def _attention_work(query, key, num_heads, head_dim):
    """The device-side description of the attention work for the selected kernel."""
    if _attention_kernel == "planned" and head_dim == 64:
        return query.attention_plan(num_heads, head_dim, kv=key)
    return query.attention_schedule(kv=key)


def _check_mha_inputs(query, key, value):
    if query.dim() != 3:
        raise RuntimeError("query needs to be 3 dim.")
    if key.dim() != 3:
        raise RuntimeError("key needs to be 3 dim.")
    if value.dim() != 3:
        raise RuntimeError("value needs to be 3 dim.")


def mha_packed(num_heads, head_dim, query, key, value, in_proj_weight, in_proj_bias, scaling,
               out_proj_weight, out_proj_bias):
    """Nested multi-head attention on packed buffers.  Semantics of min_mha
    (mha.cpp:18-69): per sequence, softmax over that sequence's own keys only.
    query/key/value are NestedTensorImpl of dim 3 with regular last dim."""
    _check_mha_inputs(query, key, value)
    opt = query.opt_sizes()
    if opt[2] is None:
        raise RuntimeError("query's third dimension must be regular.")
    E = num_heads * head_dim
    if opt[2] != E:
        raise RuntimeError("query's embedding dimension %d does not match num_heads * head_dim = %d"
                           % (opt[2], E))
    if key.opt_sizes()[2] != E or value.opt_sizes()[2] != E:
        raise RuntimeError("key and value must have the embedding dimension of query.")
    if key.B != query.B or value.B != query.B:
        raise RuntimeError("query, key and value must hold the same number of sequences.")
    if not torch.equal(key.sizes, value.sizes):
        raise RuntimeError("key and value must have the same nested size.")
    _C.require_device(query.buffer, "multi-head attention")
    dtype = query.buffer.dtype
    W = in_proj_weight.contiguous()
    if tuple(W.shape) != (3 * E, E):
        raise RuntimeError("in_proj_weight must have shape [3 * embed_dim, embed_dim].")
    xq = query.buffer.reshape(-1, E)
    same = (key is query or key.buffer.data_ptr() == query.buffer.data_ptr()) and \
        (value is query or value.buffer.data_ptr() == query.buffer.data_ptr()) and \
        torch.equal(key.sizes, query.sizes)
    max_q = int(query.sizes[:, 0].max()) if query.B > 0 else 0
    mfma_path = head_dim in (32, 64, 128) and dtype in (torch.float16, torch.bfloat16)
    fused = same and mfma_path and (2 * E) % 128 == 0
    if in_proj_bias is not None:
        in_proj_bias = in_proj_bias.contiguous()
        if in_proj_bias.dtype != dtype:
            raise RuntimeError("linear: input, weight and bias must have the same dtype")
    if W.dtype != dtype:
        raise RuntimeError("linear: input, weight and bias must have the same dtype")
    if fused:
        # self-attention, head_dim 32 / 64 / 128: Q|K row-major + V transposed straight out of
        # the projection GEMM, attention reads both without any re-layout pass, then the
        # output projection: three launches, issued by one call into the extension
        out = _mha_self_packed(xq, _attention_work(query, None, num_heads, head_dim), num_heads, head_dim, W, in_proj_bias,
                               float(scaling), out_proj_weight, out_proj_bias)
        return query.with_buffer(out.reshape(-1))
    xk, xv = key.buffer.reshape(-1, E), value.buffer.reshape(-1, E)
    if mfma_path and bool((key.sizes[:, 0] > 0).all()):
        # cross-attention (or an embedding size the fused projection does not tile),
        # head_dim 32 / 64 / 128: three projections (the value one written
        # transposed), then the same attention kernel with one key sequence per
        # query sequence: five launches issued by one call into the extension
        out = _mha_cross_packed(xq, xk, xv, _attention_work(query, key, num_heads, head_dim), num_heads, head_dim, W,
                                in_proj_bias, float(scaling), out_proj_weight, out_proj_bias)
        return query.with_buffer(out.reshape(-1))
    # V row-major: fp32 with head_dim 32 / 64 / 128 on the fp32 matrix instruction from
    # the work list (only tiles that exist, longest key sequences first), anything else
    # (other head dims, key sequences without keys) on the generic kernels over the
    # device row offsets
    sched = None
    if dtype == torch.float32 and head_dim in (32, 64, 128):
        sched = query.attention_schedule(kv=None if same else key)
    out = _mha_rowmajor_packed(xq, xk, xv, same, sched, query.row_offsets_dev(), key.row_offsets_dev(), max_q,
                               num_heads, head_dim, W, in_proj_bias, float(scaling), out_proj_weight,
                               out_proj_bias)
    return query.with_buffer(out.reshape(-1))


def min_mha(num_heads, head_dim, dropout_p, training, query, key, value, in_proj_weight,
            in_proj_bias, scaling, out_proj_weight, out_proj_bias):
    """min_mha (mha.cpp:18-69)."""
    _check_mha_inputs(query, key, value)
    if in_proj_bias is None:
        raise RuntimeError("Input projection bias needs to be defined.")
    if training and dropout_p > 0:
        raise RuntimeError("nested multi-head attention is inference only (no dropout).")
    return mha_packed(num_heads, head_dim, query, key, value, in_proj_weight, in_proj_bias,
                      scaling, out_proj_weight, out_proj_bias)


def bt_min_mha(num_heads, head_dim, dropout_p, training, query, key, value, attr_kernel,
               attr_bias, scaling, out_proj_weight, out_proj_bias):
    """bt_min_mha (cuda/mha.cpp:22-107).  As in the reference, key and value
    are taken to be query, and out_proj_bias is not added (cuda/mha.cpp:106).
    The softmax is the exact one over each sequence's own keys, which the
    reference's -10000 additive mask and +1e-6 denominator approximate."""
    _check_mha_inputs(query, key, value)
    return mha_packed(num_heads, head_dim, query, query, query, attr_kernel, attr_bias, scaling,
                      out_proj_weight, None)


# ---- row-wise ops on the packed buffer: the steps either side of attention ----

def layer_norm(impl, normalized_shape, weight=None, bias=None, eps=1e-5, residual=None):
    """NestedTensor_layer_norm (functions.cpp:65-112; device fast path
    cuda/layernorm.cpp:14-76): normalise over the regular last dim, one launch
    over the packed [T, n] view (nt_layer_norm).  `residual` (a nested tensor of
    the same nested size) is added first, rounded to the storage type, as
    ``layer_norm(nt + residual)`` does in two ops (BinaryOps.cpp:18-44)."""
    normalized_shape = tuple(normalized_shape) if not isinstance(normalized_shape, int) \
        else (normalized_shape,)
    if len(normalized_shape) != 1:
        raise RuntimeError("Currently only singleton tuples of integers supported for layer_norm.")
    opt = impl.opt_sizes()
    last = impl.dim() - 1
    if opt[last] is None:
        raise RuntimeError("Cannot normalize across irregular dimension %d" % last)
    n = opt[last]
    if n != normalized_shape[0]:
        raise RuntimeError("Normalized shape [%d] does not match the size of the last dimension (%d) of input."
                           % (normalized_shape[0], n))
    if (weight is None) != (bias is None):
        raise RuntimeError("Either both weight and bias are used or not.")
    buf = impl.buffer
    _C.require_device(buf, "layer_norm")
    for t in (weight, bias):
        if t is not None and (t.dtype != buf.dtype or t.device != buf.device or t.numel() != n):
            raise RuntimeError("layer_norm: weight and bias must have %d elements of the input's dtype "
                               "on the input's device" % n)
    res_buf = None
    if residual is not None:
        if not torch.equal(residual.sizes, impl.sizes) or residual.buffer.dtype != buf.dtype:
            raise RuntimeError("layer_norm: the residual must have the nested size and dtype of the input")
        res_buf = residual.buffer
    if n == 0 or buf.numel() == 0:
        return impl.with_buffer(torch.empty_like(buf))
    weight = weight.contiguous() if weight is not None else None
    bias = bias.contiguous() if bias is not None else None
    return impl.with_buffer(_layer_norm_packed(buf, res_buf, weight, bias, n, float(eps)))


def add(impl, other, alpha=1):
    """NestedTensor_add_Tensor on the packed buffers (BinaryOps.cpp:12-115): the
    two cases that need no per-constituent work, nested + nested of equal nested
    size (:18-44) and nested with a regular last dim + 1-D tensor (:97-107)."""
    buf = impl.buffer
    _C.require_device(buf, "add")
    if isinstance(other, NestedTensorImpl):
        if other.sizes.shape != impl.sizes.shape or not torch.equal(other.sizes, impl.sizes):
            raise NotImplementedError("add of nested tensors of different nested size is not on the packed path.")
        if not (impl.channels_last and other.channels_last):
            # two channels-last operands add buffer to buffer and stay channels-last
            # (BinaryOps.cpp:25-32); any other mix goes through the row-major layout (:33-43)
            impl, other = contiguous(impl), contiguous(other)
            buf = impl.buffer
        b, period = other.buffer, buf.numel()
    elif isinstance(other, torch.Tensor) and other.dim() == 1:
        impl = contiguous(impl)
        buf = impl.buffer
        opt = impl.opt_sizes()
        if opt[impl.dim() - 1] is None or opt[impl.dim() - 1] != other.size(0):
            raise NotImplementedError("add of a 1-D tensor needs a regular last dim of the same size.")
        b, period = other.contiguous(), other.size(0)
    else:
        raise NotImplementedError("add: only nested + nested (same nested size) and nested + 1-D tensor "
                                  "are on the packed path.")
    if b.dtype != buf.dtype or b.device != buf.device:
        raise RuntimeError("add: both operands must have the same dtype and device")
    return impl.with_buffer(_binary_packed(buf, b, float(alpha), period, False))


def softmax(impl, dim, dtype=None, log=False):
    """NestedTensor_softmax / NestedTensor_log_softmax (SoftMax.cpp:12-46) over the
    last dim, which may be ragged, in one launch over the packed buffer
    (nt_softmax_rows).  Other dims of the constituents are not on the packed
    path; dim 0 is the nested dim and is refused like in the reference."""
    name = "log_softmax" if log else "softmax"
    nd = impl.dim()
    if not -nd <= dim < nd:
        raise IndexError("Dimension out of range (expected to be in range of [%d, %d], but got %d)"
                         % (-nd, nd - 1, dim))
    dim = dim % nd
    if dim < impl.nested_dim():
        raise RuntimeError("Cannot apply %s across nested dimensions %d" % (name, dim))
    if dim != nd - 1:
        raise NotImplementedError("%s on a NestedTensor: only the last dim is on the packed path." % name)
    buf = impl.buffer
    _C.require_device(buf, name)
    if dtype is not None and dtype != buf.dtype:
        buf = buf.to(dtype)
        impl = impl.with_buffer(buf)
    if buf.numel() == 0:
        return impl.with_buffer(torch.empty_like(buf))
    row_offsets, total_rows = impl.last_dim_rows()
    return impl.with_buffer(_softmax_rows(buf, impl.offsets_dev(), row_offsets, total_rows, bool(log)))


def mul(impl, other):
    """NestedTensor_mul_Tensor on the packed buffer (BinaryOps.cpp:241-300): nested
    * scalar (the q * scaling step of min_mha, mha.cpp:46), nested * nested of
    equal nested size, nested * 1-D tensor over a regular last dim."""
    _C.require_device(impl.buffer, "mul")
    b, period, scale = None, 0, 1.0
    if isinstance(other, NestedTensorImpl):
        if other.sizes.shape != impl.sizes.shape or not torch.equal(other.sizes, impl.sizes):
            raise NotImplementedError("mul of nested tensors of different nested size is not on the packed path.")
        if not (impl.channels_last and other.channels_last):
            impl, other = contiguous(impl), contiguous(other)
        b, period = other.buffer, impl.buffer.numel()
    elif isinstance(other, (int, float)) or (isinstance(other, torch.Tensor) and other.dim() == 0):
        scale = float(other)            # the layout does not matter
    elif isinstance(other, torch.Tensor) and other.dim() == 1:
        impl = contiguous(impl)
        opt = impl.opt_sizes()
        if opt[impl.dim() - 1] is None or opt[impl.dim() - 1] != other.size(0):
            raise NotImplementedError("mul by a 1-D tensor needs a regular last dim of the same size.")
        b, period = other.contiguous(), other.size(0)
    else:
        raise NotImplementedError("mul: only nested * scalar, nested * nested (same nested size) and "
                                  "nested * 1-D tensor are on the packed path.")
    buf = impl.buffer
    if b is not None and (b.dtype != buf.dtype or b.device != buf.device):
        raise RuntimeError("mul: both operands must have the same dtype and device")
    return impl.with_buffer(_binary_packed(buf, b, scale, period, True))


def matmul(impl, other):
    """NestedTensor_matmul, packed fast path (matmul.cpp:13-41): a nested tensor
    [B, L_i, K] times a dense [K, N] matrix is one GEMM over the packed [T, K]
    buffer.  nt_linear wants the weight K-contiguous, so `other` is transposed
    first (a copy of K * N elements)."""
    if isinstance(other, NestedTensorImpl) or not isinstance(impl, NestedTensorImpl):
        raise NotImplementedError("matmul: only nested [B, L_i, K] x dense [K, N] is on the packed path.")
    opt = impl.opt_sizes()
    if impl.dim() != 3 or other.dim() != 2 or opt[2] is None or opt[2] != other.size(0):
        raise NotImplementedError("matmul: only nested [B, L_i, K] x dense [K, N] is on the packed path.")
    out = linear(impl.buffer.reshape(-1, opt[2]), other.t().contiguous(), None)
    sizes = impl.sizes.clone()
    sizes[:, 1] = other.size(1)
    return NestedTensorImpl(out.reshape(-1), sizes)


# ---- dense ops called through pad -> op -> un-pad (pooling.cpp:41-57, conv2d.cpp:77-92) ----

def _pair(v):
    if isinstance(v, int):
        return (v, v)
    v = tuple(int(x) for x in v)
    return (v[0], v[0]) if len(v) == 1 else v


def _dense_via_padding(impl, pad_value, dense_op, out_channels, k, stride, padding, dilation, ceil_mode=False):
    """to_padded_tensor -> one dense call over the whole batch -> from_padded_tensor
    with the per-constituent output sizes
    ``(s + 2 p - d (k - 1) - 1) // stride + 1`` (pooling.cpp:50-53, conv2d.cpp:80-84).
    With ceil_mode the division rounds up and a last window that would start past
    the input and its left padding is dropped, as ATen's pooling_output_shape does
    for each constituent on the reference's per-constituent route (pooling.cpp:60-72)."""
    if impl.dim() != 4:
        raise RuntimeError("Input must be 4 dimensional.")
    _C.require_device(impl.buffer, "dense op on a NestedTensor")
    was_channels_last = impl.channels_last
    impl = contiguous(impl)
    data = to_padded_tensor(impl, pad_value)
    result = dense_op(data).contiguous()
    sizes = impl.sizes.clone()
    if out_channels is not None:
        sizes[:, 0] = out_channels
    for j in (0, 1):
        extent = sizes[:, 1 + j]
        span = extent + 2 * padding[j] - dilation[j] * (k[j] - 1) - 1
        if ceil_mode:
            out = torch.div(span + stride[j] - 1, stride[j], rounding_mode="floor") + 1
            out = out - ((out - 1) * stride[j] >= extent + padding[j]).to(out.dtype)
        else:
            out = torch.div(span, stride[j], rounding_mode="floor") + 1
        sizes[:, 1 + j] = out
    if bool((sizes <= 0).any()):
        raise RuntimeError("Output size is too small")
    target = NestedTensorImpl(torch.empty(0, dtype=result.dtype, device=result.device), sizes)
    out = from_padded_tensor(result, target)
    # a channels-last input gives a channels-last result (pooling.cpp:54-56, conv2d.cpp:88-90)
    return contiguous(out, torch.channels_last) if was_channels_last else out


def max_pool2d(impl, kernel_size, stride=None, padding=0, dilation=1, ceil_mode=False,
               return_indices=False):
    """NestedTensor_max_pool2d (pooling.cpp:34-75).  The reference takes the
    padded route for fp16 only and pads with 0; here every dtype takes it and the
    pad value is -inf, which makes the result equal to pooling each constituent on
    its own (what the reference's tests assert) also for windows that reach past a
    constituent's edge."""
    if return_indices:
        # not part of the reference's operator either (pooling.cpp:34-40)
        raise NotImplementedError("max_pool2d on a NestedTensor: return_indices is not supported.")
    k = _pair(kernel_size)
    s = _pair(stride) if stride not in (None, [], ()) else k
    p, d = _pair(padding), _pair(dilation)
    # ceil_mode: a window that reaches past a constituent's edge sees -inf there, in
    # the padded batch as in the constituent pooled on its own
    return _dense_via_padding(
        impl, float("-inf"),
        lambda x: torch.nn.functional.max_pool2d(x, k, s, p, d, bool(ceil_mode)), None, k, s, p, d,
        ceil_mode=bool(ceil_mode))


def _conv1x1_row_major(impl, w2d):
    """The 1x1 convolution of row-major f16 / bf16 images as one launch on the packed
    buffer (nt_conv1x1_nchw); None when the kernel does not cover the shape."""
    buf = impl.buffer
    c_out, c_in = w2d.shape
    if impl.channels_last or buf.dtype not in (torch.float16, torch.bfloat16) or \
            not _C.lib.nt_conv1x1_supported(c_in, c_out, _C.dtype_code(buf.dtype)):
        return None
    tn = int(_C.lib.nt_conv1x1_tile_pixels())
    B = impl.B
    if impl._transpose_meta is None:
        impl._transpose_meta = {}
    key = ("conv1x1", tn)
    cached = impl._transpose_meta.get(key)
    if cached is not None and cached[0].device == buf.device:
        meta_dev, total_tiles = cached
    else:
        pix = impl.sizes[:, 1] * impl.sizes[:, 2]
        meta = torch.zeros((2, B + 1), dtype=torch.int64)
        meta[0, 1:] = torch.cumsum(pix, 0)
        # a tile is one 128-byte line of every output row; the rows' lines start up to
        # tn - 1 pixels before a multiple of tn, hence one tile more than ceil(P / tn)
        meta[1, 1:] = torch.cumsum(torch.where(pix > 0, (pix + tn - 1) // tn + 1, pix), 0)
        total_tiles = int(meta[1, B])
        meta_dev = meta.to(buf.device)
        impl._transpose_meta[key] = (meta_dev, total_tiles)
    w2d = w2d.contiguous()
    sizes = impl.sizes.clone()
    sizes[:, 0] = c_out
    out = torch.empty(int(sizes.prod(1).sum()), dtype=buf.dtype, device=buf.device)
    if total_tiles:
        with _C.on_device(buf.device):
            _C.check(_C.lib.nt_conv1x1_nchw(_C.ptr(buf), _C.ptr(w2d), _C.ptr(out), _C.ptr(meta_dev[0]),
                                            _C.ptr(meta_dev[1]), B, total_tiles, c_in, c_out,
                                            _C.dtype_code(buf.dtype), _C.current_stream(buf.device)))
    return NestedTensorImpl(out, sizes)


def conv2d(impl, weight, bias=None, stride=1, padding=0, dilation=1, groups=1):
    """NestedTensor_conv2d, padded route (conv2d.cpp:77-92; the reference takes it
    for fp16).  Padding with 0 is exact: a convolution pads with zeros itself."""
    if isinstance(padding, str):
        raise NotImplementedError("conv2d on a NestedTensor: string padding is not supported.")
    s, p, d = _pair(stride), _pair(padding), _pair(dilation)
    k = (weight.size(2), weight.size(3))
    if (impl.dim() == 4 and bias is None and k == (1, 1) and s == (1, 1) and p == (0, 0) and d == (1, 1)
            and groups == 1 and impl.opt_sizes()[1] is not None and impl.buffer.is_cuda
            and weight.dtype == impl.buffer.dtype and weight.size(1) == impl.opt_sizes()[1]):
        # 1x1 convolution = one GEMM over all pixels of all images (conv2d.cpp:33-75)
        c_in, c_out = weight.size(1), weight.size(0)
        if impl.channels_last:
            # the buffer already is the [pixels, C_in] matrix, and the product is
            # the channels-last result (conv2d.cpp:43-60): no transposes
            y = linear(impl.buffer.reshape(-1, c_in), weight.reshape(c_out, c_in), None)
            sizes = impl.sizes.clone()
            sizes[:, 0] = c_out
            res = NestedTensorImpl(y.reshape(-1), sizes, channels_last=True)
            return res
        y = _conv1x1_row_major(impl, weight.reshape(c_out, c_in))
        if y is not None:
            return y
        # NCHW -> NHWC on the packed buffer, [pixels, C_in] x W^T, and back (conv2d.cpp:61-73)
        nhwc = transpose_nchw_nhwc(impl)
        y = linear(nhwc.buffer.reshape(-1, c_in), weight.reshape(c_out, c_in), None)
        sizes = nhwc.sizes.clone()
        sizes[:, 2] = c_out
        return transpose_nhwc_nchw(NestedTensorImpl(y.reshape(-1), sizes))
    return _dense_via_padding(
        impl, 0.0, lambda x: torch.conv2d(x, weight, bias, s, p, d, groups), weight.size(0), k, s, p, d)


# ---- consumers of the offsets array: interop formats ----------------------------

# Out-of-range indices.  torch's own device embedding traps asynchronously; here
# the kernels write zero rows for such indices and count them in a counter that
# lives on the device for the life of the process (it only ever grows).  How the
# count reaches the host is a setting:
#   "immediate" (default) every call waits for its own count and raises before
#               returning, like an index error of the reference's host path.  Under
#               stream capture nothing can be waited for; a captured call behaves
#               as in "deferred".
#   "deferred"  after each call the counter is copied, asynchronously, into pinned
#               host memory; the next embedding / embedding_bag call and
#               check_index_errors() look at that copy and raise IndexError for
#               whatever has arrived.  No call waits for the device: the setting
#               for serving loops that validate their indices elsewhere.
#   "off"       indices are trusted; nothing is copied.
_INDEX_CHECK_MODES = ("deferred", "immediate", "off")
_index_check_mode = "immediate"
_index_counters = {}      # device index -> [device int32[1], pinned int32[1], count already reported]


def set_index_check(mode):
    """Select how out-of-range indices of embedding / embedding_bag are reported
    ("deferred", "immediate" or "off"); returns the previous setting."""
    global _index_check_mode
    if mode not in _INDEX_CHECK_MODES:
        raise ValueError("index check mode must be one of %s, got %r" % (", ".join(_INDEX_CHECK_MODES), mode))
    previous, _index_check_mode = _index_check_mode, mode
    return previous


def _index_counter(device):
    slot = _index_counters.get(device.index)
    if slot is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("embedding / embedding_bag: the index counter of this device cannot be created "
                               "during stream capture; run the op once before capturing (or set_index_check('off')).")
        slot = [torch.zeros(1, dtype=torch.int32, device=device),
                torch.zeros(1, dtype=torch.int32).pin_memory(), 0]
        _index_counters[device.index] = slot
    return slot


def _report_index_errors(slot, what):
    seen = int(slot[1][0])            # a read of pinned host memory, no device call
    if seen != slot[2]:
        n, slot[2] = seen - slot[2], seen
        raise IndexError("%s: %d index value(s) out of range" % (what, n))


def check_index_errors(synchronize=True):
    """Raise IndexError if an embedding / embedding_bag call issued so far met
    out-of-range indices that have not been reported yet.  With synchronize (the
    default) the devices that ran such calls are waited for first, so every call
    issued before this one is covered; without it only the counts that have
    already arrived on the host are looked at."""
    for index, slot in _index_counters.items():
        if synchronize:
            torch.cuda.synchronize(index)
        _report_index_errors(slot, "embedding / embedding_bag (an earlier call)")


def _oob_begin(device, what):
    """The device's counter slot for a launch (None when checks are off); in
    deferred mode reports what earlier calls have left.  The operator adds to the
    counter and copies it to the pinned mirror on its stream."""
    if _index_check_mode == "off":
        return None
    slot = _index_counter(device)
    if not torch.cuda.is_current_stream_capturing():
        # what earlier deferred (or captured) calls have left
        _report_index_errors(slot, what + " (an earlier call)")
    return slot


def _oob_end(slot, what):
    if _index_check_mode == "immediate" and not torch.cuda.is_current_stream_capturing():
        torch.cuda.current_stream(slot[0].device).synchronize()
        _report_index_errors(slot, what)


def embedding(weight, indices, padding_idx=None, max_norm=None, norm_type=2.0,
              scale_grad_by_freq=False, sparse=False):
    """NestedTensor_embedding (functions.cpp:14-63): one gather over the packed
    index buffer (nt_gather_rows); the result gets a trailing regular dim of
    weight.size(1).  padding_idx, scale_grad_by_freq and sparse only shape
    gradients and are accepted for the call signature; max_norm would modify the
    table and is refused."""
    if max_norm is not None:
        raise NotImplementedError("embedding on a NestedTensor: max_norm is not supported.")
    if not isinstance(indices, NestedTensorImpl) or isinstance(weight, NestedTensorImpl):
        raise NotImplementedError("embedding: expected a dense weight and NestedTensor indices.")
    if weight.dim() != 2:
        raise RuntimeError("'weight' must be 2-D")
    idx = indices.buffer
    _C.require_device(idx, "embedding")
    if idx.dtype not in (torch.int64, torch.int32):
        raise RuntimeError("Expected tensor for argument #1 'indices' to have one of the following scalar "
                           "types: Long, Int; but got %s instead" % idx.dtype)
    if weight.device != idx.device:
        raise RuntimeError("embedding: weight and indices must be on the same device")
    E = weight.size(1)
    slot = _oob_begin(weight.device, "embedding")
    if slot is None:
        out = _embedding_packed(weight, idx, None, None)
    else:
        out = _embedding_packed(weight, idx, slot[0], slot[1])
        _oob_end(slot, "embedding")
    out = out.reshape(-1)
    if indices.sizes.dim() == 0:
        sizes = indices.sizes
    else:
        sizes = torch.cat([indices.sizes, torch.full((indices.B, 1), E, dtype=torch.int64)], 1)
    return NestedTensorImpl(out, sizes)


def embedding_bag(input, weight, offsets=None, max_norm=None, norm_type=2, scale_grad_by_freq=False,
                  mode="mean", sparse=False, per_sample_weights=None, include_last_offset=False,
                  padding_idx=None):
    """_nn_functional_embedding_bag (nested/nested.py:43-118): the bags are the
    constituents of a nested tensor of 1-D index tensors; its device offsets array
    is the offsets argument the reference rebuilds in a host loop.  Returns a
    dense [B, E] tensor."""
    if max_norm is not None:
        raise NotImplementedError("NestedTensor embedding_bag: max_norm is not supported")
    if per_sample_weights is not None:
        raise NotImplementedError("NestedTensor embedding_bag: per_sample_weights is not supported")
    if not isinstance(input, NestedTensorImpl):
        raise NotImplementedError("embedding_bag: expected NestedTensor indices.")
    if input.dim() == 2:
        if offsets is not None:
            raise ValueError("if input is 2D, then offsets has to be None, as input is treated is a "
                             "mini-batch of fixed length sequences. However, found offsets of type %s"
                             % type(offsets))
    else:
        raise ValueError("input has to be 2D NestedTensor, but got NestedTensor of dimension %d"
                         % input.dim())
    modes = {"sum": 0, "mean": 1, "max": 2}
    if mode not in modes:
        raise ValueError("mode has to be one of sum, mean or max")
    if mode == "max" and scale_grad_by_freq:
        raise ValueError("max mode does not support scaling the gradient by the frequency")
    if mode == "max" and sparse:
        raise ValueError("max mode does not support sparse weights")
    if padding_idx is not None:
        raise NotImplementedError("padding_idx is not supported for NestedTensor embedding_bag")
    idx = input.buffer
    _C.require_device(idx, "embedding_bag")
    if weight.dim() != 2 or weight.device != idx.device:
        raise RuntimeError("embedding_bag: weight must be 2-D on the device of the indices")
    slot = _oob_begin(weight.device, "embedding_bag")
    if slot is None:
        return _embedding_bag_packed(weight, idx, input.offsets_dev(), modes[mode], None, None)
    out = _embedding_bag_packed(weight, idx, input.offsets_dev(), modes[mode], slot[0], slot[1])
    _oob_end(slot, "embedding_bag")
    return out


def to_sparse_csr(impl):
    """NestedTensor_to_sparse_csr (nested_tensor_impl.h:326-349): crow_indices are
    the offsets array, col_indices one arange per constituent (nt_ragged_arange),
    values the packed buffer."""
    if impl.dim() != 2:
        raise RuntimeError("Given tensor must be of dimension 2, got dimension %d" % impl.dim())
    buf = impl.buffer
    _C.require_device(buf, "to_sparse_csr")
    crow = impl.offsets_dev()
    col = torch.empty(buf.numel(), dtype=torch.int64, device=buf.device)
    mx = impl.max_sizes()
    with _C.on_device(buf.device):
        _C.check(_C.lib.nt_ragged_arange(_C.ptr(crow), impl.B, mx[0] if mx else 0, _C.ptr(col),
                                         _C.current_stream(buf.device)))
    return torch.sparse_csr_tensor(crow, col, buf, size=(impl.B, mx[0] if mx else 0))


def to_packed_sequence(impl):
    """NestedTensor.to_packed_sequence (nested/nested.py:484-488) without the
    unbind: the time-major row order of torch.nn.utils.rnn.pack_sequence(...,
    enforce_sorted=False) is built on the device (nt_packed_sequence_index) and
    the token rows are moved by one gather (nt_gather_rows)."""
    if impl.dim() < 3:
        raise RuntimeError("NestedTensor should consistent of 2d Tensors of size L x *")
    buf = impl.buffer
    _C.require_device(buf, "to_packed_sequence")
    opt = impl.opt_sizes()
    if any(v is None for v in opt[2:]):
        raise RuntimeError("to_packed_sequence: the trailing dims of the constituents must be regular")
    if impl.has_empty_constituent():
        raise RuntimeError("Length of all samples has to be greater than 0, but found an element in "
                           "'lengths' that is <= 0")
    trailing = [int(v) for v in opt[2:]]
    row_elems = 1
    for v in trailing:
        row_elems *= v
    data, batch_sizes, sorted_dev, rank_dev = _packed_sequence_lowered(
        buf, impl.sizes[:, 0].contiguous(), impl.row_offsets_dev(), row_elems)
    return torch.nn.utils.rnn.PackedSequence(data.reshape([data.size(0)] + trailing), batch_sizes, sorted_dev,
                                             rank_dev)


# ---- channels-last ragged images: per-constituent transposes ------------------------

def _transpose_tile(max_rows, max_cols, elem_bytes):
    """Tile shape for nt_transpose_ragged: the strip kernels (a workgroup per 2048
    bytes of the long side) when the other side is at most 16, images of a few
    channels; 64 x 64 otherwise.  The larger tiles the library also accepts keep
    fewer workgroups in flight and measured slower on every image shape tried."""
    strip = 2048 // elem_bytes
    if max_rows <= 16 and max_cols > 64:
        return 16, strip
    if max_cols <= 16 and max_rows > 64:
        return strip, 16
    return 64, 64


def _transpose_constituents(impl, rows, cols, new_sizes, which):
    """Every constituent, seen as a row-major [rows[b], cols[b]] matrix, is
    transposed in place of its slot of the packed buffer (nt_transpose_ragged).
    The device copy of (rows, cols, tile offsets) depends on the nested size and
    the direction `which` only and is kept with the nested size."""
    buf = impl.buffer
    _C.require_device(buf, "transpose")
    B = impl.B
    which = (which, buf.element_size())       # the tile shape depends on the element size
    if impl._transpose_meta is None:
        impl._transpose_meta = {}
    cached = impl._transpose_meta.get(which)
    if cached is not None and cached[0].device == buf.device:
        meta_dev, total_tiles, tr, tc = cached
    else:
        tr, tc = _transpose_tile(int(rows.max()) if B else 0, int(cols.max()) if B else 0, buf.element_size())
        if (tr, tc) == (64, 64) and buf.element_size() == 2 and bool((rows % 64 != 0).any()):
            # output rows that do not begin on 128-byte lines: the kernel that gives every
            # output row its own line-aligned window (tile shape recorded as 0 x 0)
            tr = tc = 0
            tiles = torch.where((rows > 0) & (cols > 0), ((rows + 63) // 64 + 1) * ((cols + 63) // 64),
                                torch.zeros_like(rows))
        else:
            tiles = ((rows + tr - 1) // tr) * ((cols + tc - 1) // tc)
        meta = torch.zeros((3, B + 1), dtype=torch.int64)
        meta[0, :B], meta[1, :B] = rows, cols
        meta[2, 1:] = torch.cumsum(tiles, 0)
        total_tiles = int(meta[2, B])
        meta_dev = meta.to(buf.device)
        impl._transpose_meta[which] = (meta_dev, total_tiles, tr, tc)
    out = torch.empty_like(buf)
    if total_tiles:
        with _C.on_device(buf.device):
            if tr == 0:
                _C.check(_C.lib.nt_transpose_ragged_lines(
                    _C.ptr(buf), _C.ptr(out), _C.ptr(impl.offsets_dev()), _C.ptr(meta_dev[0]),
                    _C.ptr(meta_dev[1]), _C.ptr(meta_dev[2]), B, total_tiles, buf.element_size(),
                    _C.current_stream(buf.device)))
            else:
                _C.check(_C.lib.nt_transpose_ragged(
                    _C.ptr(buf), _C.ptr(out), _C.ptr(impl.offsets_dev()), _C.ptr(meta_dev[0]),
                    _C.ptr(meta_dev[1]), _C.ptr(meta_dev[2]), B, total_tiles, tr, tc, buf.element_size(),
                    _C.current_stream(buf.device)))
    res = NestedTensorImpl(out, new_sizes)
    res._offsets_dev = impl._offsets_dev      # the constituents keep their extents
    return res


def transpose_nchw_nhwc(impl):
    """transpose_nchw_nhwc (transpose.cpp:122-146): constituents [C, H_i, W_i]
    with a regular C become [H_i, W_i, C]."""
    impl = contiguous(impl)
    if impl.dim() != 4:
        raise RuntimeError("transpose_nchw_nhwc needs 4d input.")
    if impl.opt_sizes()[1] is None:
        raise RuntimeError("Expected first dimension to be regular.")
    s = impl.sizes
    return _transpose_constituents(impl, s[:, 0], s[:, 1] * s[:, 2],
                                   torch.stack([s[:, 1], s[:, 2], s[:, 0]], 1).contiguous(), "nchw_nhwc")


def transpose_nhwc_nchw(impl):
    """transpose_nhwc_nchw (transpose.cpp:183-204): constituents [H_i, W_i, C]
    with a regular C become [C, H_i, W_i]."""
    impl = contiguous(impl)
    if impl.dim() != 4:
        raise RuntimeError("transpose_nhwc_nchw needs 4d input.")
    if impl.opt_sizes()[3] is None:
        raise RuntimeError("Expected last dimension to be regular.")
    s = impl.sizes
    return _transpose_constituents(impl, s[:, 0] * s[:, 1], s[:, 2],
                                   torch.stack([s[:, 2], s[:, 0], s[:, 1]], 1).contiguous(), "nhwc_nchw")


def is_contiguous(impl, memory_format=torch.contiguous_format):
    """get_is_contiguous (nested_tensor_impl.h:151-160)."""
    if memory_format in (torch.contiguous_format, 0):
        return not impl.channels_last
    if memory_format in (torch.channels_last, 2):
        # an empty buffer is contiguous in both senses (Packed.h:131-133)
        return impl.channels_last or (impl.buffer.numel() == 0 and not impl.channels_last)
    raise RuntimeError("is_contiguous does not support memory format " + str(memory_format))


def contiguous(impl, memory_format=torch.contiguous_format):
    """NestedTensor_contiguous (nested_tensor_impl.cpp:157-198): the same nested
    tensor with its buffer in the requested layout.  Going to channels-last is
    the NCHW -> NHWC transpose of every constituent with the nested size kept
    (:182-194); coming back views the buffer as [H_i, W_i, C] constituents and
    transposes them the other way (:165-179)."""
    if memory_format == torch.preserve_format:
        raise RuntimeError("preserve memory format is unsupported by the contiguous operator")
    if memory_format == torch.contiguous_format:
        if not impl.channels_last:
            return impl
        s = impl.sizes
        as_nhwc = NestedTensorImpl(impl.buffer, torch.stack([s[:, 1], s[:, 2], s[:, 0]], 1).contiguous())
        as_nhwc._offsets_dev = impl._offsets_dev
        out = transpose_nhwc_nchw(as_nhwc)
        return impl.with_buffer(out.buffer, channels_last=False)
    if memory_format == torch.channels_last:
        if impl.channels_last:
            return impl
        if impl.dim() != 4:
            raise RuntimeError("ChannelsLast memory format requires 4 dim input.")
        if impl.buffer.numel() == 0:
            return impl.with_buffer(impl.buffer, channels_last=True)
        out = transpose_nchw_nhwc(impl)
        return impl.with_buffer(out.buffer, channels_last=True)
    raise RuntimeError("Given memory format " + str(memory_format) +
                       " not supported by NestedTensor_contiguous.")
