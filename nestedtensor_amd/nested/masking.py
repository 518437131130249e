"""Dense -> nested conversions (nestedtensor/nested/masking.py:12-50 and the
native nt_from_tensor_mask they call, nestedtensor/csrc/masking.cpp:181-249).

The reference walks the mask on the host with one ``.item<bool>()`` per element.
Here the mask is reduced on the device: keep-counts per mask row (wavefront
ballot + popcount), an exclusive scan of the counts, and a compaction of the
kept data.  Only the per-row counts travel to the host, where the nested size
is derived from them; the output size depends on the mask, so that one
device-to-host copy cannot be avoided.
"""

import torch

from .. import _C
from .. import ops
from ..impl import NestedTensorImpl
from . import nested


def nested_tensor_from_padded_tensor(tensor, nested_dim=1, padding=-1):
    """``nested_tensor_from_tensor_mask(tensor, tensor != padding, nested_dim)``
    (nested/masking.py:12-14).  On the device the mask is never materialised: the
    keep-counts are taken straight from the data (nt_value_row_counts)."""
    if tensor is None:
        raise RuntimeError("Tensor can't be undefined (None).")
    if tensor.dim() == 0:
        raise RuntimeError("Can't construct nested tensor from a scalar.")
    if nested_dim == 0:
        raise RuntimeError("Nested dimension can't be 0.")
    if nested_dim is not None and nested_dim > tensor.dim():
        raise RuntimeError("Nested dimension ({0}) can't be bigger than data tensor dimension ({1}).".format(
            nested_dim, tensor.dim()))
    if not tensor.is_cuda or tensor.dim() < 2 or tensor.numel() < 2 or tensor.dtype not in _C.ELEM_TYPE:
        mask = (tensor != padding)
        return nested_tensor_from_tensor_mask(tensor, mask, nested_dim)
    buffer, sizes = torch.ops.nestedtensor.nt_from_padded_tensor(tensor, float(padding), nested_dim)
    return nested.NestedTensor(NestedTensorImpl(buffer, sizes)).contiguous()


# Constructs nested tensor from passed tensor and mask.
def nested_tensor_from_tensor_mask(tensor, mask, nested_dim=1):
    if tensor is None:
        raise RuntimeError("Tensor can't be undefined (None).")

    if mask is None:
        raise RuntimeError("Mask can't be undefined (None).")

    # Scalar was passed
    if tensor.dim() == 0:
        raise RuntimeError("Can't construct nested tensor from a scalar.")

    if nested_dim == 0:
        raise RuntimeError("Nested dimension can't be 0.")

    if nested_dim is not None and nested_dim > tensor.dim():
        raise RuntimeError("Nested dimension ({0}) can't be bigger than data tensor dimension ({1}).".format(
            nested_dim, tensor.dim()))

    if tensor.numel() == 0 and mask.numel() != 0:
        raise RuntimeError("Data tensor can't be emtpy if a mask has values.")

    if tensor.numel() != 0 and mask.numel() == 0:
        raise RuntimeError(
            "Mask tensor can't be emtpy if a data tensor has values.")

    return nt_from_tensor_mask(tensor, mask, nested_dim)


def nt_from_tensor_mask(tensor, mask, nested_dim):
    buffer, sizes = torch.ops.nestedtensor.nt_from_tensor_mask(
        tensor, mask, nested_dim)
    return nested.NestedTensor(NestedTensorImpl(buffer, sizes)).contiguous()


def from_padded_tensor(padded, target):
    """Length-based un-pad (from_padded_tensor, masking.cpp:459-533; C++-only in
    the reference): the entries of ``padded`` inside ``target``'s nested size,
    as a NestedTensor.  ``target`` is a NestedTensor or its nested_size()."""
    if isinstance(target, nested.NestedTensor):
        impl = target._impl
    else:
        shapes = [list(s) for s in target]
        sizes = torch.tensor(shapes, dtype=torch.int64).reshape(len(shapes), padded.dim() - 1)
        impl = NestedTensorImpl(torch.empty(0, dtype=padded.dtype, device=padded.device), sizes)
    return nested.NestedTensor(ops.from_padded_tensor(padded, impl))


# ---------------------------------------------------------------------------


def _empty_nt():
    # nested_tensor([]): Packed.h:77-79, EfficientSizeNode.h:10-12
    return NestedTensorImpl(torch.ones(0), torch.zeros((), dtype=torch.int64))


def _keep_all(tensor):
    """Every tensor[i] is a constituent, whole (masking.cpp:228-232)."""
    B = tensor.size(0)
    if B == 0:
        return _empty_nt()
    sizes = torch.tensor([list(tensor.shape[1:])] * B, dtype=torch.int64).reshape(B, tensor.dim() - 1)
    return NestedTensorImpl(tensor.contiguous().reshape(-1).clone(), sizes)


def _as_byte_mask(mask):
    if mask.dtype == torch.bool:
        return mask.contiguous().view(torch.uint8)
    if mask.dtype == torch.uint8:
        return mask.contiguous()
    return (mask != 0).contiguous().view(torch.uint8)


def _compact(data, bmask, R, M, chunk_elems, total_kept, counts_dev):
    """Scan the per-row keep-counts and move the kept chunks (nt_exclusive_scan_i32,
    nt_compact_rows).  Returns the packed 1-D buffer."""
    dev = data.device
    out = torch.empty(total_kept * chunk_elems, dtype=data.dtype, device=dev)
    if total_kept == 0 or chunk_elems == 0:
        return out
    row_offsets = torch.empty(R + 1, dtype=torch.int64, device=dev)
    ws_bytes = _C.lib.nt_scan_workspace_bytes(R)
    ws = torch.empty(max(ws_bytes, 8), dtype=torch.uint8, device=dev) if ws_bytes else None
    with _C.on_device(dev):
        stream = _C.current_stream(dev)
        _C.check(_C.lib.nt_exclusive_scan_i32(
            _C.ptr(counts_dev), R, _C.ptr(row_offsets), _C.ptr(ws), ws_bytes, stream))
        _C.check(_C.lib.nt_compact_rows(
            _C.ptr(data), _C.ptr(bmask), _C.ptr(row_offsets), R, M,
            chunk_elems * data.element_size(), _C.ptr(out), stream))
    return out


def _row_counts(bmask, R, M):
    """Keep-count and is-a-prefix flag per row of a byte mask [R, M]."""
    counts = torch.empty(R, dtype=torch.int32, device=bmask.device)
    prefix = torch.empty(R, dtype=torch.uint8, device=bmask.device)
    with _C.on_device(bmask.device):
        _C.check(_C.lib.nt_mask_row_counts(
            _C.ptr(bmask), R, M, _C.ptr(counts), _C.ptr(prefix), _C.current_stream(bmask.device)))
    return counts, prefix


def _value_row_counts(tensor, padding, R, M):
    """The same for the mask ``tensor != padding`` without building it."""
    counts = torch.empty(R, dtype=torch.int32, device=tensor.device)
    prefix = torch.empty(R, dtype=torch.uint8, device=tensor.device)
    with _C.on_device(tensor.device):
        _C.check(_C.lib.nt_value_row_counts(
            _C.ptr(tensor), _C.ELEM_TYPE[tensor.dtype], float(padding), R, M, _C.ptr(counts),
            _C.ptr(prefix), _C.current_stream(tensor.device)))
    return counts, prefix


def _from_mask_native(tensor, mask, nested_dim):
    """nt_from_tensor_mask (masking.cpp:181-249) at nested_dim 1."""
    if nested_dim != 1:
        raise RuntimeError("Only nested_dim of 1 is currently supported.")
    # masking.cpp:228-234: an empty mask or a single true keeps everything, a
    # single false keeps nothing.
    if mask.numel() == 0:
        return _keep_all(tensor)
    if mask.numel() == 1:
        return _keep_all(tensor) if bool(mask.reshape(-1)[0].item()) else _empty_nt()

    if tensor.device != mask.device:
        raise RuntimeError("tensor and mask must be on the same device.")
    _C.require_device(tensor, "nested_tensor_from_tensor_mask")
    if mask.dim() > tensor.dim():
        raise RuntimeError("Mask has more dimensions than the data tensor.")
    B = tensor.size(0)
    if mask.size(0) < B:
        raise IndexError("index %d is out of bounds for dimension 0 with size %d" % (mask.size(0), B))
    mask = mask[:B]
    tensor = tensor.contiguous()
    bmask = _as_byte_mask(mask)
    inner_mask_shape = tuple(mask.shape[1:])
    inner_numel = 1
    for v in inner_mask_shape:
        inner_numel *= v

    if inner_numel == 1:
        # One mask value per constituent (masking.cpp:186-201 on mask[i]):
        # true keeps tensor[i] whole; false drops it (0-d mask[i]) or leaves an
        # empty constituent of shape [1, .., 1, 0].
        row_elems = tensor[0].numel() if B > 0 else 0
        counts, _ = _row_counts(bmask, 1, B)
        kept = int(counts.item())
        keep_host = mask.reshape(B).to(torch.bool).cpu()
        buf = _compact(tensor, bmask, 1, B, row_elems, kept, counts)
        full = list(tensor.shape[1:])
        if mask.dim() == 1:
            if kept == 0:
                return _empty_nt()
            sizes = torch.tensor([full] * kept, dtype=torch.int64).reshape(kept, len(full))
            return NestedTensorImpl(buf, sizes)
        empty_shape = [1] * (mask.dim() - 2) + [0]
        shapes = [full if bool(k) else empty_shape for k in keep_host]
        return _impl_from_shapes(buf, shapes)

    if tuple(tensor.shape[1:mask.dim()]) != inner_mask_shape:
        raise RuntimeError(
            "Mask of shape %s does not match the leading dimensions of the data tensor %s."
            % (tuple(mask.shape), tuple(tensor.shape)))

    return _from_rows(tensor, mask.dim(), lambda R, M: _row_counts(bmask, R, M), lambda: bmask)


def _from_value_native(tensor, padding, nested_dim):
    """nested_tensor_from_padded_tensor on the device: the mask is
    ``tensor != padding`` with the dims of the data."""
    if nested_dim != 1:
        raise RuntimeError("Only nested_dim of 1 is currently supported.")
    _C.require_device(tensor, "nested_tensor_from_padded_tensor")
    tensor = tensor.contiguous()
    return _from_rows(tensor, tensor.dim(),
                      lambda R, M: _value_row_counts(tensor, padding, R, M),
                      lambda: _as_byte_mask(tensor != padding))


# from this many mask rows on, the lowest mask level is summarised on the device
_DEVICE_REDUCE_ROWS = 32768


def _from_rows(tensor, mask_dims, count_rows, byte_mask):
    """General case of nt_from_tensor_mask (masking.cpp:203-222) for a mask over
    the first `mask_dims` dims of `tensor`.  Rows = everything but the last mask
    dim.  `count_rows(R, M)` gives device (counts, prefix flags); `byte_mask()`
    materialises the mask, which only the non-prefix path needs."""
    B = tensor.size(0)
    inner_mask_shape = tuple(tensor.shape[1:mask_dims])
    M = tensor.size(mask_dims - 1)
    R = 1
    for v in tensor.shape[:mask_dims - 1]:
        R *= v
    rest = list(tensor.shape[mask_dims:])
    chunk = 1
    for v in rest:
        chunk *= v
    counts_dev, prefix_dev = count_rows(R, M)
    # Nested size from the counts: at every mask level the extent is the number
    # of children that keep anything (masking.cpp:203-222); the selection must
    # be rectangular or at::stack would have thrown.  `leading`: kept children
    # come first at every level.
    count_shape = (B,) + inner_mask_shape[:-1]
    if R >= _DEVICE_REDUCE_ROWS:
        # many rows: the lowest level is reduced on the device and only the
        # per-constituent summaries cross to the host, in one copy
        cd = counts_dev.reshape(count_shape).to(torch.int64)
        flat = cd.reshape(B, -1)
        pieces = [flat.sum(1), flat.max(1).values, prefix_dev.min().to(torch.int64).reshape(1)]
        has_level = cd.dim() > 1
        if has_level:
            alive_d = cd > 0
            lead_d = (alive_d[..., 1:] <= alive_d[..., :-1]).all() if alive_d.size(-1) > 1 \
                else torch.ones((), dtype=torch.bool, device=cd.device)
            pieces += [lead_d.to(torch.int64).reshape(1), alive_d.sum(-1).reshape(-1)]
        host = torch.cat(pieces).cpu()
        total, extents = host[:B], [host[B:2 * B]]
        leading = bool(host[2 * B])
        alive = None
        if has_level:
            leading = leading and bool(host[2 * B + 1])
            c = host[2 * B + 2:].reshape(count_shape[:-1])
            extents.append(c.reshape(B, -1).max(1).values)
            alive = c > 0
    else:
        # one device-to-host copy: the row counts plus "every row keeps a prefix"
        if R > 0:
            host = torch.cat([counts_dev, prefix_dev.min().to(torch.int32).reshape(1)]).cpu()
            counts, leading = host[:-1], bool(host[-1])
        else:
            counts, leading = counts_dev.cpu(), True
        counts = counts.to(torch.int64).reshape(count_shape)
        flat = counts.reshape(B, -1)
        total = flat.sum(1)
        extents = [flat.max(1).values]
        alive = counts > 0
    while alive is not None and alive.dim() > 1:
        if leading and alive.size(-1) > 1:
            leading = bool((alive[..., 1:] <= alive[..., :-1]).all())
        c = alive.sum(-1)
        extents.append(c.reshape(B, -1).max(1).values)
        alive = c > 0
    extents = torch.stack(list(reversed(extents)), 1)          # [B, k]
    if bool((extents.prod(1) != total).any()):
        raise RuntimeError("stack expects each tensor to be equal size: the mask does not select "
                           "a rectangular block in every constituent.")
    empty_shape = list(inner_mask_shape[:-1]) + [0]
    shapes = [e + rest if t else empty_shape for t, e in zip(total.tolist(), extents.tolist())]
    if leading:
        # Every constituent keeps a leading box: this is the length-based un-pad
        # (nt_remove_padding) with the nested size just derived.
        target = _impl_from_shapes(torch.empty(0, dtype=tensor.dtype, device=tensor.device), shapes)
        return ops.from_padded_tensor(tensor, target)
    buf = _compact(tensor, byte_mask(), R, M, chunk, int(total.sum()), counts_dev)
    return _impl_from_shapes(buf, shapes)


def _impl_from_shapes(buf, shapes):
    if len(shapes) == 0:
        return _empty_nt()
    d = len(shapes[0])
    for s in shapes:
        if len(s) != d:
            raise RuntimeError(
                "Given Tensor / NestedTensor constiuent of dimension %d doesn't match another "
                "constiuent of dimension %d. " % (len(s), d))
    sizes = torch.tensor(shapes, dtype=torch.int64).reshape(len(shapes), d)
    return NestedTensorImpl(buf, sizes)


def _nt_from_tensor_mask_op(tensor, mask, nested_dim):
    impl = _from_mask_native(tensor, mask, nested_dim)
    return impl.buffer, impl.sizes


# The op takes plain tensors, so it is registered with the dispatcher itself,
# one implementation for every device.  A dispatcher op cannot return the Python
# wrapper, so it returns the lowered pair (packed buffer, sizes[B, D]) that
# nt_from_tensor_mask() above wraps; sizes is 0-d for an empty result.
ops._lib.impl("nt_from_tensor_mask", _nt_from_tensor_mask_op, "CompositeExplicitAutograd")


# masking.cpp:653-655: an op on plain tensors, one implementation for every device
ops._lib.impl("merge_tensor_mask", ops.merge_tensor_mask, "CompositeExplicitAutograd")


def _nt_from_padded_tensor_op(tensor, padding, nested_dim):
    impl = _from_value_native(tensor, padding, nested_dim)
    return impl.buffer, impl.sizes


# No counterpart among the reference's ops (it builds the mask in Python,
# nested/masking.py:12-14); same lowered return convention as above.
ops._lib.define("nt_from_padded_tensor(Tensor tensor, float padding, int nested_dim) -> (Tensor, Tensor)")
ops._lib.impl("nt_from_padded_tensor", _nt_from_padded_tensor_op, "CompositeExplicitAutograd")
