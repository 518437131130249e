"""Dense -> nested conversions (nestedtensor/nested/masking.py:12-50 and the
native nt_from_tensor_mask they call, nestedtensor/csrc/masking.cpp:181-249).

The reference walks the mask on the host with one ``.item<bool>()`` per element.
Here the mask is reduced on the device: keep-counts per mask row (wavefront
ballot + popcount), an exclusive scan of the counts, and a compaction of the
kept data.  Only the per-row counts travel to the host, where the nested size
is derived from them; the output size depends on the mask, so that one
device-to-host copy cannot be avoided.  This module holds the argument checks
of the Python entry points; the work is done by operators of the extension.
"""

import torch

from .. import _C
from .. import ops
from ..impl import NestedTensorImpl
from . import nested

# The conversions themselves are operators of the C++ extension
# (csrc/torch_ops.cpp): row counts on the device, one copy of them into pinned
# host memory, the nested size derived from them in C++, then un-pad or
# compaction.  torch.ops.nestedtensor.nt_from_tensor_mask / nt_from_padded_tensor
# return the pair (buffer, sizes); the *_lowered variants also hand back the
# device metadata they had to build.
_from_tensor_mask_lowered = _C.ops.from_tensor_mask_lowered.default
_from_padded_value_lowered = _C.ops.from_padded_value_lowered.default


def _check_dense_arguments(tensor, nested_dim, mask=None, with_mask=False):
    """The argument errors of the reference's entry point (nested/masking.py:18-41),
    in its order and wording; one table, walked until the first that applies."""
    checks = [(tensor is None, "Tensor can't be undefined (None).")]
    if with_mask:
        checks.append((mask is None, "Mask can't be undefined (None)."))
    for failed, message in checks:
        if failed:
            raise RuntimeError(message)
    rank = tensor.dim()
    checks = [
        (rank == 0, "Can't construct nested tensor from a scalar."),
        (nested_dim == 0, "Nested dimension can't be 0."),
        (nested_dim is not None and nested_dim != 0 and nested_dim > rank,
         "Nested dimension ({0}) can't be bigger than data tensor dimension ({1}).".format(nested_dim, rank)),
    ]
    if with_mask:
        n_data, n_mask = tensor.numel(), mask.numel()
        checks.append((n_data == 0 and n_mask != 0, "Data tensor can't be emtpy if a mask has values."))
        checks.append((n_data != 0 and n_mask == 0, "Mask tensor can't be emtpy if a data tensor has values."))
    for failed, message in checks:
        if failed:
            raise RuntimeError(message)


def _on_host(nested_result):
    impl = nested_result._impl
    return nested.NestedTensor(impl.with_buffer(impl.buffer.cpu()))


def nested_tensor_from_padded_tensor(tensor, nested_dim=1, padding=-1):
    """``nested_tensor_from_tensor_mask(tensor, tensor != padding, nested_dim)``
    (nested/masking.py:12-14).  On the device the mask is never materialised: the
    keep-counts are taken straight from the data (nt_value_row_counts).  A host
    tensor is staged through the device and the result returned to the host."""
    _check_dense_arguments(tensor, nested_dim)
    if not tensor.is_cuda:
        staged = tensor.to(_C.staging_device("nested_tensor_from_padded_tensor"))
        return _on_host(nested_tensor_from_padded_tensor(staged, nested_dim, padding))
    if tensor.dim() < 2 or tensor.numel() < 2 or tensor.dtype not in _C.ELEM_TYPE:
        return nt_from_tensor_mask(tensor, tensor != padding, nested_dim)
    return _wrap_lowered(*_from_padded_value_lowered(tensor, float(padding), nested_dim))


def nested_tensor_from_tensor_mask(tensor, mask, nested_dim=1):
    """The nested tensor of the entries of ``tensor`` that ``mask`` keeps
    (nested/masking.py:17-43)."""
    _check_dense_arguments(tensor, nested_dim, mask, with_mask=True)
    return nt_from_tensor_mask(tensor, mask, nested_dim)


def _wrap_lowered(buffer, sizes, sizes_dev, offsets_dev):
    """NestedTensor over the lowered result of a conversion; the device copies of
    the nested size and of the offsets are adopted when the conversion built them."""
    impl = NestedTensorImpl(buffer, sizes)
    if sizes_dev.numel() > 0 or (sizes.dim() == 2 and sizes.numel() == 0 and offsets_dev.numel() > 0):
        impl.adopt_device_metadata(sizes_dev, offsets_dev)
    return nested.NestedTensor(impl).contiguous()


def nt_from_tensor_mask(tensor, mask, nested_dim):
    if not tensor.is_cuda and mask.numel() > 1:      # smaller masks are answered on the host
        dev = _C.staging_device("nested_tensor_from_tensor_mask")
        return _on_host(nt_from_tensor_mask(tensor.to(dev), mask.to(dev), nested_dim))
    return _wrap_lowered(*_from_tensor_mask_lowered(tensor, mask, nested_dim))


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


