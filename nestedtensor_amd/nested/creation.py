"""Constructors (nestedtensor/nested/creation.py:9-26 and the native
nested_tensor_impl they call, nestedtensor/csrc/creation.cpp:28-222)."""

import torch

from .. import ops
from .. import _C
from ..impl import NestedTensorImpl
from . import nested

_pack_device = _C.ops.pack_device.default

_HINT = (
    "To form a valid NestedTensor all Tensor / NestedTensor constiuents of the given list must be "
    "of the same dimension, layout, device, scalar type and either all or none require gradients.")


# host constituents of at least this many bytes on average are copied to the
# device one by one instead of being packed on the host first
_DIRECT_COPY_BYTES = 256 * 1024


def _verify_variables(tensors):
    # creation.cpp:28-171
    first = tensors[0]
    for t in tensors:
        if t.dim() != first.dim():
            raise RuntimeError(
                "Given Tensor / NestedTensor constiuent of dimension %d doesn't match another "
                "constiuent of dimension %d. %s" % (t.dim(), first.dim(), _HINT))
        if t.layout != first.layout:
            raise RuntimeError(
                "Given Tensor / NestedTensor constiuent of layout %s doesn't match another "
                "constiuent of layout %s. %s" % (t.layout, first.layout, _HINT))
        if t.device != first.device:
            raise RuntimeError(
                "Given Tensor / NestedTensor constiuent of device %s doesn't match another "
                "constiuent of device %s. " % (t.device, first.device))
        if t.dtype != first.dtype:
            raise RuntimeError(
                "Given Tensor / NestedTensor constiuent of scalar type %s doesn't match another "
                "constiuent of scalar type %s. " % (t.dtype, first.dtype))
        if t.requires_grad != first.requires_grad:
            raise RuntimeError(
                "Given Tensor / NestedTensor constiuent requires gradient in contrast to another "
                "constiuent. " + _HINT)


def nested_tensor_impl(data, dtype, device, requires_grad, pin_memory, channels_last):
    """creation.cpp:191-222.  The constituents are copied into one packed
    buffer (never aliased), cast to ``dtype`` and moved to ``device``."""
    if requires_grad:
        raise RuntimeError(
            "This version of nestedtensor currently does not support autograd. Please open an "
            "issue on https://github.com/pytorch/nestedtensor if you need this.")
    if channels_last:
        # creation.cpp:217-219: pack row-major, then change the layout
        impl = nested_tensor_impl(data, dtype, device, requires_grad, pin_memory, False)
        return ops.contiguous(impl, torch.channels_last)
    if isinstance(data, nested.NestedTensor):
        data = data.unbind()   # a NestedTensor is a sequence of its constituents
    if torch.is_tensor(data) or not isinstance(data, (list, tuple)):
        raise TypeError("nested_tensor(): argument 'data' must be a sequence of Tensors, not %s"
                        % type(data).__name__)
    tensors = list(data)
    for t in tensors:
        if isinstance(t, nested.NestedTensor):
            raise RuntimeError("Currently do not support NestedTensor entries.")
        if not torch.is_tensor(t):
            raise RuntimeError("Currently only supporting a sequence of Tensors.")
    device = torch.device(device)
    if len(tensors) == 0:
        # Packed.h:77-79: at::ones({0}); EfficientSizeNode.h:10-12: 0-d sizes
        buffer = torch.ones(0).to(device, dtype)
        return NestedTensorImpl(buffer, torch.zeros((), dtype=torch.int64))
    src_device = tensors[0].device
    if src_device.type == "cuda":
        # constituents already in HBM: checked, sized and gathered into the packed
        # buffer by one operator of the extension (one launch, one metadata upload)
        buffer, sizes, sizes_dev, offsets = _pack_device(tensors)
        impl = NestedTensorImpl(buffer, sizes)
        impl._sizes_dev, impl._offsets_dev = sizes_dev, offsets
        if buffer.dtype != dtype or buffer.device != device:
            impl = impl.with_buffer(buffer.to(device, dtype))
        return impl
    _verify_variables(tensors)
    sizes = torch.tensor([list(t.shape) for t in tensors], dtype=torch.int64).reshape(
        len(tensors), tensors[0].dim())
    total = int(sizes.prod(1).sum())
    if (device.type == "cuda" and src_device.type == "cpu"
            and total * tensors[0].element_size() >= len(tensors) * _DIRECT_COPY_BYTES):
        # large host constituents: each goes straight into its slot of the device
        # buffer; packing them on the host first would cost one more pass over
        # the data than the transfer itself
        buffer = torch.empty(total, dtype=dtype, device=device)
        off = 0
        for t in tensors:
            n = t.numel()
            buffer[off:off + n].copy_(t.detach().reshape(-1))
            off += n
        return NestedTensorImpl(buffer, sizes)
    # host constituents: pack on the host, then one H2D copy of the packed
    # buffer (what creation.cpp:210-216 does).
    buffer = torch.cat([t.detach().contiguous().reshape(-1) for t in tensors])
    if pin_memory and device.type == "cpu":
        buffer = buffer.to(dtype).pin_memory()
    else:
        buffer = buffer.to(device, dtype)
    if buffer.data_ptr() == tensors[0].data_ptr() and buffer.numel() > 0:
        buffer = buffer.clone()  # a single constituent must still be copied
    return NestedTensorImpl(buffer, sizes)


def nested_tensor(data, dtype=None, device=None, requires_grad=False, pin_memory=False,
                  channels_last=False):
    """A NestedTensor that owns a packed copy of the tensors in ``data``.  Keyword
    arguments are those of torch.tensor (nested/creation.py:9-19): dtype defaults
    to torch's default dtype, device to the host; channels_last=None means False."""
    impl = nested_tensor_impl(
        data,
        torch.get_default_dtype() if dtype is None else dtype,
        torch.device("cpu") if device is None else device,
        requires_grad, pin_memory, bool(channels_last))
    return nested.NestedTensor(impl)


def as_nested_tensor(data, dtype=None, device=None, requires_grad=False, pin_memory=False):
    """``data`` itself when it already is a NestedTensor (the other arguments are
    then ignored, nested/creation.py:22-26); otherwise nested_tensor(...)."""
    if isinstance(data, nested.NestedTensor):
        return data
    return nested_tensor(data, dtype, device, requires_grad, pin_memory)
