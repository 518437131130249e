"""Oracle for the interop formats built from the offsets array.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows nestedtensor/csrc/functions.cpp:14-63 (embedding: at::embedding over the
packed index buffer, result gains a trailing regular dim),
nestedtensor/nested/nested.py:43-118 (embedding_bag: offsets from a host loop over
nested_size, then torch.embedding_bag), nestedtensor/csrc/nested_tensor_impl.h:326-349
(to_sparse_csr: crow = [0, cumsum(lengths)], col = cat of aranges, values = buffer)
and nestedtensor/nested/nested.py:484-488 (to_packed_sequence: pack_sequence of the
constituents, enforce_sorted=False) and
nestedtensor/csrc/nested_tensor_impl.cpp:157-198 (contiguous with a memory format:
the channels-last storage of ragged images).

Pinned in tests/test_oracle_interop.py by closed forms that do not go through the
same library calls: ``weight[idx]`` indexing, explicit Python loops for the bag
reductions, ``csr.to_dense() == to_padded_tensor(0)`` (the reference's own check,
test/test_nested_tensor_class.py:741-752) and the
``pad_packed_sequence(to_packed_sequence(nt)) == to_padded_tensor(0)`` round trip;
the channels-last storage by torch's own ``contiguous(memory_format=channels_last)``
per constituent, values and strides (the reference's check,
test/test_nested_tensor_class.py:844-866).
"""

import torch

from .nt import RefNestedTensor


def embedding(weight, indices):
    outs = [torch.embedding(weight, t) for t in indices.unbind()]
    return RefNestedTensor(outs, weight.dtype)


def embedding_bag(indices, weight, mode="mean"):
    if indices.dim() != 2:
        raise ValueError("input has to be 2D NestedTensor, but got NestedTensor of dimension %d" % indices.dim())
    sizes = [int(s[0]) for s in indices._shapes]
    offsets = torch.zeros(len(sizes), dtype=torch.int64)       # nested.py:76-79
    for i in range(1, len(sizes)):
        offsets[i] = offsets[i - 1] + sizes[i - 1]
    mode_enum = {"sum": 0, "mean": 1, "max": 2}[mode]
    ret, _, _, _ = torch.embedding_bag(weight, indices.buffer, offsets, False, mode_enum, False, None, False)
    return ret


def to_sparse_csr(nt):
    if nt.dim() != 2:
        raise RuntimeError("Given tensor must be of dimension 2, got dimension %d" % nt.dim())
    lengths = nt.sizes.reshape(-1)
    crow = torch.cat([torch.tensor([0]), torch.cumsum(lengths, 0)])
    col = torch.cat([torch.arange(int(v)) for v in lengths]) if len(lengths) else torch.zeros(0, dtype=torch.int64)
    return torch.sparse_csr_tensor(crow, col, nt.buffer)


def to_packed_sequence(nt):
    if not nt.dim() == 3:
        raise RuntimeError("NestedTensor should consistent of 2d Tensors of size L x *")
    return torch.nn.utils.rnn.pack_sequence(nt.unbind(), enforce_sorted=False)


def transpose_nchw_nhwc(nt):
    """transpose.cpp:122-146: every constituent permuted (1, 2, 0) and made
    contiguous, which is what the reference's test compares with
    (test/test_nested_tensor_class.py:820-840)."""
    if nt.dim() != 4:
        raise RuntimeError("transpose_nchw_nhwc needs 4d input.")
    if nt.opt_sizes()[1] is None:
        raise RuntimeError("Expected first dimension to be regular.")
    return RefNestedTensor([t.permute(1, 2, 0).contiguous() for t in nt.unbind()], nt.dtype)


def transpose_nhwc_nchw(nt):
    """transpose.cpp:183-204: the inverse, permute (2, 0, 1)."""
    if nt.dim() != 4:
        raise RuntimeError("transpose_nhwc_nchw needs 4d input.")
    if nt.opt_sizes()[3] is None:
        raise RuntimeError("Expected last dimension to be regular.")
    return RefNestedTensor([t.permute(2, 0, 1).contiguous() for t in nt.unbind()], nt.dtype)


def to_channels_last(nt):
    """NestedTensor_contiguous(ChannelsLast) (nested_tensor_impl.cpp:182-194):
    returns ``(buffer, strides)``: the buffer of transpose_nchw_nhwc(nt) under
    the unchanged nested size, and per constituent the strides
    ``(1, C * W, C)`` written by :188-192."""
    if nt.dim() != 4:
        raise RuntimeError("ChannelsLast memory format requires 4 dim input.")
    buffer = transpose_nchw_nhwc(nt).buffer
    strides = []
    for (c, h, w) in nt._shapes:
        s2 = c
        s1 = s2 * w
        strides.append((1, s1, s2))
    return buffer, strides


def from_channels_last(buffer, shapes, dtype):
    """NestedTensor_contiguous(Contiguous) of a channels-last nested tensor
    (nested_tensor_impl.cpp:165-179): the nested size (C, H, W) is permuted to
    (H, W, C) by the two swaps of :167-175, the buffer is wrapped with it and
    transpose_nhwc_nchw is applied."""
    pieces, off = [], 0
    for size in shapes:
        p = list(size)
        p[0], p[2] = p[2], p[0]     # -> (W, H, C)
        p[0], p[1] = p[1], p[0]     # -> (H, W, C)
        n = p[0] * p[1] * p[2]
        pieces.append(buffer[off:off + n].reshape(p))
        off += n
    return transpose_nhwc_nchw(RefNestedTensor(pieces, dtype))
