"""Oracle-side nested tensor: a list of constituents, as the reference sees it.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows nestedtensor/nested/creation.py:9-26, nestedtensor/csrc/creation.cpp:28-222,
nestedtensor/csrc/storage/Packed.h:75-98 (pack) and
nestedtensor/csrc/storage/EfficientSizeNode.h:8-138 (sizes / opt_sizes / numel).
"""

import torch


class RefNestedTensor:
    """A nested tensor of nested_dim 1 held the way the reference's CPU code
    walks it: a list of constituent tensors (``get_nested_tensor_structure``)
    plus the packed buffer built from them."""

    def __init__(self, tensors, dtype, device=torch.device("cpu")):
        self.dtype = dtype
        self.device = torch.device(device)
        # impl::pack (Packed.h:75-98): empty list -> at::ones({0}); otherwise a
        # 1-D buffer holding the row-major contiguous elements of each tensor
        # in order.  creation.cpp:212 then casts the buffer to (device, dtype).
        if len(tensors) == 0:
            self.buffer = torch.ones(0).to(self.device, dtype)
            self.sizes = torch.zeros((), dtype=torch.int64)  # EfficientSizeNode.h:10-12
        else:
            flat = [t.contiguous().reshape(-1) for t in tensors]
            self.buffer = torch.cat(flat).to(self.device, dtype)
            self.sizes = torch.tensor(
                [list(t.shape) for t in tensors], dtype=torch.int64
            ).reshape(len(tensors), -1)
        self._shapes = [tuple(t.shape) for t in tensors]

    # --- metadata (EfficientSizeNode.h:86-131, py_init.cpp:169-190) -------
    def __len__(self):
        return len(self._shapes)

    def dim(self):
        return 1 + self.sizes.size(1) if self.sizes.dim() > 0 else 1

    def nested_dim(self):
        return 1

    def numel(self):
        if self.sizes.dim() == 0:
            return 0
        if self.sizes.numel() == 0:
            # B constituents of dim 0: the reference returns 0 here
            # (EfficientSizeNode.h:117-119), although the buffer holds B values.
            return 0
        return int(self.sizes.prod(1).sum())

    def opt_sizes(self):
        # construct_efficient_size (EfficientSizeNode.h:27-49)
        res = [len(self)]
        if self.sizes.dim() > 0:
            for j in range(self.sizes.size(1)):
                col = self.sizes[:, j]
                res.append(int(col[0]) if bool((col == col[0]).all()) else None)
        return res

    def size(self):
        return tuple(self.opt_sizes())

    def nested_size(self, dim=None):
        if dim is None:
            return [torch.Size(s) for s in self._shapes]
        nd = self.dim()
        if not -nd <= dim < nd:
            raise IndexError("Dimension out of range")
        dim = dim % nd
        if dim == 0:
            return len(self)
        return tuple(s[dim - 1] for s in self._shapes)

    def nested_stride(self, dim=None):
        def cont(shape):
            st, acc = [], 1
            for s in reversed(shape):
                st.append(acc)
                acc *= s
            return tuple(reversed(st))

        strides = [cont(s) for s in self._shapes]
        if dim is None:
            return strides
        if dim == 0:
            return len(self)
        return tuple(s[dim - 1] for s in strides)

    def unbind(self):
        # build_structure (Packed.h:21-64): split the buffer, view each piece.
        out, off = [], 0
        for s in self._shapes:
            n = 1
            for v in s:
                n *= v
            out.append(self.buffer[off:off + n].reshape(s))
            off += n
        return out


def _verify(tensors):
    # _verify_variables (creation.cpp:28-171)
    first = tensors[0]
    for t in tensors:
        if not torch.is_tensor(t):
            raise RuntimeError("Currently only supporting a sequence of Tensors.")
        if t.dim() != first.dim():
            raise RuntimeError(
                "Given Tensor / NestedTensor constiuent of dimension %d doesn't match "
                "another constiuent of dimension %d. " % (t.dim(), first.dim()))
        if t.layout != first.layout or t.device != first.device or t.dtype != first.dtype:
            raise RuntimeError("constiuents differ in layout, device or scalar type")


def ref_nested_tensor(data, dtype=None, device=None):
    """nestedtensor.nested_tensor (creation.py:9-19): dtype defaults to
    torch.get_default_dtype() (so integer inputs become float32), device to cpu."""
    if dtype is None:
        dtype = torch.get_default_dtype()
    if device is None:
        device = torch.device("cpu")
    if not isinstance(data, (list, tuple)):
        raise TypeError("nested_tensor expects a sequence of Tensors")
    data = list(data)
    if len(data) > 0:
        _verify(data)
    return RefNestedTensor(data, dtype, device)
