"""Oracle restatement of the reference's CPU padding / mask code.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  Follows
nestedtensor/csrc/masking.cpp and nestedtensor/nested/masking.py line by line
in behaviour (not in code): per-constituent ``constant_pad_nd`` + ``stack``,
``sum``-and-collapse for masks, the recursive ``.item()`` walk for
nt_from_tensor_mask, ``masked_select`` for the length-based un-pad.
"""

import torch
import torch.nn.functional as F

from .nt import RefNestedTensor, ref_nested_tensor


# ---------------------------------------------------------------------------
# helpers


def get_max_size(nt):
    """get_max_size_from_efficient_size (masking.cpp:83-103)."""
    if len(nt) > 0:
        if nt.sizes.size(1) == 0:
            raise RuntimeError(
                "Internal error: Expected sizes_size_1 to be greater than 0.")
        return [int(v) for v in nt.sizes.max(0).values]
    return []


def pad_tensor_to_shape(t, goal_shape, value=0):
    """pad_tensor_to_shape (masking.cpp:45-58)."""
    if t.dim() != len(goal_shape):
        raise RuntimeError("dimension doesn't match length of goal shape.")
    padd = []
    for i in range(t.dim() - 1, -1, -1):
        padd += [0, goal_shape[i] - t.shape[i]]
    out = F.pad(t, padd, mode="constant", value=value)  # at::constant_pad_nd
    return out.reshape(goal_shape)


def merge_tensor_mask(tensor, mask, mask_dim=None):
    """merge_tensor_mask (masking.cpp:12-43)."""
    if mask_dim is not None and mask.dim() == mask_dim:
        return tensor, mask
    if mask.dim() == 0:
        return tensor, mask
    last_size = mask.size(-1)
    collapsed = mask.sum(-1)
    n_full = int((collapsed == last_size).sum())
    n_zero = int((collapsed == 0).sum())
    if n_full + n_zero == collapsed.numel():
        return merge_tensor_mask(tensor, collapsed.to(torch.bool), mask_dim)
    if mask_dim is not None and mask_dim != mask.dim():
        raise RuntimeError("Mask dimension is too small to represent data tensor.")
    return tensor.contiguous(), mask.contiguous()


def _pad_leaf(t, shape):
    """pad_nt on a plain tensor (masking.cpp:139-159)."""
    if t.numel() == 0:
        raise RuntimeError("Empty tensors are not yet supported.")
    if t.dim() == 0:
        return t, torch.tensor(True)
    tensor = pad_tensor_to_shape(t, shape)
    mask = pad_tensor_to_shape(
        torch.full(t.shape, 1, dtype=torch.uint8, device=t.device), shape)
    return tensor, mask


def pad_nt(nt, shape):
    """pad_nt (masking.cpp:138-179): data padded with 0, uint8 mask of ones."""
    if len(nt) == 0:
        return torch.tensor([0]), torch.tensor([0], dtype=torch.uint8)
    res_t, res_m = [], []
    for child in nt.unbind():
        t, m = _pad_leaf(child, shape)
        res_t.append(t)
        res_m.append(m)
    return torch.stack(res_t), torch.stack(res_m)


# ---------------------------------------------------------------------------
# nested -> dense


def _check_mask_dim(nt, mask_dim):
    if mask_dim is not None and mask_dim > nt.dim():
        raise RuntimeError(
            "Requested mask dimension %d is bigger than dimension %d of given NestedTensor."
            % (mask_dim, nt.dim()))


def to_tensor_mask(nt, mask_dim=None):
    """to_tensor_mask, CPU/generic branch (masking.cpp:297-319)."""
    _check_mask_dim(nt, mask_dim)
    opt = nt.opt_sizes()
    if len(opt) == 1 and opt[0] == 1:
        buf = nt.buffer.reshape(-1)
        mask = torch.tensor(True) if (mask_dim is None or mask_dim == 0) else torch.tensor([True])
        return buf, mask
    max_size = get_max_size(nt)
    t, m = pad_nt(nt, max_size)
    return merge_tensor_mask(t, m, mask_dim)


def _create_nt_mask(sizes, shape):
    """_create_nt_mask on one constituent (masking.cpp:353-371)."""
    numel = 1
    for s in sizes:
        numel *= s
    if numel <= 0:
        raise RuntimeError("Empty tensors are not yet supported.")
    if len(sizes) == 0:
        return torch.tensor(True)
    return pad_tensor_to_shape(torch.full(sizes, 1, dtype=torch.uint8), shape)


def to_mask(nt, mask_dim=None):
    """to_mask (masking.cpp:408-457)."""
    _check_mask_dim(nt, mask_dim)
    opt = nt.opt_sizes()
    if len(opt) == 1 and opt[0] == 1:
        return torch.tensor(True) if (mask_dim is None or mask_dim == 0) else torch.tensor([True])
    if nt.dim() > 1 and mask_dim is not None and mask_dim > 1:
        tmp_max = get_max_size(nt)
        max_size = [tmp_max[i - 1] for i in range(1, mask_dim)]
        if mask_dim == 2 and nt.dim() == 3:
            # masking.cpp:436-451
            res = torch.zeros((opt[0], tmp_max[0]), dtype=torch.uint8)
            for i in range(nt.sizes.size(0)):
                res[i, : int(nt.sizes[i, 0])] = 1
            return res
        # masking.cpp:391-404: only the first len(shape) sizes are used
        masks = []
        for i in range(nt.sizes.size(0)):
            masks.append(_create_nt_mask(
                [int(nt.sizes[i, j]) for j in range(len(max_size))], max_size))
        return torch.stack(masks)
    max_size = get_max_size(nt)
    if len(nt) == 0:
        # _create_nt_mask(EfficientSizeNode) on an empty node stacks nothing;
        # at::stack of an empty list raises in ATen.
        raise RuntimeError("stack expects a non-empty TensorList")
    masks = [_create_nt_mask([int(v) for v in nt.sizes[i]], max_size)
             for i in range(nt.sizes.size(0))]
    res = torch.stack(masks)
    _, m = merge_tensor_mask(res, res, mask_dim)
    return m


def to_padded_tensor(nt, padding, replicate_scalar_double_push=False):
    """to_padded_tensor, CPU branch (masking.cpp:627-649).

    ``replicate_scalar_double_push`` reproduces masking.cpp:644-647, where a
    0-d constituent is pushed twice; it is off by default because the product
    deliberately does not follow that bug."""
    opt = nt.opt_sizes()
    if len(opt) == 1 and opt[0] == 1:
        return nt.buffer
    if len(nt) == 0:
        return torch.tensor([float(padding)])
    max_size = get_max_size(nt) if nt.sizes.size(1) > 0 else []
    res = []
    for t in nt.unbind():
        if t.numel() == 0:
            raise RuntimeError("Empty tensors are not yet supported.")
        if t.dim() == 0 and replicate_scalar_double_push:
            res.append(t)
        res.append(pad_tensor_to_shape(t, max_size, padding))
    return torch.stack(res)


# ---------------------------------------------------------------------------
# dense -> nested


def from_padded_tensor(padded, target):
    """from_padded_tensor, CPU branch (masking.cpp:511-532): length-based
    un-pad by ``masked_select`` with a mask of ones padded to the batch max.

    ``target`` is a RefNestedTensor (or anything with ``.sizes`` [B, D]) that
    gives the nested size of the result."""
    sizes = target.sizes
    if padded.dim() != 1 + sizes.size(1):
        raise RuntimeError("Target size has different dimension as input padded Tensor.")
    target_vec = [int(v) for v in sizes.max(0).values]
    masks = []
    for i in range(sizes.size(0)):
        m = torch.full([int(v) for v in sizes[i]], 1, dtype=torch.uint8)
        masks.append(pad_tensor_to_shape(m, target_vec))
    final_mask = torch.stack(masks).to(torch.bool)
    new_buffer = padded.masked_select(final_mask)
    shapes = [tuple(int(v) for v in sizes[i]) for i in range(sizes.size(0))]
    out, off = [], 0
    for s in shapes:
        n = 1
        for v in s:
            n *= v
        out.append(new_buffer[off:off + n].reshape(s))
        off += n
    return RefNestedTensor(out, padded.dtype)


def _R(tensor, mask):
    """nt_from_tensor_mask at nested_dim == 0 (masking.cpp:185-225).
    Returns a tensor or None (c10::nullopt)."""
    if mask.numel() == 0 or (mask.numel() == 1 and bool(mask.item())):
        return tensor
    if mask.dim() == 1:
        tensors = [tensor[i] for i in range(mask.size(0)) if bool(mask[i].item())]
        if len(tensors) == 0:
            return torch.tensor([]).to(tensor)
        return torch.stack(tensors)
    if mask.dim() > 1:
        tensors, all_zero = [], True
        for i in range(mask.size(0)):
            tmp = _R(tensor[i], mask[i])
            if tmp.numel() > 0:
                all_zero = False
                tensors.append(tmp)
        if all_zero:
            for i in range(mask.size(0)):
                tensors.append(_R(tensor[i], mask[i]))
        if len(tensors) == 0:
            return torch.tensor([]).to(tensor)
        return torch.stack(tensors)
    return None


def nt_from_tensor_mask(tensor, mask, nested_dim):
    """nt_from_tensor_mask at nested_dim == 1 (masking.cpp:226-248): the
    literal recursive walk with one ``.item()`` per mask element.  Returns the
    list of constituents (wrap_tensor_node of the node list)."""
    if nested_dim != 1:
        raise RuntimeError("Only nested_dim of 1 is currently supported.")
    inner = []
    if mask.numel() == 0 or (mask.numel() == 1 and bool(mask.item())):
        for i in range(tensor.size(0)):
            inner.append(_R(tensor[i], mask))
    elif mask.numel() == 1 and not bool(mask.item()):
        inner.append(None)
    else:
        for i in range(tensor.size(0)):
            inner.append(_R(tensor[i], mask[i]))
    return [t for t in inner if t is not None]


def nested_tensor_from_tensor_mask(tensor, mask, nested_dim=1):
    """nestedtensor.nested_tensor_from_tensor_mask (nested/masking.py:18-50).
    The result takes the dtype of the constituents (NestedTensorImpl(TensorNode)
    packs them as they are); an empty result is float32 (Packed.h:77-79)."""
    if tensor is None:
        raise RuntimeError("Tensor can't be undefined (None).")
    if mask is None:
        raise RuntimeError("Mask can't be undefined (None).")
    if tensor.dim() == 0:
        raise RuntimeError("Can't construct nested tensor from a scalar.")
    if nested_dim == 0:
        raise RuntimeError("Nested dimension can't be 0.")
    if nested_dim is not None and nested_dim > tensor.dim():
        raise RuntimeError(
            "Nested dimension ({0}) can't be bigger than data tensor dimension ({1}).".format(
                nested_dim, tensor.dim()))
    if tensor.numel() == 0 and mask.numel() != 0:
        raise RuntimeError("Data tensor can't be emtpy if a mask has values.")
    if tensor.numel() != 0 and mask.numel() == 0:
        raise RuntimeError("Mask tensor can't be emtpy if a data tensor has values.")
    parts = nt_from_tensor_mask(tensor, mask, nested_dim)
    if len(parts) == 0:
        return RefNestedTensor([], torch.float32)
    return RefNestedTensor(parts, parts[0].dtype, parts[0].device)


def nested_tensor_from_padded_tensor(tensor, nested_dim=1, padding=-1):
    """nestedtensor.nested_tensor_from_padded_tensor (nested/masking.py:12-14)."""
    mask = tensor != padding
    return nested_tensor_from_tensor_mask(tensor, mask, nested_dim)


def nt_from_tensor_mask_vectorised(tensor, mask):
    """The same result as nt_from_tensor_mask(tensor, mask, 1) for masks of
    dim >= 2 whose selections are rectangular, computed without per-element
    host calls so that full-size inputs finish in seconds.  It follows from
    masking.cpp:190-222 that the kept elements keep their row-major order
    (so the data is ``tensor[i][mask[i] broadcast]``) and that, at each mask
    level, the extent is the number of children with a non-empty selection.
    Checked against the literal walk on small inputs in
    tests/test_oracle_masking.py."""
    assert mask.dim() >= 2 and mask.dim() <= tensor.dim()
    parts = []
    rest = tensor.shape[mask.dim():]
    for i in range(tensor.size(0)):
        m = mask[i].to(torch.bool)
        t = tensor[i]
        if not bool(m.any()):
            # all children empty: the stack of empties keeps the leading mask
            # extents and a trailing 0 (masking.cpp:213-222)
            parts.append(torch.empty(tuple(m.shape[:-1]) + (0,), dtype=tensor.dtype))
            continue
        mm = m
        extents = []
        # extent at the last level = max count along the last dim; at upper
        # levels = number of children that keep anything.
        counts = mm.sum(-1)
        extents.append(int(counts.max()))
        alive = counts > 0
        while alive.dim() > 0:
            c = alive.sum(-1)
            extents.append(int(c.max()))
            alive = c > 0
        extents = list(reversed(extents))
        sel = t[m]  # row-major order of kept mask elements, each with `rest` trailing dims
        n = 1
        for e in extents:
            n *= e
        if sel.shape[0] != n:
            raise RuntimeError("stack expects each tensor to be equal size")
        parts.append(sel.reshape(tuple(extents) + tuple(rest)))
    return parts
