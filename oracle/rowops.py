"""Oracle for the row-wise ops either side of nested attention: layer norm and
the packed additions.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows nestedtensor/csrc/functions.cpp:65-112 (NestedTensor_layer_norm: the
checks, then ``map_nested_tensor(at::layer_norm)`` over the constituents) and
nestedtensor/csrc/BinaryOps.cpp:12-115 (NestedTensor_add_Tensor: ``at::add`` on
the packed buffers for equal nested sizes, ``at::add(buffer.reshape(-1, n),
other)`` for a 1-D tensor over a regular last dim, else per constituent).

layer_norm below is NOT a call of torch's layer_norm: it is the two-pass
definition (mean, biased variance, 1/sqrt(var + eps), affine) written out in
fp64 and rounded once, so that ``torch.nn.functional.layer_norm`` per
constituent -- what the reference's own test compares with
(test/test_nested_tensor_functional.py:894-917) -- is an independent check of it
(tests/test_oracle_rowops.py), together with the closed forms mean 0 / variance
n/(n + eps*n/var) and invariance under adding a constant to a row.
"""

import torch

from .nt import RefNestedTensor


def layer_norm(nt, normalized_shape, weight=None, bias=None, eps=1e-5):
    """functions.cpp:65-112.  Returns a RefNestedTensor."""
    normalized_shape = (normalized_shape,) if isinstance(normalized_shape, int) else tuple(normalized_shape)
    if len(normalized_shape) != 1:
        raise RuntimeError("Currently only singleton tuples of integers supported for layer_norm.")
    opt = nt.opt_sizes()
    last = nt.dim() - 1
    if opt[last] is None:
        raise RuntimeError("Cannot normalize across irregular dimension %d" % last)
    if opt[last] != normalized_shape[0]:
        raise RuntimeError("Normalized shape [%d] does not match the size of the last dimension (%d) of input."
                           % (normalized_shape[0], opt[last]))
    if (weight is None) != (bias is None):
        raise RuntimeError("Either both weight and bias are used or not.")
    outs = []
    for t in nt.unbind():
        x = t.double()
        mean = x.mean(-1, keepdim=True)
        var = ((x - mean) ** 2).mean(-1, keepdim=True)
        y = (x - mean) / torch.sqrt(var + eps)
        if weight is not None:
            y = y * weight.double() + bias.double()
        outs.append(y.to(t.dtype))
    return RefNestedTensor(outs, nt.dtype)


def add(nt, other, alpha=1):
    """BinaryOps.cpp:12-115 for the cases the packed path covers; ``at::add``
    computes ``a + alpha * b`` in the op-math type and rounds once."""
    if isinstance(other, RefNestedTensor):
        if not torch.equal(nt.sizes, other.sizes):
            raise NotImplementedError("different nested sizes")
        outs = [torch.add(a, b, alpha=alpha) for a, b in zip(nt.unbind(), other.unbind())]
    else:
        outs = [torch.add(a, other, alpha=alpha) for a in nt.unbind()]
    return RefNestedTensor(outs, nt.dtype)


def mul(nt, other):
    """NestedTensor_mul_Tensor (BinaryOps.cpp:296-299): at::mul per constituent;
    `other` a nested tensor of the same nested size, a scalar, or a tensor that
    broadcasts against every constituent."""
    if isinstance(other, RefNestedTensor):
        outs = [torch.mul(a, b) for a, b in zip(nt.unbind(), other.unbind())]
    else:
        outs = [torch.mul(a, other) for a in nt.unbind()]
    return RefNestedTensor(outs, nt.dtype)


def matmul(nt, other):
    """NestedTensor_matmul (matmul.cpp:44-49): at::matmul per constituent."""
    return RefNestedTensor([torch.matmul(a, other) for a in nt.unbind()], nt.dtype)


def softmax(nt, dim, dtype=None, log=False):
    """NestedTensor_softmax / NestedTensor_log_softmax (SoftMax.cpp:12-46):
    at::softmax(t, dim - nested_dim) per constituent; dim 0 is refused."""
    nd = nt.dim()
    dim = dim % nd
    if dim < 1:
        raise RuntimeError("Cannot apply %s across nested dimensions %d" % ("log_softmax" if log else "softmax", dim))
    fn = torch.log_softmax if log else torch.softmax
    outs = [fn(t, dim - 1, dtype=dtype) for t in nt.unbind()]
    return RefNestedTensor(outs, outs[0].dtype if outs else nt.dtype)


def activation(nt, kind):
    """NestedTensor_relu / NestedTensor_gelu (activation.cpp:11-19, 34-46): at::relu
    / at::gelu (erf form) per constituent."""
    fn = {"relu": torch.relu, "gelu": torch.nn.functional.gelu}[kind]
    return RefNestedTensor([fn(t) for t in nt.unbind()], nt.dtype)
