"""Oracle for the dense ops the reference runs through pad -> op -> un-pad.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows the per-constituent definition the reference's CPU path implements and
its tests assert (nestedtensor/csrc/pooling.cpp:59-72, conv2d.cpp:93-110:
``map_nested_tensor`` of ``at::max_pool2d`` / ``at::conv2d`` on
``t.unsqueeze(0)``; test/test_nested_tensor_functional.py:44-135, 251-266,
788-811).  The dense arithmetic is ATen's; what is restated is the mapping over
constituents and the resulting nested size.
"""

import torch

from .nt import RefNestedTensor


def max_pool2d(nt, kernel_size, stride=None, padding=0, dilation=1, ceil_mode=False):
    if nt.dim() != 4:
        raise RuntimeError("Input must be 4 dimensional.")
    outs = [torch.nn.functional.max_pool2d(t.unsqueeze(0), kernel_size, stride, padding, dilation,
                                           ceil_mode).squeeze(0) for t in nt.unbind()]
    return RefNestedTensor(outs, nt.dtype)


def conv2d(nt, weight, bias=None, stride=1, padding=0, dilation=1, groups=1):
    if nt.dim() != 4:
        raise RuntimeError("Expected input to be dim 4, but got %d." % nt.dim())
    outs = [torch.conv2d(t.unsqueeze(0), weight, bias, stride, padding, dilation, groups).squeeze(0)
            for t in nt.unbind()]
    return RefNestedTensor(outs, nt.dtype)
