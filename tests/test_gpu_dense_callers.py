"""max_pool2d / conv2d on a NestedTensor through pad -> dense op -> un-pad
(pooling.cpp:41-57, conv2d.cpp:77-92), against the per-constituent oracle.  The
shapes are the reference's (test/test_nested_tensor_functional.py:81-135,
251-266, 788-811, the 500x600 images scaled down where noted)."""

import pytest
import torch

import nestedtensor_amd as nt
import oracle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _rand(shapes, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=g).to(dtype) for s in shapes]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("shapes", [[(3, 500, 600), (3, 128, 128)], [(3, 50, 60), (3, 50, 60)],
                                    [(2, 7, 5), (2, 3, 9), (2, 8, 8)]])
def test_max_pool2d_equals_per_constituent(shapes, dtype):
    ts = _rand(shapes, dtype, 1)
    ts = [t - 3.0 for t in ts]      # mostly negative: a 0-padded window would show
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    got = torch.nn.functional.max_pool2d(a, kernel_size=(3, 3), stride=(2, 2), padding=(1, 1),
                                         dilation=(1, 1), ceil_mode=False)
    exp = oracle.max_pool2d(oracle.ref_nested_tensor(ts, dtype=dtype), (3, 3), (2, 2), (1, 1), (1, 1))
    assert got.nested_size() == nt.nested_tensor(list(exp.unbind())).nested_size()
    assert torch.equal(got._impl.buffer.cpu(), exp.buffer)          # max is exact
    pool = torch.nn.MaxPool2d(kernel_size=(3, 3), stride=2, padding=(1, 1), dilation=1, ceil_mode=False)
    assert torch.equal(pool(a)._impl.buffer.cpu(), exp.buffer)


@pytest.mark.parametrize("k,s,p,d", [((3, 3), (2, 2), (1, 1), (1, 1)), ((2, 2), (2, 2), (0, 0), (1, 1)),
                                     ((3, 2), (3, 2), (1, 0), (1, 1)), ((3, 3), (2, 3), (1, 1), (2, 1))])
def test_max_pool2d_ceil_mode_equals_per_constituent(k, s, p, d):
    # pooling.cpp:60-72: the per-constituent route passes ceil_mode on; odd and even
    # extents so that some last windows reach past the edge and some are dropped
    shapes = [(2, 7, 5), (2, 3, 9), (2, 8, 8), (2, 6, 10), (2, 13, 4), (2, 5, 5)]
    ts = [t - 3.0 for t in _rand(shapes, torch.float32, 5)]
    a = nt.nested_tensor(ts, device=DEV)
    got = torch.nn.functional.max_pool2d(a, kernel_size=k, stride=s, padding=p, dilation=d, ceil_mode=True)
    exp = oracle.max_pool2d(oracle.ref_nested_tensor(ts), k, s, p, d, ceil_mode=True)
    assert got.nested_size() == nt.nested_tensor(list(exp.unbind())).nested_size()
    assert torch.equal(got._impl.buffer.cpu(), exp.buffer)
    with pytest.raises(NotImplementedError):
        torch.nn.functional.max_pool2d(a, 2, return_indices=True)


CONV_CASES = [
    # shapes, weight shape, stride, padding, dilation, groups
    ([(2, 2, 3), (2, 4, 2), (2, 2, 2)], (3, 2, 1, 1), 1, 0, 1, 1),
    ([(2, 4, 5), (2, 5, 3), (2, 3, 3)], (3, 2, 3, 3), 1, 0, 1, 1),
    ([(32, 4, 5), (32, 5, 3), (32, 3, 3)], (32, 1, 3, 3), 1, 1, 1, 32),
    ([(4, 3, 2), (4, 3, 3), (4, 2, 3)], (5, 4, 2, 2), 1, 1, 1, 1),
    ([(8, 40, 33), (8, 17, 64)], (16, 8, 3, 3), 2, 1, 1, 1),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_equals_per_constituent(case, dtype):
    shapes, wshape, stride, padding, dilation, groups = case
    ts = _rand(shapes, dtype, 2)
    g = torch.Generator().manual_seed(3)
    w = (torch.randn(*wshape, generator=g) * 0.3).to(dtype)
    b = torch.randn(wshape[0], generator=g).to(dtype)
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    got = torch.conv2d(a, w.to(DEV), b.to(DEV), stride=stride, padding=padding, dilation=dilation,
                       groups=groups)
    # oracle in fp32 on the host (no fp16 convolution there), rounded once
    ref = oracle.conv2d(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), w.float(),
                        b.float(), stride, padding, dilation, groups)
    assert [tuple(x.shape) for x in got.unbind()] == [tuple(x.shape) for x in ref.unbind()]
    err = (got._impl.buffer.float().cpu() - ref.buffer).abs().max().item()
    scale = max(1.0, ref.buffer.abs().max().item())
    assert err <= (1e-5 if dtype == torch.float32 else 2e-2) * scale, err
    # and the same dense library applied per constituent on the device
    for gi, t in zip(got.unbind(), ts):
        ti = torch.conv2d(t.to(DEV).unsqueeze(0), w.to(DEV), b.to(DEV), stride, padding, dilation, groups).squeeze(0)
        assert (gi.float() - ti.float()).abs().max().item() <= (1e-5 if dtype == torch.float32 else 2e-2) * scale


def test_dense_callers_errors():
    a = nt.nested_tensor([torch.randn(3, 4), torch.randn(2, 4)], device=DEV)
    with pytest.raises(RuntimeError, match="Input must be 4 dimensional."):
        torch.nn.functional.max_pool2d(a, 2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_conv2d_1x1_runs_as_one_gemm(dtype):
    # conv2d.cpp:33-75: no bias, 1x1, unit stride -> transpose, packed GEMM, transpose back;
    # shapes of the reference's 1x1 test plus an image-sized case
    for shapes, c_out in (([(2, 2, 3), (2, 4, 2), (2, 2, 2)], 3), ([(64, 37, 50), (64, 128, 9), (64, 1, 1)], 96)):
        ts = _rand(shapes, dtype, 5)
        c_in = shapes[0][0]
        w = (torch.randn(c_out, c_in, 1, 1, generator=torch.Generator().manual_seed(6)) * 0.3).to(dtype)
        a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
        got = torch.conv2d(a, w.to(DEV))
        ref = oracle.conv2d(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), w.float())
        assert [tuple(x.shape) for x in got.unbind()] == [tuple(x.shape) for x in ref.unbind()]
        err = (got._impl.buffer.float().cpu() - ref.buffer).abs().max().item()
        scale = max(1.0, ref.buffer.abs().max().item())
        assert err <= (1e-5 if dtype == torch.float32 else 2e-2) * scale, err


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("c_in,c_out", [(16, 32), (64, 256), (64, 96), (128, 256), (32, 512), (48, 160), (128, 64)])
def test_conv2d_1x1_row_major_in_one_launch(dtype, c_in, c_out, monkeypatch):
    """Row-major f16 / bf16 images with depths the kernel covers take nt_conv1x1_nchw:
    no transposes (conv2d.cpp:33-75 does two around its matmul), same numbers as the
    per-constituent convolution.  Pixel counts around the 8-pixel pieces and the
    64-pixel tiles, images of one pixel, and more tiles than workgroups."""
    from nestedtensor_amd import ops

    def boom(*a, **k):
        raise AssertionError("this 1x1 convolution must not transpose")
    monkeypatch.setattr(ops, "transpose_nchw_nhwc", boom)
    shapes = [(c_in, 1, 1), (c_in, 1, 7), (c_in, 8, 8), (c_in, 5, 13), (c_in, 9, 7), (c_in, 16, 8), (c_in, 3, 43),
              (c_in, 37, 50), (c_in, 250, 300)]
    g = torch.Generator().manual_seed(c_in + c_out)
    ts = [torch.randn(s, generator=g).to(dtype) for s in shapes]
    w = (torch.randn(c_out, c_in, 1, 1, generator=g) * c_in ** -0.5).to(dtype)
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    got = torch.conv2d(a, w.to(DEV))
    again = torch.conv2d(a, w.to(DEV))                       # the cached tile table
    assert torch.equal(got._impl.buffer, again._impl.buffer)
    ref = oracle.conv2d(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), w.float())
    assert [tuple(x.shape) for x in got.unbind()] == [tuple(x.shape) for x in ref.unbind()]
    assert torch.isfinite(got._impl.buffer).all()
    err = (got._impl.buffer.float().cpu() - ref.buffer).abs().max().item()
    scale = max(1.0, ref.buffer.abs().max().item())
    assert err <= (1e-2 if dtype == torch.float16 else 4e-2) * scale, err
    # exactly the packed GEMM's numbers: the channels-last route computes the same
    # products in the same order of K
    monkeypatch.undo()                                       # building a channels-last tensor transposes
    cl = torch.conv2d(nt.nested_tensor(ts, device=DEV, dtype=dtype, channels_last=True), w.to(DEV))
    diff = (cl.contiguous()._impl.buffer.float() - got._impl.buffer.float()).abs().max().item()
    assert diff <= (4e-3 if dtype == torch.float16 else 3e-2) * scale, diff


def test_conv2d_1x1_depths_outside_the_kernel_keep_the_transposes():
    ts = [torch.randn(24, 9, 11).half(), torch.randn(24, 4, 4).half()]     # 24 input channels: not a multiple of 16
    w = (torch.randn(40, 24, 1, 1) * 0.2).half()
    a = nt.nested_tensor(ts, device=DEV, dtype=torch.float16)
    got = torch.conv2d(a, w.to(DEV))
    ref = oracle.conv2d(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), w.float())
    assert (got._impl.buffer.float().cpu() - ref.buffer).abs().max().item() <= 2e-2 * max(1.0, ref.buffer.abs().max().item())
