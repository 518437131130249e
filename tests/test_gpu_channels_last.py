"""The channels-last storage of ragged images (nested_tensor_impl.cpp:157-198) and
the ops that look at it (creation.cpp:217-219, BinaryOps.cpp:25-43,
conv2d.cpp:43-60, 88-90, pooling.cpp:54-56), against the oracle.  Layout changes
are copies: bit-exact."""

import random

import pytest
import torch

import nestedtensor_amd as nt
import oracle
from nestedtensor_amd import ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _images(seed=1010, n=7, c=30, lo=20, hi=40):
    rnd = random.Random(seed)
    shapes = [(c, rnd.randint(lo, hi), rnd.randint(lo, hi)) for _ in range(n)]
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=g) for s in shapes]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_channels_last_creation(dtype):
    # test/test_nested_tensor_class.py:844-866
    ts = _images()
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype, channels_last=True)
    assert a.is_contiguous(memory_format=torch.channels_last) and not a.is_contiguous()
    buffer, strides = oracle.to_channels_last(oracle.ref_nested_tensor(ts, dtype=dtype))
    assert torch.equal(a._impl.buffer.cpu(), buffer)
    assert list(a.nested_stride()) == strides
    for t, got in zip(ts, a):
        want = t.to(dtype).unsqueeze(0).contiguous(memory_format=torch.channels_last).squeeze(0)
        assert got.stride() == want.stride()
        assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.int64])
def test_channels_last_round_trip(dtype):
    ts = [(t * 100).to(dtype) for t in _images(seed=5, n=5, c=3, lo=1, hi=70)]
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    cl = a.to(memory_format=torch.channels_last)
    assert cl.is_contiguous(memory_format=torch.channels_last)
    assert cl.nested_size() == a.nested_size()
    assert cl.contiguous(memory_format=torch.channels_last) is cl
    back = cl.contiguous()
    assert back.is_contiguous() and torch.equal(back._impl.buffer, a._impl.buffer)
    exp = oracle.from_channels_last(cl._impl.buffer.cpu(), [tuple(t.shape) for t in ts], dtype)
    assert torch.equal(back._impl.buffer.cpu(), exp.buffer)
    # an op that reads row-major constituents sees the same nested tensor
    assert torch.equal(cl.to_padded_tensor(0), a.to_padded_tensor(0))
    d1, m1 = cl.to_tensor_mask()
    d0, m0 = a.to_tensor_mask()
    assert torch.equal(d1, d0) and torch.equal(m1, m0)


def test_channels_last_errors():
    a = nt.nested_tensor([torch.randn(3, 4), torch.randn(2, 4)], device=DEV)
    with pytest.raises(RuntimeError, match="ChannelsLast memory format requires 4 dim input."):
        a.contiguous(memory_format=torch.channels_last)
    with pytest.raises(RuntimeError, match="ChannelsLast memory format requires 4 dim input."):
        nt.nested_tensor([torch.randn(3, 4)], device=DEV, channels_last=True)
    # irregular channel count: the transpose underneath refuses it (transpose.cpp:126-128)
    b = nt.nested_tensor([torch.randn(2, 3, 3), torch.randn(3, 3, 3)], device=DEV)
    with pytest.raises(RuntimeError, match="Expected first dimension to be regular."):
        b.contiguous(memory_format=torch.channels_last)
    with pytest.raises(RuntimeError, match="preserve memory format is unsupported"):
        ops.contiguous(b._impl, torch.preserve_format)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_add_keeps_channels_last_only_when_both_are(dtype):
    ts = [t.to(dtype) for t in _images(seed=7, n=4, c=8, lo=3, hi=30)]
    us = [torch.randn(t.shape, generator=torch.Generator().manual_seed(9)).to(dtype) for t in ts]
    a, b = nt.nested_tensor(ts, device=DEV, dtype=dtype), nt.nested_tensor(us, device=DEV, dtype=dtype)
    exp = oracle.add(oracle.ref_nested_tensor(ts, dtype=dtype), oracle.ref_nested_tensor(us, dtype=dtype))
    acl, bcl = a.to(memory_format=torch.channels_last), b.to(memory_format=torch.channels_last)
    both = acl + bcl
    assert both.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(both.contiguous()._impl.buffer.cpu(), exp.buffer)
    for mixed in (acl + b, a + bcl):
        assert mixed.is_contiguous()
        assert torch.equal(mixed._impl.buffer.cpu(), exp.buffer)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_conv2d_1x1_on_channels_last_is_the_gemm_alone(dtype, monkeypatch):
    # conv2d.cpp:43-60: the buffer is the [pixels, C_in] matrix already
    ts = [t.to(dtype) for t in _images(seed=11, n=5, c=64, lo=1, hi=60)]
    c_out = 96
    w = (torch.randn(c_out, 64, 1, 1, generator=torch.Generator().manual_seed(12)) * 0.3).to(dtype)
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype, channels_last=True)

    def no_transpose(*args, **kwargs):
        raise AssertionError("a channels-last 1x1 convolution must not transpose")
    monkeypatch.setattr(ops, "_transpose_constituents", no_transpose)
    got = torch.conv2d(a, w.to(DEV))
    monkeypatch.undo()
    assert got.is_contiguous(memory_format=torch.channels_last)
    ref = oracle.conv2d(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), w.float())
    assert [tuple(x.shape) for x in got.unbind()] == [tuple(x.shape) for x in ref.unbind()]
    err = (got.contiguous()._impl.buffer.float().cpu() - ref.buffer).abs().max().item()
    scale = max(1.0, ref.buffer.abs().max().item())
    assert err <= (1e-5 if dtype == torch.float32 else 2e-2) * scale, err
    # the same numbers as the row-major route (same GEMM, two more copies)
    rm = torch.conv2d(a.contiguous(), w.to(DEV))
    assert torch.equal(rm._impl.buffer, got.contiguous()._impl.buffer)


def test_padded_route_returns_the_input_layout():
    # pooling.cpp:54-56, conv2d.cpp:88-90
    dtype = torch.float16
    ts = [t.to(dtype) for t in _images(seed=13, n=3, c=4, lo=9, hi=33)]
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype, channels_last=True)
    ref_in = oracle.ref_nested_tensor(ts, dtype=dtype)
    got = torch.nn.functional.max_pool2d(a, kernel_size=3, stride=2, padding=1)
    exp = oracle.max_pool2d(ref_in, (3, 3), (2, 2), (1, 1), (1, 1))
    assert got.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(got.contiguous()._impl.buffer.cpu(), exp.buffer)
    w = (torch.randn(6, 4, 3, 3, generator=torch.Generator().manual_seed(14)) * 0.2).to(dtype)
    got = torch.conv2d(a, w.to(DEV), None, 1, 1)
    assert got.is_contiguous(memory_format=torch.channels_last)
    ref = oracle.conv2d(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), w.float(),
                        None, (1, 1), (1, 1))
    err = (got.contiguous()._impl.buffer.float().cpu() - ref.buffer).abs().max().item()
    assert err <= 2e-2 * max(1.0, ref.buffer.abs().max().item()), err
