"""Pins oracle.layer_norm / oracle.add (CPU only)."""
import pytest
import torch

import oracle


def _nt(shapes, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    return oracle.ref_nested_tensor([torch.randn(*s, generator=g) * 3 + 1 for s in shapes], dtype=dtype)


@pytest.mark.parametrize("size", [1024, 512, 256, 128, 2, 4, 32, 7])
def test_layer_norm_matches_torch_per_constituent(size):
    # the reference's own check (test/test_nested_tensor_functional.py:894-917):
    # nn.LayerNorm applied to the nested tensor equals it applied per constituent
    nt = _nt([(2, size), (2, size), (5, size), (1, size)], seed=size)
    ln = torch.nn.LayerNorm(size)
    with torch.no_grad():
        ln.weight.copy_(torch.randn(size))
        ln.bias.copy_(torch.randn(size))
    got = oracle.layer_norm(nt, (size,), ln.weight.detach(), ln.bias.detach(), ln.eps)
    for a, t in zip(got.unbind(), nt.unbind()):
        exp = ln(t).detach()
        assert (a - exp).abs().max() <= 2e-6 * max(1.0, exp.abs().max().item())


def test_layer_norm_closed_forms():
    nt = _nt([(3, 64), (9, 64)], seed=3)
    eps = 1e-5
    y = oracle.layer_norm(nt, 64, None, None, eps)
    for a, t in zip(y.unbind(), nt.unbind()):
        var = t.double().var(-1, unbiased=False)
        assert a.double().mean(-1).abs().max() < 1e-6                                    # zero mean
        assert (a.double().var(-1, unbiased=False) - var / (var + eps)).abs().max() < 1e-5  # var / (var + eps)
    shifted = oracle.ref_nested_tensor([t.double() + 5.0 for t in nt.unbind()], dtype=torch.float64)
    y64 = oracle.layer_norm(oracle.ref_nested_tensor(nt.unbind(), dtype=torch.float64), 64, None, None, eps)
    ys = oracle.layer_norm(shifted, 64, None, None, eps)
    for a, b in zip(y64.unbind(), ys.unbind()):
        assert (a - b).abs().max() < 1e-9                                                  # shift invariance


def test_layer_norm_errors():
    nt = _nt([(3, 4), (2, 5)])
    with pytest.raises(RuntimeError, match="Cannot normalize across irregular dimension 2"):
        oracle.layer_norm(nt, 4)
    nt = _nt([(3, 4), (2, 4)])
    with pytest.raises(RuntimeError, match=r"Normalized shape \[3\] does not match the size of the last dimension \(4\) of input."):
        oracle.layer_norm(nt, 3)
    with pytest.raises(RuntimeError, match="Currently only singleton tuples of integers supported for layer_norm."):
        oracle.layer_norm(nt, (3, 2, 4))
    with pytest.raises(RuntimeError, match="Either both weight and bias are used or not."):
        oracle.layer_norm(nt, 4, torch.ones(4), None)


def test_add_matches_packed_buffer_add():
    a = _nt([(3, 8), (5, 8)], seed=1)
    b = _nt([(3, 8), (5, 8)], seed=2)
    got = oracle.add(a, b, alpha=2)
    assert torch.equal(got.buffer, a.buffer + 2 * b.buffer)          # BinaryOps.cpp:18-44
    v = torch.arange(8.0)
    got = oracle.add(a, v)
    assert torch.equal(got.buffer, (a.buffer.reshape(-1, 8) + v).reshape(-1))   # BinaryOps.cpp:97-107


def test_dense_ops_output_sizes_closed_form():
    # pooling.cpp:50-53 / conv2d.cpp:80-84: (s + 2p - d(k-1) - 1) // stride + 1
    nt = _nt([(3, 50, 60), (3, 28, 17), (3, 9, 33)])
    k, s, p, d = (3, 3), (2, 2), (1, 1), (1, 1)
    got = oracle.max_pool2d(nt, k, s, p, d)
    for t, o in zip(nt.unbind(), got.unbind()):
        exp = tuple((t.shape[1 + j] + 2 * p[j] - d[j] * (k[j] - 1) - 1) // s[j] + 1 for j in (0, 1))
        assert tuple(o.shape) == (3,) + exp
    w = torch.randn(5, 3, 2, 2)
    got = oracle.conv2d(nt, w, None, (1, 2), (1, 0), (2, 1))
    for t, o in zip(nt.unbind(), got.unbind()):
        exp = ((t.shape[1] + 2 - 2 * 1 - 1) // 1 + 1, (t.shape[2] + 0 - 1 * 1 - 1) // 2 + 1)
        assert tuple(o.shape) == (5,) + exp


def test_mul_and_matmul_known_answers():
    a = oracle.ref_nested_tensor([torch.tensor([[1.0, 2.0], [3.0, 4.0]]), torch.tensor([[5.0, 6.0]])])
    b = oracle.ref_nested_tensor([torch.tensor([[2.0, 2.0], [0.5, -1.0]]), torch.tensor([[0.0, 1.0]])])
    assert oracle.mul(a, b).buffer.tolist() == [2.0, 4.0, 1.5, -4.0, 0.0, 6.0]
    assert oracle.mul(a, 0.5).buffer.tolist() == [0.5, 1.0, 1.5, 2.0, 2.5, 3.0]
    assert oracle.mul(a, torch.tensor([10.0, -1.0])).buffer.tolist() == [10.0, -2.0, 30.0, -4.0, 50.0, -6.0]
    w = torch.tensor([[1.0, 0.0, 2.0], [0.0, 1.0, -1.0]])              # [K=2, N=3]
    got = oracle.matmul(a, w)
    assert got.opt_sizes() == [2, None, 3]
    assert got.buffer.tolist() == [1.0, 2.0, 0.0, 3.0, 4.0, 2.0, 5.0, 6.0, 4.0]
    # against an fp64 product of the packed buffer (matmul.cpp:13-41: the fast path is one GEMM)
    x = _nt([(3, 8), (5, 8)], seed=5)
    w8 = torch.randn(8, 6, generator=torch.Generator().manual_seed(6))
    ref = (x.buffer.reshape(-1, 8).double() @ w8.double()).reshape(-1)
    assert (oracle.matmul(x, w8).buffer.double() - ref).abs().max() < 1e-5


def test_softmax_closed_forms():
    import math
    ts = [torch.randn(2, 3, 5, generator=torch.Generator().manual_seed(1)),
          torch.randn(2, 4, 2, generator=torch.Generator().manual_seed(2))]      # ragged last dim
    a = oracle.ref_nested_tensor(ts)
    got = oracle.softmax(a, -1)
    lg = oracle.softmax(a, 3, log=True)
    for t, o, l in zip(ts, got.unbind(), lg.unbind()):
        assert o.shape == t.shape
        for h in range(t.size(0)):
            for r in range(t.size(1)):
                row = [float(v) for v in t[h, r]]
                den = sum(math.exp(v) for v in row)
                for c, v in enumerate(row):
                    assert abs(float(o[h, r, c]) - math.exp(v) / den) < 1e-6
                    assert abs(float(l[h, r, c]) - math.log(math.exp(v) / den)) < 1e-5
        assert torch.allclose(o.sum(-1), torch.ones(t.shape[:-1]), atol=1e-6)
    shifted = oracle.ref_nested_tensor([t + 3.0 for t in ts])
    assert (oracle.softmax(shifted, -1).buffer - got.buffer).abs().max() < 1e-6
    with pytest.raises(RuntimeError, match="Cannot apply softmax across nested dimensions 0"):
        oracle.softmax(a, 0)
    # dims other than the last follow at::softmax per constituent too (SoftMax.cpp:24-27)
    other = oracle.softmax(a, 1)
    assert torch.allclose(other.unbind()[0].sum(0), torch.ones(3, 5), atol=1e-6)


def test_activation_closed_forms():
    import math
    x = _nt([(3, 8), (5, 8)], seed=9)
    r = oracle.activation(x, "relu")
    assert torch.equal(r.buffer, torch.clamp(x.buffer, min=0))
    ge = oracle.activation(x, "gelu")
    exp = torch.tensor([0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0))) for v in x.buffer.double().tolist()])
    assert (ge.buffer.double() - exp).abs().max() < 1e-6
