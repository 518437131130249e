"""Parity of the packed row-wise ops (layer norm, packed add) with the oracle.

Tolerances: fp32 <= 1e-5 relative to the output scale, fp16 / bf16 <= 2e-2
absolute (outputs are O(1)).  The size list is the reference's
(test/test_nested_tensor_functional.py:935-939) plus the encoder widths of the
benchmark configurations C3 and C4."""

import pytest
import torch

import nestedtensor_amd as nt
import oracle
from nestedtensor_amd import ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _tol(dtype):
    return 1e-5 if dtype == torch.float32 else 2e-2


def _close(got, exp, dtype):
    got, exp = got.float().cpu(), exp.float()
    assert got.shape == exp.shape and torch.isfinite(got).all()
    err = (got - exp).abs().max().item()
    if dtype == torch.float32:
        assert err <= 1e-5 * max(1.0, exp.abs().max().item()), err
    else:
        assert err <= 2e-2, err


def _tensors(shapes, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(*s, generator=g) * 2 + 0.5).to(dtype) for s in shapes]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("size", [1024, 512, 256, 128, 2, 4, 32, 768, 2048, 4096, 100, 7])
def test_layer_norm_module(size, dtype):
    # reference test: two [2, size] constituents repeated; here ragged lengths too
    ts = _tensors([(2, size), (2, size), (5, size), (1, size), (17, size)], dtype, size)
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    ln = torch.nn.LayerNorm(size).to(dtype)
    with torch.no_grad():
        ln.weight.copy_(torch.randn(size))
        ln.bias.copy_(torch.randn(size))
    got = ln.to(DEV)(a)
    assert isinstance(got, nt.NestedTensor) and got.nested_size() == a.nested_size()
    exp = oracle.layer_norm(oracle.ref_nested_tensor(ts, dtype=dtype), (size,), ln.weight.detach().cpu(),
                            ln.bias.detach().cpu(), ln.eps)
    _close(got._impl.buffer, exp.buffer, dtype)


def test_layer_norm_no_affine_and_4d():
    ts = _tensors([(3, 2, 64), (1, 5, 64)], torch.float32, 5)
    a = nt.nested_tensor(ts, device=DEV)
    got = torch.nn.functional.layer_norm(a, (64,))
    exp = oracle.layer_norm(oracle.ref_nested_tensor(ts), 64)
    _close(got._impl.buffer, exp.buffer, torch.float32)


def test_layer_norm_errors():
    a = nt.nested_tensor([torch.randn(3, 4), torch.randn(2, 5)], device=DEV)
    with pytest.raises(RuntimeError, match="Cannot normalize across irregular dimension 2"):
        torch.nn.functional.layer_norm(a, (4,))
    a = nt.nested_tensor([torch.randn(3, 4), torch.randn(2, 4)], device=DEV)
    with pytest.raises(RuntimeError, match=r"Normalized shape \[3\] does not match the size of the last dimension \(4\) of input."):
        torch.nn.functional.layer_norm(a, (3,))
    with pytest.raises(RuntimeError, match="Currently only singleton tuples of integers supported for layer_norm."):
        torch.nn.functional.layer_norm(a, (3, 2, 4))
    with pytest.raises(RuntimeError, match="Either both weight and bias are used or not."):
        torch.nn.functional.layer_norm(a, (4,), torch.ones(4, device=DEV), None)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_add_nested_and_vector(dtype):
    shapes = [(3, 40), (7, 40), (1, 40)]
    ta, tb = _tensors(shapes, dtype, 1), _tensors(shapes, dtype, 2)
    a, b = nt.nested_tensor(ta, device=DEV, dtype=dtype), nt.nested_tensor(tb, device=DEV, dtype=dtype)
    ra, rb = oracle.ref_nested_tensor(ta, dtype=dtype), oracle.ref_nested_tensor(tb, dtype=dtype)
    # one rounding of an fp32 sum: bit-exact against at::add
    assert torch.equal((a + b)._impl.buffer.cpu(), oracle.add(ra, rb).buffer)
    assert torch.equal(torch.add(a, b, alpha=2)._impl.buffer.cpu(), oracle.add(ra, rb, alpha=2).buffer)
    v = torch.randn(40, generator=torch.Generator().manual_seed(3)).to(dtype)
    assert torch.equal((a + v.to(DEV))._impl.buffer.cpu(), oracle.add(ra, v).buffer)
    assert torch.equal((v.to(DEV) + a)._impl.buffer.cpu(), oracle.add(ra, v).buffer)
    odd = nt.nested_tensor(_tensors([(3, 7), (2, 7)], dtype, 4), device=DEV, dtype=dtype)   # unaligned rows
    ro = oracle.ref_nested_tensor(_tensors([(3, 7), (2, 7)], dtype, 4), dtype=dtype)
    v7 = torch.arange(7.0).to(dtype)
    assert torch.equal((odd + v7.to(DEV))._impl.buffer.cpu(), oracle.add(ro, v7).buffer)
    with pytest.raises(NotImplementedError):
        a + odd


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_mul_scalar_nested_and_vector(dtype):
    # BinaryOps.cpp:241-300; one rounding of an fp32 product: bit-exact against at::mul
    shapes = [(3, 40), (7, 40), (1, 40)]
    ta, tb = _tensors(shapes, dtype, 1), _tensors(shapes, dtype, 2)
    a, b = nt.nested_tensor(ta, device=DEV, dtype=dtype), nt.nested_tensor(tb, device=DEV, dtype=dtype)
    ra, rb = oracle.ref_nested_tensor(ta, dtype=dtype), oracle.ref_nested_tensor(tb, dtype=dtype)
    assert torch.equal((a * b)._impl.buffer.cpu(), oracle.mul(ra, rb).buffer)
    assert torch.equal(torch.mul(a, b)._impl.buffer.cpu(), oracle.mul(ra, rb).buffer)
    for sc in (0.125, 3, -1.7):                                   # 0.125 = the head_dim 64 scaling of min_mha
        assert torch.equal((a * sc)._impl.buffer.cpu(), oracle.mul(ra, sc).buffer)
        assert torch.equal((sc * a)._impl.buffer.cpu(), oracle.mul(ra, sc).buffer)
    v = torch.randn(40, generator=torch.Generator().manual_seed(3)).to(dtype)
    assert torch.equal((a * v.to(DEV))._impl.buffer.cpu(), oracle.mul(ra, v).buffer)
    assert torch.equal((v.to(DEV) * a)._impl.buffer.cpu(), oracle.mul(ra, v).buffer)
    odd_t = _tensors([(3, 7), (2, 7)], dtype, 4)                      # unaligned rows
    odd = nt.nested_tensor(odd_t, device=DEV, dtype=dtype)
    ro = oracle.ref_nested_tensor(odd_t, dtype=dtype)
    v7 = torch.arange(7.0).to(dtype)
    assert torch.equal((odd * v7.to(DEV))._impl.buffer.cpu(), oracle.mul(ro, v7).buffer)
    assert torch.equal((odd * 0.3)._impl.buffer.cpu(), oracle.mul(ro, 0.3).buffer)
    with pytest.raises(NotImplementedError):
        a * odd
    with pytest.raises(NotImplementedError):
        a * torch.ones(3, 40, device=DEV, dtype=dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("log", [False, True])
def test_softmax_last_dim(dtype, log):
    # SoftMax.cpp:12-46; the shapes: per-sequence attention scores [H, L_i, L_i] (ragged last dim),
    # a regular last dim, 1-D constituents, rows longer than a wavefront, a single element
    import torch.nn.functional as F
    cases = [[(4, 5, 5), (4, 130, 130), (4, 1, 1)], [(3, 40), (7, 40)], [(9,), (300,), (1,)],
             [(2, 1100), (3, 513)], [(2, 3, 1023), (2, 3, 1025)], [(2, 511), (1, 4097), (1, 9001)],   # around the register-cached row limits
             # a wavefront takes four consecutive rows: groups that straddle constituents of other
             # row lengths, with a constituent without rows between them, and a ragged last group
             [(3, 5), (0, 5), (2, 9), (5, 1024), (1, 1025), (6, 2)], [(1, 7)] * 9 + [(2, 33)]]
    for k, shapes in enumerate(cases):
        ts = [t * 3 for t in _tensors(shapes, dtype, 20 + k)]
        a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
        fn = F.log_softmax if log else F.softmax
        got = fn(a, -1)
        ref = oracle.softmax(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), -1, log=log)
        assert got.nested_size() == a.nested_size() and got.dtype == dtype
        # probabilities are at most 1: absolute; log-probabilities reach -20 or so: relative to |value|
        err = ((got._impl.buffer.float().cpu() - ref.buffer).abs() / ref.buffer.abs().clamp(min=1.0)).max().item()
        assert err <= (1e-5 if dtype == torch.float32 else 2e-2), err
        assert torch.equal((a.log_softmax(a.dim() - 1) if log else a.softmax(a.dim() - 1))._impl.buffer,
                           got._impl.buffer)
    a = nt.nested_tensor(_tensors([(2, 3, 4), (2, 5, 4)], dtype, 30), device=DEV, dtype=dtype)
    with pytest.raises(RuntimeError, match="across nested dimensions 0"):
        torch.softmax(a, 0)
    with pytest.raises(NotImplementedError):
        torch.softmax(a, 1)
    if dtype != torch.float32 and not log:
        up = torch.softmax(a, -1, dtype=torch.float32)          # at::softmax's dtype argument
        assert up.dtype == torch.float32
        assert torch.equal(torch.softmax(a, -1, torch.float32)._impl.buffer, up._impl.buffer)   # positional
        assert torch.equal(torch.nn.functional.softmax(a, -1, dtype=torch.float32)._impl.buffer, up._impl.buffer)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_relu_gelu_packed(dtype):
    import torch.nn.functional as F
    for shapes in ([(3, 40), (7, 40), (1, 40)], [(3, 7), (2, 7)], [(2, 3, 5, 4), (2, 1, 2, 4)]):
        ts = [t * 2 for t in _tensors(shapes, dtype, 40)]
        a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
        ref = oracle.ref_nested_tensor(ts, dtype=dtype)
        assert torch.equal(F.relu(a)._impl.buffer.cpu(), oracle.activation(ref, "relu").buffer)
        assert torch.equal(torch.relu(a)._impl.buffer.cpu(), oracle.activation(ref, "relu").buffer)
        got = F.gelu(a)
        exp = oracle.activation(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), "gelu")
        assert got.nested_size() == a.nested_size()
        err = (got._impl.buffer.float().cpu() - exp.buffer).abs().max().item()
        assert err <= (1e-5 if dtype == torch.float32 else 2e-2), err
        assert torch.equal(torch.nn.GELU()(a)._impl.buffer, got._impl.buffer)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("act", ["relu", "gelu"])
def test_linear_act_equals_linear_then_activation(dtype, act):
    import torch.nn.functional as F
    K, N = 64, 200
    ts = _tensors([(5, K), (300, K), (1, K)], dtype, 41)
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(42)) * 0.3).to(dtype)
    b = torch.randn(N, generator=torch.Generator().manual_seed(43)).to(dtype)
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    fused = nt.linear_act(a, w.to(DEV), b.to(DEV), activation=act)
    xs = oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32)
    lin = oracle.ref_nested_tensor([F.linear(t, w.float(), b.float()) for t in xs.unbind()], dtype=torch.float32)
    exp = oracle.activation(lin, act)
    assert [tuple(x.shape) for x in fused.unbind()] == [tuple(x.shape) for x in exp.unbind()]
    err = (fused._impl.buffer.float().cpu() - exp.buffer).abs().max().item()
    assert err <= (1e-5 if dtype == torch.float32 else 2e-2) * max(1.0, exp.buffer.abs().max().item()), err
    # the fused launch rounds once; applying the activation to the rounded linear output
    # may differ by that rounding only
    two = (F.relu if act == "relu" else F.gelu)(F.linear(a, w.to(DEV), b.to(DEV)))
    d = (fused._impl.buffer.float() - two._impl.buffer.float()).abs().max().item()
    assert d <= (1e-5 if dtype == torch.float32 else 2e-2) * max(1.0, exp.buffer.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_matmul_packed_fast_path(dtype):
    # matmul.cpp:13-41: nested [B, L_i, K] x dense [K, N] is one GEMM on the packed buffer
    K, N = 64, 96
    ts = _tensors([(5, K), (130, K), (1, K)], dtype, 7)
    w = (torch.randn(K, N, generator=torch.Generator().manual_seed(8)) * 0.2).to(dtype)
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    got = torch.matmul(a, w.to(DEV))
    assert (a @ w.to(DEV)).nested_size() == got.nested_size()
    ref = oracle.matmul(oracle.ref_nested_tensor([t.float() for t in ts], dtype=torch.float32), w.float())
    assert [tuple(x.shape) for x in got.unbind()] == [tuple(x.shape) for x in ref.unbind()]
    err = (got._impl.buffer.float().cpu() - ref.buffer).abs().max().item()
    assert err <= (1e-5 if dtype == torch.float32 else 2e-2) * max(1.0, ref.buffer.abs().max().item()), err
    with pytest.raises(NotImplementedError):
        torch.matmul(a, torch.randn(K + 1, N, device=DEV).to(dtype))
    with pytest.raises(NotImplementedError):
        torch.matmul(a, a)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_residual_layer_norm_equals_two_ops(dtype):
    # ops.layer_norm(x, residual=r) == layer_norm(x + r): the sum is rounded to the
    # storage type first, so the fused launch is bit-identical to the two launches
    E = 768
    shapes = [(L, E) for L in (5, 131, 64, 1)]
    tx, tr = _tensors(shapes, dtype, 7), _tensors(shapes, dtype, 8)
    x, r = nt.nested_tensor(tx, device=DEV, dtype=dtype), nt.nested_tensor(tr, device=DEV, dtype=dtype)
    g = torch.Generator().manual_seed(9)
    w, b = torch.randn(E, generator=g).to(dtype).to(DEV), torch.randn(E, generator=g).to(dtype).to(DEV)
    fused = ops.layer_norm(x._impl, (E,), w, b, 1e-5, residual=r._impl)
    two = torch.nn.functional.layer_norm(x + r, (E,), w, b, 1e-5)
    assert torch.equal(fused.buffer, two._impl.buffer)
    exp = oracle.layer_norm(oracle.add(oracle.ref_nested_tensor(tx, dtype=dtype), oracle.ref_nested_tensor(tr, dtype=dtype)),
                            (E,), w.cpu(), b.cpu(), 1e-5)
    _close(fused.buffer, exp.buffer, dtype)


def test_row_ops_at_encoder_size_properties():
    # C3-sized buffer: rows normalised without affine have mean 0 and variance 1
    g = torch.Generator().manual_seed(11)
    lens = [int(v) for v in torch.randint(32, 513, (32,), generator=g)]
    ts = [torch.randn(L, 768, generator=g).half() * 3 + 1 for L in lens]
    a = nt.nested_tensor(ts, device=DEV, dtype=torch.float16)
    y = torch.nn.functional.layer_norm(a, (768,))._impl.buffer.float().reshape(-1, 768)
    assert y.mean(1).abs().max().item() < 2e-3
    assert (y.var(1, unbiased=False) - 1).abs().max().item() < 5e-3
