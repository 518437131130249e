"""Parity of the HIP nested multi-head attention path with the CPU oracle.

Tolerances of the benchmark definition: fp32 <= 1e-5 relative to the output scale
(max |a-b| / max |b|), fp16 / bf16 <= 2e-2 absolute.  The shape list is the
reference's (test/test_nested_tensor_functional.py:1142-1160) plus the benchmark
configurations C3 (BERT-base, fp16) and C4 (bf16, high raggedness)."""

import random

import pytest
import torch

import nestedtensor_amd as nt
import oracle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)

FP32_REL = 1e-5
FP32_ELEM_ABS = 1e-5
HALF_ABS = 2e-2


def make_case(E, lens, seed, dtype, w_std=0.02, bias_std=0.0, x_std=1.0):
    g = torch.Generator().manual_seed(seed)
    xs = [(torch.randn(L, E, generator=g) * x_std).to(dtype) for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * w_std).to(dtype)
    W_out = (torch.randn(E, E, generator=g) * w_std).to(dtype)
    b_in = (torch.randn(3 * E, generator=g) * bias_std).to(dtype)
    b_out = (torch.randn(E, generator=g) * bias_std).to(dtype)
    return xs, W_in, b_in, W_out, b_out


def check(got_nt, exp_parts, dtype, exp64=None):
    got = got_nt._impl.buffer.float().cpu()
    exp = torch.cat([p.reshape(-1) for p in exp_parts]).float()
    assert got.shape == exp.shape
    assert torch.isfinite(got).all()
    err = (got - exp).abs().max().item()
    if dtype == torch.float32:
        scale = max(exp.abs().max().item(), 1e-30)
        assert err / scale <= FP32_REL, (err, scale)
        # and element by element, the way the reference's own tests compare
        # (assertEqual at 1e-5, test/utils_test_case.py:21,102-118) together with the
        # 1e-5 relative bound of the target: |a - b| <= 1e-5 + 1e-5 |b|
        excess = ((got - exp).abs() - (FP32_ELEM_ABS + FP32_REL * exp.abs())).max().item()
        assert excess <= 0.0, "worst element exceeds 1e-5 + 1e-5 |b| by %g" % excess
    else:
        assert err <= HALF_ABS, err
    if exp64 is not None:
        # the fused path accumulates in fp32 and must not be further from the
        # float64 answer than the reference's own dtype-rounded chain, up to
        # one unit of output rounding
        e64 = torch.cat([p.reshape(-1) for p in exp64]).float()
        assert (got - e64).abs().max().item() <= (exp - e64).abs().max().item() + HALF_ABS / 4
    return err


def run_min_mha(H, hd, xs, W_in, b_in, W_out, b_out, dtype, via="op"):
    E = H * hd
    a = nt.nested_tensor(xs, device=DEV, dtype=dtype)
    args = (H, hd, 0.0, False, a, a, a, W_in.to(DEV), b_in.to(DEV), float(hd) ** -0.5,
            W_out.to(DEV), b_out.to(DEV))
    return torch.ops.nestedtensor.min_mha(*args)


REF_SHAPES = [  # (num_heads, batch_size, seq_len_, head_size)
    (2, 1, 2, 1), (1, 3, 5, 4), (2, 3, 5, 2), (2, 1, 2, 2), (8, 8, 50, 16),
    (16, 64, 50, 16), (4, 32, 50, 256), (16, 32, 50, 64),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,B,Lmax,hd", REF_SHAPES)
def test_min_mha_reference_shapes(dtype, H, B, Lmax, hd):
    random.seed(H * 1000 + B)
    lens = [random.randint(1, Lmax) for _ in range(B)]
    E = H * hd
    xs, W_in, b_in, W_out, b_out = make_case(E, lens, 17, dtype, w_std=E ** -0.5, bias_std=0.1)
    got = run_min_mha(H, hd, xs, W_in, b_in, W_out, b_out, dtype)
    ref = oracle.ref_nested_tensor(xs, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)
    assert got.nested_size() == nt.nested_tensor(xs).nested_size()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,hd,lens", [(8, 32, (1, 64, 65, 300, 129)), (4, 128, (130, 7, 257, 64)),
                                       (2, 32, (513,)), (3, 128, (1, 2, 3)),
                                       (3, 32, (70, 200))])     # E = 96: not a multiple of the fused tile
def test_mfma_attention_head_dims_32_and_128(dtype, H, hd, lens):
    """head_dim 32 and 128 take the same MFMA kernels as 64 (self- and cross-attention);
    fp32 runs on the fp32 matrix instruction."""
    E = H * hd
    amp = 0.5 if dtype == torch.bfloat16 else 1.0
    xs, W_in, b_in, W_out, b_out = make_case(E, list(lens), 23, dtype, w_std=E ** -0.5, bias_std=0.1, x_std=amp)
    got = run_min_mha(H, hd, xs, W_in, b_in, W_out, b_out, dtype)
    ref = oracle.ref_nested_tensor(xs, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)
    # cross-attention: the same queries over memories of other lengths
    g = torch.Generator().manual_seed(29)
    kv_lens = [max(1, (L * 3) // 2 + 5) for L in lens]
    kv = [(torch.randn(L, E, generator=g) * amp).to(dtype) for L in kv_lens]
    qa, ka = nt.nested_tensor(xs, device=DEV, dtype=dtype), nt.nested_tensor(kv, device=DEV, dtype=dtype)
    got = torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, qa, ka, ka, W_in.to(DEV), b_in.to(DEV),
                                         hd ** -0.5, W_out.to(DEV), b_out.to(DEV))
    rk = oracle.ref_nested_tensor(kv, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, rk, rk, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("hd", [32, 64, 128])
def test_mfma_attention_boundary_lengths(hd, dtype):
    """Every length around the 32-row wavefront blocks, the 32- and 64-key tiles and
    the 128-row query tiles, in one batch, as queries and (rotated) as keys."""
    H = 2
    E = H * hd
    lens = [1, 2, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 191, 192, 193, 255, 256, 257]
    xs, W_in, b_in, W_out, b_out = make_case(E, lens, 31, dtype, w_std=E ** -0.5, bias_std=0.1)
    got = run_min_mha(H, hd, xs, W_in, b_in, W_out, b_out, dtype)
    ref = oracle.ref_nested_tensor(xs, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)
    g = torch.Generator().manual_seed(37)
    kv_lens = lens[7:] + lens[:7]
    kv = [torch.randn(L, E, generator=g).to(dtype) for L in kv_lens]
    qa, ka = nt.nested_tensor(xs, device=DEV, dtype=dtype), nt.nested_tensor(kv, device=DEV, dtype=dtype)
    got = torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, qa, ka, ka, W_in.to(DEV), b_in.to(DEV),
                                         hd ** -0.5, W_out.to(DEV), b_out.to(DEV))
    rk = oracle.ref_nested_tensor(kv, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, rk, rk, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_bt_min_mha_op_and_module_hook(dtype):
    # test_nested_tensor_functional.py:1087-1140: bt_min_mha == mha(nt, nt, nt)
    # == dense MHA with key_padding_mask (zero biases, as nn.MultiheadAttention
    # initialises them)
    random.seed(3)
    H, hd, B, Lmax = 8, 16, 8, 50
    E = H * hd
    lens = [random.randint(1, Lmax) for _ in range(B)]
    torch.manual_seed(1010)
    mha = torch.nn.MultiheadAttention(E, H).to(dtype).eval()
    xs = [torch.randn(L, E).to(dtype) for L in lens]
    a = nt.nested_tensor(xs, device=DEV, dtype=dtype)
    W_in = mha.in_proj_weight.detach().clone()
    b_in = mha.in_proj_bias.detach().clone()
    W_out = mha.out_proj.weight.detach().clone()
    b_out = mha.out_proj.bias.detach().clone()
    with torch.inference_mode():
        r_bt = torch.ops.nestedtensor.bt_min_mha(H, hd, 0.5, False, a, a, a, W_in.to(DEV), b_in.to(DEV),
                                                 float(hd) ** -0.5, W_out.to(DEV), b_in.to(DEV))
        mha_dev = mha.to(DEV)
        r_mod, w = mha_dev(a, a, a)
    assert w is None and isinstance(r_mod, nt.NestedTensor)
    assert torch.equal(r_bt._impl.buffer, r_mod._impl.buffer)       # zero out-bias: same result
    ref = oracle.ref_nested_tensor(xs, dtype=dtype)
    exp_bt = oracle.bt_min_mha(H, hd, 0.5, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_in)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(r_bt, exp, dtype)
    check(r_bt, exp_bt, dtype)
    # dense differential of the reference test: atol 5e-4 (fp32)
    if dtype == torch.float32:
        mha_cpu = mha.to("cpu").float()
        padded = torch.nn.utils.rnn.pad_sequence(xs)
        kpm = torch.ones(B, max(lens), dtype=torch.bool)
        for b, L in enumerate(lens):
            kpm[b, :L] = False
        with torch.no_grad():
            dense, _ = mha_cpu(padded, padded, padded, key_padding_mask=kpm, need_weights=False)
        dense = dense.transpose(0, 1) * (~kpm).unsqueeze(-1)
        assert torch.allclose(r_bt.to_padded_tensor(padding=0).cpu(), dense, atol=5e-4, rtol=1e-8)


def test_bt_min_mha_ignores_out_bias_and_min_mha_adds_it():
    H, hd = 2, 64
    E = H * hd
    xs, W_in, b_in, W_out, b_out = make_case(E, [5, 70, 33], 4, torch.float16, bias_std=0.5)
    a = nt.nested_tensor(xs, device=DEV, dtype=torch.float16)
    args = (H, hd, 0.0, False, a, a, a, W_in.to(DEV), b_in.to(DEV), hd ** -0.5, W_out.to(DEV))
    r_bt = torch.ops.nestedtensor.bt_min_mha(*args, b_out.to(DEV))
    r_min = torch.ops.nestedtensor.min_mha(*args, b_out.to(DEV))
    r_zero = torch.ops.nestedtensor.min_mha(*args, torch.zeros_like(b_out).to(DEV))
    assert torch.equal(r_bt._impl.buffer, r_zero._impl.buffer)
    assert not torch.equal(r_bt._impl.buffer, r_min._impl.buffer)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("q_lens,kv_lens", [((3, 130, 64), (77, 2, 200)),
                                            ((100, 100, 100, 1), (1, 64, 65, 513)),     # DETR-like: fixed queries
                                            ((257, 5), (128, 129))])
def test_cross_attention_different_kv_lengths(dtype, q_lens, kv_lens):
    # fp16 / bf16 with head_dim 64 take the MFMA kernel with one key sequence per query
    # sequence; fp32 the general kernel
    H, hd = 4, 64
    E = H * hd
    g = torch.Generator().manual_seed(5)
    # bf16 keeps 8 bits: inputs at half the scale hold the outputs below 2, where one unit of
    # output rounding (the fused path rounds once, the reference after every op) is under 2e-2
    amp = 0.5 if dtype == torch.bfloat16 else 1.0
    q = [(torch.randn(L, E, generator=g) * amp).to(dtype) for L in q_lens]
    kv = [(torch.randn(L, E, generator=g) * amp).to(dtype) for L in kv_lens]
    _, W_in, b_in, W_out, b_out = make_case(E, [1], 6, dtype, w_std=E ** -0.5, bias_std=0.1)
    qa, ka = nt.nested_tensor(q, device=DEV, dtype=dtype), nt.nested_tensor(kv, device=DEV, dtype=dtype)
    got = torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, qa, ka, ka, W_in.to(DEV), b_in.to(DEV),
                                         hd ** -0.5, W_out.to(DEV), b_out.to(DEV))
    rq, rk = oracle.ref_nested_tensor(q, dtype=dtype), oracle.ref_nested_tensor(kv, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, rq, rk, rk, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)
    # key and value of the same nested size but different contents (key = memory + position)
    v2 = [(torch.randn(L, E, generator=g) * amp).to(dtype) for L in kv_lens]
    va = nt.nested_tensor(v2, device=DEV, dtype=dtype)
    got = torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, qa, ka, va, W_in.to(DEV), b_in.to(DEV),
                                         hd ** -0.5, W_out.to(DEV), b_out.to(DEV))
    rv = oracle.ref_nested_tensor(v2, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, rq, rk, rv, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(300, 256, 128), (1000, 192, 64), (257, 70, 96), (5, 64, 40)])
def test_linear_transposed(M, N, K, dtype):
    from nestedtensor_amd import _C
    g = torch.Generator().manual_seed(17)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.2).to(dtype)
    b = torch.randn(N, generator=g).to(dtype)
    ld = (M + 72 + 7) // 8 * 8
    ct = torch.full((N, ld), 7.0, dtype=dtype, device=DEV)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    _C.check(_C.lib.nt_linear_transposed(_C.ptr(xd), K, _C.ptr(wd), _C.ptr(bd), _C.ptr(ct), ld, M, N, K,
                                         _C.dtype_code(dtype), _C.current_stream(DEV)))
    ref = (x.double() @ w.double().t() + b.double()).t()
    got = ct[:, :M].double().cpu()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (got - ref).abs().max().item() <= tol * max(1.0, ref.abs().max().item())
    assert bool((ct[:, M:] == 7.0).all())          # nothing is written past column M


@pytest.mark.parametrize("M,E,K", [(300, 128, 128), (777, 256, 64), (5, 384, 200)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_linear_kv_one_launch(M, E, K, dtype):
    # key projection row-major and value projection transposed from one launch
    # (mha.cpp:45-54 for key and value that are one tensor), against float64
    from nestedtensor_amd import _C
    g = torch.Generator().manual_seed(23)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(2 * E, K, generator=g) * 0.2).to(dtype)
    b = torch.randn(2 * E, generator=g).to(dtype)
    ld = (M + 72 + 7) // 8 * 8
    kp = torch.full((M, E), 7.0, dtype=dtype, device=DEV)
    vt = torch.full((E, ld), 7.0, dtype=dtype, device=DEV)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    _C.check(_C.lib.nt_linear_kv(_C.ptr(xd), K, _C.ptr(wd), _C.ptr(bd), _C.ptr(kp), E, _C.ptr(vt), ld, M, E, K,
                                 _C.dtype_code(dtype), _C.current_stream(DEV)))
    ref = x.double() @ w.double().t() + b.double()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    scale = max(1.0, ref.abs().max().item())
    assert (kp.double().cpu() - ref[:, :E]).abs().max().item() <= tol * scale
    assert (vt[:, :M].double().cpu() - ref[:, E:].t()).abs().max().item() <= tol * scale
    assert bool((vt[:, M:] == 7.0).all())          # nothing is written past column M


def test_mha_input_errors():
    a = nt.nested_tensor([torch.randn(3, 4), torch.randn(2, 4)], device=DEV)
    b2 = nt.nested_tensor([torch.randn(3), torch.randn(2)], device=DEV)
    W, bi, Wo, bo = (torch.randn(12, 4, device=DEV), torch.randn(12, device=DEV),
                     torch.randn(4, 4, device=DEV), torch.randn(4, device=DEV))
    with pytest.raises(RuntimeError, match="query needs to be 3 dim."):
        torch.ops.nestedtensor.min_mha(2, 2, 0.0, False, b2, a, a, W, bi, 1.0, Wo, bo)
    with pytest.raises(RuntimeError, match="key needs to be 3 dim."):
        torch.ops.nestedtensor.bt_min_mha(2, 2, 0.0, False, a, b2, a, W, bi, 1.0, Wo, bo)
    with pytest.raises(RuntimeError, match="Input projection bias needs to be defined."):
        torch.ops.nestedtensor.min_mha(2, 2, 0.0, False, a, a, a, W, None, 1.0, Wo, bo)
    irregular = nt.nested_tensor([torch.randn(3, 4), torch.randn(2, 5)], device=DEV)
    with pytest.raises(RuntimeError, match="query's third dimension must be regular."):
        torch.ops.nestedtensor.min_mha(2, 2, 0.0, False, irregular, a, a, W, bi, 1.0, Wo, bo)


def test_weights_on_the_host_raise_before_any_launch():
    # a module left on the host must raise, not hand the kernels a host pointer
    H, hd = 2, 64
    E = H * hd
    for dtype in (torch.float16, torch.float32):
        xs, W_in, b_in, W_out, b_out = make_case(E, [5, 9], 3, dtype)
        a = nt.nested_tensor(xs, device=DEV, dtype=dtype)
        dev = [t.to(DEV) for t in (W_in, b_in, W_out, b_out)]
        host = [W_in, b_in, W_out, b_out]
        for i in range(4):
            w = list(dev)
            w[i] = host[i]
            with pytest.raises(RuntimeError, match="is on cpu"):
                torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, a, a, a, w[0], w[1], hd ** -0.5, w[2], w[3])
        # cross-attention takes the operator with three projections
        k = nt.nested_tensor([torch.randn(7, E).to(dtype), torch.randn(3, E).to(dtype)], device=DEV, dtype=dtype)
        with pytest.raises(RuntimeError, match="is on cpu"):
            torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, a, k, k, dev[0], dev[1], hd ** -0.5, W_out, dev[3])
        # biases of the wrong length are refused too
        with pytest.raises(RuntimeError, match="in_proj_bias must have"):
            torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, a, a, a, dev[0], dev[1][:E], hd ** -0.5, dev[2], dev[3])
        with pytest.raises(RuntimeError, match="out_proj_bias must have"):
            torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, a, a, a, dev[0], dev[1], hd ** -0.5, dev[2], dev[3][:5])
    a = nt.nested_tensor([torch.randn(4, 8), torch.randn(2, 8)], device=DEV)
    with pytest.raises(RuntimeError, match="is on cpu"):
        torch.nn.functional.linear(a, torch.randn(16, 8))
    with pytest.raises(RuntimeError, match="is on cpu"):
        torch.nn.functional.linear(a, torch.randn(16, 8, device=DEV), torch.randn(16))
    with pytest.raises(RuntimeError, match="bias of 3 elements"):
        torch.nn.functional.linear(a, torch.randn(16, 8, device=DEV), torch.randn(3, device=DEV))
    with pytest.raises(RuntimeError, match="weight and bias must have 8 elements"):
        torch.ops.nestedtensor.layer_norm_packed(a._impl.buffer, None, torch.ones(4, device=DEV), None, 8, 1e-5)


def _c3():
    g = torch.Generator().manual_seed(1010 + 2)
    lens = [int(v) for v in torch.randint(32, 513, (32,), generator=g)]
    E = 768
    xs = [torch.randn(L, E, generator=g).half() for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * 0.02).half()
    W_out = (torch.randn(E, E, generator=g) * 0.02).half()
    return lens, xs, W_in, torch.zeros(3 * E).half(), W_out, torch.zeros(E).half()


def test_config_c3_bert_base_fp16():
    lens, xs, W_in, b_in, W_out, b_out = _c3()
    got = run_min_mha(12, 64, xs, W_in, b_in, W_out, b_out, torch.float16)
    ref = oracle.ref_nested_tensor(xs, dtype=torch.float16)
    exp = oracle.min_mha(12, 64, 0.0, False, ref, ref, ref, W_in, b_in, 64 ** -0.5, W_out, b_out)
    ref64 = oracle.ref_nested_tensor([x.double() for x in xs], dtype=torch.float64)
    exp64 = oracle.min_mha(12, 64, 0.0, False, ref64, ref64, ref64, W_in.double(), b_in.double(),
                           64 ** -0.5, W_out.double(), b_out.double())
    err = check(got, exp, torch.float16, exp64)
    print("C3 fp16 max abs err vs oracle: %.3e" % err)
    # the module route gives the same tensor
    mha = torch.nn.MultiheadAttention(768, 12).half().eval()
    with torch.no_grad():
        mha.in_proj_weight.copy_(W_in)
        mha.in_proj_bias.zero_()
        mha.out_proj.weight.copy_(W_out)
        mha.out_proj.bias.zero_()
    a = nt.nested_tensor(xs, device=DEV, dtype=torch.float16)
    with torch.inference_mode():
        r_mod, _ = mha.to(DEV)(a, a, a)
    assert torch.equal(r_mod._impl.buffer, got._impl.buffer)


def test_config_c4_bf16_high_raggedness():
    g = torch.Generator().manual_seed(1010 + 3)
    raw = torch.empty(128).exponential_(1.0 / 96.0, generator=g)
    lens = [int(v) for v in raw.round().clamp(8, 512)]
    E, H = 1024, 16
    xs = [torch.randn(L, E, generator=g).bfloat16() for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * 0.02).bfloat16()
    W_out = (torch.randn(E, E, generator=g) * 0.02).bfloat16()
    b_in, b_out = torch.zeros(3 * E).bfloat16(), torch.zeros(E).bfloat16()
    a = nt.nested_tensor(xs, device=DEV, dtype=torch.bfloat16)
    got = torch.ops.nestedtensor.bt_min_mha(H, 64, 0.0, False, a, a, a, W_in.to(DEV), b_in.to(DEV),
                                            64 ** -0.5, W_out.to(DEV), b_out.to(DEV))
    ref = oracle.ref_nested_tensor(xs, dtype=torch.bfloat16)
    exp = oracle.min_mha(H, 64, 0.0, False, ref, ref, ref, W_in, b_in, 64 ** -0.5, W_out, b_out)
    err = check(got, exp, torch.bfloat16)
    print("C4 bf16 max abs err vs oracle: %.3e" % err)


def test_linear_packed_fast_path():
    # F.linear on a NestedTensor: one GEMM on the packed view (matmul.cpp:13-41)
    g = torch.Generator().manual_seed(8)
    for dtype, tol in ((torch.float32, 1e-5), (torch.float16, 2e-2)):
        xs = [torch.randn(L, 96, generator=g).to(dtype) for L in (5, 131, 64)]
        W = (torch.randn(200, 96, generator=g) * 0.1).to(dtype)
        b = torch.randn(200, generator=g).to(dtype)
        a = nt.nested_tensor(xs, device=DEV, dtype=dtype)
        y = torch.nn.functional.linear(a, W.to(DEV), b.to(DEV))
        assert y.size() == (3, None, 200)
        for yi, xi in zip(y.unbind(), xs):
            exp = torch.nn.functional.linear(xi, W, b).float()
            assert (yi.float().cpu() - exp).abs().max() <= tol * max(1.0, exp.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [
    (300, 200, 64),        # far fewer 256-row tiles than CUs: 128 x 64 tiles, whole K tiles
    (300, 200, 72),        # K tail: element-wise loads
    (1000, 500, 200),      # 128 x 64 tiles, ragged in every dimension
    (3200, 768, 128),      # more 128 x 64 tiles than CUs: 128 x 128 tiles
    (3210, 760, 104),
    (8200, 1000, 64),      # one partly filled round of 256 x 128 tiles
    (9813, 2304, 64),      # two rounds of 256 x 192 tiles beat three of 256 x 128
    (9813, 2304, 40),
    (4096, 4096, 64),      # one round of 256 x 256 tiles
    (4100, 4090, 24),
])
def test_linear_tile_shapes(M, N, K, dtype):
    # the launcher picks one of five tile shapes per problem; every shape, with
    # and without a K tail, against an fp32 reference of the same product
    from nestedtensor_amd import ops
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.25).to(dtype)
    b = torch.randn(N, generator=g).to(dtype)
    y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV)).float().cpu()
    exp = x.float() @ w.float().t() + b.float()
    tol = 2e-2 if dtype == torch.float16 else 6e-2   # one rounding of |y| <= ~16 to the output type
    assert (y - exp).abs().max().item() <= tol


def test_linear_qkv_tile_shapes():
    # fused in-projection: Q | K row-major, V transposed, on the shape that takes
    # the 256 x 192 tiles (2E = 1536 is a multiple of 192) and on small ones (128 x 64
    # tiles; 128 x 128 where those would be more than the CUs)
    from nestedtensor_amd import _C
    for (T, E) in ((9813, 768), (70, 64), (471, 768), (645, 1024)):
        g = torch.Generator().manual_seed(T)
        x = torch.randn(T, E, generator=g).half()
        w = (torch.randn(3 * E, E, generator=g) * 0.05).half()
        b = torch.randn(3 * E, generator=g).half()
        xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
        ldvt = (T + 72 + 7) // 8 * 8
        qk = torch.empty(T, 2 * E, dtype=torch.float16, device=DEV)
        vt = torch.zeros(E, ldvt, dtype=torch.float16, device=DEV)
        _C.check(_C.lib.nt_linear_qkv(_C.ptr(xd), E, _C.ptr(wd), _C.ptr(bd), _C.ptr(qk), 2 * E,
                                      _C.ptr(vt), ldvt, T, E, E, _C.dtype_code(torch.float16),
                                      _C.current_stream(xd.device)))
        exp = x.float() @ w.float().t() + b.float()
        assert (qk.float().cpu() - exp[:, :2 * E]).abs().max().item() <= 2e-2
        assert (vt[:, :T].float().cpu() - exp[:, 2 * E:].t()).abs().max().item() <= 2e-2
        assert vt[:, T:].abs().max().item() == 0      # nothing written past the last token


def test_min_mha_under_hip_graph_replays():
    # the three launches of a layer captured in a graph: every replay, with new
    # input contents and eager work in between, must equal the eager result
    E, H = 256, 4
    xs, W_in, b_in, W_out, b_out = make_case(E, [37, 200, 64, 129], 21, torch.float16, bias_std=0.1)
    a = nt.nested_tensor(xs, device=DEV, dtype=torch.float16)
    dW_in, db_in, dW_out, db_out = (t.to(DEV) for t in (W_in, b_in, W_out, b_out))

    def layer():
        return torch.ops.nestedtensor.min_mha(H, 64, 0.0, False, a, a, a, dW_in, db_in, 0.125, dW_out, db_out)

    for _ in range(3):          # warm up: schedule upload, kernel attributes, allocator
        eager = layer()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer()
        with torch.cuda.graph(graph, stream=side):
            out = layer()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.Generator().manual_seed(22)
    for rep in range(4):
        new = torch.randn(a._impl.buffer.shape, generator=g).half().to(DEV)
        a._impl.buffer.copy_(new)
        graph.replay()
        torch.cuda.synchronize()
        got = out._impl.buffer.clone()
        exp = layer()._impl.buffer
        torch.cuda.synchronize()
        assert torch.equal(got, exp), "replay %d differs from the eager layer" % rep


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("K", [128, 320, 512, 896])
def test_linear_k_tile_counts_on_the_256x128_shape(K, dtype):
    # K = 2, 5, 8, 14 tiles of 64: every residue of the three-buffer ring of the
    # 256 x 128 tile shape (N = 128 admits no other shape), whose last iterations
    # re-read the final K tile into a buffer the epilogue then reuses
    from nestedtensor_amd import ops
    M, N = 700, 128
    g = torch.Generator().manual_seed(K)
    x = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * K ** -0.5).to(dtype)
    b = torch.randn(N, generator=g).to(dtype)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    exp = x.float() @ w.float().t() + b.float()
    first = ops.linear(xd, wd, bd)
    for _ in range(5):     # the same launch again and again: no run may differ
        assert torch.equal(ops.linear(xd, wd, bd), first)
    tol = 2e-2 if dtype == torch.float16 else 6e-2
    assert (first.float().cpu() - exp).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("order", ["rising", "falling", "spike"])
def test_attention_reference_maximum_moves(dtype, order):
    """Scores that grow along the keys by far more than the slack the kernel allows
    its reference maximum (2^8): the maximum is raised and the accumulators are
    rescaled on every tile ("rising"), never after the first ("falling"), or once in
    the middle ("spike")."""
    H, hd = 2, 64
    E = H * hd
    L = 300
    g = torch.Generator().manual_seed(5)
    u = torch.randn(E, generator=g)
    u = u / u.norm() * 8.0
    amp = torch.linspace(0.2, 3.0, L)
    if order == "falling":
        amp = amp.flip(0)
    elif order == "spike":
        amp = torch.full((L,), 0.3)
        amp[170] = 3.0
    x = (amp[:, None] * u[None, :] + 0.05 * torch.randn(L, E, generator=g)).to(dtype)
    short = (0.5 * torch.randn(40, E, generator=g)).to(dtype)
    # identity-like projections keep q . k ~ amp_i amp_j |u|^2 / H per head
    W_in = torch.cat([torch.eye(E), torch.eye(E), torch.eye(E)]).to(dtype)
    b_in = torch.zeros(3 * E, dtype=dtype)
    W_out = torch.eye(E).to(dtype)
    b_out = torch.zeros(E, dtype=dtype)
    xs = [x, short]
    got = run_min_mha(H, hd, xs, W_in, b_in, W_out, b_out, dtype)
    ref = oracle.ref_nested_tensor(xs, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_out)
    # the reference rounds q * scaling and the scores to the storage type, which
    # at scores of this size (up to ~36) moves its own result; compare with the
    # float64 answer as well
    ref64 = oracle.ref_nested_tensor([p.double() for p in xs], dtype=torch.float64)
    exp64 = oracle.min_mha(H, hd, 0.0, False, ref64, ref64, ref64, W_in.double(), b_in.double(),
                           hd ** -0.5, W_out.double(), b_out.double())
    gotf = got._impl.buffer.float().cpu()
    e64 = torch.cat([p.reshape(-1) for p in exp64]).float()
    e = torch.cat([p.reshape(-1) for p in exp]).float()
    assert torch.isfinite(gotf).all()
    err64 = (gotf - e64).abs().max().item()
    ref_err64 = (e - e64).abs().max().item()
    assert err64 <= max(HALF_ABS, ref_err64 + HALF_ABS / 4), (err64, ref_err64)


def test_attention_vt_items_without_keys_or_queries():
    # through the C ABI: a work item with key length 0 writes zeros to its query
    # rows, one with query length 0 writes nothing
    from nestedtensor_amd import _C
    H, hd = 2, 64
    E = H * hd
    T = 200
    g = torch.Generator().manual_seed(9)
    q = torch.randn(T, E, generator=g).half().to(DEV)
    k = torch.randn(T, E, generator=g).half().to(DEV)
    ldvt = T + 72
    vt = torch.randn(E, ldvt, generator=g).half().to(DEV)
    out = torch.full((T, E), 7.0, dtype=torch.float16, device=DEV)
    # item 0: queries 0..129 (two tiles) without keys; item 2: no queries; item 3: a real one
    sched = torch.tensor([[0, 130, 0, 0, 0, 0, 0, 0],
                          [0, 130, 128, 0, 0, 0, 0, 0],
                          [130, 0, 0, 0, 130, 20, 0, 0],
                          [150, 50, 0, 0, 150, 50, 0, 0]], dtype=torch.int32, device=DEV)
    _C.check(_C.lib.nt_varlen_attention_vt(_C.ptr(q), E, _C.ptr(k), E, _C.ptr(vt), ldvt, _C.ptr(out), E,
                                           _C.ptr(sched), 4, H, hd, T, 0.125, _C.dtype_code(torch.float16),
                                           _C.current_stream(DEV)))
    torch.cuda.synchronize()
    o = out.float().cpu()
    assert (o[:130] == 0).all()
    assert (o[130:150] == 7).all()
    qs, ks, vs = q[150:].float().cpu(), k[150:].float().cpu(), vt[:, 150:200].float().cpu().t()
    for h in range(H):
        sl = slice(h * hd, (h + 1) * hd)
        p = torch.softmax(qs[:, sl] @ ks[:, sl].t() * 0.125, dim=-1)
        assert (o[150:, sl] - p @ vs[:, sl]).abs().max().item() <= HALF_ABS


# (num_heads, batch_size, seq_len_, head_size): the four largest shapes of
# test/test_nested_tensor_functional.py:1155-1160
REF_SHAPES_LARGE = [(16, 128, 50, 16), (16, 256, 50, 16), (4, 256, 50, 256), (16, 256, 50, 64)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("H,B,Lmax,hd", REF_SHAPES_LARGE)
def test_min_mha_reference_shapes_large(dtype, H, B, Lmax, hd):
    random.seed(H * 1000 + B)
    lens = [random.randint(1, Lmax) for _ in range(B)]
    E = H * hd
    xs, W_in, b_in, W_out, b_out = make_case(E, lens, 19, dtype, w_std=E ** -0.5, bias_std=0.1)
    got = run_min_mha(H, hd, xs, W_in, b_in, W_out, b_out, dtype)
    ref = oracle.ref_nested_tensor(xs, dtype=dtype)
    exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_out)
    check(got, exp, dtype)


@pytest.mark.parametrize("hd", [32, 64, 128])
def test_fp32_attention_padded_grid_and_work_list(hd):
    # the two C entry points of the fp32 matrix-pipe kernel: nt_varlen_attention (grid
    # padded to the longest sequence, device offsets) and nt_varlen_attention_scheduled
    # (work list); same tiles, same arithmetic, so the same bits, and both against
    # a float64 softmax(q k^T) v per sequence and head
    from nestedtensor_amd import _C
    from nestedtensor_amd.impl import NestedTensorImpl
    H = 3
    E = H * hd
    q_lens, k_lens = [5, 130, 64, 1, 257], [77, 33, 200, 1, 64]
    g = torch.Generator().manual_seed(hd)
    Tq, Tk = sum(q_lens), sum(k_lens)
    q = torch.randn(Tq, E, generator=g)
    k = torch.randn(Tk, E, generator=g)
    v = torch.randn(Tk, E, generator=g)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    qi = NestedTensorImpl(qd.reshape(-1), torch.tensor([[L, E] for L in q_lens], dtype=torch.int64))
    ki = NestedTensorImpl(kd.reshape(-1), torch.tensor([[L, E] for L in k_lens], dtype=torch.int64))
    scale = hd ** -0.5
    out_a = torch.full((Tq, E), float("nan"), device=DEV)
    out_b = torch.full((Tq, E), float("nan"), device=DEV)
    stream = _C.current_stream(DEV)
    _C.check(_C.lib.nt_varlen_attention(
        _C.ptr(qd), E, _C.ptr(kd), E, _C.ptr(vd), E, _C.ptr(out_a), E, _C.ptr(qi.row_offsets_dev()),
        _C.ptr(ki.row_offsets_dev()), len(q_lens), H, hd, max(q_lens), scale, _C.dtype_code(torch.float32), stream))
    sched = qi.attention_schedule(kv=ki)
    _C.check(_C.lib.nt_varlen_attention_scheduled(
        _C.ptr(qd), E, _C.ptr(kd), E, _C.ptr(vd), E, _C.ptr(out_b), E, _C.ptr(sched), sched.size(0), H, hd,
        scale, _C.dtype_code(torch.float32), stream))
    torch.cuda.synchronize()
    assert torch.equal(out_a, out_b)
    exp = torch.empty(Tq, E, dtype=torch.float64)
    qo = ko = 0
    for Lq, Lk in zip(q_lens, k_lens):
        for h in range(H):
            c = slice(h * hd, (h + 1) * hd)
            s = (q[qo:qo + Lq, c].double() @ k[ko:ko + Lk, c].double().t()) * scale
            exp[qo:qo + Lq, c] = torch.softmax(s, -1) @ v[ko:ko + Lk, c].double()
        qo, ko = qo + Lq, ko + Lk
    err = (out_a.cpu().double() - exp).abs().max().item()
    assert err <= FP32_REL * exp.abs().max().item(), err
    # rows that are not 16-byte aligned are refused by the work-list entry point and
    # take the scalar kernel in the other
    rc = _C.lib.nt_varlen_attention_scheduled(
        _C.ptr(qd), E + 1, _C.ptr(kd), E, _C.ptr(vd), E, _C.ptr(out_b), E, _C.ptr(sched), sched.size(0), H, hd,
        scale, _C.dtype_code(torch.float32), stream)
    assert rc != 0


def test_encoder_layer_under_hip_graph_replays():
    # a whole encoder layer on the packed layout (attention, add + layer norm, feed-forward
    # with gelu in the GEMM epilogue, add + layer norm: seven launches) captured once and
    # replayed with new token values; every replay must equal the eager layer
    from nestedtensor_amd import ops
    E, H = 256, 4
    xs, W_in, b_in, W_out, b_out = make_case(E, [37, 200, 64, 129, 5], 41, torch.float16, bias_std=0.1)
    a = nt.nested_tensor(xs, device=DEV, dtype=torch.float16)
    g = torch.Generator().manual_seed(43)
    W1 = (torch.randn(4 * E, E, generator=g) * E ** -0.5).half().to(DEV)
    W2 = (torch.randn(E, 4 * E, generator=g) * (4 * E) ** -0.5).half().to(DEV)
    b1, b2 = (torch.randn(4 * E, generator=g) * 0.1).half().to(DEV), (torch.randn(E, generator=g) * 0.1).half().to(DEV)
    ln_w, ln_b = torch.ones(E, device=DEV).half(), torch.zeros(E, device=DEV).half()
    dW_in, db_in, dW_out, db_out = (t.to(DEV) for t in (W_in, b_in, W_out, b_out))

    def layer():
        y = torch.ops.nestedtensor.min_mha(H, 64, 0.0, False, a, a, a, dW_in, db_in, 0.125, dW_out, db_out)
        h = ops.layer_norm(y._impl, (E,), ln_w, ln_b, 1e-5, residual=a._impl)
        f = ops.linear_nt(h, W1, b1, "gelu")
        o = ops.linear_nt(f, W2, b2)
        return ops.layer_norm(o, (E,), ln_w, ln_b, 1e-5, residual=h).buffer

    for _ in range(3):
        layer()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer()
        with torch.cuda.graph(graph, stream=side):
            out = layer()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        a._impl.buffer.copy_(torch.randn(a._impl.buffer.shape, generator=g).half().to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        exp = layer()
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, exp), "replay %d differs from the eager layer" % rep
