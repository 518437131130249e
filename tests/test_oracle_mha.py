"""Pins the CPU oracle for nested multi-head attention against library routines
and a float64 brute force.  No GPU, no product code."""

import math
import random

import torch

import oracle


def _mk(E, H, lens, seed, dtype=torch.float32, bias_scale=0.1):
    g = torch.Generator().manual_seed(seed)
    xs = [torch.randn(L, E, generator=g).to(dtype) for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * 0.2).to(dtype)
    b_in = (torch.randn(3 * E, generator=g) * bias_scale).to(dtype)
    W_out = (torch.randn(E, E, generator=g) * 0.2).to(dtype)
    b_out = (torch.randn(E, generator=g) * bias_scale).to(dtype)
    return xs, W_in, b_in, W_out, b_out


def _brute_force_f64(xs, W_in, b_in, W_out, b_out, H):
    """Textbook multi-head attention in float64 with explicit loops over heads."""
    outs = []
    for x in xs:
        x = x.double()
        E = x.size(1)
        hd = E // H
        q = x @ W_in[:E].double().t() + b_in[:E].double()
        k = x @ W_in[E:2 * E].double().t() + b_in[E:2 * E].double()
        v = x @ W_in[2 * E:].double().t() + b_in[2 * E:].double()
        o = torch.zeros_like(q)
        for h in range(H):
            sl = slice(h * hd, (h + 1) * hd)
            s = (q[:, sl] @ k[:, sl].t()) / math.sqrt(hd)
            p = torch.softmax(s, -1)
            o[:, sl] = p @ v[:, sl]
        outs.append(o @ W_out.double().t() + b_out.double())
    return outs


def test_min_mha_equals_torch_mha_per_sequence():
    # the reference's own differential: test_nested_tensor_functional.py:648-667
    E, H = 16, 4
    lens = [3, 7, 1, 12]
    xs, W_in, b_in, W_out, b_out = _mk(E, H, lens, 5)
    nt = oracle.ref_nested_tensor(xs)
    got = oracle.min_mha(H, E // H, 0.0, False, nt, nt, nt, W_in, b_in, (E // H) ** -0.5, W_out, b_out)
    mha = torch.nn.MultiheadAttention(E, H)
    with torch.no_grad():
        mha.in_proj_weight.copy_(W_in)
        mha.in_proj_bias.copy_(b_in)
        mha.out_proj.weight.copy_(W_out)
        mha.out_proj.bias.copy_(b_out)
    mha.eval()
    for x, o in zip(xs, got):
        with torch.no_grad():
            ref, _ = mha(x.unsqueeze(1), x.unsqueeze(1), x.unsqueeze(1), need_weights=False)
        assert torch.allclose(o, ref.squeeze(1), atol=1e-5, rtol=1e-5)


def test_min_mha_equals_dense_mha_with_key_padding_mask():
    # test_nested_tensor_functional.py:1118-1140
    E, H = 32, 4
    lens = [5, 9, 2]
    xs, W_in, b_in, W_out, b_out = _mk(E, H, lens, 6)
    nt = oracle.ref_nested_tensor(xs)
    got = oracle.min_mha(H, E // H, 0.0, False, nt, nt, nt, W_in, b_in, (E // H) ** -0.5, W_out, b_out)
    mha = torch.nn.MultiheadAttention(E, H)
    with torch.no_grad():
        mha.in_proj_weight.copy_(W_in)
        mha.in_proj_bias.copy_(b_in)
        mha.out_proj.weight.copy_(W_out)
        mha.out_proj.bias.copy_(b_out)
    mha.eval()
    padded = torch.nn.utils.rnn.pad_sequence(xs)              # [Lmax, B, E]
    kpm = torch.ones(len(lens), max(lens), dtype=torch.bool)
    for b, L in enumerate(lens):
        kpm[b, :L] = False
    with torch.no_grad():
        dense, _ = mha(padded, padded, padded, key_padding_mask=kpm, need_weights=False)
    for b, L in enumerate(lens):
        assert torch.allclose(got[b], dense[:L, b], atol=1e-5, rtol=1e-5)


def test_min_mha_equals_f64_brute_force():
    E, H = 24, 3
    lens = [4, 11, 6]
    xs, W_in, b_in, W_out, b_out = _mk(E, H, lens, 8)
    nt = oracle.ref_nested_tensor(xs)
    got = oracle.min_mha(H, E // H, 0.0, False, nt, nt, nt, W_in, b_in, (E // H) ** -0.5, W_out, b_out)
    ref = _brute_force_f64(xs, W_in, b_in, W_out, b_out, H)
    for a, b in zip(got, ref):
        assert (a.double() - b).abs().max() < 1e-5


def test_min_mha_cross_attention_shapes():
    E, H = 8, 2
    g = torch.Generator().manual_seed(2)
    q = [torch.randn(L, E, generator=g) for L in (3, 5)]
    kv = [torch.randn(L, E, generator=g) for L in (7, 2)]
    _, W_in, b_in, W_out, b_out = _mk(E, H, [1], 9)
    got = oracle.min_mha(H, E // H, 0.0, False, oracle.ref_nested_tensor(q), oracle.ref_nested_tensor(kv),
                         oracle.ref_nested_tensor(kv), W_in, b_in, (E // H) ** -0.5, W_out, b_out)
    mha = torch.nn.MultiheadAttention(E, H)
    with torch.no_grad():
        mha.in_proj_weight.copy_(W_in)
        mha.in_proj_bias.copy_(b_in)
        mha.out_proj.weight.copy_(W_out)
        mha.out_proj.bias.copy_(b_out)
    for a, qq, kk in zip(got, q, kv):
        with torch.no_grad():
            ref, _ = mha(qq.unsqueeze(1), kk.unsqueeze(1), kk.unsqueeze(1), need_weights=False)
        assert torch.allclose(a, ref.squeeze(1), atol=1e-5, rtol=1e-5)


def test_bt_min_mha_equals_min_mha_without_out_bias():
    # test_nested_tensor_functional.py:1115 asserts equality at 1e-5 (zero biases there)
    random.seed(1010)
    for (H, B, Lmax, hd) in [(2, 1, 2, 1), (1, 3, 5, 4), (2, 3, 5, 2), (8, 8, 50, 16)]:
        E = H * hd
        lens = [random.randint(1, Lmax) for _ in range(B)]
        xs, W_in, b_in, W_out, b_out = _mk(E, H, lens, 12)
        nt = oracle.ref_nested_tensor(xs)
        a = oracle.bt_min_mha(H, hd, 0.5, False, nt, nt, nt, W_in, b_in, hd ** -0.5, W_out, b_in)
        b = oracle.min_mha(H, hd, 0.0, False, nt, nt, nt, W_in, b_in, hd ** -0.5, W_out,
                           torch.zeros(E))
        for x, y in zip(a, b):
            # the 1e-6 in the softmax denominator and exp(-10000) leakage are
            # below 1e-5 relative to the output scale
            assert (x - y).abs().max() < 1e-5 * max(1.0, float(y.abs().max()))
