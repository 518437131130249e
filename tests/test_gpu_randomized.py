"""Seeded random shapes through the whole path: the projection GEMM over every tile
shape its launcher can pick, pack -> to_tensor_mask -> nested_tensor_from_tensor_mask
round trips on ragged image batches, the row-major 1x1 convolution, and attention
layers of random head counts and lengths against the oracle's min_mha
(mha.cpp:18-69).  The fixed cases of the other files sit on the boundaries their
kernels have; these look for the ones nobody thought of."""

import random

import pytest
import torch

import nestedtensor_amd as nt
import oracle
from nestedtensor_amd import ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_linear_random_shapes(seed):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for _ in range(40):
        M = rng.choice([1, 7, 100, 129, 300, 1000, 2047, 3200, 5000, 9000])
        N = rng.choice([8, 64, 72, 200, 512, 768, 1000])
        K = rng.choice([8, 24, 64, 72, 200, 512])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        x = torch.randn(M, K, generator=g).to(dtype)
        w = (torch.randn(N, K, generator=g) * 0.2).to(dtype)
        b = torch.randn(N, generator=g).to(dtype)
        y = ops.linear(x.to(DEV), w.to(DEV), b.to(DEV)).float().cpu()
        exp = x.float() @ w.float().t() + b.float()
        # one rounding of the result to the storage type
        tol = (2e-2 if dtype == torch.float16 else 1.2e-1) * max(1.0, exp.abs().max().item() / 16)
        assert (y - exp).abs().max().item() <= tol, (M, N, K, dtype)


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_image_batches_round_trip(seed):
    # bit-exact: what comes back from the dense (tensor, mask) pair is what went in,
    # and every constituent sits in its corner of the padded tensor
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for _ in range(30):
        B = rng.randint(1, 9)
        C = rng.choice([1, 3, 5])
        Hm = rng.randint(1, 70)
        Wm = rng.choice([1, 5, 17, 64, 95, 96, 97, 130, 300, 1015])
        dtype = rng.choice([torch.float32, torch.float16, torch.int64])
        parts = []
        for _b in range(B):
            t = torch.randn(C, rng.randint(1, Hm), rng.randint(1, Wm), generator=g)
            parts.append((t * 10).to(dtype) if dtype == torch.int64 else t.to(dtype))
        a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
        data, mask = a.to_tensor_mask()
        ref_data, ref_mask = oracle.to_tensor_mask(oracle.ref_nested_tensor(parts, dtype=dtype))
        assert torch.equal(mask.cpu(), ref_mask)
        assert torch.equal(data.cpu().view(torch.uint8), ref_data.contiguous().view(torch.uint8))
        back = nt.nested_tensor_from_tensor_mask(data, mask)
        got = [t.cpu() for t in back.unbind()]
        assert len(got) == len(parts)
        for x, y in zip(got, parts):
            assert x.shape == y.shape and torch.equal(x.view(torch.uint8), y.view(torch.uint8))
        padded = a.to_padded_tensor(0)
        for b, p in enumerate(parts):
            assert torch.equal(padded[b][tuple(slice(0, s) for s in p.shape)].cpu(), p)


@pytest.mark.parametrize("seed", [31, 32])
def test_conv1x1_random_images(seed):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for _ in range(20):
        B = rng.randint(1, 6)
        c_in = rng.choice([16, 32, 48, 64, 128])
        c_out = rng.choice([32, 64, 96, 160, 256])
        dtype = rng.choice([torch.float16, torch.bfloat16])
        imgs = [torch.randn(c_in, rng.randint(1, 40), rng.randint(1, 90), generator=g).to(dtype) for _b in range(B)]
        w = (torch.randn(c_out, c_in, 1, 1, generator=g) * 0.1).to(dtype)
        y = torch.nn.functional.conv2d(nt.nested_tensor(imgs, device=DEV, dtype=dtype), w.to(DEV))
        for yi, xi in zip(y.unbind(), imgs):
            exp = torch.nn.functional.conv2d(xi.float()[None], w.float())[0]
            assert yi.shape == exp.shape
            assert (yi.float().cpu() - exp).abs().max().item() <= (3e-2 if dtype == torch.float16 else 1.5e-1)


@pytest.mark.parametrize("seed", [41, 42, 43])
def test_attention_layers_random_batches(seed):
    # fp16 / bf16 within 2e-2 absolute of the oracle's layer in fp32 on the same
    # (rounded) inputs and weights, scaled where the outputs are larger than 1
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for _ in range(12):
        B = rng.randint(1, 12)
        H = rng.choice([2, 4, 8])
        hd = rng.choice([32, 64, 128])
        E = H * hd
        dtype = rng.choice([torch.float16, torch.bfloat16])
        lens = [rng.randint(1, rng.choice([8, 40, 130, 300])) for _b in range(B)]
        xs = [torch.randn(L, E, generator=g).to(dtype) for L in lens]
        W_in = (torch.randn(3 * E, E, generator=g) * E ** -0.5).to(dtype)
        W_out = (torch.randn(E, E, generator=g) * E ** -0.5).to(dtype)
        b_in = (torch.randn(3 * E, generator=g) * 0.1).to(dtype)
        b_out = (torch.randn(E, generator=g) * 0.1).to(dtype)
        a = nt.nested_tensor(xs, device=DEV, dtype=dtype)
        out = torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, a, a, a, W_in.to(DEV), b_in.to(DEV), hd ** -0.5,
                                             W_out.to(DEV), b_out.to(DEV))
        ref = oracle.ref_nested_tensor([x.float() for x in xs], dtype=torch.float32)
        exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in.float(), b_in.float(), hd ** -0.5,
                             W_out.float(), b_out.float())
        for o, e in zip(out.unbind(), exp):
            tol = (2e-2 if dtype == torch.float16 else 1.2e-1) * max(1.0, e.abs().max().item())
            assert (o.float().cpu() - e).abs().max().item() <= tol, (B, H, hd, dtype, tuple(e.shape))
