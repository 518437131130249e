"""The planned attention kernel (persistent workgroups, a sequence's keys streamed
through LDS from a host-made plan; selected with set_attention_kernel("planned"))
against the CPU oracle of min_mha (nestedtensor/csrc/mha.cpp:18-69) and against
the default work-list kernel on the same inputs.  Tolerance as for the other
f16 / bf16 attention tests: 2e-2 absolute against the oracle."""

import pytest
import torch

import nestedtensor_amd as nt
import oracle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)
HALF_ABS = 2e-2


@pytest.fixture
def planned():
    previous = nt.set_attention_kernel("planned")
    yield
    nt.set_attention_kernel(previous)


def weights(E, seed, dtype, w_std, bias_std=0.1):
    g = torch.Generator().manual_seed(seed)
    W_in = (torch.randn(3 * E, E, generator=g) * w_std).to(dtype)
    W_out = (torch.randn(E, E, generator=g) * w_std).to(dtype)
    b_in = (torch.randn(3 * E, generator=g) * bias_std).to(dtype)
    b_out = (torch.randn(E, generator=g) * bias_std).to(dtype)
    return W_in, b_in, W_out, b_out


def both_kernels(H, q, kv, W, dtype):
    """min_mha on the device with the planned kernel and with the work list;
    returns (planned, work list) as host float vectors."""
    hd = 64
    qa = nt.nested_tensor(q, device=DEV, dtype=dtype)
    ka = qa if kv is None else nt.nested_tensor(kv, device=DEV, dtype=dtype)
    args = (H, hd, 0.0, False, qa, ka, ka) + (W[0].to(DEV), W[1].to(DEV), hd ** -0.5, W[2].to(DEV), W[3].to(DEV))
    assert nt.set_attention_kernel("planned") == "planned"     # the fixture selected it
    got = torch.ops.nestedtensor.min_mha(*args)._impl.buffer.float().cpu()
    plan = qa._impl._attn_plan
    assert plan is not None and plan[2].dim() == 1, "the planned kernel did not run"
    nt.set_attention_kernel("work_list")
    try:
        qb = nt.nested_tensor(q, device=DEV, dtype=dtype)
        kb = qb if kv is None else nt.nested_tensor(kv, device=DEV, dtype=dtype)
        base = torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, qb, kb, kb, *args[7:])._impl.buffer.float().cpu()
        assert qb._impl._attn_plan is None
    finally:
        nt.set_attention_kernel("planned")
    return got, base


def expect(H, q, kv, W, dtype):
    rq = oracle.ref_nested_tensor(q, dtype=dtype)
    rk = rq if kv is None else oracle.ref_nested_tensor(kv, dtype=dtype)
    parts = oracle.min_mha(H, 64, 0.0, False, rq, rk, rk, W[0], W[1], 64 ** -0.5, W[2], W[3])
    return torch.cat([p.reshape(-1) for p in parts]).float()


def compare(got, base, exp):
    assert got.shape == exp.shape and torch.isfinite(got).all()
    assert (got - exp).abs().max().item() <= HALF_ABS
    # the two kernels do the same arithmetic per 64-key tile; they differ in when the
    # reference maximum moves, which is worth a few units of output rounding at most
    assert (got - base).abs().max().item() <= HALF_ABS / 4


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_boundary_lengths_self_and_cross(planned, dtype):
    """Every length around the 32-row query blocks, the 64-key tiles, the 256-key
    steps and the twelve-block chunks, as queries and (rotated) as keys."""
    H, E = 2, 128
    lens = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 383, 384, 385, 511, 512, 513, 769, 1025]
    g = torch.Generator().manual_seed(31)
    amp = 0.5 if dtype == torch.bfloat16 else 1.0
    q = [(torch.randn(L, E, generator=g) * amp).to(dtype) for L in lens]
    W = weights(E, 32, dtype, E ** -0.5)
    compare(*both_kernels(H, q, None, W, dtype), expect(H, q, None, W, dtype))
    kv_lens = lens[9:] + lens[:9]
    kv = [(torch.randn(L, E, generator=g) * amp).to(dtype) for L in kv_lens]
    compare(*both_kernels(H, q, kv, W, dtype), expect(H, q, kv, W, dtype))


def test_config_c3_bert_base_fp16(planned):
    g = torch.Generator().manual_seed(1010 + 2)
    lens = [int(v) for v in torch.randint(32, 513, (32,), generator=g)]
    E = 768
    q = [torch.randn(L, E, generator=g).half() for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * 0.02).half()
    W_out = (torch.randn(E, E, generator=g) * 0.02).half()
    W = (W_in, torch.zeros(3 * E).half(), W_out, torch.zeros(E).half())
    compare(*both_kernels(12, q, None, W, torch.float16), expect(12, q, None, W, torch.float16))


def test_config_c4_bf16_high_raggedness(planned):
    g = torch.Generator().manual_seed(1010 + 3)
    raw = torch.empty(128).exponential_(1.0 / 96.0, generator=g)
    lens = [int(v) for v in raw.round().clamp(8, 512)]
    E, H = 1024, 16
    q = [torch.randn(L, E, generator=g).bfloat16() for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * 0.02).bfloat16()
    W_out = (torch.randn(E, E, generator=g) * 0.02).bfloat16()
    W = (W_in, torch.zeros(3 * E).bfloat16(), W_out, torch.zeros(E).bfloat16())
    compare(*both_kernels(H, q, None, W, torch.bfloat16), expect(H, q, None, W, torch.bfloat16))


@pytest.mark.parametrize("order", ["rising", "falling", "spike"])
def test_reference_maximum_moves_across_steps(planned, order):
    """Scores that grow along 700 keys (three steps of a chain) by far more than
    the slack the kernel allows its reference maximum: the softmax state carried
    from step to step is rescaled on every tile, never, or once in the middle."""
    H, E, L = 2, 128, 700
    dtype = torch.float16
    g = torch.Generator().manual_seed(5)
    u = torch.randn(E, generator=g)
    u = u / u.norm() * 8.0
    amp = torch.linspace(0.2, 3.0, L)
    if order == "falling":
        amp = amp.flip(0)
    elif order == "spike":
        amp = torch.full((L,), 0.3)
        amp[430] = 3.0
    x = (amp[:, None] * u[None, :] + 0.05 * torch.randn(L, E, generator=g)).to(dtype)
    short = (0.5 * torch.randn(40, E, generator=g)).to(dtype)
    W = (torch.cat([torch.eye(E)] * 3).to(dtype), torch.zeros(3 * E, dtype=dtype), torch.eye(E).to(dtype),
         torch.zeros(E, dtype=dtype))
    q = [x, short]
    got, base = both_kernels(H, q, None, W, dtype)
    # at scores of this size the reference's own rounding of q * scaling and of the
    # scores moves its result: judge both against the float64 answer
    r64 = oracle.ref_nested_tensor([p.double() for p in q], dtype=torch.float64)
    e64 = torch.cat([p.reshape(-1) for p in oracle.min_mha(H, 64, 0.0, False, r64, r64, r64, W[0].double(),
                                                           W[1].double(), 64 ** -0.5, W[2].double(),
                                                           W[3].double())]).float()
    ref_err = (expect(H, q, None, W, dtype) - e64).abs().max().item()
    assert torch.isfinite(got).all()
    assert (got - e64).abs().max().item() <= max(HALF_ABS, ref_err + HALF_ABS / 4)
    assert (got - base).abs().max().item() <= HALF_ABS / 2


def test_other_head_dims_keep_the_work_list(planned):
    H, hd = 2, 32
    E = H * hd
    g = torch.Generator().manual_seed(9)
    q = [torch.randn(L, E, generator=g).half() for L in (70, 3)]
    W = weights(E, 10, torch.float16, E ** -0.5)
    a = nt.nested_tensor(q, device=DEV, dtype=torch.float16)
    got = torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, a, a, a, W[0].to(DEV), W[1].to(DEV), hd ** -0.5,
                                         W[2].to(DEV), W[3].to(DEV))._impl.buffer.float().cpu()
    assert a._impl._attn_plan is None and a._impl._attn_schedule is not None
    r = oracle.ref_nested_tensor(q, dtype=torch.float16)
    exp = torch.cat([p.reshape(-1) for p in oracle.min_mha(H, hd, 0.0, False, r, r, r, W[0], W[1], hd ** -0.5,
                                                           W[2], W[3])]).float()
    assert (got - exp).abs().max().item() <= HALF_ABS


def test_selector_refuses_unknown_names():
    with pytest.raises(ValueError):
        nt.set_attention_kernel("fastest")
