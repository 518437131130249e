"""Parity of the HIP pack / pad / un-pad / mask path with the CPU oracle
(bit-exact), through the product's Python surface down to the C ABI.  The cases
mirror the reference's GPU-vs-CPU tests (test/test_nested_tensor_class.py:754-817)
and replay its literal masking cases (tests/golden/masking_cases.py) on the device."""

import random

import pytest
import torch

import nestedtensor_amd as nt
import oracle
from nestedtensor_amd import _C
from nestedtensor_amd.impl import device_offsets
from masking_cases import (TO_TENSOR_MASK, FROM_TENSOR_MASK, ROUND_TRIP_DATA, ROUND_TRIP_MASK)

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)

_INT_VIEW = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def bits_equal(a, b):
    """Same shape, dtype and bit pattern (NaN payloads and -0.0 included)."""
    a, b = a.cpu().contiguous(), b.cpu().contiguous()
    assert a.shape == b.shape, (a.shape, b.shape)
    assert a.dtype == b.dtype, (a.dtype, b.dtype)
    if a.numel() == 0:
        return
    if a.dtype == torch.bool:
        assert torch.equal(a, b)
        return
    v = _INT_VIEW[a.element_size()]
    assert torch.equal(a.view(v), b.view(v))


def rand_parts(g, B, dims, lo, hi, dtype):
    parts = []
    for _ in range(B):
        shape = [int(v) for v in torch.randint(lo, hi + 1, (dims,), generator=g)]
        if dtype.is_floating_point:
            parts.append(torch.randn(*shape, generator=g).to(dtype))
        else:
            parts.append(torch.randint(0, 100, shape, generator=g).to(dtype))
    return parts


# ---- device prefix scan -------------------------------------------------------

@pytest.mark.parametrize("B,D", [(1, 1), (5, 2), (64, 0), (2048, 1), (2049, 3), (5000, 2), (300001, 1)])
def test_offsets_scan(B, D):
    g = torch.Generator().manual_seed(B * 7 + D)
    sizes = torch.randint(0, 50, (B, D), generator=g, dtype=torch.int64)
    got = device_offsets(sizes.to(DEV), B, D)
    exp = torch.cat([torch.zeros(1, dtype=torch.int64), sizes.prod(1).cumsum(0)])
    assert torch.equal(got.cpu(), exp)


def test_offsets_scan_beyond_int32():
    sizes = torch.full((4096, 2), 4096, dtype=torch.int64)      # 6.9e10 elements in total
    got = device_offsets(sizes.to(DEV), 4096, 2)
    exp = torch.arange(4097, dtype=torch.int64) * (4096 * 4096)
    assert torch.equal(got.cpu(), exp)


# ---- to_padded_tensor ---------------------------------------------------------

@pytest.mark.parametrize("dims", [1, 2, 3])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.float64,
                                   torch.int64, torch.uint8])
def test_to_padded_tensor_reference_gpu_cases(dims, dtype):
    # test_nested_tensor_class.py:754-791: 5 tensors, sizes 3..30, padding=1
    random.seed(1010)
    parts = [torch.randn(*[random.randint(3, 30) for _ in range(dims)]) for _ in range(5)]
    if not dtype.is_floating_point:
        parts = [(p * 10).to(dtype) for p in parts]
    a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
    got = a.to_padded_tensor(padding=1)
    ref = oracle.ref_nested_tensor(parts, dtype=dtype)
    exp = oracle.to_padded_tensor(ref, 1)
    bits_equal(got, exp)
    # and the reference's own formulation of the expected value
    d1, m1 = oracle.to_tensor_mask(ref)
    m1 = m1.to(torch.bool)
    while m1.dim() < d1.dim():
        m1 = m1.unsqueeze(-1)
    bits_equal(got, d1.masked_fill(m1.logical_not().expand_as(d1), 1))


@pytest.mark.parametrize("inner", [1, 3, 8, 33, 256])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_to_padded_tensor_regular_last_dim_alignments(inner, dtype):
    # dim-3 nested tensor with regular last dim: the collapsed fast shape
    # (masking.cpp:566-568); odd inner sizes exercise unaligned rows
    g = torch.Generator().manual_seed(inner)
    parts = [torch.randn(int(l), inner, generator=g).to(dtype)
             for l in torch.randint(1, 40, (17,), generator=g)]
    a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
    for pad in (0.0, -1.0, 0.1):
        bits_equal(a.to_padded_tensor(pad), oracle.to_padded_tensor(oracle.ref_nested_tensor(parts, dtype=dtype), pad))


def test_to_padded_tensor_mixed_regular_dims():
    g = torch.Generator().manual_seed(2)
    # [3, H_i, W_i]: regular first dim, ragged trailing dims (the image shape class)
    parts = [torch.rand(3, int(h), int(w), generator=g) for h, w in torch.randint(5, 40, (6, 2), generator=g)]
    a = nt.nested_tensor(parts, device=DEV)
    bits_equal(a.to_padded_tensor(0.5), oracle.to_padded_tensor(oracle.ref_nested_tensor(parts), 0.5))
    # [L_i, 4, 8]: two trailing regular dims
    parts = [torch.rand(int(l), 4, 8, generator=g) for l in torch.randint(1, 9, (6,), generator=g)]
    a = nt.nested_tensor(parts, device=DEV)
    bits_equal(a.to_padded_tensor(-2), oracle.to_padded_tensor(oracle.ref_nested_tensor(parts), -2))
    # all regular
    parts = [torch.rand(4, 5, generator=g) for _ in range(3)]
    a = nt.nested_tensor(parts, device=DEV)
    bits_equal(a.to_padded_tensor(-2), oracle.to_padded_tensor(oracle.ref_nested_tensor(parts), -2))


def test_nan_payload_and_negative_zero_survive():
    bits = torch.tensor([0x7fc00001, 0x7f800001, 0x80000000, 0xffc12345 - (1 << 32), 0x00000001],
                        dtype=torch.int64).to(torch.int32)
    x = bits.view(torch.float32)
    parts = [x[:2].clone(), x.clone(), x[1:4].clone()]
    a = nt.nested_tensor(parts, device=DEV)
    got = a.to_padded_tensor(0.0)
    exp = oracle.to_padded_tensor(oracle.ref_nested_tensor(parts), 0.0)
    bits_equal(got, exp)
    back = nt.from_padded_tensor(got, a)
    bits_equal(back._impl.buffer, oracle.ref_nested_tensor(parts).buffer)


def test_special_shapes():
    with pytest.raises(RuntimeError, match="Empty tensors are not yet supported."):
        nt.nested_tensor([torch.randn(0, 3), torch.randn(2, 3)], device=DEV).to_padded_tensor(0)
    s = nt.nested_tensor([torch.tensor(3.0)], device=DEV)
    assert s.to_padded_tensor(0).data_ptr() == s._impl.buffer.data_ptr()   # alias, masking.cpp:628-631
    one = nt.nested_tensor([torch.randn(7, 5)], device=DEV)
    bits_equal(one.to_padded_tensor(0), one.unbind()[0].unsqueeze(0))


# ---- nested_tensor from device tensors (pack kernel) ----------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.uint8])
def test_pack_device_constituents(dtype):
    g = torch.Generator().manual_seed(9)
    parts = rand_parts(g, 23, 2, 1, 37, dtype)
    dev_parts = [p.to(DEV) for p in parts]
    dev_parts[3] = dev_parts[3].t().contiguous().t()       # non-contiguous constituent
    a = nt.nested_tensor(dev_parts, dtype=dtype, device=DEV)
    ref = oracle.ref_nested_tensor(parts, dtype=dtype)
    bits_equal(a._impl.buffer, ref.buffer)
    assert a.nested_size().unbind() == ref.nested_size()
    for u, p in zip(a.unbind(), parts):
        bits_equal(u, p)
    # copies, not views
    assert a._impl.buffer.data_ptr() != dev_parts[0].data_ptr()


# ---- to_tensor_mask / to_mask ---------------------------------------------------

@pytest.mark.parametrize("name,parts,dtype,checks", TO_TENSOR_MASK, ids=[c[0] for c in TO_TENSOR_MASK])
def test_to_tensor_mask_literals_on_device(name, parts, dtype, checks):
    a = nt.nested_tensor(parts, dtype=dtype, device=DEV)
    for mask_dim, exp_t, exp_m in checks:
        t, m = a.to_tensor_mask(mask_dim=mask_dim)
        assert t.shape == exp_t.shape and m.shape == exp_m.shape
        assert torch.equal(t.cpu().to(exp_t.dtype), exp_t)
        assert torch.equal(m.cpu().to(torch.bool), exp_m)


def test_mask_dim_too_small_on_device():
    a = nt.nested_tensor([torch.tensor([1, 2]), torch.tensor([3, 4, 5, 6])], device=DEV)
    with pytest.raises(RuntimeError, match="Mask dimension is too small to represent data tensor."):
        a.to_tensor_mask(mask_dim=1)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_to_tensor_mask_cuda_reference_case(dtype):
    # test_nested_tensor_class.py:793-807
    random.seed(110)
    lens = [random.randint(2, 4) for _ in range(3)]
    parts = [torch.arange(t * 3).reshape(t, 3).float() for t in lens]
    a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
    data, mask = a.to_tensor_mask(mask_dim=2)
    d1, m1 = oracle.to_tensor_mask(oracle.ref_nested_tensor(parts, dtype=dtype), 2)
    bits_equal(data, d1)
    assert mask.dtype == torch.bool and torch.equal(mask.cpu(), m1.to(torch.bool))
    # to_mask == to_tensor_mask()[1] (test_nested_tensor_class.py:809-817)
    assert torch.equal(torch.ops.nestedtensor.to_mask(a, 2), mask)


@pytest.mark.parametrize("dims", [1, 2, 3])
def test_to_tensor_mask_every_mask_dim(dims):
    g = torch.Generator().manual_seed(40 + dims)
    for trial in range(6):
        regular = [bool(torch.randint(0, 2, (1,), generator=g)) for _ in range(dims)]
        base = [int(torch.randint(1, 7, (1,), generator=g)) for _ in range(dims)]
        parts = [torch.randn(*[base[k] if regular[k] else int(torch.randint(1, 7, (1,), generator=g))
                               for k in range(dims)], generator=g) for _ in range(4)]
        a = nt.nested_tensor(parts, device=DEV)
        ref = oracle.ref_nested_tensor(parts)
        for md in [None] + list(range(0, dims + 2)):
            try:
                exp_t, exp_m = oracle.to_tensor_mask(ref, md)
            except RuntimeError as e:
                with pytest.raises(RuntimeError, match=str(e)[:30]):
                    a.to_tensor_mask(mask_dim=md)
                continue
            t, m = a.to_tensor_mask(mask_dim=md)
            bits_equal(t, exp_t)
            assert m.shape == exp_m.shape and torch.equal(m.cpu(), exp_m.to(torch.bool))
            try:
                exp_tm = oracle.to_mask(ref, md)
            except RuntimeError:
                continue
            got_tm = torch.ops.nestedtensor.to_mask(a, md)
            assert got_tm.shape == exp_tm.shape and torch.equal(got_tm.cpu(), exp_tm.to(torch.bool))


# ---- nested_tensor_from_tensor_mask / from_padded ---------------------------------

def nt_matches(res, parts, dtype):
    assert res.dtype == dtype, (res.dtype, dtype)
    assert len(res) == len(parts)
    assert res.nested_size().unbind() == [torch.Size(p.shape) for p in parts]
    for r, p in zip(res.unbind(), parts):
        bits_equal(r, p.to(dtype))


@pytest.mark.parametrize("name,tensor,mask,parts,dtype", FROM_TENSOR_MASK,
                         ids=[c[0] for c in FROM_TENSOR_MASK])
def test_from_tensor_mask_literals_on_device(name, tensor, mask, parts, dtype):
    res = nt.nested_tensor_from_tensor_mask(tensor.to(DEV), mask.to(DEV))
    nt_matches(res, parts, dtype)
    assert res.nested_dim() == 1


def test_reference_round_trip_literal_on_device():
    # test_nested_tensor_masking.py:454-477
    data1, mask1 = ROUND_TRIP_DATA.to(DEV), ROUND_TRIP_MASK.to(DEV)
    nt2 = nt.nested_tensor_from_tensor_mask(data1, mask1)
    data2, mask2 = nt2.to_tensor_mask()
    bits_equal(data2, ROUND_TRIP_DATA)
    assert torch.equal(mask2.cpu(), ROUND_TRIP_MASK)
    data3 = nt2.to_padded_tensor(padding=-10)
    exp = oracle.to_padded_tensor(
        oracle.ref_nested_tensor(oracle.nt_from_tensor_mask(ROUND_TRIP_DATA, ROUND_TRIP_MASK, 1)), -10)
    bits_equal(data3, exp)


@pytest.mark.parametrize("mask_dims", [2, 3, 4])
def test_from_tensor_mask_random_boxes_vs_literal_walk(mask_dims):
    g = torch.Generator().manual_seed(100 + mask_dims)
    for trial in range(8):
        B = 4
        dims = [int(v) for v in torch.randint(1, 7, (3,), generator=g)]
        t = torch.randn(B, *dims, generator=g)
        mask = torch.zeros([B] + dims[: mask_dims - 1], dtype=torch.bool)
        for b in range(B):
            ext = [int(torch.randint(0, d + 1, (1,), generator=g)) for d in dims[: mask_dims - 1]]
            if b == 0:
                ext = [max(e, 1) for e in ext]
            mask[b][tuple(slice(0, e) for e in ext)] = True
        exp = oracle.nt_from_tensor_mask(t, mask, 1)
        shapes = {p.dim() for p in exp}
        if len(shapes) != 1:
            with pytest.raises(RuntimeError):
                nt.nested_tensor_from_tensor_mask(t.to(DEV), mask.to(DEV))
            continue
        res = nt.nested_tensor_from_tensor_mask(t.to(DEV), mask.to(DEV))
        nt_matches(res, exp, torch.float32)


def test_from_tensor_mask_literals_and_subset_selections():
    for name, tensor, mask, parts, dtype in FROM_TENSOR_MASK:
        res = nt.nested_tensor_from_tensor_mask(tensor.to(DEV), mask.to(DEV))
        nt_matches(res, parts, dtype)
    # a subset selection that is not a prefix, and a ragged one
    t = torch.arange(24.).reshape(2, 3, 4)
    m = torch.tensor([[[0, 1, 1, 0], [0, 1, 1, 0], [0, 0, 0, 0]], [[1, 1, 0, 0], [0, 0, 0, 0], [1, 1, 0, 0]]]).bool()
    exp = oracle.nt_from_tensor_mask(t, m, 1)
    nt_matches(nt.nested_tensor_from_tensor_mask(t.to(DEV), m.to(DEV)), exp, torch.float32)
    bad = torch.tensor([[[1, 1, 1, 0], [1, 0, 0, 0], [0, 0, 0, 0]], [[1, 1, 0, 0], [0, 0, 0, 0], [0, 0, 0, 0]]]).bool()
    with pytest.raises(RuntimeError):
        nt.nested_tensor_from_tensor_mask(t.to(DEV), bad.to(DEV))


def test_from_tensor_mask_subset_selection_and_ragged_error():
    t = torch.arange(24.0).reshape(2, 3, 4)
    mask = torch.tensor([[[1, 0, 1, 0], [0, 0, 0, 0], [0, 1, 1, 0]],
                         [[1, 1, 1, 1], [1, 1, 1, 1], [1, 1, 1, 1]]], dtype=torch.bool)
    exp = oracle.nt_from_tensor_mask(t, mask, 1)
    nt_matches(nt.nested_tensor_from_tensor_mask(t.to(DEV), mask.to(DEV)), exp, torch.float32)
    bad = mask.clone()
    bad[0, 2, 0] = True          # rows keep 2 and 3 elements: at::stack would throw
    with pytest.raises(RuntimeError):
        oracle.nt_from_tensor_mask(t, bad, 1)
    with pytest.raises(RuntimeError):
        nt.nested_tensor_from_tensor_mask(t.to(DEV), bad.to(DEV))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_nested_tensor_from_padded_tensor_value_based(dtype):
    g = torch.Generator().manual_seed(77)
    parts = [torch.rand(int(l), 6, generator=g).to(dtype) + 1 for l in torch.randint(1, 9, (5,), generator=g)]
    padded = oracle.to_padded_tensor(oracle.ref_nested_tensor(parts, dtype=dtype), -1)
    res = nt.nested_tensor_from_padded_tensor(padded.to(DEV))          # padding=-1 default
    exp = oracle.nested_tensor_from_padded_tensor(padded)
    nt_matches(res, exp.unbind(), dtype)
    nt_matches(res, parts, dtype)


@pytest.mark.parametrize("dims", [1, 2, 3])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.int64])
def test_from_padded_tensor_length_based(dims, dtype):
    g = torch.Generator().manual_seed(dims)
    parts = rand_parts(g, 7, dims, 1, 21, dtype)
    a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
    ref = oracle.ref_nested_tensor(parts, dtype=dtype)
    padded = a.to_padded_tensor(5)
    back = nt.from_padded_tensor(padded, a)
    exp = oracle.from_padded_tensor(oracle.to_padded_tensor(ref, 5), ref)
    bits_equal(back._impl.buffer, exp.buffer)
    bits_equal(back._impl.buffer, ref.buffer)
    assert back.nested_size() == a.nested_size()
    # target given as a nested size, padded larger than the batch maximum
    bigger = torch.nn.functional.pad(padded, [0, 3] * dims, value=9)
    back2 = nt.from_padded_tensor(bigger, a.nested_size())
    bits_equal(back2._impl.buffer, ref.buffer)


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_sweep_against_oracle(seed):
    """Many small random nested tensors (1 to 3 constituent dims, extents 1..37 so
    that every alignment of rows and of the valid / pad boundary turns up, some
    dims regular at random, five element sizes): pad, mask and both inverses
    against the oracle, bit for bit."""
    g = torch.Generator().manual_seed(9000 + seed)
    dtypes = [torch.float32, torch.float16, torch.uint8, torch.int64, torch.bfloat16, torch.float64]
    for case in range(40):
        D = int(torch.randint(1, 4, (1,), generator=g))
        B = int(torch.randint(1, 9, (1,), generator=g))
        dtype = dtypes[int(torch.randint(0, len(dtypes), (1,), generator=g))]
        regular = [bool(torch.randint(0, 3, (1,), generator=g) == 0) for _ in range(D)]
        fixed = [int(torch.randint(1, 38, (1,), generator=g)) for _ in range(D)]
        parts = []
        for _ in range(B):
            shape = [fixed[k] if regular[k] else int(torch.randint(1, 38, (1,), generator=g)) for k in range(D)]
            parts.append((torch.randn(*shape, generator=g) * 50).to(dtype))
        a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
        ref = oracle.ref_nested_tensor(parts, dtype=dtype)
        pad_value = 3 if dtype in (torch.uint8, torch.int64) else -1.5
        padded = a.to_padded_tensor(pad_value)
        bits_equal(padded, oracle.to_padded_tensor(ref, pad_value))
        data, mask = a.to_tensor_mask()
        exp_d, exp_m = oracle.to_tensor_mask(ref)
        bits_equal(data, exp_d)
        assert mask.shape == exp_m.shape and torch.equal(mask.cpu(), exp_m.to(torch.bool)), (case, parts[0].shape)
        back = nt.from_padded_tensor(padded, a)
        bits_equal(back._impl.buffer, ref.buffer)
        full_mask = torch.ops.nestedtensor.to_mask(a, a.dim())
        again = nt.nested_tensor_from_tensor_mask(data, full_mask)
        nt_matches(again, parts, dtype)


def test_constructor_direct_copy_of_large_host_constituents():
    # constituents of 256 KiB or more go to the device one by one (no host packing); with a dtype
    # change and a non-contiguous constituent
    g = torch.Generator().manual_seed(55)
    parts = [torch.randn(300, 300, generator=g, dtype=torch.float64), torch.randn(700, 300, generator=g,
                                                                                  dtype=torch.float64).t()]
    parts[1] = parts[1].t()[:, :300].t()       # a strided view, shape [300, 700]
    for dtype in (torch.float64, torch.float16):
        a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
        ref = oracle.ref_nested_tensor(parts, dtype=dtype)
        bits_equal(a._impl.buffer, ref.buffer)
        assert a.nested_size().unbind() == [torch.Size(p.shape) for p in parts]


def test_pad_nt_to_a_given_shape():
    # pad_nt (masking.cpp:138-179): a caller-given goal shape, data padded with 0, full-shape mask
    parts = [torch.randn(3, 5), torch.randn(1, 5), torch.randn(4, 2)]
    a = nt.nested_tensor(parts, device=DEV)
    ref = oracle.ref_nested_tensor(parts)
    for shape in ([4, 5], [6, 9]):
        data, mask = torch.ops.nestedtensor.pad_nt(a, shape)
        exp_d, exp_m = oracle.pad_nt(ref, shape)
        bits_equal(data, exp_d)
        assert mask.dtype == torch.bool and torch.equal(mask.cpu(), exp_m.to(torch.bool))
    # a regular dim shorter than the goal shape
    reg = [torch.randn(2, 3), torch.randn(2, 3)]
    data, mask = torch.ops.nestedtensor.pad_nt(nt.nested_tensor(reg, device=DEV), [2, 8])
    exp_d, exp_m = oracle.pad_nt(oracle.ref_nested_tensor(reg), [2, 8])
    bits_equal(data, exp_d)
    assert torch.equal(mask.cpu(), exp_m.to(torch.bool))
    with pytest.raises(RuntimeError, match="does not hold"):
        torch.ops.nestedtensor.pad_nt(a, [3, 5])


# ---- benchmark configurations -----------------------------------------------------

def test_config_c1_round_trip_bit_exact():
    g = torch.Generator().manual_seed(1010 + 0)
    lengths = torch.randint(1, 129, (64,), generator=g)
    lengths[0] = 128
    parts = [torch.randn(int(l), 256, generator=g) for l in lengths]
    a = nt.nested_tensor(parts, device=DEV)
    padded = a.to_padded_tensor(0)
    assert tuple(padded.shape) == (64, 128, 256)
    ref = oracle.ref_nested_tensor(parts)
    bits_equal(padded, oracle.to_padded_tensor(ref, 0))
    # value-based inverse, as configs[0] names it; a padding value that no
    # N(0,1) sample equals
    padded_m = a.to_padded_tensor(-1e30)
    back = nt.nested_tensor_from_padded_tensor(padded_m, padding=-1e30)
    bits_equal(back._impl.buffer, ref.buffer)
    assert back.nested_size().unbind() == ref.nested_size()
    back2 = nt.from_padded_tensor(padded, a)
    bits_equal(back2._impl.buffer, ref.buffer)


def test_config_c2_images_tensor_mask_round_trip():
    g = torch.Generator().manual_seed(1010 + 1)
    hw = torch.randint(480, 1025, (16, 2), generator=g)
    parts = [torch.rand(3, int(h), int(w), generator=g) for h, w in hw]
    a = nt.nested_tensor(parts, device=DEV)
    ref = oracle.ref_nested_tensor(parts)
    data, mask = a.to_tensor_mask()
    exp_d, exp_m = oracle.to_tensor_mask(ref)
    bits_equal(data, exp_d)
    assert mask.dtype == torch.bool and mask.shape == exp_m.shape == data.shape
    assert torch.equal(mask.cpu(), exp_m.to(torch.bool))
    back = nt.nested_tensor_from_tensor_mask(data, mask)
    exp_parts = oracle.nt_from_tensor_mask_vectorised(exp_d, exp_m.to(torch.bool))
    nt_matches(back, exp_parts, torch.float32)
    nt_matches(back, parts, torch.float32)


def test_config_c5_chunk_full_size_properties():
    """One chunk of the largest configuration at its real shape: 512 fp16
    constituents [L_i, 4096], L_i ~ U[1, 2048], generated on the device (more
    than 2^31 packed elements, so every index is exercised as int64).  Checked
    through properties that do not need the oracle at this size: the round trip
    is bit-exact, every constituent's bits sum to the same value before and after
    padding, the padding holds the pad value and nothing else, and three
    constituents (first, longest, last) are compared element by element."""
    from nestedtensor_amd.impl import NestedTensorImpl
    from nestedtensor_amd.nested.nested import NestedTensor
    g = torch.Generator().manual_seed(1010 + 4)
    E = 4096
    lens = torch.randint(1, 2049, (512,), generator=g)
    sizes = torch.stack([lens, torch.full_like(lens, E)], 1).contiguous()
    total = int(lens.sum()) * E
    assert total > 2 ** 31
    bits = torch.randint(-32768, 32767, (total,), device=DEV, dtype=torch.int16)     # any bit pattern
    a = NestedTensor(NestedTensorImpl(bits.view(torch.float16), sizes))
    Lmax = int(lens.max())
    padded = torch.ops.nestedtensor.to_padded_tensor(a, float("nan"))
    assert tuple(padded.shape) == (512, Lmax, E)
    pview = padded.view(torch.int16)
    # the canonical fp16 NaN the pad value converts to
    nan_bits = int(torch.tensor(float("nan"), dtype=torch.float16).view(torch.int16))
    # round trip
    back = nt.from_padded_tensor(padded, a)
    assert torch.equal(back._impl.buffer.view(torch.int16), bits)
    # per-constituent checksums and pad region
    starts = (torch.cumsum(lens, 0) - lens) * E
    row_valid = torch.arange(Lmax, device=DEV).unsqueeze(0) < lens.to(DEV).unsqueeze(1)      # [512, Lmax]
    row_sums = pview.sum(2, dtype=torch.int64)                                            # [512, Lmax]
    got_valid = (row_sums * row_valid).sum(1)
    cs = torch.zeros(total // E + 1, dtype=torch.int64, device=DEV)
    cs[1:] = torch.cumsum(bits.view(-1, E).sum(1, dtype=torch.int64), 0)
    tok = torch.cumsum(lens, 0).to(DEV)
    exp_valid = cs[tok] - cs[tok - lens.to(DEV)]
    assert torch.equal(got_valid, exp_valid)
    pad_rows = ~row_valid
    assert bool((pview[pad_rows] == nan_bits).all())
    for b in (0, int(lens.argmax()), 511):
        L, s0 = int(lens[b]), int(starts[b])
        assert torch.equal(pview[b, :L].reshape(-1), bits[s0:s0 + L * E])
    del padded, pview, back, row_sums


# ---- row statistics kernels (C ABI level) -------------------------------------------

def _cpu_counts_prefix(keep):
    counts = keep.sum(1).to(torch.int32)
    M = keep.size(1)
    idx = torch.arange(M).unsqueeze(0)
    prefix = (keep == (idx < counts.unsqueeze(1))).all(1).to(torch.uint8)
    return counts, prefix


@pytest.mark.parametrize("M", [1, 7, 16, 33, 64, 100, 1024, 1029, 4096])
def test_mask_row_counts_and_prefix_flags(M):
    g = torch.Generator().manual_seed(M)
    R = 37
    keep = torch.zeros(R, M, dtype=torch.bool)
    for r in range(R):
        kind = r % 4
        n = int(torch.randint(0, M + 1, (1,), generator=g))
        if kind == 0:
            keep[r, :n] = True                                   # prefix
        elif kind == 1:
            keep[r] = torch.rand(M, generator=g) < 0.5           # random subset
        elif kind == 2:
            keep[r, :n] = True
            if M > 1:
                keep[r, int(torch.randint(0, M, (1,), generator=g))] ^= True   # prefix with one flip
        else:
            keep[r, M - n:] = True                               # suffix
    exp_c, exp_p = _cpu_counts_prefix(keep)
    mask = keep.to(DEV).view(torch.uint8)
    counts = torch.empty(R, dtype=torch.int32, device=DEV)
    prefix = torch.empty(R, dtype=torch.uint8, device=DEV)
    _C.check(_C.lib.nt_mask_row_counts(_C.ptr(mask), R, M, _C.ptr(counts), _C.ptr(prefix), _C.current_stream(DEV)))
    assert torch.equal(counts.cpu(), exp_c)
    assert torch.equal(prefix.cpu(), exp_p)
    # value mode on the same pattern: kept = 1.5, dropped = padding (-1)
    for dtype in (torch.float16, torch.float32, torch.bfloat16, torch.int64, torch.float64):
        data = torch.where(keep, torch.tensor(3, dtype=dtype), torch.tensor(-1, dtype=dtype)).to(DEV)
        _C.check(_C.lib.nt_value_row_counts(_C.ptr(data), _C.ELEM_TYPE[dtype], -1.0, R, M, _C.ptr(counts),
                                            _C.ptr(prefix), _C.current_stream(DEV)))
        assert torch.equal(counts.cpu(), exp_c), dtype
        assert torch.equal(prefix.cpu(), exp_p), dtype


@pytest.mark.parametrize("M", [16, 333, 1015, 4096])
def test_mask_row_counts_take_any_nonzero_byte_as_true(M):
    # a uint8 mask is true wherever it is non-zero (nested/masking.py:18-50 hands the
    # mask to the kernels as it is): 0x80, 0x7f, 0x01 and 0xff bytes in every position
    # of a lane's sixteen
    g = torch.Generator().manual_seed(100 + M)
    R = 64
    values = torch.tensor([0, 0, 1, 2, 0x7f, 0x80, 0x81, 0xff], dtype=torch.uint8)
    mask = values[torch.randint(0, values.numel(), (R, M), generator=g)]
    for r in range(0, R, 4):                     # every fourth row: a prefix of odd bytes
        n = int(torch.randint(0, M + 1, (1,), generator=g))
        mask[r] = 0
        mask[r, :n] = values[2 + torch.randint(0, 6, (n,), generator=g)]
    exp_c, exp_p = _cpu_counts_prefix(mask != 0)
    counts = torch.empty(R, dtype=torch.int32, device=DEV)
    prefix = torch.empty(R, dtype=torch.uint8, device=DEV)
    dmask = mask.to(DEV)
    _C.check(_C.lib.nt_mask_row_counts(_C.ptr(dmask), R, M, _C.ptr(counts), _C.ptr(prefix), _C.current_stream(DEV)))
    assert torch.equal(counts.cpu(), exp_c)
    assert torch.equal(prefix.cpu(), exp_p)


def _box_by_brute_force(c, pf, dims):
    """(ok, w, extents) of one constituent's row statistics, every candidate box
    tried: the definition nt_leading_boxes implements, not its algorithm."""
    c = c.reshape(dims if dims else [1])
    if not bool((pf == 1).all()):
        return 0, int(c.flatten()[0]), None
    w = int(c.flatten()[0])
    if w == 0:
        return (1 if int(c.abs().sum()) == 0 else 0), 0, [0] * len(dims)
    import itertools
    for ext in itertools.product(*[range(1, d + 1) for d in dims]):
        box = torch.zeros_like(c)
        box[tuple(slice(0, e) for e in ext)] = w
        if torch.equal(box, c):
            return 1, w, list(ext)
    return 0, w, None


@pytest.mark.parametrize("dims", [[], [5], [3, 4], [2, 3, 4], [300], [2, 260]])
def test_leading_boxes_against_every_candidate_box(dims):
    g = torch.Generator().manual_seed(len(dims) * 7 + sum(dims))
    rows_per = 1
    for d in dims:
        rows_per *= d
    cases = []
    for trial in range(24):
        w = int(torch.randint(1, 9, (1,), generator=g))
        ext = [int(torch.randint(1, d + 1, (1,), generator=g)) for d in dims]
        c = torch.zeros(dims if dims else [1], dtype=torch.int32)
        c[tuple(slice(0, e) for e in ext)] = w
        pf = torch.ones(rows_per, dtype=torch.uint8)
        kind = trial % 6
        if kind == 1:
            c.zero_()                                              # an empty constituent
        elif kind == 2 and rows_per > 1:
            flat = c.flatten()
            r = int(torch.randint(1, rows_per, (1,), generator=g))
            flat[r] = w if int(flat[r]) == 0 else 0                # one row flipped
            c = flat.reshape(c.shape)
        elif kind == 3 and rows_per > 1:
            flat = c.flatten()
            flat[int(torch.randint(0, rows_per, (1,), generator=g))] += 1      # one row of another width
            c = flat.reshape(c.shape)
        elif kind == 4:
            pf[int(torch.randint(0, rows_per, (1,), generator=g))] = 0        # a row that keeps no prefix
        elif kind == 5 and dims:
            c = c.flip(0)                                          # the box at the far end of the first dim
        cases.append((c.flatten(), pf))
    B = len(cases)
    counts = torch.cat([c for c, _ in cases]).to(DEV)
    prefix = torch.cat([p for _, p in cases]).to(DEV)
    K = int(_C.lib.nt_leading_boxes_max_dims())
    boxes = torch.full((B, K + 2), -7, dtype=torch.int32, device=DEV)
    # the completion word lives in pinned host memory; the arrival counter on the device
    done = torch.zeros(4, dtype=torch.int32).pin_memory()
    arrivals = torch.zeros(1, dtype=torch.int32, device=DEV)
    for value in (41, 42):                    # twice: the counter must be back at zero
        boxes.fill_(-7)
        _C.check(_C.lib.nt_leading_boxes(_C.ptr(counts), _C.ptr(prefix), B, rows_per, _C.i64_array(dims or [1]),
                                         len(dims), _C.ptr(boxes), _C.ptr(done), value, _C.ptr(arrivals),
                                         _C.current_stream(DEV)))
        torch.cuda.synchronize()
        assert int(done[0]) == value and int(arrivals.cpu()[0]) == 0
    got = boxes.cpu()
    # without an arrival counter: a completion word per constituent, same lines
    words = torch.zeros(B, dtype=torch.int32).pin_memory()
    boxes.fill_(-7)
    _C.check(_C.lib.nt_leading_boxes(_C.ptr(counts), _C.ptr(prefix), B, rows_per, _C.i64_array(dims or [1]),
                                     len(dims), _C.ptr(boxes), _C.ptr(words), 43, None, _C.current_stream(DEV)))
    torch.cuda.synchronize()
    assert bool((words == 43).all()) and torch.equal(boxes.cpu(), got)
    # stamped lines: every entry {value, stamp} in one 8-byte word, nothing else to wait for
    lines = torch.zeros(B, K + 2, dtype=torch.int64).pin_memory()
    _C.check(_C.lib.nt_leading_boxes_stamped(_C.ptr(counts), _C.ptr(prefix), B, rows_per, _C.i64_array(dims or [1]),
                                             len(dims), _C.ptr(lines), 44, _C.current_stream(DEV)))
    torch.cuda.synchronize()
    assert bool(((lines >> 32) == 44).all())
    assert torch.equal((lines & 0xffffffff).to(torch.int32), got)
    n_ok = 0
    for b, (c, pf) in enumerate(cases):
        ok, w, ext = _box_by_brute_force(c, pf, dims)
        assert int(got[b, 0]) == ok, (b, c, pf)
        if ok:
            n_ok += 1
            assert int(got[b, 1]) == w
            if w:
                assert [int(v) for v in got[b, 2:2 + len(dims)]] == ext
    assert 0 < n_ok < B or not dims


def test_from_tensor_mask_falls_back_when_one_constituent_is_no_leading_box():
    # two constituents keep a leading box, the third keeps a box that starts at
    # column 1: same result as the reference's walk (masking.cpp:203-222)
    g = torch.Generator().manual_seed(77)
    t = torch.randn(3, 4, 6, generator=g)
    m = torch.zeros(3, 4, 6, dtype=torch.bool)
    m[0, :2, :3] = True
    m[1, :4, :6] = True
    m[2, :3, 1:5] = True
    exp = oracle.nested_tensor_from_tensor_mask(t, m)
    got = nt.nested_tensor_from_tensor_mask(t.to(DEV), m.to(DEV))
    assert got.nested_size().unbind() == exp.nested_size()
    bits_equal(got._impl.buffer, exp.buffer)


def test_from_padded_value_comparison_semantics():
    # `tensor != padding` of torch: NaN is kept, -0.0 equals the padding 0.0
    t = torch.tensor([[1.0, float("nan"), 0.0, 0.0], [2.0, -0.0, 0.0, 0.0], [3.0, 4.0, 5.0, 6.0]])
    exp = oracle.nested_tensor_from_padded_tensor(t, padding=0.0)
    got = nt.nested_tensor_from_padded_tensor(t.to(DEV), padding=0.0)
    assert got.nested_size().unbind() == exp.nested_size()
    bits_equal(got._impl.buffer, exp.buffer)


def test_dense_to_nested_operators_refuse_a_tensor_without_rows():
    # the registered operators can be called directly; a 1-D tensor has no mask rows
    # below the batch dim
    t = torch.arange(6.0, device=DEV)
    with pytest.raises(RuntimeError, match="batch dim and at least one more"):
        torch.ops.nestedtensor.nt_from_padded_tensor(t, -1.0, 1)
    with pytest.raises(RuntimeError, match="batch dim and at least one more"):
        torch.ops.nestedtensor.from_padded_value_lowered(t, -1.0, 1)


def test_from_padded_value_non_prefix_takes_compaction_path():
    t = torch.tensor([[[1.0, -1.0, 2.0, -1.0], [3.0, -1.0, 4.0, -1.0]],
                      [[5.0, 6.0, -1.0, -1.0], [7.0, 8.0, -1.0, -1.0]]])
    exp = oracle.nested_tensor_from_padded_tensor(t)
    got = nt.nested_tensor_from_padded_tensor(t.to(DEV))
    assert got.nested_size().unbind() == exp.nested_size()
    bits_equal(got._impl.buffer, exp.buffer)
    # rows that are dropped in the middle: kept children are not leading
    t2 = torch.tensor([[[1.0, 2.0], [-1.0, -1.0], [3.0, 4.0]]])
    exp2 = oracle.nested_tensor_from_padded_tensor(t2)
    got2 = nt.nested_tensor_from_padded_tensor(t2.to(DEV))
    assert got2.nested_size().unbind() == exp2.nested_size()
    bits_equal(got2._impl.buffer, exp2.buffer)


@pytest.mark.parametrize("dtype,padding", [(torch.float16, 0.1), (torch.bfloat16, 0.1), (torch.bfloat16, 1e-3),
                                           (torch.float32, 0.1), (torch.int64, -1), (torch.int32, 0.5)])
def test_from_padded_tensor_compares_in_the_tensors_own_type(dtype, padding):
    # `tensor != padding` rounds the padding to the tensor's type first: 0.1 as a
    # half is 0.0999755859375, and elements holding exactly that are padding
    B, L, E = 6, 9, 4
    g = torch.Generator().manual_seed(77)
    lens = [int(v) for v in torch.randint(1, L + 1, (B,), generator=g)]
    lens[0] = L
    if dtype.is_floating_point:
        pad_t = torch.tensor(padding, dtype=dtype)
        padded = pad_t.expand(B, L, E).clone()
        for b, n in enumerate(lens):
            padded[b, :n] = torch.randn(n, E, generator=g).to(dtype) + 3.0
    else:
        padded = torch.full((B, L, E), int(padding) if float(padding).is_integer() else 0, dtype=dtype)
        for b, n in enumerate(lens):
            padded[b, :n] = torch.randint(1 << 40 if dtype == torch.int64 else 5, (1 << 40) + 50 if dtype == torch.int64 else 90,
                                          (n, E), generator=g).to(dtype)
    mask = padded != padding          # torch's own comparison, on the host
    got = nt.nested_tensor_from_padded_tensor(padded.to(DEV), padding=padding)
    exp = oracle.nested_tensor_from_tensor_mask(padded, mask)
    nt_matches(got, exp.unbind(), dtype)


# ---- nested tensors in host memory: staged through the device -----------------

def test_host_nested_tensors_are_staged_through_the_device():
    # the reference's default device is the host (nested/creation.py:15-16); its
    # conversions there are CPU loops (masking.cpp:297-319, 511-532, 627-649)
    g = torch.Generator().manual_seed(77)
    parts = [torch.randn(int(l), 5, generator=g) for l in (3, 1, 7, 4)]
    a = nt.nested_tensor(parts)
    assert a.device.type == "cpu"
    ref = oracle.ref_nested_tensor(parts)
    padded = a.to_padded_tensor(-2.0)
    assert padded.device.type == "cpu" and torch.equal(padded, oracle.to_padded_tensor(ref, -2.0))
    t, m = a.to_tensor_mask()
    exp_t, exp_m = oracle.to_tensor_mask(ref)
    assert t.device.type == "cpu" and m.device.type == "cpu"
    assert torch.equal(t, exp_t) and torch.equal(m, exp_m.to(torch.bool))
    for md in (2, 3):
        got = torch.ops.nestedtensor.to_mask(a, md)
        assert got.device.type == "cpu" and torch.equal(got, oracle.to_mask(ref, md).to(torch.bool))
    back = nt.nested_tensor_from_tensor_mask(t, m)
    assert back.device.type == "cpu" and torch.equal(back._impl.buffer, ref.buffer)
    assert back.nested_size() == a.nested_size()
    back = nt.nested_tensor_from_padded_tensor(padded, padding=-2.0)
    assert back.device.type == "cpu" and torch.equal(back._impl.buffer, ref.buffer)
    back = nt.from_padded_tensor(padded, a)
    assert back.device.type == "cpu" and torch.equal(back._impl.buffer, ref.buffer)
    back = nt.from_padded_tensor(padded, a.nested_size())
    assert torch.equal(back._impl.buffer, ref.buffer)


# ---- many short rows: the kernels that share the row decode ----------------------

def _short_row_case(kind, g):
    """Shapes with at least 4096 output rows of at most 4 KiB."""
    if kind == "one ragged dim, rows up to 600 bytes":
        return [(int(l),) for l in torch.randint(1, 301, (6000,), generator=g)]
    if kind == "one ragged dim, rows up to 3840 bytes":
        return [(int(l), 24) for l in torch.randint(1, 41, (5000,), generator=g)]
    if kind == "two ragged dims":
        hw = torch.randint(1, 201, (40, 2), generator=g)
        hw[0] = torch.tensor([150, 200])
        return [(min(int(h), 150), int(w)) for h, w in hw]
    if kind == "three ragged dims":
        chw = torch.randint(1, 7, (8, 1), generator=g), torch.randint(1, 201, (8, 1), generator=g), \
            torch.randint(1, 151, (8, 1), generator=g)
        shapes = [(int(c), int(h), int(w)) for c, h, w in zip(*chw)]
        shapes[0] = (6, 200, 150)
        return shapes
    if kind == "two ragged dims and a regular tail":
        hw = torch.randint(1, 121, (50, 2), generator=g)
        hw[0] = torch.tensor([120, 120])
        return [(int(h), int(w), 3) for h, w in hw]
    raise AssertionError(kind)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.float16, torch.float32, torch.float64])
@pytest.mark.parametrize("kind", ["one ragged dim, rows up to 600 bytes", "one ragged dim, rows up to 3840 bytes",
                                  "two ragged dims", "three ragged dims", "two ragged dims and a regular tail"])
def test_many_short_rows(kind, dtype):
    # from 4096 rows of at most 4 KiB on, pad / un-pad take the row-batch / row-group
    # kernels and masks of 1 MiB or more the flat plane kernel: every element size,
    # one to three ragged dims, rows at every alignment
    g = torch.Generator().manual_seed(len(kind))
    shapes = _short_row_case(kind, g)
    if dtype == torch.float64 and kind == "one ragged dim, rows up to 3840 bytes":
        shapes = [(l, 12) for l, _ in shapes]
    if dtype.is_floating_point:
        parts = [torch.randn(*s, generator=g).to(dtype) for s in shapes]
    else:
        parts = [torch.randint(1, 200, s, generator=g).to(dtype) for s in shapes]
    a = nt.nested_tensor(parts, device=DEV, dtype=dtype)
    ref = oracle.ref_nested_tensor(parts, dtype=dtype)
    pad_value = 7 if dtype == torch.uint8 else -10000.0      # no N(0, 1) sample rounds to it
    padded = a.to_padded_tensor(pad_value)
    bits_equal(padded, oracle.to_padded_tensor(ref, pad_value))
    bits_equal(nt.from_padded_tensor(padded, a)._impl.buffer, ref.buffer)
    data, mask = a.to_tensor_mask()
    exp_d, exp_m = oracle.to_tensor_mask(ref)
    bits_equal(data, exp_d)
    assert mask.shape == exp_m.shape and torch.equal(mask.cpu(), exp_m.to(torch.bool))
    full = torch.ops.nestedtensor.to_mask(a, a.dim())
    assert torch.equal(full.cpu(), oracle.to_mask(ref, a.dim()).to(torch.bool))
    # a goal shape larger than the batch maximum in every dim: regular dims are
    # walked as ragged, the extra region is padding in the data and zeros in the mask
    goal = [m + 3 for m in a._impl.max_sizes()]
    big_d, big_m = torch.ops.nestedtensor.pad_nt(a, goal)
    exp_bd, exp_bm = oracle.pad_nt(ref, goal)
    bits_equal(big_d, exp_bd)
    assert torch.equal(big_m.cpu(), exp_bm.to(torch.bool))
    bits_equal(nt.from_padded_tensor(big_d, a)._impl.buffer, ref.buffer)
    # dense -> nested from the full mask and from the padding value
    again = nt.nested_tensor_from_tensor_mask(data, full)
    bits_equal(again._impl.buffer, ref.buffer)
    assert again.nested_size() == a.nested_size()
    if dtype != torch.uint8:
        again = nt.nested_tensor_from_padded_tensor(padded, padding=pad_value)
        bits_equal(again._impl.buffer, ref.buffer)


@pytest.mark.parametrize("dtype", [torch.float32, torch.uint8, torch.float16, torch.float64])
def test_pack_table_in_kernel_arguments_and_uploaded(dtype):
    # up to nt_pack_table_max_entries() int64 of metadata ride in the kernel arguments of
    # the pack launch, which also writes their device copy; larger batches upload the
    # table first.  Both sides of the limit, empty constituents, and the adopted metadata.
    from nestedtensor_amd import _C
    limit = int(_C.lib.nt_pack_table_max_entries())
    g = torch.Generator().manual_seed(91)
    for B, D in ((1, 1), (16, 3), (limit // 4, 2), (limit // 4 + 5, 2), (3, 2)):
        shapes = [[int(v) for v in torch.randint(0 if B == 3 else 1, 9, (D,), generator=g)] for _ in range(B)]
        parts = [(torch.randn(*s, generator=g) * 40).to(dtype) for s in shapes]
        dev_parts = [p.to(DEV) for p in parts]
        a = nt.nested_tensor(dev_parts, device=DEV, dtype=dtype)
        ref = oracle.ref_nested_tensor(parts, dtype=dtype)
        bits_equal(a._impl.buffer, ref.buffer)
        assert a.nested_size().unbind() == [torch.Size(p.shape) for p in parts]
        assert torch.equal(a._impl.sizes_dev().cpu(), a._impl.sizes)
        exp_off = torch.zeros(B + 1, dtype=torch.int64)
        exp_off[1:] = torch.cumsum(a._impl.sizes.prod(1), 0)
        assert torch.equal(a._impl.offsets_dev().cpu(), exp_off)
        if not a._impl.has_empty_constituent():
            bits_equal(a.to_padded_tensor(0), oracle.to_padded_tensor(ref, 0))


def test_pad_unpad_mask_under_hip_graph_replays():
    # pad, length-based un-pad and masks enqueue on the current stream, allocate through
    # torch and never wait for the device, so they can be captured; every replay, with new
    # contents in the packed buffer, must equal the eager result.  (The dense -> nested
    # conversions size their output from device data and cannot be captured.)
    g = torch.Generator().manual_seed(123)
    parts = [torch.randn(int(l), 40, generator=g) for l in (5, 17, 1, 33, 12)]
    a = nt.nested_tensor(parts, device=DEV)

    def work():
        padded = a.to_padded_tensor(-3.0)
        data, mask = a.to_tensor_mask()
        back = nt.from_padded_tensor(padded, a)
        return padded, data, mask, back._impl.buffer

    for _ in range(3):
        work()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()
        with torch.cuda.graph(graph, stream=side):
            outs = work()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        a._impl.buffer.copy_(torch.randn(a._impl.buffer.shape, generator=g).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        exp = work()
        torch.cuda.synchronize()
        for x, y in zip(got, exp):
            assert torch.equal(x, y), "replay %d differs from the eager call" % rep
        ref = oracle.ref_nested_tensor([p.cpu() for p in a.unbind()])
        bits_equal(got[0], oracle.to_padded_tensor(ref, -3.0))
        bits_equal(got[3], ref.buffer)
