"""Pins the CPU oracle for packing / padding / masks: replay of the reference's
literal test cases (tests/golden/masking_cases.py), independent library cross-checks and
closed forms.  No GPU, no product code."""

import random

import pytest
import torch

import oracle
from masking_cases import (TO_TENSOR_MASK, TO_TENSOR_MASK_ERRORS, FROM_TENSOR_MASK,
                   FROM_TENSOR_MASK_ERRORS, ROUND_TRIP_DATA, ROUND_TRIP_MASK)


def same(a, b):
    """The reference's comparison (test/utils_test_case.py:76-118): same size,
    then b cast to a's type, max abs diff <= 1e-5."""
    assert a.size() == b.size(), (a.size(), b.size())
    if a.numel() == 0:
        return
    b = b.to(a)
    if a.dtype == torch.bool:
        a, b = a.int(), b.int()
    assert (a.double() - b.double()).abs().max() <= 1e-5


def nt_equal(res, expected_parts, expected_dtype):
    assert res.dtype == expected_dtype
    assert len(res) == len(expected_parts)
    for r, e in zip(res.unbind(), expected_parts):
        assert tuple(r.shape) == tuple(e.shape)
        same(r, e.to(expected_dtype))


# ---- pack / metadata -------------------------------------------------------

def test_pack_is_concatenation():
    g = torch.Generator().manual_seed(1)
    ts = [torch.randn(int(l), 5, generator=g) for l in torch.randint(1, 9, (6,), generator=g)]
    nt = oracle.ref_nested_tensor(ts)
    assert torch.equal(nt.buffer, torch.cat([t.reshape(-1) for t in ts]))
    for a, b in zip(nt.unbind(), ts):
        assert torch.equal(a, b)
    # non-contiguous inputs are packed contiguous (test_nested_tensor_functional.py:137-150)
    ts2 = [torch.randn(4, 6, generator=g).t(), torch.randn(3, 7, generator=g)[:, ::2]]
    nt2 = oracle.ref_nested_tensor(ts2)
    assert torch.equal(nt2.buffer, torch.cat([t.contiguous().reshape(-1) for t in ts2]))


def test_metadata_literals():
    # test_nested_tensor_class.py:199-231, 449-472
    a = oracle.ref_nested_tensor([])
    assert len(a.nested_size()) == 0 and a.size() == (0,) and a.dim() == 1
    a = oracle.ref_nested_tensor([torch.tensor(1)])
    assert a.nested_size()[0] == torch.Size([]) and a.nested_size(0) == 1 and a.size() == (1,)
    with pytest.raises(IndexError):
        a.nested_size(1)
    a = oracle.ref_nested_tensor([torch.randn(1, 2)])
    assert a.nested_size(1) == (1,) and a.nested_size(2) == (2,)
    a = oracle.ref_nested_tensor([torch.rand(1, 2), torch.rand(1, 8)])
    assert a.size() == (2, 1, None)
    a = oracle.ref_nested_tensor([torch.rand(3, 4), torch.rand(5, 4)])
    assert a.size() == (2, None, 4)
    # default dtype cast (creation.py:13-14)
    assert oracle.ref_nested_tensor([torch.tensor([1, 2])]).dtype == torch.float32
    # nested_stride (test_nested_tensor_class.py:256-265)
    ts = [torch.rand(1, 2, 4)[:, :, 0], torch.rand(2, 3, 4)[:, 1, :], torch.rand(3, 4, 5)[1, :, :]]
    a = oracle.ref_nested_tensor(ts)
    assert [list(s) for s in a.nested_stride()] == [list(t.contiguous().stride()) for t in ts]


# ---- to_tensor_mask / to_mask ----------------------------------------------

@pytest.mark.parametrize("name,parts,dtype,checks", TO_TENSOR_MASK, ids=[c[0] for c in TO_TENSOR_MASK])
def test_to_tensor_mask_literals(name, parts, dtype, checks):
    nt = oracle.ref_nested_tensor(parts, dtype=dtype)
    for mask_dim, exp_t, exp_m in checks:
        t, m = oracle.to_tensor_mask(nt, mask_dim)
        same(t, exp_t)
        same(m, exp_m)


@pytest.mark.parametrize("parts,dtype,mask_dim,msg", TO_TENSOR_MASK_ERRORS)
def test_to_tensor_mask_errors(parts, dtype, mask_dim, msg):
    nt = oracle.ref_nested_tensor(parts, dtype=dtype)
    with pytest.raises(RuntimeError, match=msg):
        oracle.to_tensor_mask(nt, mask_dim)


def _closed_form_mask(sizes, max_size):
    B = sizes.size(0)
    mask = torch.ones([B] + max_size, dtype=torch.bool)
    for k in range(len(max_size)):
        idx = torch.arange(max_size[k]).reshape([1] + [max_size[k] if j == k else 1 for j in range(len(max_size))])
        lim = sizes[:, k].reshape([B] + [1] * len(max_size))
        mask &= idx < lim
    return mask


def test_to_tensor_mask_closed_form_and_to_mask():
    random.seed(110)
    for dims in (1, 2, 3):
        parts = [torch.randn(*[random.randint(1, 5) for _ in range(dims)]) for _ in range(4)]
        nt = oracle.ref_nested_tensor(parts)
        full = dims + 1
        t, m = oracle.to_tensor_mask(nt, full)
        cf = _closed_form_mask(nt.sizes, oracle.get_max_size(nt))
        assert torch.equal(m.to(torch.bool), cf)
        # data: inside == constituent, outside == 0
        for b, p in enumerate(parts):
            sl = tuple(slice(0, s) for s in p.shape)
            assert torch.equal(t[b][sl], p)
        assert torch.equal(t[~cf], torch.zeros(int((~cf).sum())))
        # to_mask == to_tensor_mask()[1] (test_nested_tensor_class.py:809-817)
        for md in [None] + list(range(2, full + 1)):
            try:
                _, m0 = oracle.to_tensor_mask(nt, md)
            except RuntimeError:
                continue
            m1 = oracle.to_mask(nt, md)
            same(m0, m1)


def test_to_mask_reference_case():
    # test_nested_tensor_class.py:809-817
    random.seed(110)
    lens = [random.randint(2, 4) for _ in range(3)]
    parts = [torch.arange(t * 3).reshape(t, 3).float() for t in lens]
    nt = oracle.ref_nested_tensor(parts)
    _, m0 = oracle.to_tensor_mask(nt, 2)
    m1 = oracle.to_mask(nt, 2)
    same(m0, m1)
    exp = torch.zeros(3, max(lens), dtype=torch.bool)
    for b, l in enumerate(lens):
        exp[b, :l] = True
    assert torch.equal(m1.to(torch.bool), exp)


# ---- to_padded_tensor --------------------------------------------------------

def test_to_padded_tensor_library_cross_checks():
    g = torch.Generator().manual_seed(7)
    parts = [torch.randn(int(l), 6, generator=g) for l in torch.randint(1, 12, (9,), generator=g)]
    nt = oracle.ref_nested_tensor(parts)
    got = oracle.to_padded_tensor(nt, -3.5)
    ref1 = torch.nn.utils.rnn.pad_sequence(parts, batch_first=True, padding_value=-3.5)
    assert torch.equal(got, ref1)
    ref2 = torch.nested.nested_tensor(parts).to_padded_tensor(-3.5)
    assert torch.equal(got, ref2)
    # irregular in every dim, 3-D constituents, against core torch.nested
    parts = [torch.randn(int(a), int(b), int(c), generator=g)
             for a, b, c in torch.randint(1, 6, (5, 3), generator=g)]
    got = oracle.to_padded_tensor(oracle.ref_nested_tensor(parts), 2.0)
    assert torch.equal(got, torch.nested.nested_tensor(parts).to_padded_tensor(2.0))


def test_reference_round_trip_literal():
    # test_nested_tensor_masking.py:454-477
    parts = oracle.nt_from_tensor_mask(ROUND_TRIP_DATA, ROUND_TRIP_MASK, 1)
    nt2 = oracle.ref_nested_tensor(parts)
    d2, m2 = oracle.to_tensor_mask(nt2)
    same(ROUND_TRIP_DATA, d2)
    same(ROUND_TRIP_MASK, m2)
    d3 = oracle.to_padded_tensor(nt2, -10)
    same(ROUND_TRIP_DATA + ~ROUND_TRIP_MASK * -10, d3)


# ---- nested_tensor_from_tensor_mask ------------------------------------------

@pytest.mark.parametrize("name,tensor,mask,parts,dtype", FROM_TENSOR_MASK,
                         ids=[c[0] for c in FROM_TENSOR_MASK])
def test_from_tensor_mask_literals(name, tensor, mask, parts, dtype):
    res = oracle.nested_tensor_from_tensor_mask(tensor, mask)
    nt_equal(res, parts, dtype)
    res = oracle.nested_tensor_from_tensor_mask(tensor, mask, nested_dim=1)
    nt_equal(res, parts, dtype)


@pytest.mark.parametrize("tensor,mask,nested_dim,exc,msg", FROM_TENSOR_MASK_ERRORS)
def test_from_tensor_mask_errors(tensor, mask, nested_dim, exc, msg):
    with pytest.raises(exc, match=msg):
        oracle.nested_tensor_from_tensor_mask(tensor, mask, nested_dim)


def test_from_tensor_mask_vectorised_equals_literal_walk():
    g = torch.Generator().manual_seed(3)
    for trial in range(20):
        B = 3
        dims = [int(v) for v in torch.randint(1, 5, (3,), generator=g)]
        t = torch.randn(B, *dims, generator=g)
        mdim = 1 + int(torch.randint(1, 4, (1,), generator=g))   # mask dims incl. batch: 2..4
        # rectangular prefix boxes, some constituents empty
        mask = torch.zeros([B] + dims[: mdim - 1], dtype=torch.bool)
        for b in range(B):
            ext = [int(torch.randint(0, d + 1, (1,), generator=g)) for d in dims[: mdim - 1]]
            if b == 0:
                ext = [max(e, 1) for e in ext]
            mask[b][tuple(slice(0, e) for e in ext)] = True
        lit = oracle.nt_from_tensor_mask(t, mask, 1)
        vec = oracle.nt_from_tensor_mask_vectorised(t, mask)
        assert len(lit) == len(vec)
        for a, b_ in zip(lit, vec):
            assert tuple(a.shape) == tuple(b_.shape), (a.shape, b_.shape, mask.shape)
            assert torch.equal(a, b_)


# ---- from_padded_tensor (length based) ----------------------------------------

def test_from_padded_round_trip_and_masked_select():
    g = torch.Generator().manual_seed(11)
    for dims in (1, 2, 3):
        parts = [torch.randn(*[int(v) for v in torch.randint(1, 6, (dims,), generator=g)], generator=g)
                 for _ in range(5)]
        nt = oracle.ref_nested_tensor(parts)
        padded = oracle.to_padded_tensor(nt, 9.0)
        back = oracle.from_padded_tensor(padded, nt)
        assert torch.equal(back.buffer, nt.buffer)
        cf = _closed_form_mask(nt.sizes, oracle.get_max_size(nt))
        assert torch.equal(back.buffer, padded[cf])
