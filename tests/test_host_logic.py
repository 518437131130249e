"""Host-side logic of the product that needs no GPU: the C-ABI library loads and
exports every declared symbol, constructors and metadata accessors behave like
the reference's (test/test_nested_tensor_class.py), error messages match, and
compute ops refuse host tensors instead of falling back."""

import ctypes
import os
import re

import pytest
import torch

import nestedtensor_amd as nt
from nestedtensor_amd import _C
from masking_cases import FROM_TENSOR_MASK_ERRORS, TO_TENSOR_MASK_ERRORS

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "nestedtensor_amd.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(nt_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 14
    lib = ctypes.CDLL(_C.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(_C.SIGNATURES), declared ^ set(_C.SIGNATURES)
    assert lib.nt_abi_version() == 1


def test_argument_validation_needs_no_gpu():
    # invalid geometry is rejected on the host before any launch
    rc = _C.lib.nt_add_padding(None, None, None, None, 4, 2, 5, _C.i64_array([1, 1]), 4, 0, None)
    assert rc == 1 and b"bad geometry" in _C.lib.nt_last_error()
    rc = _C.lib.nt_linear(None, 0, None, None, None, 0, 4, 4, 4, 0, None)
    assert rc == 1
    rc = _C.lib.nt_varlen_attention(None, 0, None, 0, None, 0, None, 0, None, None, 1, 0, 64, 1, 1.0, 1, None)
    assert rc == 1


def _constructors():
    yield nt.as_nested_tensor
    yield nt.nested_tensor


def test_constructor_copies():
    # test_nested_tensor_class.py:48-88
    tensors = [torch.arange(float((i + 1) * 4)).reshape(i + 1, 4) + 1 for i in range(5)]
    for ctor in _constructors():
        a = ctor(tensors)
        for i, t in enumerate(tensors):
            t.mul_(i + 2)
        for t, u in zip(tensors, a.unbind()):
            assert not torch.equal(t, u)
            assert t.untyped_storage().data_ptr() != u.untyped_storage().data_ptr()
    a = nt.nested_tensor([torch.tensor([3.0])])
    assert nt.as_nested_tensor(a) is a
    assert nt.as_nested_tensor(a, dtype=torch.int64) is a
    one = torch.tensor([1.0, 2.0])
    b = nt.nested_tensor([one])
    one.mul_(3)
    assert torch.equal(b.unbind()[0], torch.tensor([1.0, 2.0]))


def test_constructor_errors():
    # test_nested_tensor_class.py:90-102
    for ctor in _constructors():
        with pytest.raises(RuntimeError):
            ctor([3.0])
        with pytest.raises(TypeError):
            ctor(torch.tensor([3.0]))
        with pytest.raises(TypeError):
            ctor(4.0)
        with pytest.raises(TypeError):
            ctor()
        for ctor2 in _constructors():
            ctor(ctor2([torch.tensor([3.0])]))
            with pytest.raises(RuntimeError):
                ctor([torch.tensor([2.0]), ctor2([torch.tensor([3.0])])])
        with pytest.raises(RuntimeError):
            ctor([torch.randn(2), torch.randn(2, 2)])
        with pytest.raises(RuntimeError):
            ctor([torch.randn(2), torch.randn(2).double()])
    with pytest.raises(RuntimeError, match="does not support autograd"):
        nt.nested_tensor([torch.randn(2)], requires_grad=True)


def test_default_constructor():
    # test_nested_tensor_class.py:104-122
    for ctor in _constructors():
        a = ctor([])
        d = torch.tensor([])
        assert a.nested_dim() == 1
        assert a.nested_size().unbind() == []
        assert a.dim() == d.dim() and a.layout == d.layout and a.device == d.device
        assert a.dtype == d.dtype and a.requires_grad == d.requires_grad
        assert a.is_pinned() == d.is_pinned()


def test_nested_size_size_stride_len():
    # test_nested_tensor_class.py:199-231, 256-265, 449-472
    for ctor in _constructors():
        a = ctor([])
        assert len(a.nested_size()) == 0 and a.size() == (0,)
        with pytest.raises(RuntimeError):
            a.nested_size()[0]
        a = ctor([torch.tensor(1)])
        assert len(a.nested_size()) == 1 and a.nested_size()[0] == torch.Size([])
        assert a.nested_size(0) == 1 and a.size() == (1,)
        with pytest.raises(IndexError):
            a.nested_size(1)
        a = ctor([torch.randn(1)])
        assert a.nested_size()[0] == torch.Size([1]) and a.nested_size(1) == (1,)
        with pytest.raises(IndexError):
            a.nested_size(2)
        a = ctor([torch.randn(1, 2)])
        assert a.nested_size(1) == (1,) and a.nested_size(2) == (2,)
        b = a.nested_size()
        del a
        assert len(b) == 1 and b[0] == torch.Size([1, 2])
        assert ctor([torch.tensor(1), torch.tensor(2)]).size() == (2,)
        assert ctor([torch.rand(1, 2), torch.rand(1, 8)]).size() == (2, 1, None)
        a = ctor([torch.rand(3, 4), torch.rand(5, 4)])
        assert a.size() == (2, None, 4) and len(a) == 2 and a.dim() == 3 and a.numel() == 32
        assert a.is_contiguous() and a.nested_size() == ctor([torch.rand(3, 4), torch.rand(5, 4)]).nested_size()
        ts = [torch.rand(1, 2, 4)[:, :, 0], torch.rand(2, 3, 4)[:, 1, :], torch.rand(3, 4, 5)[1, :, :]]
        a = ctor(ts)
        assert [list(s) for s in a.nested_stride()] == [list(t.contiguous().stride()) for t in ts]
        # non-contiguous inputs are packed contiguous (test_nested_tensor_functional.py:137-150)
        for t, u in zip(ts, a.unbind()):
            assert torch.equal(t, u) and u.is_contiguous()
    assert nt.nested_tensor([torch.tensor([1, 2])]).dtype == torch.float32
    assert nt.nested_tensor([torch.tensor([1, 2])], dtype=torch.int64).dtype == torch.int64


def test_host_only_special_cases():
    # results that need no kernel (masking.cpp:305-313, 164-167, 628-636)
    e = nt.nested_tensor([])
    t, m = e.to_tensor_mask()
    assert torch.equal(t, torch.tensor([0])) and torch.equal(m, torch.tensor(False))
    assert torch.equal(e.to_padded_tensor(2.0), torch.tensor([2.0]))
    s = nt.nested_tensor([torch.tensor(1, dtype=torch.uint8)], dtype=torch.uint8)
    for md, exp in ((None, torch.tensor(True)), (0, torch.tensor(True)), (1, torch.tensor([True]))):
        t, m = s.to_tensor_mask(mask_dim=md)
        assert torch.equal(t, torch.tensor([1], dtype=torch.uint8)) and torch.equal(m, exp)
    assert torch.equal(torch.ops.nestedtensor.to_mask(s, 1), torch.tensor([True]))


@pytest.mark.parametrize("parts,dtype,mask_dim,msg", TO_TENSOR_MASK_ERRORS)
def test_to_tensor_mask_error_messages(parts, dtype, mask_dim, msg):
    a = nt.nested_tensor(parts, dtype=dtype)
    with pytest.raises(RuntimeError, match=msg):
        a.to_tensor_mask(mask_dim=mask_dim)


@pytest.mark.parametrize("tensor,mask,nested_dim,exc,msg", FROM_TENSOR_MASK_ERRORS)
def test_from_tensor_mask_error_messages(tensor, mask, nested_dim, exc, msg):
    with pytest.raises(exc, match=msg):
        nt.nested_tensor_from_tensor_mask(tensor, mask, nested_dim)


def test_from_tensor_mask_host_only_cases():
    # keep-all / keep-nothing masks need no kernel (masking.cpp:228-234)
    r = nt.nested_tensor_from_tensor_mask(torch.tensor([1, 2, 3]), torch.tensor(True))
    assert r.dtype == torch.int64 and r.nested_size().unbind() == [torch.Size([])] * 3
    assert torch.equal(r._impl.buffer, torch.tensor([1, 2, 3]))
    r = nt.nested_tensor_from_tensor_mask(torch.tensor([0]), torch.tensor(False))
    assert len(r) == 0 and r.dtype == torch.float32 and r.nested_dim() == 1
    r = nt.nested_tensor_from_tensor_mask(torch.tensor([[], []]), torch.tensor([[], []]))
    assert r.nested_size().unbind() == [torch.Size([0]), torch.Size([0])]
    r = nt.nested_tensor_from_tensor_mask(torch.tensor([]), torch.tensor([]))
    assert len(r) == 0


def test_host_tensors_need_the_device():
    # conversions of host nested tensors are staged through the device; compute ops
    # want the nested tensor moved first.  Nothing falls back to host arithmetic:
    # without a visible device every one of them raises.
    if torch.cuda.is_available():
        pytest.skip("a device is visible: staging is covered by the device tests")
    a = nt.nested_tensor([torch.randn(2, 3), torch.randn(4, 3)])
    with pytest.raises(RuntimeError, match="staged through the HIP device"):
        a.to_padded_tensor(0)
    with pytest.raises(RuntimeError, match="staged through the HIP device"):
        a.to_tensor_mask()
    with pytest.raises(RuntimeError, match="staged through the HIP device"):
        torch.ops.nestedtensor.to_mask(a, 2)
    with pytest.raises(RuntimeError, match="staged through the HIP device"):
        nt.nested_tensor_from_tensor_mask(torch.randn(2, 3), torch.ones(2, 3, dtype=torch.bool))
    with pytest.raises(RuntimeError, match="staged through the HIP device"):
        nt.nested_tensor_from_padded_tensor(torch.randn(2, 3), padding=0)
    with pytest.raises(RuntimeError, match="staged through the HIP device"):
        nt.from_padded_tensor(torch.randn(2, 4, 3), a)
    mha = torch.nn.MultiheadAttention(3, 1).eval()
    with pytest.raises(RuntimeError, match="HIP device only"):
        mha(a, a, a)
    with pytest.raises(RuntimeError, match="HIP device only"):
        torch.relu(a)
    with pytest.raises(NotImplementedError):
        torch.sigmoid(a)


def test_mask_collapse_closed_form_matches_oracle():
    import oracle
    from nestedtensor_amd import ops
    g = torch.Generator().manual_seed(4)
    for trial in range(40):
        dims = int(torch.randint(1, 4, (1,), generator=g))
        B = int(torch.randint(1, 4, (1,), generator=g))
        regular = [bool(torch.randint(0, 2, (1,), generator=g)) for _ in range(dims)]
        base = [int(torch.randint(1, 4, (1,), generator=g)) for _ in range(dims)]
        parts = []
        for b in range(B):
            shape = [base[k] if regular[k] else int(torch.randint(1, 4, (1,), generator=g)) for k in range(dims)]
            parts.append(torch.randn(*shape, generator=g))
        a = nt.nested_tensor(parts)
        ref = oracle.ref_nested_tensor(parts)
        for md in [None] + list(range(0, dims + 2)):
            try:
                _, m = oracle.to_tensor_mask(ref, md)
                exp = m.dim()
            except RuntimeError as e:
                exp = str(e)
            try:
                got = ops._collapsed_mask_dims(a._impl, md)
            except RuntimeError as e:
                got = str(e)
            assert got == exp, (parts and [p.shape for p in parts], md, got, exp)


def test_channels_last_metadata_and_views():
    """A channels-last impl over a host buffer: strides, is_contiguous and the
    constituent views need no device work (nested_tensor_impl.cpp:182-194,
    Packed.h:125-163)."""
    from nestedtensor_amd.impl import NestedTensorImpl
    from nestedtensor_amd.nested.nested import NestedTensor
    import oracle
    ts = [torch.randn(4, 3, 5), torch.randn(4, 2, 7)]
    ref = oracle.ref_nested_tensor(ts)
    buffer, strides = oracle.to_channels_last(ref)
    a = NestedTensor(NestedTensorImpl(buffer, ref.sizes, channels_last=True))
    assert a.is_contiguous(memory_format=torch.channels_last)
    assert not a.is_contiguous()
    assert a.nested_size() == nt.nested_tensor(ts).nested_size()
    assert list(a.nested_stride()) == strides
    assert a.nested_stride(1) == (1, 1) and a.nested_stride(3) == (4, 4)
    for got, t in zip(a.unbind(), ts):
        want = t.unsqueeze(0).contiguous(memory_format=torch.channels_last).squeeze(0)
        assert got.stride() == want.stride() and torch.equal(got, t)
    b = nt.nested_tensor(ts)
    assert b.is_contiguous() and not b.is_contiguous(memory_format=torch.channels_last)
    assert b.contiguous() is b and a.contiguous(memory_format=torch.channels_last) is a
    with pytest.raises(RuntimeError, match="not supported"):
        b.is_contiguous(memory_format=torch.channels_last_3d)
    with pytest.raises(RuntimeError, match="requires 4 dim input"):
        NestedTensorImpl(torch.zeros(6), torch.tensor([[2, 3]]), channels_last=True)
    with pytest.raises(RuntimeError, match="runs on the HIP device only"):
        b.contiguous(memory_format=torch.channels_last)
    with pytest.raises(RuntimeError, match="requires 4 dim input"):
        nt.nested_tensor([torch.randn(2, 3)]).contiguous(memory_format=torch.channels_last)


def test_unbind_across_constituent_dims():
    # test/test_nested_tensor_class.py:394-429
    for unbind_fn in (lambda x, dim: x.unbind(dim), lambda x, dim: torch.unbind(x, dim)):
        a = torch.rand(3, 2)
        x = nt.nested_tensor([a])
        for d in (1, 2):
            got = unbind_fn(x, d)
            exp = [nt.nested_tensor([p]) for p in a.unbind(d - 1)]
            assert len(got) == len(exp)
            for g_, e_ in zip(got, exp):
                assert g_.nested_size() == e_.nested_size()
                assert all(torch.equal(u, v) for u, v in zip(g_.unbind(), e_.unbind()))
        b = torch.rand(2, 3)
        x = nt.nested_tensor([a, b])
        assert all(torch.equal(u, v) for u, v in zip(unbind_fn(x, 0), (a, b)))
        got = unbind_fn(x, 1)
        exp = [nt.nested_tensor([a[0], b[0]]), nt.nested_tensor([a[1], b[1]]), nt.nested_tensor([a[2]])]
        assert len(got) == 3
        for g_, e_ in zip(got, exp):
            assert g_.nested_size() == e_.nested_size()
            assert all(torch.equal(u, v) for u, v in zip(g_.unbind(), e_.unbind()))
        assert len(unbind_fn(x, -1)) == 3          # slices along the last dim: 2 and 3 columns
        with pytest.raises(IndexError):
            unbind_fn(x, 3)


def test_to_tensor_needs_regular_sizes():
    # totensor.cpp:30-42, 45-63
    ts = [torch.rand(3, 2), torch.rand(3, 2)]
    a = nt.nested_tensor(ts)
    got = a.to_tensor()
    assert torch.equal(got, torch.stack(ts)) and got.data_ptr() != a._impl.buffer.data_ptr()
    assert torch.equal(a.to_tensor(0), torch.stack(ts))
    with pytest.raises(IndexError, match="only works if there is no None in size"):
        nt.nested_tensor([torch.rand(3, 2), torch.rand(2, 2)]).to_tensor()
    with pytest.raises(RuntimeError, match="Non-zero dimension 1 is currently not supported."):
        a.to_tensor(1)
    assert nt.nested_tensor([]).to_tensor().numel() == 0


def test_getitem_int_slice_tuple():
    # py_init.cpp:26-108 at nested_dim 1 (cases of test/test_nested_tensor_class.py:679-707 that need no deeper nesting)
    a, b, c = torch.randn(3, 4), torch.randn(4, 3), torch.randn(1, 3)
    x = nt.nested_tensor([a, b, c])
    assert torch.equal(x[0], a) and torch.equal(x[-1], c)
    assert x[0].data_ptr() == x._impl.buffer.data_ptr()                 # a view
    assert x[:].nested_size() == x.nested_size()
    assert [tuple(t.shape) for t in x[-1:].unbind()] == [(1, 3)]
    assert torch.equal(x[0, 1:], a[1:]) and torch.equal(x[1, :, 0], b[:, 0])
    got = x[:, 0]
    assert all(torch.equal(u, v) for u, v in zip(got.unbind(), (a[0], b[0], c[0])))
    got = x[:2, :, -1:]
    assert all(torch.equal(u, v) for u, v in zip(got.unbind(), (a[:, -1:], b[:, -1:])))
    assert x[()] is x
    with pytest.raises(IndexError, match=r"expected to be in range of \[-3, 2\], but got 3"):
        x[3]
    with pytest.raises(RuntimeError, match="Only nested_dim of 1"):
        x[None]


def test_merge_tensor_mask_op_matches_oracle():
    # masking.cpp:12-43 as an op on plain tensors
    import oracle
    g = torch.Generator().manual_seed(3)
    t = torch.randn(4, 3, 5, generator=g)
    full_rows = torch.tensor([[1, 1, 0], [1, 0, 0], [1, 1, 1], [0, 0, 0]], dtype=torch.uint8)
    cases = [full_rows.unsqueeze(-1).expand(4, 3, 5).contiguous(),            # collapses to [4, 3]
             torch.ones(4, 3, 5, dtype=torch.uint8),                         # collapses to a scalar
             (torch.rand(4, 3, 5, generator=g) > 0.5).to(torch.uint8)]       # does not collapse
    for m in cases:
        for mask_dim in (None, 1, 2, 3):
            try:
                exp = oracle.merge_tensor_mask(t, m, mask_dim)
            except RuntimeError as e:
                with pytest.raises(RuntimeError, match=str(e)):
                    torch.ops.nestedtensor.merge_tensor_mask(t, m, mask_dim)
                continue
            got = torch.ops.nestedtensor.merge_tensor_mask(t, m, mask_dim)
            assert got[1].shape == exp[1].shape
            assert torch.equal(got[1].to(torch.bool), exp[1].to(torch.bool))
            assert torch.equal(got[0], exp[0])
