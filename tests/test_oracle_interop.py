"""Pins the interop oracle functions (CPU only)."""
import pytest
import torch

import oracle


def _idx_nt(lens, V, seed=0):
    g = torch.Generator().manual_seed(seed)
    return oracle.ref_nested_tensor([torch.randint(V, (L,), generator=g) for L in lens], dtype=torch.int64)


def test_embedding_is_row_indexing():
    w = torch.randn(50, 6, generator=torch.Generator().manual_seed(1))
    nt = _idx_nt([5, 1, 9], 50)
    got = oracle.embedding(w, nt)
    for o, i in zip(got.unbind(), nt.unbind()):
        assert torch.equal(o, w[i])
    assert got.opt_sizes() == [3, None, 6]


@pytest.mark.parametrize("mode", ["sum", "mean", "max"])
def test_embedding_bag_against_loops(mode):
    w = torch.randn(100, 8, generator=torch.Generator().manual_seed(2))
    nt = _idx_nt([5, 5, 1, 12], 100, seed=3)            # reference case: two bags of 5 (functional.py:189-190)
    got = oracle.embedding_bag(nt, w, mode)
    for b, idx in enumerate(nt.unbind()):
        rows = [w[int(i)] for i in idx]
        if mode == "max":
            exp = torch.stack(rows).max(0).values
        else:
            exp = rows[0].clone()
            for r in rows[1:]:
                exp = exp + r
            if mode == "mean":
                exp = exp / len(rows)
        assert (got[b] - exp).abs().max() <= 1e-6 * max(1.0, exp.abs().max().item())


def test_to_sparse_csr_to_dense_is_padded():
    # test/test_nested_tensor_class.py:741-752
    a, b, c = torch.arange(3) + 1, torch.arange(4) + 1, torch.arange(2) + 1
    nt = oracle.ref_nested_tensor([a, b, c], dtype=torch.int64)
    st = oracle.to_sparse_csr(nt)
    assert torch.equal(st.to_dense(), oracle.to_padded_tensor(nt, 0))
    nt = oracle.ref_nested_tensor([a.unsqueeze(1), b.unsqueeze(1)], dtype=torch.int64)
    with pytest.raises(RuntimeError, match="Given tensor must be of dimension 2, got dimension 3"):
        oracle.to_sparse_csr(nt)


def test_to_packed_sequence_round_trip():
    g = torch.Generator().manual_seed(4)
    ts = [torch.randn(L, 3, generator=g) for L in (4, 7, 1, 7, 2)]
    nt = oracle.ref_nested_tensor(ts)
    ps = oracle.to_packed_sequence(nt)
    padded, lengths = torch.nn.utils.rnn.pad_packed_sequence(ps, batch_first=True)
    assert torch.equal(padded, oracle.to_padded_tensor(nt, 0))
    assert lengths.tolist() == [4, 7, 1, 7, 2]
    assert ps.batch_sizes.tolist() == [5, 4, 3, 3, 2, 2, 2]


def test_transposes_are_inverse_permutations():
    g = torch.Generator().manual_seed(5)
    ts = [torch.randn(4, h, w, generator=g) for h, w in ((3, 5), (7, 2), (1, 1))]
    nt = oracle.ref_nested_tensor(ts)
    a = oracle.transpose_nchw_nhwc(nt)
    for t, o in zip(ts, a.unbind()):
        assert o.shape == (t.shape[1], t.shape[2], 4)
        for c in range(4):
            assert torch.equal(o[:, :, c], t[c])           # element [h, w, c] == [c, h, w]
    back = oracle.transpose_nhwc_nchw(a)
    assert torch.equal(back.buffer, nt.buffer)
    with pytest.raises(RuntimeError, match="Expected first dimension to be regular."):
        oracle.transpose_nchw_nhwc(oracle.ref_nested_tensor([torch.randn(2, 3, 3), torch.randn(3, 3, 3)]))


def _images(seed=1010, n=7, c=30):
    # shapes of the reference's case (test/test_nested_tensor_class.py:852-856)
    import random
    rnd = random.Random(seed)
    shapes = [(c, rnd.randint(20, 40), rnd.randint(20, 40)) for _ in range(n)]
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=g) for s in shapes]


def test_channels_last_storage_is_torch_channels_last_per_constituent():
    ts = _images()
    nt = oracle.ref_nested_tensor(ts)
    buffer, strides = oracle.to_channels_last(nt)
    off = 0
    for t, st in zip(ts, strides):
        want = t.unsqueeze(0).contiguous(memory_format=torch.channels_last).squeeze(0)
        assert tuple(want.stride()) == st
        got = torch.as_strided(buffer, t.shape, st, off)
        assert torch.equal(got, t) and torch.equal(got, want)
        # the storage order itself: [H, W, C] row-major
        assert torch.equal(buffer[off:off + t.numel()], t.permute(1, 2, 0).reshape(-1))
        off += t.numel()
    assert off == buffer.numel()


def test_channels_last_round_trip():
    ts = _images(seed=3, n=4, c=5)
    nt = oracle.ref_nested_tensor(ts)
    buffer, _ = oracle.to_channels_last(nt)
    back = oracle.from_channels_last(buffer, nt._shapes, nt.dtype)
    assert torch.equal(back.buffer, nt.buffer)
    assert [tuple(t.shape) for t in back.unbind()] == [tuple(t.shape) for t in ts]
    with pytest.raises(RuntimeError, match="requires 4 dim input"):
        oracle.to_channels_last(oracle.ref_nested_tensor([torch.randn(3, 4), torch.randn(2, 4)]))
