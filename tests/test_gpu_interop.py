"""Parity of the interop formats (embedding, embedding_bag, CSR, PackedSequence)
built on the device from the offsets array, against the oracle.  Copies and
integer work are bit-exact; bag sums are fp32 in token order (1e-5 relative)."""

import pytest
import torch

import nestedtensor_amd as nt
import oracle

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda", 0)


def _idx(lens, V, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(V, (L,), generator=g) for L in lens]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("E", [8, 768, 7])
def test_embedding(E, dtype):
    V = 1000
    ids = _idx([5, 1, 131, 64], V, 1)
    w = torch.randn(V, E, generator=torch.Generator().manual_seed(2)).to(dtype)
    a = nt.nested_tensor(ids, device=DEV, dtype=torch.int64)
    emb = torch.nn.Embedding(V, E).to(dtype)
    with torch.no_grad():
        emb.weight.copy_(w)
    got = emb.to(DEV)(a)
    exp = oracle.embedding(w, oracle.ref_nested_tensor(ids, dtype=torch.int64))
    assert got.nested_size() == nt.nested_tensor(list(exp.unbind())).nested_size()
    assert torch.equal(got._impl.buffer.cpu(), exp.buffer)
    got2 = torch.nn.functional.embedding(a, w.to(DEV))
    assert torch.equal(got2._impl.buffer.cpu(), exp.buffer)


def _bad_and_good():
    bad = nt.nested_tensor([torch.tensor([1, 2, 50]), torch.tensor([3, -1])], device=DEV, dtype=torch.int64)
    good = nt.nested_tensor([torch.tensor([1, 2, 5]), torch.tensor([3])], device=DEV, dtype=torch.int64)
    return bad, good, torch.randn(10, 4, device=DEV)


@pytest.mark.parametrize("op", ["embedding", "embedding_bag"])
def test_out_of_range_indices_immediate(op):
    fn = getattr(torch.nn.functional, op)
    bad, good, w = _bad_and_good()
    previous = nt.set_index_check("immediate")
    try:
        with pytest.raises(IndexError, match="2 index value"):
            fn(bad, w)
        fn(good, w)                       # nothing is left over for the next call
        nt.check_index_errors()
    finally:
        nt.set_index_check(previous)


@pytest.mark.parametrize("op", ["embedding", "embedding_bag"])
def test_out_of_range_indices_deferred(op):
    # opt-in: the call itself returns (zero rows for the bad indices, no wait for the
    # device); the count is raised by check_index_errors() or by the next call
    fn = getattr(torch.nn.functional, op)
    bad, good, w = _bad_and_good()
    previous = nt.set_index_check("deferred")
    try:
        _deferred_reports(op, fn, bad, good, w)
    finally:
        nt.set_index_check(previous)


def test_out_of_range_indices_raise_by_default():
    # without any setting a bad index raises from the call that met it, as the
    # reference's host embedding does
    bad, good, w = _bad_and_good()
    with pytest.raises(IndexError, match="2 index value"):
        torch.nn.functional.embedding(bad, w)
    torch.nn.functional.embedding(good, w)
    nt.check_index_errors()


def _deferred_reports(op, fn, bad, good, w):
    nt.check_index_errors()
    out = fn(bad, w)
    dense = out.to_padded_tensor(0) if op == "embedding" else out
    if op == "embedding":
        assert torch.equal(dense[0, 2], torch.zeros(4, device=DEV))       # index 50: a zero row
        assert torch.equal(dense[0, 1], w[2])
    with pytest.raises(IndexError, match="2 index value"):
        nt.check_index_errors()
    nt.check_index_errors()               # reported once
    fn(bad, w)
    torch.cuda.synchronize()
    with pytest.raises(IndexError, match="earlier call"):
        fn(good, w)
    fn(good, w)
    nt.check_index_errors()


def test_out_of_range_indices_off():
    bad, good, w = _bad_and_good()
    previous = nt.set_index_check("off")
    try:
        torch.nn.functional.embedding(bad, w)
        torch.cuda.synchronize()
        nt.check_index_errors()
    finally:
        nt.set_index_check(previous)
    with pytest.raises(ValueError):
        nt.set_index_check("sometimes")


@pytest.mark.parametrize("op", ["embedding", "embedding_bag"])
def test_embedding_ops_under_hip_graph_replays(op):
    # neither op reads anything back from the device, so both can be captured; every
    # replay, with new indices and eager work in between, must equal the eager result
    V, E = 500, 72
    fn = getattr(torch.nn.functional, op)
    kw = dict(mode="sum") if op == "embedding_bag" else {}
    g = torch.Generator().manual_seed(31)
    lens = [17, 1, 300, 64, 5]
    a = nt.nested_tensor([torch.randint(V, (L,), generator=g) for L in lens], device=DEV, dtype=torch.int64)
    w = torch.randn(V, E, generator=g).half().to(DEV)

    def buf(t):
        return t._impl.buffer if op == "embedding" else t

    for _ in range(3):
        fn(a, w, **kw)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn(a, w, **kw)
        with torch.cuda.graph(graph, stream=side):
            out = fn(a, w, **kw)
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(4):
        a._impl.buffer.copy_(torch.randint(V, (sum(lens),), generator=g).to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = buf(out).clone()
        exp = buf(fn(a, w, **kw))
        torch.cuda.synchronize()
        assert torch.equal(got, exp), "replay %d differs from the eager call" % rep
    # an out-of-range index met during a replay (nothing waits inside a graph) is
    # reported by the next check
    a._impl.buffer[3] = V + 7
    graph.replay()
    with pytest.raises(IndexError, match="1 index value"):
        nt.check_index_errors()


@pytest.mark.parametrize("mode", ["sum", "mean", "max"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("E", [8, 7, 776])     # 16-byte column pieces, the scalar path, two column blocks
def test_embedding_bag(mode, dtype, E):
    V = 100
    for lens in ([5, 5], [5, 1, 12, 300], [3] * 70):       # first: the reference's case
        ids = _idx(lens, V, 3)
        w = torch.randn(V, E, generator=torch.Generator().manual_seed(4)).to(dtype)
        a = nt.nested_tensor(ids, device=DEV, dtype=torch.int64)
        bag = torch.nn.EmbeddingBag(V, E, mode=mode).to(dtype)
        with torch.no_grad():
            bag.weight.copy_(w)
        got = bag.to(DEV)(a)
        exp = oracle.embedding_bag(oracle.ref_nested_tensor(ids, dtype=torch.int64), w.float(), mode)
        assert got.shape == (len(lens), E) and got.dtype == dtype
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert (got.float().cpu() - exp).abs().max().item() <= tol * max(1.0, exp.abs().max().item())


def test_embedding_bag_errors():
    a = nt.nested_tensor([torch.tensor([[1, 2]]), torch.tensor([[3, 4]])], device=DEV, dtype=torch.int64)
    with pytest.raises(ValueError, match="input has to be 2D NestedTensor"):
        torch.nn.functional.embedding_bag(a, torch.randn(10, 4, device=DEV))
    a = nt.nested_tensor([torch.tensor([1, 2]), torch.tensor([3])], device=DEV, dtype=torch.int64)
    with pytest.raises(ValueError, match="if input is 2D, then offsets has to be None"):
        torch.nn.functional.embedding_bag(a, torch.randn(10, 4, device=DEV), offsets=torch.tensor([0, 2]))
    with pytest.raises(ValueError, match="mode has to be one of sum, mean or max"):
        torch.nn.functional.embedding_bag(a, torch.randn(10, 4, device=DEV), mode="prod")


def test_to_sparse_csr():
    # test/test_nested_tensor_class.py:741-752
    a, b, c = torch.arange(3) + 1, torch.arange(4) + 1, torch.arange(2) + 1
    x = nt.nested_tensor([a, b, c], device=DEV, dtype=torch.int64)
    st = x.to_sparse_csr_tensor()
    assert torch.equal(st.to_dense(), x.to_padded_tensor(padding=0))
    ref = oracle.to_sparse_csr(oracle.ref_nested_tensor([a, b, c], dtype=torch.int64))
    assert torch.equal(st.crow_indices().cpu(), ref.crow_indices())
    assert torch.equal(st.col_indices().cpu(), ref.col_indices())
    assert torch.equal(st.values().cpu(), ref.values())
    y = nt.nested_tensor([a.unsqueeze(1), b.unsqueeze(1)], device=DEV, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="Given tensor must be of dimension 2, got dimension 3"):
        y.to_sparse_csr_tensor()
    # long rows: more than one block per row
    g = torch.Generator().manual_seed(5)
    ts = [torch.randn(L, generator=g) for L in (5000, 1, 70000)]
    z = nt.nested_tensor(ts, device=DEV)
    ref = oracle.to_sparse_csr(oracle.ref_nested_tensor(ts))
    st = z.to_sparse_csr_tensor()
    assert torch.equal(st.col_indices().cpu(), ref.col_indices())
    assert torch.equal(st.crow_indices().cpu(), ref.crow_indices())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_to_packed_sequence(dtype):
    g = torch.Generator().manual_seed(6)
    for lens, E in (((4, 7, 1, 7, 2), 3), ((33, 512, 32, 100, 512, 77), 768)):
        ts = [torch.randn(L, E, generator=g).to(dtype) for L in lens]
        a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
        ps = a.to_packed_sequence()
        ref = oracle.to_packed_sequence(oracle.ref_nested_tensor(ts, dtype=dtype))
        assert torch.equal(ps.data.cpu(), ref.data)
        assert torch.equal(ps.batch_sizes, ref.batch_sizes)
        assert torch.equal(ps.sorted_indices.cpu(), ref.sorted_indices)
        assert torch.equal(ps.unsorted_indices.cpu(), ref.unsorted_indices)
        padded, lengths = torch.nn.utils.rnn.pad_packed_sequence(ps, batch_first=True)
        assert torch.equal(padded, a.to_padded_tensor(0))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.int64, torch.uint8])
def test_transpose_nchw_nhwc_round_trip(dtype):
    # test/test_nested_tensor_class.py:820-840: 20 images [32, H, W], H, W in [20, 100]
    import random
    random.seed(1010)
    shapes = [(32, random.randint(20, 100), random.randint(20, 100)) for _ in range(20)] + [(32, 1, 1), (32, 129, 3)]
    g = torch.Generator().manual_seed(7)
    ts = [(torch.randn(*s, generator=g) * 50).to(dtype) for s in shapes]
    a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
    ref = oracle.ref_nested_tensor(ts, dtype=dtype)
    a0 = nt.transpose_nchw_nhwc(a)
    e0 = oracle.transpose_nchw_nhwc(ref)
    assert a0.nested_size() == nt.nested_tensor(list(e0.unbind())).nested_size()
    assert torch.equal(a0._impl.buffer.cpu(), e0.buffer)
    a2 = nt.transpose_nhwc_nchw(a0)
    assert a2.nested_size() == a.nested_size()
    assert torch.equal(a2._impl.buffer, a._impl.buffer)


def test_transpose_errors_and_irregular_channels():
    a = nt.nested_tensor([torch.randn(2, 3, 3), torch.randn(3, 3, 3)], device=DEV)
    with pytest.raises(RuntimeError, match="Expected first dimension to be regular."):
        nt.transpose_nchw_nhwc(a)
    with pytest.raises(RuntimeError, match="transpose_nchw_nhwc needs 4d input."):
        nt.transpose_nchw_nhwc(nt.nested_tensor([torch.randn(2, 3)], device=DEV))


@pytest.mark.parametrize("dtype", [torch.uint8, torch.float16, torch.float32, torch.int64])
def test_transpose_ragged_every_tile_shape(dtype):
    """nt_transpose_ragged through the C ABI with each tile shape it accepts, on
    matrices whose extents are not multiples of any of them (one is a single
    row, one a single column)."""
    from nestedtensor_amd import _C
    from nestedtensor_amd.impl import device_offsets
    shapes = [(1, 300), (300, 1), (64, 257), (130, 67), (255, 129), (7, 5)]
    g = torch.Generator().manual_seed(21)
    mats = [torch.randint(0, 200, s, generator=g).to(dtype) for s in shapes]
    buf = torch.cat([m.reshape(-1) for m in mats]).to(DEV)
    exp = torch.cat([m.t().contiguous().reshape(-1) for m in mats])
    B = len(shapes)
    rows = torch.tensor([s[0] for s in shapes], dtype=torch.int64)
    cols = torch.tensor([s[1] for s in shapes], dtype=torch.int64)
    offsets = device_offsets(torch.stack([rows, cols], 1).contiguous().to(DEV), B, 2)
    eb = buf.element_size()
    stream = _C.current_stream(DEV)
    rows_d, cols_d = rows.to(DEV), cols.to(DEV)
    for tr, tc in ((64, 64), (64, 128), (128, 64), (128, 128), (64, 256), (256, 64)):
        tiles = ((rows + tr - 1) // tr) * ((cols + tc - 1) // tc)
        toff = torch.zeros(B + 1, dtype=torch.int64)
        toff[1:] = torch.cumsum(tiles, 0)
        toff_d = toff.to(DEV)
        out = torch.full_like(buf, 201 if dtype != torch.uint8 else 255)
        rc = _C.lib.nt_transpose_ragged(_C.ptr(buf), _C.ptr(out), _C.ptr(offsets), _C.ptr(rows_d),
                                        _C.ptr(cols_d), _C.ptr(toff_d), B, int(toff[B]), tr, tc, eb, stream)
        if tr * tc * eb > 32768:
            assert rc != 0 and b"tile" in _C.lib.nt_last_error()
            continue
        assert rc == 0, _C.lib.nt_last_error()
        assert torch.equal(out.cpu(), exp), (tr, tc)
    rc = _C.lib.nt_transpose_ragged(_C.ptr(buf), _C.ptr(out), _C.ptr(offsets), _C.ptr(rows_d),
                                    _C.ptr(cols_d), _C.ptr(toff_d), B, 1, 32, 64, eb, stream)
    assert rc != 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.int16])
@pytest.mark.parametrize("first", [(64, 7, 9), (64, 1, 1)])
def test_transpose_two_byte_elements_with_whole_line_rows(dtype, first):
    """Two-byte elements take a kernel of their own, which stores whole cache lines
    where every output row is a multiple of 64 elements in a constituent that starts
    on a line (64 and 256 channels, NCHW -> NHWC) and ordinary pieces elsewhere: both
    store paths in one batch, in both directions (transpose.cpp:122-204)."""
    g = torch.Generator().manual_seed(31)
    for ch in (64, 256, 192, 72):
        shapes = [(ch,) + first[1:], (ch, 33, 65), (ch, 64, 64), (ch, 100, 3), (ch, 5, 129)]
        ts = [torch.randint(-300, 300, s, generator=g).to(dtype) for s in shapes]
        a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
        ref = oracle.ref_nested_tensor(ts, dtype=dtype)
        a0 = nt.transpose_nchw_nhwc(a)
        e0 = oracle.transpose_nchw_nhwc(ref)
        assert torch.equal(a0._impl.buffer.cpu().view(torch.int16), e0.buffer.view(torch.int16)), ch
        a2 = nt.transpose_nhwc_nchw(a0)
        assert torch.equal(a2._impl.buffer.view(torch.int16), a._impl.buffer.view(torch.int16)), ch


@pytest.mark.parametrize("shift", [0, 1, 37])
def test_transpose_ragged_lines_through_the_c_abi(shift):
    """nt_transpose_ragged_lines (every output row written as whole 128-byte lines
    from its own window) on matrices whose extents are multiples of nothing, one
    with a single row and one with a single column, with the output buffer starting
    `shift` elements into an allocation so that the lines' phase moves."""
    from nestedtensor_amd import _C
    from nestedtensor_amd.impl import device_offsets
    shapes = [(1, 300), (300, 1), (64, 257), (130, 67), (255, 129), (7, 5), (1000, 64), (513, 100)]
    g = torch.Generator().manual_seed(23)
    mats = [torch.randint(-300, 300, s, generator=g).to(torch.int16) for s in shapes]
    buf = torch.cat([m.reshape(-1) for m in mats]).to(DEV)
    exp = torch.cat([m.t().contiguous().reshape(-1) for m in mats])
    B = len(shapes)
    rows = torch.tensor([s[0] for s in shapes], dtype=torch.int64)
    cols = torch.tensor([s[1] for s in shapes], dtype=torch.int64)
    offsets = device_offsets(torch.stack([rows, cols], 1).contiguous().to(DEV), B, 2)
    tiles = ((rows + 63) // 64 + 1) * ((cols + 63) // 64)
    toff = torch.zeros(B + 1, dtype=torch.int64)
    toff[1:] = torch.cumsum(tiles, 0)
    store = torch.full((buf.numel() + shift + 64,), 777, dtype=torch.int16, device=DEV)
    out = store[shift:shift + buf.numel()]
    rows_d, cols_d, toff_d = rows.to(DEV), cols.to(DEV), toff.to(DEV)      # alive until the kernels have run
    rc = _C.lib.nt_transpose_ragged_lines(_C.ptr(buf), _C.ptr(out), _C.ptr(offsets), _C.ptr(rows_d),
                                          _C.ptr(cols_d), _C.ptr(toff_d), B, int(toff[B]), 2,
                                          _C.current_stream(DEV))
    assert rc == 0, _C.lib.nt_last_error()
    assert torch.equal(out.cpu(), exp)
    # nothing outside the output was touched
    assert bool((store[:shift] == 777).all()) and bool((store[shift + buf.numel():] == 777).all())
    rc = _C.lib.nt_transpose_ragged_lines(_C.ptr(buf), _C.ptr(out), _C.ptr(offsets), _C.ptr(rows_d),
                                          _C.ptr(cols_d), _C.ptr(toff_d), B, int(toff[B]), 4,
                                          _C.current_stream(DEV))
    assert rc != 0 and b"2-byte" in _C.lib.nt_last_error()


@pytest.mark.parametrize("dtype", [torch.uint8, torch.float16, torch.float32, torch.int64])
@pytest.mark.parametrize("narrow", [1, 3, 4, 7, 16])
def test_transpose_ragged_strips(dtype, narrow):
    """Images of a few channels take the strip kernels in both directions; the
    long sides straddle one, two and many strips."""
    strip = 2048 // torch.empty(0, dtype=dtype).element_size()
    longs = [1, 65, strip - 1, strip, strip + 1, 2 * strip + 13, 5 * strip + 7]
    g = torch.Generator().manual_seed(22)
    for shapes in ([(narrow, n, 1) for n in longs], ):
        ts = [torch.randint(0, 200, s, generator=g).to(dtype) for s in shapes]
        a = nt.nested_tensor(ts, device=DEV, dtype=dtype)
        from nestedtensor_amd import ops
        assert ops._transpose_tile(narrow, max(longs), a.element_size()) == (16, strip)
        assert ops._transpose_tile(max(longs), narrow, a.element_size()) == (strip, 16)
        fwd = nt.transpose_nchw_nhwc(a)
        exp = oracle.transpose_nchw_nhwc(oracle.ref_nested_tensor(ts, dtype=dtype))
        assert torch.equal(fwd._impl.buffer.cpu(), exp.buffer)
        back = nt.transpose_nhwc_nchw(fwd)
        assert torch.equal(back._impl.buffer, a._impl.buffer)
