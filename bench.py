#!/usr/bin/env python3
"""Benchmark of the ragged hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass over the headline configuration C5: 4096 fp16 constituents
[L_i, 4096], L_i uniform in [1, 2048] (1.7e10 elements, 34 GB packed), padded to
the chunk maximum in chunks of 512 constituents (nt_add_padding) and un-padded
again (nt_remove_padding).  All data is generated on the device and is resident
in HBM before the timed region.  `value` is the algorithmic bytes of the whole
step (pad: valid read + padded written; un-pad: valid read + valid written)
divided by the step time.

The LAST line of the output is the headline JSON record.  It carries
  roofline     - the dominant kernel (row_kernel<2, pad>): algorithmic bytes per
                 launch / mean launch time from HIP events, against 8 TB/s; and in
                 roofline.mha the second half of the metric: the C3 attention
                 layer's tokens/s and fraction of the dense fp16 MFMA peak;
  cpu_baseline - the CPU oracle (the reference's CPU algorithm restated) timed on
                 a bounded sample of the same workload on the host cores (and in
                 cpu_baseline.mha the oracle's attention layer on the C3 batch);
  mha          - the C3 leg in full: per-kernel times, the same layer from a HIP
                 graph, the whole encoder layer, and the reference benchmark's own
                 comparison, torch's dense nn.MultiheadAttention on the padded batch.
A line before it, {"rows": ...}, holds the remaining rows of the path
(to_tensor_mask, to_mask, nested_tensor_from_tensor_mask / _from_padded_tensor,
pack, the offsets scan, C4 attention, ...) on configurations C1, C2 and C4.

Every row is the median over timed batches of calls, with the slowest batch
and the mean beside it.  All device legs run first; what the CPU oracle times
runs after the last of them.  Two more modes issue dispatches for profiler runs
and print only the sizes the counters are to be set against:
  --pmc-probe  a plain copy of known size, then one pad and one un-pad launch;
  --mha-probe  the kernels of the C3 and C4 attention layers and the vendor GEMM
               on C3's projection shapes.
"""

import argparse
import contextlib
import ctypes
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, GB/s
# HBM bytes per launch / algorithmic bytes per launch of the pad kernel, from the
# rocprofv3 FETCH_SIZE and WRITE_SIZE runs of `bench.py --pmc-probe`, each scaled
# by what the same counter reads for a 4 GiB plain copy (FETCH_SIZE: 2.0 KiB per
# unit, WRITE_SIZE: 1.0 KiB per unit).
PAD_TRAFFIC_RATIO = 1.0001
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16, TFLOP/s
MFMA_F32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix, TFLOP/s

METRIC = "ragged->padded HBM GB/s + nested BERT MHA tokens/s (B=32, L<=512, d=768)"


@contextlib.contextmanager
def _no_gc(collect=True):
    """Timed regions run with Python's cyclic collector off (and collected just
    before, unless the caller has done that ahead of its warm-up).  A full
    collection walks every tracked object of the interpreter, about 40 ms with
    torch imported, and starts whenever the allocation counters say so: inside a
    loop of 20-microsecond calls it is a stall of two thousand calls' worth that
    has nothing to do with the call being timed."""
    was = gc.isenabled()
    if collect:
        gc.collect()
    gc.disable()
    try:
        yield
    finally:
        if was:
            gc.enable()


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--chunk", type=int, default=512, help="constituents per chunk")
    ap.add_argument("--batch", type=int, default=4096, help="constituents in total (C5: 4096)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-mha", action="store_true", help="skip the C3 attention leg")
    ap.add_argument("--no-rows", action="store_true", help="skip the per-row measurements (C1, C2, C4)")
    ap.add_argument("--no-encoder", action="store_true",
                    help="skip the whole-encoder-layer figure of the attention leg (so that a kernel "
                         "trace of that leg holds the three kernels of the attention layer only)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="one plain copy of known size, then one pad and one un-pad launch of the "
                         "first C5 chunk; meant to run under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--mha-probe", action="store_true",
                    help="the kernels of the C3 fp16 and C4 bf16 attention layers, each layer issued twice "
                         "(the second pass with warm caches), then the vendor GEMM (torch.addmm) on the two "
                         "C3 projection shapes; meant to run under rocprofv3 --kernel-trace or --pmc")
    return ap.parse_args()


def build_c5(torch, nt_impl, dev, batch, chunk):
    """Lengths on the host (seeded), values on the device, chunk by chunk."""
    g = torch.Generator().manual_seed(1010 + 4)
    lengths = torch.randint(1, 2049, (batch,), generator=g)
    E = 4096
    total_rows = int(lengths.sum())
    packed = torch.empty(total_rows * E, dtype=torch.float16, device=dev)
    torch.manual_seed(1010 + 4)
    chunks = []
    row0 = 0
    for c0 in range(0, batch, chunk):
        ls = lengths[c0:c0 + chunk]
        rows = int(ls.sum())
        view = packed[row0 * E:(row0 + rows) * E]
        # N(0,1) values, generated in place in slabs to bound temporaries
        slab = 1 << 28
        for s in range(0, view.numel(), slab):
            view[s:s + slab].normal_()
        sizes = torch.stack([ls, torch.full_like(ls, E)], 1).contiguous()
        impl = nt_impl(view, sizes)
        chunks.append(impl)
        row0 += rows
    return lengths, packed, chunks


def bench_c5(args, torch, dev):
    from nestedtensor_amd import _C
    from nestedtensor_amd.impl import NestedTensorImpl

    lengths, packed, chunks = build_c5(torch, NestedTensorImpl, dev, args.batch, args.chunk)
    E, eb = 4096, 2
    max_padded = max(c.B * c.max_sizes()[0] * E for c in chunks)
    max_valid = max(c.numel() for c in chunks)
    padded_buf = torch.empty(max_padded, dtype=torch.float16, device=dev)
    unpacked_buf = torch.empty(max_valid, dtype=torch.float16, device=dev)
    stream = _C.current_stream(dev)

    meta = []
    for c in chunks:
        ext = c.max_sizes()
        meta.append(dict(impl=c, ext=_C.i64_array(ext), offsets=c.offsets_dev(), sizes=c.sizes_dev(),
                         valid_bytes=c.numel() * eb, padded_bytes=c.B * ext[0] * E * eb))
    torch.cuda.synchronize()

    def pad(m):
        _C.check(_C.lib.nt_add_padding(_C.ptr(m["impl"].buffer), _C.ptr(padded_buf), _C.ptr(m["offsets"]),
                                       _C.ptr(m["sizes"]), m["impl"].B, 2, 1, m["ext"], eb, 0, stream))

    def unpad(m):
        _C.check(_C.lib.nt_remove_padding(_C.ptr(padded_buf), _C.ptr(unpacked_buf), _C.ptr(m["offsets"]),
                                          _C.ptr(m["sizes"]), m["impl"].B, 2, 1, m["ext"], eb, stream))

    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(len(meta) * args.steps)]
    step_start = torch.cuda.Event(enable_timing=True)
    step_end = torch.cuda.Event(enable_timing=True)
    # (the collector runs here, before the warm-up, not between it and the timed steps:
    # its 40 ms would be an idle spell after which the device's clocks start low)
    gc.collect()
    # warm-up, with the size-independent parity property of the full-size run:
    # un-pad(pad(x)) == x bit-exact, and the padding region reads as the pad value
    for w in range(max(args.warmup, 1)):
        for m in meta:
            pad(m)
            unpad(m)
            if w == 0:
                n = m["impl"].numel()
                assert torch.equal(unpacked_buf[:n].view(torch.int16), m["impl"].buffer.view(torch.int16)), \
                    "round trip is not bit-exact"
                B, L = m["impl"].B, m["impl"].max_sizes()[0]
                pv = padded_buf[:B * L * E].view(B, L, E)
                lens = m["impl"].sizes[:, 0]
                b_short = int(torch.argmin(lens))
                assert bool((pv[b_short, int(lens[b_short]):] == 0).all()), "padding region is not the pad value"
    torch.cuda.synchronize()
    with _no_gc(collect=False):
        t0 = time.perf_counter()
        step_start.record()
        i = 0
        for s in range(args.steps):
            for m in meta:
                e = ev[i]
                e[0].record()
                pad(m)
                e[1].record()
                unpad(m)
                e[2].record()
                i += 1
        step_end.record()
        torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    total_ms = step_start.elapsed_time(step_end)
    ms_per_step = total_ms / args.steps

    pad_ms = [e[0].elapsed_time(e[1]) for e in ev]
    unpad_ms = [e[1].elapsed_time(e[2]) for e in ev]
    pad_bytes = [m["valid_bytes"] + m["padded_bytes"] for m in meta] * args.steps
    unpad_bytes = [2 * m["valid_bytes"] for m in meta] * args.steps
    step_bytes = sum(m["valid_bytes"] + m["padded_bytes"] + 2 * m["valid_bytes"] for m in meta)
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    pad_gbs = sum(pad_bytes) / (sum(pad_ms) * 1e-3) / 1e9
    unpad_gbs = sum(unpad_bytes) / (sum(unpad_ms) * 1e-3) / 1e9
    res = dict(
        value=value, ms_per_step=ms_per_step, wall_ms_per_step=wall_ms / args.steps,
        roofline=dict(bound="hbm", kernel="row_kernel<2, pad> (nt_add_padding)",
                      achieved=pad_gbs, peak=HBM_PEAK_GBS, unit="GB/s", frac=pad_gbs / HBM_PEAK_GBS,
                      traffic=PAD_TRAFFIC_RATIO * sum(pad_bytes) / len(pad_bytes),
                      bytes_per_launch=sum(pad_bytes) / len(pad_bytes),
                      ms_per_launch=sum(pad_ms) / len(pad_ms), launches=len(pad_ms)),
        unpad=dict(kernel="row_kernel<2, unpad> (nt_remove_padding)", achieved=unpad_gbs,
                   peak=HBM_PEAK_GBS, unit="GB/s", frac=unpad_gbs / HBM_PEAK_GBS,
                   bytes_per_launch=sum(unpad_bytes) / len(unpad_bytes),
                   ms_per_launch=sum(unpad_ms) / len(unpad_ms)),
        workload=dict(constituents=int(lengths.numel()), packed_elements=int(lengths.sum()) * E,
                      packed_GB=int(lengths.sum()) * E * eb / 1e9,
                      padded_GB=sum(m["padded_bytes"] for m in meta) / 1e9, chunks=len(meta)))
    del padded_buf, unpacked_buf, packed, chunks, meta
    torch.cuda.empty_cache()
    return res


def pmc_probe(args, torch, dev):
    """Dispatches for hardware-counter runs: a plain device copy of 4 GiB (reads
    4 GiB, writes 4 GiB: the calibration for the counters' unit), one
    nt_add_padding and one nt_remove_padding launch on the first C5 chunk, then
    one launch each of the short-row kernels on C2."""
    from nestedtensor_amd import _C
    from nestedtensor_amd.impl import NestedTensorImpl
    _, packed, chunks = build_c5(torch, NestedTensorImpl, dev, args.chunk, args.chunk)
    m = chunks[0]
    E, eb = 4096, 2
    ext = m.max_sizes()
    padded = torch.empty(m.B * ext[0] * E, dtype=torch.float16, device=dev)
    back = torch.empty(m.numel(), dtype=torch.float16, device=dev)
    src = torch.ones(1 << 31, dtype=torch.float16, device=dev)
    dst = torch.empty_like(src)
    offsets, sizes = m.offsets_dev(), m.sizes_dev()
    stream = _C.current_stream(dev)
    torch.cuda.synchronize()
    dst.copy_(src)
    _C.check(_C.lib.nt_add_padding(_C.ptr(m.buffer), _C.ptr(padded), _C.ptr(offsets), _C.ptr(sizes),
                                   m.B, 2, 1, _C.i64_array(ext), eb, 0, stream))
    _C.check(_C.lib.nt_remove_padding(_C.ptr(padded), _C.ptr(back), _C.ptr(offsets), _C.ptr(sizes),
                                      m.B, 2, 1, _C.i64_array(ext), eb, stream))
    torch.cuda.synchronize()
    assert torch.equal(back.view(torch.int16), m.buffer.view(torch.int16))
    info = {"copy_bytes_read": src.numel() * 2, "copy_bytes_written": src.numel() * 2,
            "pad_valid_bytes": m.numel() * eb, "pad_padded_bytes": padded.numel() * eb,
            "unpad_valid_bytes": m.numel() * eb}
    del src, dst, padded, back, packed, chunks
    # then the short-row kernels on C2 (16 fp32 images [3, H, W]), one launch each through
    # the package: pad, mask, length-based un-pad, pack of device tensors, row counts + un-pad
    import nestedtensor_amd as nt
    g = torch.Generator().manual_seed(1010 + 1)
    hw = torch.randint(480, 1025, (16, 2), generator=g)
    imgs = [torch.rand(3, int(h), int(w), generator=g).to(dev) for h, w in hw]
    a2 = nt.nested_tensor(imgs, device=dev)           # pack
    padded2 = a2.to_padded_tensor(0)                  # pad
    mask2 = torch.ops.nestedtensor.to_mask(a2, 4)     # mask
    back2 = nt.from_padded_tensor(padded2, a2)        # un-pad
    again = nt.nested_tensor_from_tensor_mask(padded2, mask2)   # row counts, un-pad
    torch.cuda.synchronize()
    assert torch.equal(back2._impl.buffer, a2._impl.buffer) and torch.equal(again._impl.buffer, a2._impl.buffer)
    info.update(c2_valid_bytes=a2.numel() * 4, c2_padded_bytes=padded2.numel() * 4, c2_mask_bytes=mask2.numel(),
                c2_launch_order="pack_table_kernel, row_group_kernel<4,0> (pad), mask_plane_kernel, "
                                "row_group_kernel<4,1> (un-pad), row_counts_kernel, row_group_kernel<4,1>")
    print(json.dumps(info))


def mha_probe(args, torch, dev):
    """Dispatches for kernel-trace and hardware-counter runs of the attention
    layers: min_mha on C3 (fp16) twice, torch.addmm (the vendor GEMM) on C3's two
    projection shapes twice, bt_min_mha on C4 (bf16) twice and min_mha on C3 in
    fp32 twice.  Prints the shapes and flop counts the counters are to be set
    against."""
    import nestedtensor_amd as nt
    out = {}
    for tag, seed, B, E, H, dtype in (("C3", 1010 + 2, 32, 768, 12, torch.float16),
                                      ("C4", 1010 + 3, 128, 1024, 16, torch.bfloat16),
                                      ("C3_fp32", 1010 + 2, 32, 768, 12, torch.float32)):
        g = torch.Generator().manual_seed(seed)
        if tag != "C4":
            lens = [int(v) for v in torch.randint(32, 513, (B,), generator=g)]
        else:
            lens = [int(v) for v in torch.empty(B).exponential_(1.0 / 96.0, generator=g).round().clamp(8, 512)]
        xs = [torch.randn(L, E, generator=g).to(dtype) for L in lens]
        W_in = (torch.randn(3 * E, E, generator=g) * 0.02).to(dtype).to(dev)
        W_out = (torch.randn(E, E, generator=g) * 0.02).to(dtype).to(dev)
        b_in, b_out = torch.zeros(3 * E, dtype=dtype, device=dev), torch.zeros(E, dtype=dtype, device=dev)
        a = nt.nested_tensor(xs, device=dev, dtype=dtype)
        op = torch.ops.nestedtensor.bt_min_mha if tag == "C4" else torch.ops.nestedtensor.min_mha
        torch.cuda.synchronize()
        for _ in range(2):
            op(H, 64, 0.0, False, a, a, a, W_in, b_in, 64 ** -0.5, W_out, b_out)
        torch.cuda.synchronize()
        T = sum(lens)
        out[tag] = dict(tokens=T, embed=E, heads=H, sum_L2=sum(L * L for L in lens),
                        flops_in_proj=2 * T * E * 3 * E, flops_out_proj=2 * T * E * E,
                        flops_attention=4 * E * sum(L * L for L in lens))
        if dtype != torch.float32:
            # the same layer with the planned attention kernel (two more dispatches of the
            # projections and two of varlen_attention_planned_kernel), and both timed
            def layer():
                return op(H, 64, 0.0, False, a, a, a, W_in, b_in, 64 ** -0.5, W_out, b_out)
            out[tag]["layer_us_work_list"] = round(_event_us(torch, layer), 2)
            nt.set_attention_kernel("planned")
            try:
                for _ in range(2):
                    layer()
                torch.cuda.synchronize()
                out[tag]["layer_us_planned"] = round(_event_us(torch, layer), 2)
            finally:
                nt.set_attention_kernel("work_list")
            # and the default once more, so that a drift of the clocks between the two
            # measurements above would show
            out[tag]["layer_us_work_list_again"] = round(_event_us(torch, layer), 2)
        if tag == "C3":
            x = a._impl.buffer.reshape(T, E)
            for _ in range(2):
                torch.addmm(b_in, x, W_in.t())
                torch.addmm(b_out, x, W_out.t())
            torch.cuda.synchronize()
            # the in-projection shape at 1x, 2x and 4x the depth, on the whole batch (two
            # rounds of output tiles) and on 4096 rows (192 tiles, 24 per XCD: one round): the
            # differences between depths are the steady-state cost of a K tile, what is
            # left at depth 0 is a tile's fill and drain
            from nestedtensor_amd import ops as _ops
            for rows in (T, 4096):
                for depth in (E, 2 * E, 4 * E):
                    xk = torch.randn(rows, depth, device=dev, dtype=dtype)
                    wk = torch.randn(3 * E, depth, device=dev, dtype=dtype) * 0.02
                    for _ in range(2):
                        _ops.linear(xk, wk, b_in)
                    torch.cuda.synchronize()
            out["gemm_depth_sweep"] = dict(N=3 * E, rows=[T, 4096], depths=[E, 2 * E, 4 * E],
                                           order="rows-major, two dispatches per (rows, depth)")
            # the attention kernel alone on batches of equal-length sequences (random
            # operands in the layout the projection writes): what a key tile costs when
            # sequences are long, and what a workgroup costs when they are short
            import ctypes
            from nestedtensor_amd import _C
            from nestedtensor_amd.impl import NestedTensorImpl
            sweep = []
            for count, length in ((8, 2048), (64, 512), (16, 512), (64, 256), (128, 128), (256, 64)):
                Tn = count * length
                ldvt = (Tn + 72 + 7) // 8 * 8
                qk = torch.randn(Tn, 2 * E, device=dev, dtype=dtype)
                vt = torch.randn(E, ldvt, device=dev, dtype=dtype)
                o = torch.empty(Tn, E, device=dev, dtype=dtype)
                impl = NestedTensorImpl(torch.empty(Tn * E, device=dev, dtype=dtype),
                                        torch.tensor([[length, E]] * count, dtype=torch.int64))
                sched = impl.attention_schedule()
                kptr = ctypes.c_void_p(qk.data_ptr() + E * qk.element_size())
                for _ in range(2):
                    _C.check(_C.lib.nt_varlen_attention_vt(
                        _C.ptr(qk), 2 * E, kptr, 2 * E, _C.ptr(vt), ldvt, _C.ptr(o), E, _C.ptr(sched),
                        sched.size(0), H, 64, Tn, 0.125, _C.dtype_code(dtype), _C.current_stream(dev)))
                torch.cuda.synchronize()
                plan = impl.attention_plan(H, 64)
                n_wg = torch.cuda.get_device_properties(dev).multi_processor_count

                def work_list():
                    _C.check(_C.lib.nt_varlen_attention_vt(
                        _C.ptr(qk), 2 * E, kptr, 2 * E, _C.ptr(vt), ldvt, _C.ptr(o), E, _C.ptr(sched),
                        sched.size(0), H, 64, Tn, 0.125, _C.dtype_code(dtype), _C.current_stream(dev)))

                def planned():
                    _C.check(_C.lib.nt_varlen_attention_planned(
                        _C.ptr(qk), 2 * E, kptr, 2 * E, _C.ptr(vt), ldvt, _C.ptr(o), E, _C.ptr(plan), n_wg,
                        H, 64, Tn, 0.125, _C.dtype_code(dtype), _C.current_stream(dev)))
                for _ in range(2):
                    planned()
                torch.cuda.synchronize()
                q_tiles, k_tiles = (length + 127) // 128, (length + 63) // 64
                sweep.append(dict(sequences=count, length=length, workgroups=count * q_tiles * H,
                                  wavefront_key_tiles=count * q_tiles * 4 * k_tiles * H,
                                  flops=4 * E * count * length * length,
                                  us_work_list=round(_event_us(torch, work_list), 2),
                                  us_planned=round(_event_us(torch, planned), 2)))
            out["attention_length_sweep"] = sweep
    out["instruction_rates"] = instruction_rates()
    # the vendor's GEMM at a size that fills the chip, on operands that do not toggle
    # and on N(0, 1) operands: how far the matrix rate of this part depends on the data
    by_data = {}
    n_big = 8192
    for tag in ("zeros", "normal", "zeros_again"):
        if tag == "normal":
            a = torch.randn(n_big, n_big, device=dev).half()
            b = torch.randn(n_big, n_big, device=dev).half()
        else:
            a = torch.zeros(n_big, n_big, device=dev, dtype=torch.float16)
            b = torch.zeros(n_big, n_big, device=dev, dtype=torch.float16)
        us = _event_us(torch, lambda: torch.mm(a, b), iters=20, warmup=5)
        by_data[tag] = dict(us=round(us, 1), TFLOPs=round(2 * n_big ** 3 / us / 1e6, 1))
        del a, b
    out["vendor_gemm_8192_fp16_by_operand_data"] = by_data
    print(json.dumps(out))


def _event_us(torch, fn, iters=20, warmup=3):
    """Mean time of one call of fn in microseconds, from events on the current
    stream around `iters` back-to-back calls."""
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1000.0 / iters


def instruction_rates():
    """Nanoseconds a SIMD spends per wavefront-wide instruction (every SIMD of the
    chip loaded alike, 1 to 3 wavefronts per SIMD), from libnt_probe.so: the
    transcendental and conversion instructions of the softmax against v_fma_f32,
    the matrix instruction, 16-byte LDS reads, and three mixed streams (16 matrix
    instructions with 128 multiply-adds and / or 32 exponentials per iteration)
    whose time beside the sum of their parts says how much of the vector work
    runs in the shadow of the matrix pipe."""
    path = os.path.join(ROOT, "nestedtensor_amd", "libnt_probe.so")
    if not os.path.exists(path):
        return "libnt_probe.so is not built (make -C nestedtensor_amd/csrc)"
    lib = ctypes.CDLL(path)
    lib.nt_probe_rate.restype = ctypes.c_int
    lib.nt_probe_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float),
                                  ctypes.POINTER(ctypes.c_int)]
    names = ["v_fma_f32", "v_exp_f32", "v_exp_f16", "v_cvt_pk_f16_f32", "v_dot2_f32_f16", "v_max3_f32 (2 x v_max)",
             "v_mfma_f32_32x32x16_f16", "ds_read_b128", "16 mfma + 128 fma (per iteration)",
             "16 mfma + 32 exp (per iteration)", "16 mfma + 128 fma + 32 exp (per iteration)",
             "v_mfma_f32_32x32x16_f16, accumulators in VGPRs",
             "16 mfma + 128 fma + 32 exp (per iteration), accumulators in VGPRs",
             "attention key tile: 8 mfma -> max, 32 exp, pack, sum -> 8 mfma (per tile)",
             "the same with the 16 operand fragments read from LDS (per tile)",
             "the same, and 4 LDS stores and a workgroup barrier per tile",
             "the same, the stored data loaded from global memory during the tile",
             "the same, LDS tiles as rows of 144 bytes read 16 bytes per lane and row",
             "the same, the exponentials behind a wavefront-uniform test of the tile maximum"]
    iters = 2000
    res = {}
    for kind, name in enumerate(names):
        row = {}
        for waves in (1, 2, 3):
            ms, per = ctypes.c_float(), ctypes.c_int()
            rc = lib.nt_probe_rate(kind, waves, iters, ctypes.byref(ms), ctypes.byref(per))
            if rc != 0:
                row["%d_waves_per_simd" % waves] = "probe failed (%d)" % rc
                continue
            # the SIMD runs `waves` wavefronts, each `iters * per` instructions
            row["%d_waves_per_simd" % waves] = round(ms.value * 1e6 / (iters * per.value * waves), 3)
        res[name] = row
    res["unit"] = "ns per instruction (mixed rows: per iteration) and SIMD"
    # the full tile stream on regular operands and on operands with random signs and
    # mantissas: same instructions, different switching activity, and the shader clock
    # the chip held meanwhile (shader-clock counter against the constant 100 MHz one)
    lib.nt_probe_tile_clock.restype = ctypes.c_int
    lib.nt_probe_tile_clock.argtypes = [ctypes.c_uint, ctypes.c_int, ctypes.c_int] + [ctypes.POINTER(ctypes.c_float)] * 3
    clock_iters = 20000   # ~30 ms per launch: long enough for the power management to settle
    tile = {}
    for tag, noise in (("regular_operands", 0), ("random_operands", 12345), ("regular_operands_again", 0)):
        ms, cyc, ticks = ctypes.c_float(), ctypes.c_float(), ctypes.c_float()
        rc = lib.nt_probe_tile_clock(noise, 3, clock_iters, ctypes.byref(ms), ctypes.byref(cyc), ctypes.byref(ticks))
        if rc != 0:
            tile[tag] = "probe failed (%d)" % rc
            continue
        tile[tag] = dict(ns_per_tile_and_simd=round(ms.value * 1e6 / (clock_iters * 3), 1),
                         shader_cycles_per_100mhz_tick=round(cyc.value / max(ticks.value, 1.0), 3))
    res["attention key tile, 3 wavefronts per SIMD, by operand data"] = tile
    return res


def cpu_baseline_c5(torch, n_sample=128):
    """The oracle's to_padded_tensor + from_padded_tensor on the first n_sample
    constituents of C5 (same seeded lengths), timed on the host cores."""
    import oracle
    torch.set_num_threads(_host_threads())
    g = torch.Generator().manual_seed(1010 + 4)
    lengths = torch.randint(1, 2049, (4096,), generator=g)[:n_sample]
    E = 4096
    parts = [torch.randn(int(l), E, generator=g).half() for l in lengths]
    ref = oracle.ref_nested_tensor(parts, dtype=torch.float16)
    valid = ref.buffer.numel() * 2
    padded_bytes = n_sample * int(lengths.max()) * E * 2
    best = None
    for it in range(3):
        t0 = time.perf_counter()
        padded = oracle.to_padded_tensor(ref, 0)
        t1 = time.perf_counter()
        back = oracle.from_padded_tensor(padded, ref)
        t2 = time.perf_counter()
        if it == 0:
            assert torch.equal(back.buffer.view(torch.int16), ref.buffer.view(torch.int16))
        if best is None or (t2 - t0) < best[0]:
            best = (t2 - t0, t1 - t0, t2 - t1)
    step_bytes = valid + padded_bytes + 2 * valid
    return dict(value=step_bytes / best[0] / 1e9, unit="GB/s", cores=torch.get_num_threads(),
                kind="port",
                sample="first %d of 4096 C5 constituents (%.2f GB packed fp16), oracle "
                       "to_padded_tensor + from_padded_tensor, best of 3; pad %.2f GB/s, un-pad %.2f GB/s"
                       % (n_sample, valid / 1e9, (valid + padded_bytes) / best[1] / 1e9,
                          2 * valid / best[2] / 1e9),
                host_cpus=os.cpu_count())


def bench_mha_c3(args, torch, dev, later):
    import nestedtensor_amd as nt
    import oracle
    g = torch.Generator().manual_seed(1010 + 2)
    lens = [int(v) for v in torch.randint(32, 513, (32,), generator=g)]
    E, H, hd = 768, 12, 64
    xs = [torch.randn(L, E, generator=g).half() for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * 0.02).half()
    W_out = (torch.randn(E, E, generator=g) * 0.02).half()
    b_in, b_out = torch.zeros(3 * E).half(), torch.zeros(E).half()
    a = nt.nested_tensor(xs, device=dev, dtype=torch.float16)
    dW_in, db_in, dW_out, db_out = W_in.to(dev), b_in.to(dev), W_out.to(dev), b_out.to(dev)

    def layer():
        return torch.ops.nestedtensor.min_mha(H, hd, 0.0, False, a, a, a, dW_in, db_in, hd ** -0.5,
                                              dW_out, db_out)

    out = layer()
    ms = _time_gpu(torch, layer, iters=50, warmup=5)
    ms_drained = _time_gpu(torch, layer, iters=50, warmup=5, from_idle=True)
    iters = 50
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # the same three launches replayed from a HIP graph (no host work between them)
    graph_ms = None
    try:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            layer()
            with torch.cuda.graph(graph, stream=side):
                gout = layer()
        torch.cuda.current_stream().wait_stream(side)
        graph_ms = float(_time_gpu(torch, graph.replay, iters=iters, warmup=5))
        assert torch.equal(gout._impl.buffer, out._impl.buffer)
    except Exception as exc:      # report, do not hide
        graph_ms = "graph capture failed: %r" % (exc,)
    T = sum(lens)
    flops = 8 * T * E * E + 4 * E * sum(L * L for L in lens)
    # the three launches one by one through the C ABI (each timed as batches of
    # five with an event between batches, like the layer): what each costs when the
    # device has nothing else queued
    kernel_us = _mha_kernel_times(torch, dev, a, dW_in, db_in, dW_out, db_out, H, hd)
    # The reference's own benchmark method (benchmarks/mha_cuda.py:26-83): the same
    # batch, padded to the longest sequence, through torch's dense
    # nn.MultiheadAttention with a key-padding mask on the same GPU.  Context, not a
    # target: the dense layer computes the padded tokens too.
    dense = None
    try:
        mha = torch.nn.MultiheadAttention(E, H, bias=True, batch_first=True, device=dev, dtype=torch.float16)
        with torch.no_grad():
            mha.in_proj_weight.copy_(dW_in)
            mha.in_proj_bias.copy_(db_in)
            mha.out_proj.weight.copy_(dW_out)
            mha.out_proj.bias.copy_(db_out)
        mha.eval()
        Lmax = max(lens)
        x_pad = a.to_padded_tensor(0)
        kpm = torch.arange(Lmax, device=dev)[None, :] >= torch.tensor(lens, device=dev)[:, None]

        def dense_layer():
            with torch.no_grad():
                return mha(x_pad, x_pad, x_pad, key_padding_mask=kpm, need_weights=False)[0]

        y_dense = dense_layer()
        ms_dense = _time_gpu(torch, dense_layer, iters=30, warmup=3)
        got_pad = out.to_padded_tensor(0)
        valid = ~kpm
        dense = dict(what="torch.nn.MultiheadAttention (dense, batch_first, key_padding_mask) on the batch padded to "
                          "[%d, %d, %d], same GPU, fp16" % (len(lens), Lmax, E),
                     ms=float(ms_dense), ms_max=ms_dense.max, speedup=float(ms_dense) / float(ms),
                     padded_tokens=len(lens) * Lmax, valid_tokens=T,
                     max_abs_diff_on_valid_tokens=float((y_dense[valid].float() - got_pad[valid].float()).abs().max()))
        del mha, x_pad, y_dense, got_pad
    except Exception as exc:      # report, do not hide
        dense = "dense comparison failed: %r" % (exc,)
    # the whole encoder layer on the packed layout: attention, residual + layer norm,
    # feed-forward 768 -> 3072 (gelu in the GEMM epilogue) -> 768, residual + layer norm
    from nestedtensor_amd import ops as _ops
    W1 = (torch.randn(4 * E, E, generator=g) * 0.02).half().to(dev)
    W2 = (torch.randn(E, 4 * E, generator=g) * 0.02).half().to(dev)
    b1, b2 = torch.zeros(4 * E, device=dev).half(), torch.zeros(E, device=dev).half()
    ln_w, ln_b = torch.ones(E, device=dev).half(), torch.zeros(E, device=dev).half()

    def encoder_layer():
        y = layer()
        h = _ops.layer_norm(y._impl, (E,), ln_w, ln_b, 1e-5, residual=a._impl)
        f = _ops.linear_nt(h, W1, b1, "gelu")
        o = _ops.linear_nt(f, W2, b2)
        return _ops.layer_norm(o, (E,), ln_w, ln_b, 1e-5, residual=h)

    ms_enc = None if args.no_encoder else _time_gpu(torch, encoder_layer, iters=50, warmup=5)
    enc_graph_ms = None
    if ms_enc is not None:
        # the seven launches replayed from a HIP graph
        try:
            egraph = torch.cuda.CUDAGraph()
            eside = torch.cuda.Stream()
            eside.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(eside):
                encoder_layer()
                with torch.cuda.graph(egraph, stream=eside):
                    encoder_layer()
            torch.cuda.current_stream().wait_stream(eside)
            enc_graph_ms = float(_time_gpu(torch, egraph.replay, iters=50, warmup=5))
        except Exception as exc:      # report, do not hide
            enc_graph_ms = "graph capture failed: %r" % (exc,)
    flops_enc = flops + 16 * T * E * E
    res = dict(workload="C3: nested BERT-base self-attention, fp16, B=32, L~U[32,512], d=768, 12x64",
               tokens=T, ms_per_layer=float(ms), ms_per_layer_max=ms.max, ms_per_layer_mean=ms.mean,
               timing=ms.fields()["timing"] + ", queued behind 30 ms of the same calls",
               ms_per_layer_queue_drained_first=float(ms_drained), ms_per_layer_hip_graph=graph_ms,
               tokens_per_s=T / (ms * 1e-3), flops=flops, kernel_us=kernel_us, dense_padded_torch=dense,
               roofline=dict(bound="mfma", achieved=flops / (ms * 1e-3) / 1e12, peak=MFMA_F16_PEAK_TFLOPS,
                             unit="TFLOP/s", frac=flops / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS))
    if ms_enc is not None:
        res["encoder_layer"] = dict(
            workload="the same batch through a whole BERT-base encoder layer (attention, add + layer norm, "
                     "768-3072-768 feed-forward with gelu, add + layer norm), 7 launches",
            ms_per_layer=float(ms_enc), ms_per_layer_max=ms_enc.max, ms_per_layer_hip_graph=enc_graph_ms,
            tokens_per_s=T / (ms_enc * 1e-3),
            flops=flops_enc, TFLOPs=flops_enc / (ms_enc * 1e-3) / 1e12,
            frac_of_mfma_peak=flops_enc / (ms_enc * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS)
    if not args.no_cpu:
        got = out._impl.buffer.float().cpu()

        def _cpu_layer():
            ref = oracle.ref_nested_tensor(xs, dtype=torch.float16)
            best = None
            for it in range(2):
                t0 = time.perf_counter()
                exp = oracle.min_mha(H, hd, 0.0, False, ref, ref, ref, W_in, b_in, hd ** -0.5, W_out, b_out)
                dt = time.perf_counter() - t0
                best = dt if best is None else min(best, dt)
            err = (got - torch.cat([p.reshape(-1) for p in exp]).float()).abs().max()
            res["max_abs_err_vs_oracle"] = float(err)
            res["cpu_baseline"] = dict(value=T / best, unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                                       sample="full C3 layer, oracle min_mha in fp16 on the host, best of 2")
        later.append(_cpu_layer)
    return res


def _mha_kernel_times(torch, dev, a, W_in, b_in, W_out, b_out, H, hd):
    """Microseconds of each of the three launches of the fused self-attention
    layer (nt_linear_qkv, nt_varlen_attention_vt, nt_linear_act), issued through
    the C ABI on torch's current stream with the operator's own buffers' shapes."""
    from nestedtensor_amd import _C
    impl = a._impl
    E = H * hd
    x = impl.buffer.reshape(-1, E)
    T = x.size(0)
    ldvt = (T + 72 + 63) // 64 * 64
    qk = torch.empty(T, 2 * E, device=dev, dtype=x.dtype)
    vt = torch.zeros(E, ldvt, device=dev, dtype=x.dtype)
    attn = torch.empty(T, E, device=dev, dtype=x.dtype)
    out = torch.empty(T, E, device=dev, dtype=x.dtype)
    sched = impl.attention_schedule()
    stream = _C.current_stream(dev)
    dt = _C.dtype_code(x.dtype)

    def qkv():
        _C.check(_C.lib.nt_linear_qkv(_C.ptr(x), E, _C.ptr(W_in), _C.ptr(b_in), _C.ptr(qk), 2 * E, _C.ptr(vt), ldvt,
                                      T, E, E, dt, stream))

    def attention():
        _C.check(_C.lib.nt_varlen_attention_vt(_C.ptr(qk), 2 * E, ctypes.c_void_p(qk.data_ptr() + 2 * E), 2 * E,
                                               _C.ptr(vt), ldvt, _C.ptr(attn), E, _C.ptr(sched), sched.size(0), H, hd,
                                               T, hd ** -0.5, dt, stream))

    def out_proj():
        _C.check(_C.lib.nt_linear_act(_C.ptr(attn), E, _C.ptr(W_out), _C.ptr(b_out), _C.ptr(out), E, T, E, E, 0, dt,
                                      stream))

    res = {}
    for name, fn in (("qkv_projection", qkv), ("attention", attention), ("out_projection", out_proj)):
        res[name] = float(_time_gpu(torch, fn, iters=50, warmup=5)) * 1e3
    res["sum"] = sum(res.values())
    return res


class Ms(float):
    """Milliseconds per call: the median over timed batches, with the slowest
    batch, the mean and the batch shape beside it.  A one-off stall (a host
    thread descheduled while the device waits for the next launch, an allocator
    growth, a first-use cost) moves `max` and `mean` and leaves the median."""

    def fields(self):
        return dict(ms=float(self), ms_max=self.max, ms_mean=self.mean,
                    timing="median / max / mean over %d batches of %d calls" % (self.batches, self.per))


def _time_gpu(torch, fn, iters=20, warmup=3, per=5, warm_s=0.03, from_idle=False):
    """`iters` calls of fn (rounded up to whole batches of `per`), an event
    between batches.  Events are not put between single calls: an event costs
    the device a few microseconds, which is the size of the smallest rows.
    The untimed calls go on for at least `warm_s` seconds of queued work, and
    the timed batches follow them at once (the collector runs BEFORE the untimed
    calls: its 40 ms are an idle spell for the device): after an idle spell the
    device takes about 15 ms of continuous load to reach the clocks it then
    holds, and a 100 us layer timed over its first fifty calls reads 10 to 15 %
    slower than in a loop that keeps the device busy.  from_idle=True drains the
    queue before the timed batches (the device then starts each call as the
    host issues it)."""
    with _no_gc():
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(per):
            fn()
        torch.cuda.synchronize()
        per_call = max((time.perf_counter() - t0) / per, 1e-6)
        batches = max(3, -(-iters // per))
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(batches + 1)]
        for _ in range(min(int(warm_s / per_call), 4000)):
            fn()
        if from_idle:
            torch.cuda.synchronize()
        ev[0].record()
        for b in range(batches):
            for _ in range(per):
                fn()
            ev[b + 1].record()
        torch.cuda.synchronize()
    t = sorted(ev[b].elapsed_time(ev[b + 1]) / per for b in range(batches))
    mid = batches // 2
    ms = Ms(t[mid] if batches % 2 else 0.5 * (t[mid - 1] + t[mid]))
    ms.max, ms.mean, ms.batches, ms.per = t[-1], ev[0].elapsed_time(ev[batches]) / (batches * per), batches, per
    return ms


def _host_threads():
    """Threads for the CPU legs: the visible cores, at most the 16 a one-GPU box grants."""
    return max(1, min(os.cpu_count() or 1, 16))


def _time_cpu(fn, runs=2):
    best = None
    for _ in range(runs):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return best * 1e3


def bench_rows(args, torch, dev, later):
    """The other rows of the hot path, each on the benchmark configuration that
    exercises it, through the package's Python surface (so allocation of the
    result and, for dense -> nested, the device-to-host copy of the row counts
    are inside the timed region).  GB/s = algorithmic bytes / median time.

    Only device work is timed here.  What the CPU oracle has to time is appended
    to `later` as closures over host copies of the inputs; main() runs them after
    every device leg, so that no host thread pool is busy (or still spinning)
    while a device row is being timed."""
    import nestedtensor_amd as nt
    import oracle
    from nestedtensor_amd import _C
    from nestedtensor_amd import ops as _ops
    from nestedtensor_amd.impl import NestedTensorImpl, device_offsets
    rows = {}
    cpu = not args.no_cpu

    def entry(ms, nbytes, **kw):
        d = ms.fields()
        d.update(GBps=nbytes / (ms * 1e-3) / 1e9, frac_of_hbm_peak=nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                 algorithmic_bytes=nbytes)
        d.update(kw)
        return d

    def cpu_leg(key, fn, runs, nbytes=None):
        """Time fn on the host later and file it under rows[key]."""
        if not cpu:
            return

        def job():
            c_ms = _time_cpu(fn, runs)
            rows[key]["cpu_oracle_ms"] = c_ms
            nb = rows[key]["algorithmic_bytes"] if nbytes is None else nbytes
            rows[key]["cpu_oracle_GBps"] = nb / (c_ms * 1e-3) / 1e9
        later.append(job)

    # ---- C1: 64 fp32 [L_i, 256], round trip ---------------------------------
    g = torch.Generator().manual_seed(1010 + 0)
    lengths = torch.randint(1, 129, (64,), generator=g)
    lengths[0] = 128
    parts = [torch.randn(int(l), 256, generator=g) for l in lengths]
    a = nt.nested_tensor(parts, device=dev)
    ref = oracle.ref_nested_tensor(parts)
    nvalid, npadded = a.numel(), 64 * 128 * 256
    padded = a.to_padded_tensor(-1e30)
    ms_pad = _time_gpu(torch, lambda: a.to_padded_tensor(0), iters=40)
    ms_back = _time_gpu(torch, lambda: nt.nested_tensor_from_padded_tensor(padded, padding=-1e30), iters=40)
    ms_len = _time_gpu(torch, lambda: nt.from_padded_tensor(padded, a), iters=40)
    back = nt.nested_tensor_from_padded_tensor(padded, padding=-1e30)
    assert torch.equal(back._impl.buffer.view(torch.int32).cpu(), ref.buffer.view(torch.int32))
    rows["C1_to_padded_tensor"] = entry(ms_pad, 4 * (nvalid + npadded))
    rows["C1_nested_tensor_from_padded_tensor"] = entry(
        ms_back, 4 * (npadded + 2 * nvalid),
        note="value-based; includes the device-to-host copy of the row counts")
    rows["C1_from_padded_tensor_length_based"] = entry(ms_len, 4 * 2 * nvalid)
    cp = oracle.to_padded_tensor(ref, -1e30)
    cpu_leg("C1_to_padded_tensor", lambda: oracle.to_padded_tensor(ref, 0), 3)
    cpu_leg("C1_from_padded_tensor_length_based", lambda: oracle.from_padded_tensor(cp, ref), 3)
    cpu_leg("C1_nested_tensor_from_padded_tensor",
            lambda: oracle.nt_from_tensor_mask_vectorised(cp, cp != -1e30), 3)

    # ---- C2: 16 fp32 images [3, H_i, W_i] -----------------------------------
    g = torch.Generator().manual_seed(1010 + 1)
    hw = torch.randint(480, 1025, (16, 2), generator=g)
    imgs = [torch.rand(3, int(h), int(w), generator=g) for h, w in hw]
    a2 = nt.nested_tensor(imgs, device=dev)
    nvalid2 = a2.numel()
    mx = a2._impl.max_sizes()
    npadded2 = 16 * mx[0] * mx[1] * mx[2]
    data, mask = a2.to_tensor_mask()
    ms_tm = _time_gpu(torch, lambda: a2.to_tensor_mask())
    ms_m = _time_gpu(torch, lambda: torch.ops.nestedtensor.to_mask(a2, 4))
    ms_fm = _time_gpu(torch, lambda: nt.nested_tensor_from_tensor_mask(data, mask))
    dev_imgs = [p.to(dev) for p in imgs]
    ms_pack = _time_gpu(torch, lambda: nt.nested_tensor(dev_imgs, device=dev))
    back2 = nt.nested_tensor_from_tensor_mask(data, mask)
    assert torch.equal(back2._impl.buffer, a2._impl.buffer)
    rows["C2_to_tensor_mask"] = entry(ms_tm, 4 * (nvalid2 + npadded2) + npadded2)
    rows["C2_to_mask"] = entry(ms_m, npadded2)
    rows["C2_nested_tensor_from_tensor_mask"] = entry(
        ms_fm, npadded2 + 2 * 4 * nvalid2,
        note="includes the device-to-host copy of the row counts; CPU figure is the vectorised "
             "restatement, the reference's literal walk does one host call per mask element")
    rows["C2_nested_tensor_pack_from_device_tensors"] = entry(ms_pack, 2 * 4 * nvalid2)
    # for scale: torch's own device copy of the padded tensor and fill of the mask
    # (a plain copy / fill of the same bytes, no ragged structure)
    data2 = torch.empty_like(data)
    ms_cp = _time_gpu(torch, lambda: data2.copy_(data))
    ms_fill = _time_gpu(torch, lambda: mask.fill_(True))
    rows["C2_plain_copy_of_padded_bytes_torch"] = entry(ms_cp, 2 * 4 * npadded2)
    rows["C2_plain_fill_of_mask_bytes_torch"] = entry(ms_fill, npadded2)
    del data2
    if cpu:
        ref2 = oracle.ref_nested_tensor(imgs)
        dcpu, mcpu = data.cpu(), mask.cpu()
        cpu_leg("C2_to_tensor_mask", lambda: oracle.to_tensor_mask(ref2), 1)
        cpu_leg("C2_nested_tensor_from_tensor_mask", lambda: oracle.nt_from_tensor_mask_vectorised(dcpu, mcpu), 1)
        cpu_leg("C2_to_mask", lambda: oracle.to_mask(ref2, 4), 1)

        def _literal_walk():
            # the reference's own algorithm (one host call per mask element) on every
            # eighth row and column: 1/64 of the elements, the same kind of mask
            d8, m8 = dcpu[:, :, ::8, ::8].contiguous(), mcpu[:, :, ::8, ::8].contiguous()
            t0 = time.perf_counter()
            oracle.nt_from_tensor_mask(d8, m8, 1)
            dt = time.perf_counter() - t0
            rows["C2_nested_tensor_from_tensor_mask"]["cpu_literal_walk"] = dict(
                sample="every eighth row and column of the C2 tensor and mask (1/64 of the elements)",
                mask_elements=int(m8.numel()), ms=dt * 1e3, ns_per_mask_element=dt * 1e9 / m8.numel())
        later.append(_literal_walk)
        cpu_leg("C2_nested_tensor_pack_from_device_tensors", lambda: oracle.ref_nested_tensor(imgs), 1)
    del data, mask, back2, dev_imgs, a2

    # ---- metadata scan --------------------------------------------------------
    sizes = torch.randint(1, 2049, (4096, 2), dtype=torch.int64).to(dev)
    ms_scan = _time_gpu(torch, lambda: device_offsets(sizes, 4096, 2), iters=40)
    rows["offsets_scan_B4096"] = ms_scan.fields()

    # ---- row-wise ops either side of attention: C3 encoder width and a large buffer
    for tag, lens_rw, E_rw in (("C3", [int(v) for v in torch.randint(32, 513, (32,), generator=torch.Generator().manual_seed(1012))], 768),
                               ("large", [2048] * 256, 4096)):
        T_rw = sum(lens_rw)
        buf = torch.randn(T_rw * E_rw, device=dev, dtype=torch.float16)
        sizes_rw = torch.tensor([[L, E_rw] for L in lens_rw], dtype=torch.int64)
        x_rw = NestedTensorImpl(buf, sizes_rw)
        r_rw = NestedTensorImpl(torch.randn_like(buf), sizes_rw)
        w_rw, b_rw = torch.randn(E_rw, device=dev).half(), torch.randn(E_rw, device=dev).half()
        nb = 2 * T_rw * E_rw
        ms_ln = _time_gpu(torch, lambda: _ops.layer_norm(x_rw, (E_rw,), w_rw, b_rw, 1e-5))
        ms_rln = _time_gpu(torch, lambda: _ops.layer_norm(x_rw, (E_rw,), w_rw, b_rw, 1e-5, residual=r_rw))
        ms_add = _time_gpu(torch, lambda: _ops.add(x_rw, r_rw))
        rows[tag + "_layer_norm_fp16"] = entry(ms_ln, 2 * nb, rows=T_rw, width=E_rw)
        rows[tag + "_residual_layer_norm_fp16"] = entry(ms_rln, 3 * nb, rows=T_rw, width=E_rw)
        rows[tag + "_packed_add_fp16"] = entry(ms_add, 3 * nb, rows=T_rw, width=E_rw)
        if cpu and tag == "C3":
            def _split(t, lens_rw=lens_rw, E_rw=E_rw):
                return [p.reshape(L, E_rw) for p, L in zip(t.cpu().split([L * E_rw for L in lens_rw]), lens_rw)]
            ref_rw = oracle.ref_nested_tensor(_split(buf), dtype=torch.float16)
            ref_res = oracle.ref_nested_tensor(_split(r_rw.buffer), dtype=torch.float16)
            w_c, b_c = w_rw.cpu(), b_rw.cpu()
            cpu_leg("C3_layer_norm_fp16", lambda: oracle.layer_norm(ref_rw, (768,), w_c, b_c, 1e-5), 2)
            cpu_leg("C3_packed_add_fp16", lambda: oracle.add(ref_rw, ref_res), 2)
            cpu_leg("C3_residual_layer_norm_fp16",
                    lambda: oracle.layer_norm(oracle.add(ref_rw, ref_res), (768,), w_c, b_c, 1e-5), 2)
        del buf, x_rw, r_rw

    # ---- softmax over the ragged last dim: the [H, L_i, L_i] score blocks of C3 -------
    g = torch.Generator().manual_seed(1010 + 2)
    lens_sm = [int(v) for v in torch.randint(32, 513, (32,), generator=g)]
    sizes_sm = torch.tensor([[12, L, L] for L in lens_sm], dtype=torch.int64)
    buf_sm = torch.randn(int(sizes_sm.prod(1).sum()), device=dev, dtype=torch.float16)
    x_sm = NestedTensorImpl(buf_sm, sizes_sm)
    ms_sm = _time_gpu(torch, lambda: _ops.softmax(x_sm, -1))
    rows["C3_scores_softmax_fp16"] = entry(ms_sm, 2 * 2 * buf_sm.numel(), rows=int((sizes_sm[:, 0] * sizes_sm[:, 1]).sum()),
                                           note="what the fused attention kernel never writes: the per-sequence score blocks")
    if cpu:
        parts_sm = [p.reshape(12, L, L) for p, L in zip(buf_sm.cpu().split([12 * L * L for L in lens_sm]), lens_sm)]
        ref_sm = oracle.ref_nested_tensor(parts_sm, dtype=torch.float16)
        cpu_leg("C3_scores_softmax_fp16", lambda: oracle.softmax(ref_sm, -1), 2)
    del buf_sm, x_sm

    # ---- interop formats built from the offsets array ------------------------------
    g = torch.Generator().manual_seed(1010 + 2)
    lens_io = [int(v) for v in torch.randint(32, 513, (32,), generator=g)]
    V_io, E_io = 30522, 768
    ids_io = [torch.randint(V_io, (L,), generator=g) for L in lens_io]
    table = torch.randn(V_io, E_io, generator=g).half().to(dev)
    a_ids = nt.nested_tensor(ids_io, device=dev, dtype=torch.int64)
    T_io = sum(lens_io)
    # timed as a serving loop would run them: index errors reported later, no wait per call
    previous_check = nt.set_index_check("deferred")
    ms_emb = _time_gpu(torch, lambda: torch.nn.functional.embedding(a_ids, table), iters=40)
    ms_bag = _time_gpu(torch, lambda: torch.nn.functional.embedding_bag(a_ids, table, mode="sum"), iters=40)
    nt.check_index_errors()
    nt.set_index_check(previous_check)
    x_io = torch.nn.functional.embedding(a_ids, table)
    ms_ps = _time_gpu(torch, lambda: x_io.to_packed_sequence())
    rows["C3_embedding_fp16"] = entry(ms_emb, T_io * (8 + 2 * 2 * E_io),
                                      note="out-of-range indices are counted on the device and reported later "
                                           "(deferred index check): no device-to-host read in the call")
    rows["C3_embedding_bag_sum_fp16"] = entry(ms_bag, T_io * (8 + 2 * E_io) + 32 * 2 * E_io,
                                              note="CPU figure on an fp32 table (torch's CPU embedding_bag has no fp16 path)")
    rows["C3_to_packed_sequence_fp16"] = entry(ms_ps, T_io * (8 + 2 * 2 * E_io))
    if cpu:
        ref_ids = oracle.ref_nested_tensor(ids_io, dtype=torch.int64)
        tcpu = table.cpu()
        tcpu32 = tcpu.float()
        ref_x = oracle.ref_nested_tensor([p.cpu() for p in x_io.unbind()], dtype=torch.float16)
        cpu_leg("C3_embedding_fp16", lambda: oracle.embedding(tcpu, ref_ids), 2)
        cpu_leg("C3_embedding_bag_sum_fp16", lambda: oracle.embedding_bag(ref_ids, tcpu32, "sum"), 2)
        cpu_leg("C3_to_packed_sequence_fp16", lambda: oracle.to_packed_sequence(ref_x), 2)
    big_T, big_E = 1 << 20, 1024
    big_idx = torch.randint(V_io, (big_T,), device=dev)
    big_tab = torch.randn(V_io, big_E, device=dev, dtype=torch.float16)
    big_out = torch.empty(big_T, big_E, device=dev, dtype=torch.float16)
    stream = _C.current_stream(dev)
    ms_big = _time_gpu(torch, lambda: _C.check(_C.lib.nt_gather_rows(
        _C.ptr(big_tab), V_io, big_E * 2, _C.ptr(big_idx), _C.ptr(big_out), big_T, None, stream)))
    rows["large_gather_rows_fp16"] = entry(ms_big, big_T * (8 + 2 * 2 * big_E), rows=big_T, width=big_E,
                                           note="2 GiB written; the 62 MB table is re-read from cache")
    del big_idx, big_tab, big_out, table, x_io

    # ---- channels-last ragged images: per-constituent transpose -----------------------
    g = torch.Generator().manual_seed(1010 + 1)
    hw_t = torch.randint(480, 1025, (16, 2), generator=g)
    sizes_t = torch.tensor([[64, int(h), int(w)] for h, w in hw_t], dtype=torch.int64)
    buf_t = torch.randn(int(sizes_t.prod(1).sum()), device=dev, dtype=torch.float16)
    img = NestedTensorImpl(buf_t, sizes_t)
    nhwc = _ops.transpose_nchw_nhwc(img)
    ms_t0 = _time_gpu(torch, lambda: _ops.transpose_nchw_nhwc(img))
    ms_t1 = _time_gpu(torch, lambda: _ops.transpose_nhwc_nchw(nhwc))
    assert torch.equal(_ops.transpose_nhwc_nchw(nhwc).buffer, buf_t)
    rows["C2x64ch_transpose_nchw_nhwc_fp16"] = entry(ms_t0, 2 * 2 * buf_t.numel())
    rows["C2x64ch_transpose_nhwc_nchw_fp16"] = entry(ms_t1, 2 * 2 * buf_t.numel())
    # 1x1 convolution 64 -> 256 channels: row-major input (transpose, GEMM, transpose)
    # against the channels-last storage of the same images (the GEMM alone)
    w11 = (torch.randn(256, 64, 1, 1, device=dev) * 0.1).half()
    img_cl = _ops.contiguous(img, torch.channels_last)
    pix = buf_t.numel() // 64
    ms_c0 = _time_gpu(torch, lambda: _ops.conv2d(img, w11), iters=10)
    ms_c1 = _time_gpu(torch, lambda: _ops.conv2d(img_cl, w11), iters=10)
    conv_bytes = 2 * pix * (64 + 256)
    for key, ms_c in (("C2x64ch_conv2d_1x1_to_256ch_fp16", ms_c0),
                      ("C2x64ch_conv2d_1x1_to_256ch_channels_last_fp16", ms_c1)):
        rows[key] = entry(ms_c, conv_bytes, pixels=pix)
        rows[key]["tflops"] = 2.0 * pix * 64 * 256 / (ms_c * 1e-3) / 1e12
    if cpu:
        # CPU side on the first two images (GB/s does not depend on the count)
        n2 = int(sizes_t[:2].prod(1).sum())
        parts_t = [p.reshape(tuple(int(v) for v in sz)) for p, sz in
                   zip(buf_t[:n2].cpu().split([int(v) for v in sizes_t[:2].prod(1)]), sizes_t[:2])]
        ref_t = oracle.ref_nested_tensor(parts_t, dtype=torch.float16)
        h0, w0 = int(sizes_t[0, 1]), int(sizes_t[0, 2])
        x0 = buf_t[:64 * h0 * w0].reshape(64, h0, w0).float().cpu()
        ref_c = oracle.ref_nested_tensor([x0], dtype=torch.float32)
        w_c11 = w11.float().cpu()

        def _cpu_images():
            ref_nhwc = oracle.transpose_nchw_nhwc(ref_t)
            for key, fn in (("C2x64ch_transpose_nchw_nhwc_fp16", lambda: oracle.transpose_nchw_nhwc(ref_t)),
                            ("C2x64ch_transpose_nhwc_nchw_fp16", lambda: oracle.transpose_nhwc_nchw(ref_nhwc))):
                c_ms = _time_cpu(fn, 2)
                rows[key]["cpu_oracle_GBps"] = 2 * 2 * n2 / (c_ms * 1e-3) / 1e9
                rows[key]["cpu_oracle_sample"] = "first 2 of 16 images, %.1f ms" % c_ms
            c_ms = _time_cpu(lambda: oracle.conv2d(ref_c, w_c11), 1)
            for key in ("C2x64ch_conv2d_1x1_to_256ch_fp16", "C2x64ch_conv2d_1x1_to_256ch_channels_last_fp16"):
                rows[key]["cpu_oracle_tflops"] = 2.0 * h0 * w0 * 64 * 256 / (c_ms * 1e-3) / 1e12
                rows[key]["cpu_oracle_sample"] = "first of 16 images in fp32, %.1f ms" % c_ms
        later.append(_cpu_images)
    del buf_t, img, nhwc, img_cl, w11

    def mha_row(ms, n_tok, flops, **kw):
        d = ms.fields()
        d.update(kw)
        d.update(tokens_per_s=n_tok / (ms * 1e-3), flops=flops, TFLOPs=flops / (ms * 1e-3) / 1e12,
                 frac_of_mfma_peak=flops / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS)
        return d

    # ---- C4: bt_min_mha bf16, high raggedness ---------------------------------
    g = torch.Generator().manual_seed(1010 + 3)
    raw = torch.empty(128).exponential_(1.0 / 96.0, generator=g)
    lens = [int(v) for v in raw.round().clamp(8, 512)]
    E, H = 1024, 16
    xs = [torch.randn(L, E, generator=g).bfloat16() for L in lens]
    W_in = (torch.randn(3 * E, E, generator=g) * 0.02).bfloat16().to(dev)
    W_out = (torch.randn(E, E, generator=g) * 0.02).bfloat16().to(dev)
    b_in, b_out = torch.zeros(3 * E).bfloat16().to(dev), torch.zeros(E).bfloat16().to(dev)
    a4 = nt.nested_tensor(xs, device=dev, dtype=torch.bfloat16)
    ms4 = _time_gpu(torch, lambda: torch.ops.nestedtensor.bt_min_mha(
        H, 64, 0.0, False, a4, a4, a4, W_in, b_in, 64 ** -0.5, W_out, b_out), iters=50, warmup=5)
    T4 = sum(lens)
    rows["C4_bt_min_mha_bf16"] = mha_row(ms4, T4, 8 * T4 * E * E + 4 * E * sum(L * L for L in lens), tokens=T4)

    # ---- C3 in fp32: the reference's own dtype for this test configuration ------------
    g = torch.Generator().manual_seed(1010 + 2)
    lens3 = [int(v) for v in torch.randint(32, 513, (32,), generator=g)]
    E3, H3 = 768, 12
    a3 = nt.nested_tensor([torch.randn(L, E3, generator=g) for L in lens3], device=dev, dtype=torch.float32)
    W3_in = (torch.randn(3 * E3, E3, generator=g) * 0.02).to(dev)
    W3_out = (torch.randn(E3, E3, generator=g) * 0.02).to(dev)
    b3_in, b3_out = torch.zeros(3 * E3, device=dev), torch.zeros(E3, device=dev)
    ms3 = _time_gpu(torch, lambda: torch.ops.nestedtensor.min_mha(
        H3, 64, 0.0, False, a3, a3, a3, W3_in, b3_in, 64 ** -0.5, W3_out, b3_out), iters=20, warmup=3)
    T3 = sum(lens3)
    fl3 = 8 * T3 * E3 * E3 + 4 * E3 * sum(L * L for L in lens3)
    rows["C3_min_mha_fp32"] = mha_row(ms3, T3, fl3, tokens=T3)
    rows["C3_min_mha_fp32"]["frac_of_mfma_peak"] = fl3 / (ms3 * 1e-3) / 1e12 / MFMA_F32_PEAK_TFLOPS
    rows["C3_min_mha_fp32"]["peak"] = "fp32 MFMA, %.1f TFLOP/s" % MFMA_F32_PEAK_TFLOPS
    del a3, W3_in, W3_out

    # ---- a larger layer for scale: 16 sequences of 256..2048 tokens, d = 2048, 16 heads of 128 ----
    g = torch.Generator().manual_seed(1010 + 6)
    El, Hl = 2048, 16
    lens_l = [int(v) for v in torch.randint(256, 2049, (16,), generator=g)]
    bufl = torch.randn(sum(lens_l) * El, device=dev, dtype=torch.float16)
    al = nt.NestedTensor(NestedTensorImpl(bufl, torch.tensor([[L, El] for L in lens_l], dtype=torch.int64)))
    Wl_in = (torch.randn(3 * El, El, device=dev) * 0.02).half()
    Wl_out = (torch.randn(El, El, device=dev) * 0.02).half()
    bl_in, bl_out = torch.zeros(3 * El, device=dev).half(), torch.zeros(El, device=dev).half()
    msl = _time_gpu(torch, lambda: torch.ops.nestedtensor.min_mha(
        Hl, 128, 0.0, False, al, al, al, Wl_in, bl_in, 128 ** -0.5, Wl_out, bl_out), iters=20, warmup=3)
    Tl = sum(lens_l)
    rows["large_min_mha_fp16"] = mha_row(msl, Tl, 8 * Tl * El * El + 4 * El * sum(L * L for L in lens_l),
                                         workload="B=16, L~U[256,2048], d=2048, 16x128", tokens=Tl)
    del bufl, al, Wl_in, Wl_out

    # ---- cross-attention: 100 queries per sequence over ragged memories (decoder-style) ----
    g = torch.Generator().manual_seed(1010 + 5)
    Ex, Hx = 512, 8
    kv_lens = [int(v) for v in torch.randint(256, 1025, (32,), generator=g)]
    qs = [torch.randn(100, Ex, generator=g).half() for _ in kv_lens]
    mems = [torch.randn(L, Ex, generator=g).half() for L in kv_lens]
    Wx_in = (torch.randn(3 * Ex, Ex, generator=g) * 0.03).half()
    Wx_out = (torch.randn(Ex, Ex, generator=g) * 0.03).half()
    bx_in, bx_out = torch.zeros(3 * Ex).half(), torch.zeros(Ex).half()
    aq, am = nt.nested_tensor(qs, device=dev, dtype=torch.float16), nt.nested_tensor(mems, device=dev, dtype=torch.float16)
    xargs = (Wx_in.to(dev), bx_in.to(dev), 64 ** -0.5, Wx_out.to(dev), bx_out.to(dev))
    msx = _time_gpu(torch, lambda: torch.ops.nestedtensor.min_mha(Hx, 64, 0.0, False, aq, am, am, *xargs),
                    iters=50, warmup=5)
    Tq, Tk = 100 * len(kv_lens), sum(kv_lens)
    rows["cross_attention_fp16"] = mha_row(
        msx, Tq, 2 * Ex * Ex * (2 * Tq + 2 * Tk) + 4 * Ex * 100 * Tk,
        workload="B=32, 100 queries per sequence, memory L~U[256,1024], d=512, 8x64",
        query_tokens=Tq, memory_tokens=Tk)
    if cpu:
        got = torch.ops.nestedtensor.min_mha(Hx, 64, 0.0, False, aq, am, am, *xargs)._impl.buffer.float().cpu()

        def _cpu_cross():
            rq, rm = oracle.ref_nested_tensor(qs, dtype=torch.float16), oracle.ref_nested_tensor(mems, dtype=torch.float16)
            t0 = time.perf_counter()
            ref_out = oracle.min_mha(Hx, 64, 0.0, False, rq, rm, rm, Wx_in, bx_in, 64 ** -0.5, Wx_out, bx_out)
            rows["cross_attention_fp16"]["cpu_oracle_ms"] = (time.perf_counter() - t0) * 1e3
            exp = torch.cat([p.reshape(-1) for p in ref_out]).float()
            rows["cross_attention_fp16"]["max_abs_err_vs_oracle"] = float((got - exp).abs().max())
        later.append(_cpu_cross)
    return rows


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported "
              "(the path shards by constituent ranges; nothing here uses a second GPU)." % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)

    if args.pmc_probe:
        pmc_probe(args, torch, dev)
        return
    if args.mha_probe:
        mha_probe(args, torch, dev)
        return
    c5 = bench_c5(args, torch, dev)
    line = {
        "metric": METRIC,
        "value": c5["value"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": c5["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "C5: 4096 fp16 [L_i,4096], L_i~U[1,2048], pad to chunk max in chunks of %d "
                               "+ reverse remove_padding; value = algorithmic GB per step / step time"
                               % args.chunk,
                   **c5["workload"]},
        "roofline": c5["roofline"],
        "unpad": c5["unpad"],
    }
    # every device leg first, then everything the CPU oracle has to time
    later = []
    if not args.no_mha:
        line["mha"] = bench_mha_c3(args, torch, dev, later)
    if not args.no_rows:
        line["rows"] = bench_rows(args, torch, dev, later)
    if not args.no_cpu:
        torch.set_num_threads(_host_threads())
        for job in later:
            job()
        line["cpu_baseline"] = cpu_baseline_c5(torch)
    # The metric has two halves; `value` is the first (C5 pad + un-pad GB/s).  The
    # second, the C3 attention layer, rides inside `roofline` and `cpu_baseline`
    # as well, next to the figures of the first half.
    mha = line.get("mha")
    if isinstance(mha, dict):
        r = mha["roofline"]
        line["roofline"]["mha"] = dict(bound="mfma", achieved=r["achieved"], peak=r["peak"], unit=r["unit"],
                                       frac=r["frac"], ms_per_layer=mha["ms_per_layer"],
                                       tokens_per_s=mha["tokens_per_s"], kernel_us=mha["kernel_us"],
                                       workload=mha["workload"])
        if "cpu_baseline" in mha and "cpu_baseline" in line:
            line["cpu_baseline"]["mha"] = mha["cpu_baseline"]
    # the per-operator rows go out first, on a line of their own; the last line of
    # the output is the headline record
    rows = line.pop("rows", None)
    if rows is not None:
        print(json.dumps({"rows": rows}))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
