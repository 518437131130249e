"""The host planner of the planned attention kernel (nt_attention_plan), checked
without a device: a plan is replayed on the CPU the way the kernel walks it, and
every (head, query row) must meet every key of its sequence exactly once, in key
order, inside the slots its step loads.  The attention of the reference visits
every key of a sequence for every query row of that sequence
(nestedtensor/csrc/mha.cpp:58-65); a plan that drops, repeats or misplaces a
tile would change the softmax."""

import ctypes

import numpy as np
import pytest

from nestedtensor_amd import _C

WAVES = 12
STEP = 16 + 4 * WAVES
HEADER = 4


def build_plan(q_lens, k_lens, heads, n_wg):
    q = np.asarray(q_lens, dtype=np.int64)
    k = np.asarray(k_lens, dtype=np.int64)
    qp = q.ctypes.data_as(ctypes.c_void_p)
    kp = k.ctypes.data_as(ctypes.c_void_p)
    n = _C.lib.nt_attention_plan(qp, kp, len(q), heads, 64, n_wg, None, 0)
    assert n > 0, _C.lib.nt_last_error()
    plan = np.zeros(n, dtype=np.int32)
    m = _C.lib.nt_attention_plan(qp, kp, len(q), heads, 64, n_wg, plan.ctypes.data_as(ctypes.c_void_p), n)
    assert m == n
    return plan


def replay(plan, q_lens, k_lens, heads):
    """Walks the plan like the kernel; returns the busiest workgroup's tile count
    and the total."""
    n_wg, off, n_steps = int(plan[0]), int(plan[1]), int(plan[2])
    assert plan[3] == 64 and off % 4 == 0 and off >= HEADER + n_wg + 1
    first = plan[HEADER:HEADER + n_wg + 1]
    assert first[0] == 0 and first[-1] == n_steps and (np.diff(first) >= 0).all()
    steps = plan[off:off + n_steps * STEP].reshape(n_steps, STEP)
    q_start = np.concatenate([[0], np.cumsum(q_lens)])
    k_start = np.concatenate([[0], np.cumsum(k_lens)])
    seq_of_q = np.repeat(np.arange(len(q_lens)), q_lens)
    done = np.zeros((heads, int(q_start[-1])), dtype=np.int32)
    loads = []
    for wg in range(n_wg):
        state = [None] * WAVES          # per wavefront: (head, q_tok, nq, next key token expected)
        tiles_of_wg = 0
        for s in range(first[wg], first[wg + 1]):
            d = steps[s]
            head = int(d[3])
            assert 0 <= head < heads
            slots = [(int(d[4 * i]), int(d[4 * i + 1]), int(d[4 * i + 2])) for i in range(4)]
            for tok0, nv, last in slots:
                assert 0 <= nv <= 64
                if nv:
                    assert tok0 + nv - 1 <= last and (nv == 64 or tok0 + nv - 1 == last)
            busiest = 0
            per_wave = [0] * WAVES
            for w in range(WAVES):
                q_tok, nq, bits, n_last = (int(v) for v in d[16 + 4 * w:20 + 4 * w])
                if nq == 0:
                    assert state[w] is None, "a wavefront went idle in the middle of a chain"
                    continue
                slot0, nt = bits & 15, (bits >> 4) & 15
                is_first, is_last = (bits >> 8) & 1, (bits >> 9) & 1
                assert 1 <= nq <= 32 and nt >= 1 and slot0 + nt <= 4
                b = int(seq_of_q[q_tok])
                assert seq_of_q[q_tok + nq - 1] == b, "a query block straddles two sequences"
                if is_first:
                    assert state[w] is None
                    state[w] = (head, q_tok, nq, int(k_start[b]))
                else:
                    assert state[w] is not None and state[w][:3] == (head, q_tok, nq)
                expect = state[w][3]
                for t in range(nt):
                    tok0, nv, last = slots[slot0 + t]
                    assert nv > 0 and tok0 == expect and last == k_start[b + 1] - 1
                    final = t == nt - 1
                    assert nv == (n_last if final else 64)
                    expect += nv
                per_wave[w] = nt
                state[w] = (head, q_tok, nq, expect)
                if is_last:
                    assert expect == k_start[b + 1], "chain ended before the sequence's last key"
                    done[head, q_tok:q_tok + nq] += 1
                    state[w] = None
                else:
                    assert n_last == 64
            busiest = max(sum(per_wave[i::4]) for i in range(4))
            tiles_of_wg += busiest
        assert all(st is None for st in state), "a workgroup's list ends inside a chain"
        loads.append(tiles_of_wg)
    assert (done == 1).all(), "every (head, query row) is finished exactly once"
    return max(loads), sum(loads)


CASES = {
    "c3": (np.random.default_rng(1012).integers(32, 513, 32), 12),
    "c4": (np.clip(np.round(np.random.default_rng(1013).exponential(96.0, 128)), 8, 512).astype(np.int64), 16),
    "tiny": (np.array([1, 2, 31, 32, 33, 63, 64, 65]), 3),
    "boundaries": (np.array([255, 256, 257, 511, 512, 513, 1024, 1025, 96, 128, 129]), 2),
    "one_long": (np.array([4000]), 5),
    "with_empty": (np.array([0, 17, 0, 300, 0]), 4),
}


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("n_wg", [1, 7, 256])
def test_plan_covers_every_key_once(name, n_wg):
    lens, heads = CASES[name]
    plan = build_plan(lens, lens, heads, n_wg)
    replay(plan, lens, lens, heads)


def test_plan_for_cross_attention_lengths():
    q = np.array([5, 300, 64, 0, 129])
    k = np.array([700, 3, 64, 0, 257])
    plan = build_plan(q, k, 4, 16)
    replay(plan, q, k, 4)


def test_plan_balances_the_c3_batch():
    lens, heads = CASES["c3"]
    plan = build_plan(lens, lens, heads, 256)
    worst, total = replay(plan, lens, lens, heads)
    # longest-first dealing: the busiest workgroup is within a third of the mean
    assert worst <= 1.34 * total / 256 + 4


def test_plan_refuses_queries_without_keys_and_other_head_dims():
    q = np.array([4, 4], dtype=np.int64)
    k = np.array([4, 0], dtype=np.int64)
    rc = _C.lib.nt_attention_plan(q.ctypes.data_as(ctypes.c_void_p), k.ctypes.data_as(ctypes.c_void_p), 2, 2, 64,
                                  8, None, 0)
    assert rc < 0 and b"no keys" in _C.lib.nt_last_error()
    rc = _C.lib.nt_attention_plan(q.ctypes.data_as(ctypes.c_void_p), q.ctypes.data_as(ctypes.c_void_p), 2, 2, 128,
                                  8, None, 0)
    assert rc < 0 and b"head_dim" in _C.lib.nt_last_error()


def test_plan_of_an_empty_batch():
    plan = build_plan(np.zeros(0, dtype=np.int64), np.zeros(0, dtype=np.int64), 2, 8)
    assert plan[0] == 8 and plan[2] == 0
