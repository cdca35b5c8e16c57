"""Host-side planning code of the C-ABI library (no GPU): the evaluation schedule (trails of a
layer's wiring), the destinations that dl_backward_schedule_build derives from it for the
one-pass backward, checked by replaying the kernel's walk in numpy, and the neuron order of the
fused count."""
import ctypes

import numpy as np
import pytest

from difflogic_amd import _lib
from oracle import connections as oc


def _schedule(a, b, in_dim):
    lib = _lib.load()
    chunk = lib.dl_eval_schedule_chunk()
    cap = lib.dl_eval_schedule_capacity(len(a), chunk)
    verts = np.empty(cap + 1, np.int32)
    neuron = np.empty(cap, np.int32)
    flip = np.empty(cap, np.uint8)
    steps = lib.dl_eval_schedule_build(a.ctypes.data, b.ctypes.data, in_dim, len(a), chunk, verts.ctypes.data,
                                       neuron.ctypes.data, flip.ctypes.data)
    assert steps >= len(a)
    return verts[:steps + 1].copy(), neuron[:steps].copy(), flip[:steps].copy(), int(steps)


def _plan(verts, neuron, steps, in_dim):
    lib = _lib.load()
    dst = np.empty(steps + 1, np.int32)
    fix_vertex = np.empty(in_dim, np.int32)
    fix_start = np.empty(in_dim + 1, np.int32)
    n_fix = ctypes.c_int64(0)
    rows = lib.dl_backward_schedule_build(verts.ctypes.data, neuron.ctypes.data, steps, in_dim, dst.ctypes.data,
                                          fix_vertex.ctypes.data, fix_start.ctypes.data, ctypes.byref(n_fix))
    assert rows >= 0
    n = int(n_fix.value)
    return dst, fix_vertex[:n], fix_start[:n + 1], int(rows)


def _np(pair):
    return tuple(np.asarray(t, dtype=np.int64) for t in pair)


def _wirings():
    import torch
    torch.manual_seed(11)
    rng = np.random.default_rng(5)
    yield "random_square", 64, *_np(oc.random_connections(64, 64))
    yield "unique_square", 50, *_np(oc.unique_connections(50, 50))
    yield "random_wide", 20, *_np(oc.random_connections(20, 90))
    a = rng.integers(0, 12, 30)
    yield "self_loops_and_unused", 16, a, np.where(rng.random(30) < 0.3, a, rng.integers(0, 12, 30))


@pytest.mark.parametrize("name,in_dim,a,b", list(_wirings()), ids=lambda v: v if isinstance(v, str) else None)
def test_every_input_is_completed_exactly_once(name, in_dim, a, b):
    a = np.ascontiguousarray(a, np.int64)
    b = np.ascontiguousarray(b, np.int64)
    verts, neuron, flip, steps = _schedule(a, b, in_dim)
    dst, fix_vertex, fix_start, rows = _plan(verts, neuron, steps, in_dim)
    # Replay: each neuron n hands one token (n, 'a') to input a[n] and (n, 'b') to input b[n]; position p
    # receives the token of neuron[p-1] for its far end and of neuron[p] for its near end.
    direct = [None] * in_dim
    overflow = [None] * rows
    for p in range(steps + 1):
        tokens = []
        if p > 0 and neuron[p - 1] >= 0:
            n = neuron[p - 1]
            tokens.append((n, "a" if flip[p - 1] else "b"))      # the step's new vertex is `a` when flipped
        if p < steps and neuron[p] >= 0:
            n = neuron[p]
            tokens.append((n, "b" if flip[p] else "a"))          # the step's old vertex is `b` when flipped
        for n, side in tokens:
            assert (a if side == "a" else b)[n] == verts[p]
        if not tokens:
            assert dst[p] == -1
            continue
        if dst[p] < in_dim:
            assert dst[p] == verts[p] and direct[dst[p]] is None
            direct[dst[p]] = tokens
        else:
            assert overflow[dst[p] - in_dim] is None
            overflow[dst[p] - in_dim] = (verts[p], tokens)
    assert all(o is not None for o in overflow)
    got = {v: sorted(t) for v, t in enumerate(direct) if t is not None}
    assert len(set(fix_vertex.tolist())) == len(fix_vertex)
    for i, v in enumerate(fix_vertex):
        assert v not in got
        parts = overflow[fix_start[i]:fix_start[i + 1]]
        assert all(pv == v for pv, _ in parts)
        got[int(v)] = sorted(t for _, ts in parts for t in ts)
    assert fix_start[-1] == rows
    want = {v: [] for v in range(in_dim)}
    for n in range(len(a)):
        want[int(a[n])].append((n, "a"))
        want[int(b[n])].append((n, "b"))
    assert got == {v: sorted(t) for v, t in want.items()}


def test_rejects_out_of_range_vertices():
    lib = _lib.load()
    verts = np.array([0, 7], np.int32)
    neuron = np.array([0], np.int32)
    out = np.empty(4, np.int32)
    n_fix = ctypes.c_int64(0)
    st = lib.dl_backward_schedule_build(verts.ctypes.data, neuron.ctypes.data, 1, 4, out.ctypes.data, out.ctypes.data,
                                        out.ctypes.data, ctypes.byref(n_fix))
    assert st == -_lib.DL_ERR_INVALID_ARGUMENT


@pytest.mark.parametrize("depth", [1, 2])
@pytest.mark.parametrize("rows,mid,out,k", [(40, 60, 60, 3), (16, 30, 20, 10), (9, 5, 7, 7), (100, 200, 500, 10)])
def test_count_order_is_a_class_preserving_permutation_that_gathers_readers(depth, rows, mid, out, k):
    """dl_count_order_build: every class is permuted onto itself, and walking a class in that order
    never needs more distinct input rows per workgroup than the natural order (that is its purpose)."""
    lib = _lib.load()
    rng = np.random.default_rng(rows + out + depth)
    top_in = mid if depth == 2 else rows
    a_top = rng.integers(0, top_in, out).astype(np.int64)
    b_top = rng.integers(0, top_in, out).astype(np.int64)
    a_low = rng.integers(0, rows, mid).astype(np.int64) if depth == 2 else None
    b_low = rng.integers(0, rows, mid).astype(np.int64) if depth == 2 else None
    order = np.full(out, -1, np.int32)
    group = 4
    st = lib.dl_count_order_build(a_top.ctypes.data, b_top.ctypes.data, a_low.ctypes.data if depth == 2 else None,
                                  b_low.ctypes.data if depth == 2 else None, rows, mid if depth == 2 else 0, out, k, group,
                                  order.ctypes.data)
    if out % k:
        assert st == _lib.DL_ERR_NOT_DIVISIBLE
        return
    assert st == 0
    per = out // k
    for c in range(k):
        assert sorted(order[c * per:(c + 1) * per].tolist()) == list(range(c * per, (c + 1) * per))
    if depth == 2:
        leaves = np.stack([a_low[a_top], b_low[a_top], a_low[b_top], b_low[b_top]], 1)
    else:
        leaves = np.stack([a_top, b_top], 1)

    def distinct(seq):
        return sum(len(np.unique(leaves[seq[c * per + g:min(c * per + g + group, (c + 1) * per)]]))
                   for c in range(k) for g in range(0, per, group))
    assert distinct(order) <= distinct(np.arange(out))


def test_count_order_rejects_bad_wiring():
    lib = _lib.load()
    a = np.array([0, 5], np.int64)
    order = np.empty(2, np.int32)
    assert lib.dl_count_order_build(a.ctypes.data, a.ctypes.data, None, None, 4, 0, 2, 1, 4,
                                    order.ctypes.data) == _lib.DL_ERR_INVALID_ARGUMENT


def test_schedules_of_random_multigraphs():
    """Many small random wirings (parallel edges, self loops, isolated inputs): every neuron is
    scheduled exactly once between its two inputs, chunks are whole, and the backward plan gives
    every input its tokens exactly once (the replay of test_every_input_is_completed_exactly_once)."""
    rng = np.random.default_rng(2024)
    for _ in range(300):
        in_dim = int(rng.integers(1, 40))
        out_dim = int(rng.integers(0, 80))
        a = rng.integers(0, in_dim, out_dim).astype(np.int64)
        b = rng.integers(0, in_dim, out_dim).astype(np.int64)
        if out_dim == 0:
            a = np.zeros(1, np.int64)[:0]
            b = a.copy()
        verts, neuron, flip, steps = _schedule(a, b, in_dim) if out_dim else (np.zeros(1, np.int32), np.zeros(0, np.int32),
                                                                             np.zeros(0, np.uint8), 0)
        assert steps % 8 == 0 and steps <= 2 * out_dim + 16
        seen = np.zeros(out_dim, int)
        for s in range(steps):
            n = neuron[s]
            if n < 0:
                continue
            seen[n] += 1
            u, v = verts[s], verts[s + 1]
            assert (a[n], b[n]) == ((v, u) if flip[s] else (u, v))
        assert (seen == 1).all()
        if out_dim:
            test_every_input_is_completed_exactly_once("random", in_dim, a, b)


def test_launch_plan_follows_the_traffic_model():
    """plan_groups / lds_tail choose from modelled bytes and measured rates, not from constants
    fitted to one workload: the plans measured fastest on MI355X for the three packed BASELINE
    configurations come out, and the model prices them within 25 % of the measured times."""
    from difflogic_amd import packbitstensor as pbt
    headline, c2, c4 = [784] + [64000] * 6, [784] + [8000] * 6, [9216] + [256000] * 4
    assert pbt.plan_groups(headline, True, 16384) == [4, 2] and pbt.lds_tail(headline, 16384) == 0
    assert pbt.plan_groups(c4, True, 4096) == [2, 2] and pbt.lds_tail(c4, 4096) == 0
    assert pbt.lds_tail(c2, 16384) == 6                       # the whole narrow net runs resident in LDS
    # measured launch times in ms on MI355X of the groups called on their own (4-layer prefix + 2 layers with the
    # count), gate ids drawn uniformly (a quarter of all gate inputs are ignored by their gate and not fetched) but
    # neither folded nor thinned by what the layers above look at, as they are inside PackBitsTensor
    measured = {"headline": (headline, [4, 2], 16384, 2.18 + 2.20), "C4": (c4, [2, 2], 4096, 2.74 + 2.23)}
    for name, (dims, groups, words, ms) in measured.items():
        model = pbt.plan_cost(dims, groups, True, words) * 1e3
        assert abs(model - ms) <= 0.25 * ms, (name, model, ms)
    assert abs(pbt.lds_cost(c2, 16384) * 1e3 - 0.68) <= 0.25 * 0.68      # from packed words
    # single groups against their measured times: 784 -> 64000 prefixes of depth 2, 3, 4 and square 64000-wide groups
    for depth, ms in ((2, 1.56), (3, 1.68), (4, 2.18)):
        assert abs(pbt.group_cost(784, 64000, depth, 16384, False) * 1e3 - ms) <= 0.25 * ms, depth
    assert abs(pbt.group_cost(64000, 64000, 1, 16384, False) * 1e3 - 2.99) <= 0.25 * 2.99
    assert abs(pbt.group_cost(64000, 64000, 2, 16384, False) * 1e3 - 3.00) <= 0.25 * 3.00
    # the last layers with the count, one and two layers deep
    assert abs(pbt.group_cost(64000, 64000, 1, 16384, True) * 1e3 - 1.82) <= 0.25 * 1.82
    assert abs(pbt.group_cost(64000, 64000, 2, 16384, True) * 1e3 - 2.20) <= 0.25 * 2.20
    # the model scales with the row length: the plan of a 16x shorter batch is the same, its cost 16x lower (up to
    # the per-launch overhead: 6 kernels x 3 us)
    assert pbt.plan_groups(headline, True, 1024) == [4, 2]
    assert abs(pbt.plan_cost(headline, [4, 2], True, 1024) * 16 - pbt.plan_cost(headline, [4, 2], True, 16384)) < 6 * 3e-6 * 16
    # The LDS kernel pays where it takes the WHOLE net from the bool input (C2: 0.78 ms against 0.88 streamed; the
    # model prices both within 25 %).  A narrow END of a wide net does not: staging 8000 packed rows of 128 KB
    # in 16-byte pieces costs more than streaming the last layers (784 -> 64000 -> 32000 -> 16000 -> 3 x 8000,
    # batch 2^20: 0.94 ms streamed, 1.68 ms with the last two layers in LDS).
    taper = [784, 64000, 32000, 16000, 8000, 8000, 8000]
    assert pbt.lds_tail(taper, 16384) == 0 and pbt.lds_tail(taper, 16384, 1.0) == 0
    assert pbt.lds_tail(c2, 16384, from_bool=True) == 6 and pbt.lds_tail(c2, 16384, 1.0, from_bool=True) == 6
    assert abs(pbt.lds_cost(c2, 16384, True) * 1e3 - 0.78) <= 0.25 * 0.78
    assert abs((pbt.plan_cost(c2, pbt.plan_groups(c2, True, 16384), True, 16384) + pbt._STREAM_CALL_SECONDS) * 1e3 + 0.19 - 0.88) <= 0.25 * 0.88
    # where a good part of the gate inputs is ignored the LDS kernel runs the net thinned: 0.61-0.63 ms for shares of
    # 0.5 to 0.75 against 0.74 whole, which also beats streaming for pass-through gates only (0.71 ms)
    assert abs(pbt.lds_cost(c2, 16384, True, 0.75) * 1e3 - 0.62) <= 0.15 * 0.62
    assert pbt.lds_cost(c2, 16384, True, 0.95) == pbt.lds_cost(c2, 16384, True)
    assert pbt.lds_tail(c2, 16384, 0.5, from_bool=True) == 6
    assert pbt.plan_groups([784], True) == []
