"""Temporal most-recent-neighbour sampler: bit-exact against golden vectors
written by the reference's own sampler (tests/golden/make_sampler_golden.py), a
brute-force statement of the rule, and -- where oracle/_ref is present -- the
compiled reference itself on fresh random streams."""
import glob
import importlib.util
import os

import numpy as np
import pytest

from yitu_amd import sampler_core

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "sampler_recent.npz"))
FIELDS = ("row", "col", "eid", "ts", "dts", "nodes")


def _block_arrays(blk):
    return {f: getattr(blk, f)() for f in FIELDS}


@pytest.mark.parametrize("case", range(int(GOLD["n_cases"])))
def test_matches_reference_golden_vectors(case):
    pre = "c%d_" % case
    s = sampler_core.ParallelSampler(GOLD[pre + "indptr"], GOLD[pre + "indices"], GOLD[pre + "eid"],
                                     GOLD[pre + "ts"], 2, 1, 1, [int(GOLD[pre + "fan"])], True,
                                     bool(GOLD[pre + "prop_time"]), 1, 0.0)
    for b in range(int(GOLD[pre + "n_batches"])):
        bp = pre + "b%d_" % b
        s.sample(GOLD[bp + "roots"], GOLD[bp + "root_ts"])
        ret = s.get_ret()
        assert len(ret) == 1
        got = _block_arrays(ret[0])
        for f in FIELDS:
            want = GOLD[bp + f]
            assert got[f].dtype == want.dtype and got[f].shape == want.shape, (case, b, f)
            assert np.array_equal(got[f], want), (case, b, f)
        assert [ret[0].dim_in(), ret[0].dim_out()] == GOLD[bp + "dims"].tolist()


def _bruteforce(indptr, indices, eid, ts, cursor, roots, rts, fan):
    """The rule in plain Python: cursor = running max of 'last edge with ts <= t - 1e-7';
    emit k = cursor, cursor-1, ... while k > max(first, cursor - fan) and ts[k] < t - 1e-7."""
    for n, t in zip(roots, rts):
        thr = np.float32(np.float32(t) - np.float32(1e-7))
        ok = [j for j in range(indptr[n], indptr[n + 1]) if ts[j] <= thr]
        if ok:
            cursor[n] = max(cursor[n], ok[-1])
    row, nodes, eids, dts = [], [], [], []
    for i, (n, t) in enumerate(zip(roots, rts)):
        thr = np.float32(np.float32(t) - np.float32(1e-7))
        e = cursor[n]
        k = e
        while k > max(indptr[n], e - fan):
            if ts[k] < thr:
                row.append(i)
                nodes.append(indices[k])
                eids.append(eid[k])
                dts.append(np.float32(t) - ts[k])
            k -= 1
    return row, nodes, eids, dts


def test_bruteforce_rule_and_shared_cursor():
    rng = np.random.default_rng(5)
    n_nodes, n_edges = 30, 400
    owner = np.sort(rng.integers(0, n_nodes, n_edges))
    indptr = np.searchsorted(owner, np.arange(n_nodes + 1)).astype(np.int32)
    ts = np.concatenate([np.sort(rng.uniform(0, 100, indptr[v + 1] - indptr[v]))
                         for v in range(n_nodes)]).astype(np.float32)
    indices = rng.integers(0, n_nodes, n_edges).astype(np.int32)
    eid = rng.permutation(n_edges).astype(np.int32)
    s = sampler_core.ParallelSampler(indptr, indices, eid, ts, 4, 1, 1, [4], True, False, 1, 0.0)
    cursor = indptr[:-1].copy()
    for lo in (20, 50, 40, 90):  # the third batch looks back in time: cursors must not move back
        roots = rng.integers(0, n_nodes, 25).astype(np.int32)
        roots[3] = roots[7]  # duplicated root with a different time
        rts = rng.uniform(lo, lo + 10, 25).astype(np.float32)
        s.sample(roots, rts)
        blk = s.get_ret()[0]
        row, nodes, eids, dts = _bruteforce(indptr, indices, eid, ts, cursor, roots, rts, 4)
        assert blk.row().tolist() == row
        assert blk.eid().tolist() == eids
        assert blk.nodes().tolist() == roots.tolist() + nodes
        assert np.array_equal(blk.dts()[25:], np.asarray(dts, np.float32))
        assert np.all(blk.dts()[:25] == 0)
        assert blk.col().tolist() == list(range(25, 25 + len(row)))
    s.reset()
    s.sample(np.asarray([0], np.int32), np.asarray([1000.0], np.float32))
    first = s.get_ret()[0]
    assert first.dim_out() == 1 and len(first.row()) == min(4, max(0, indptr[1] - indptr[0] - 1))


def test_edge_cases():
    indptr = np.asarray([0, 0, 1, 4], np.int32)  # node 0 empty, node 1 one edge, node 2 three
    indices = np.asarray([2, 0, 1, 1], np.int32)
    eid = np.asarray([10, 11, 12, 13], np.int32)
    ts = np.asarray([5.0, 1.0, 2.0, 3.0], np.float32)
    s = sampler_core.ParallelSampler(indptr, indices, eid, ts, 1, 1, 1, [10], True, False, 1, 0.0)
    s.sample(np.zeros(0, np.int32), np.zeros(0, np.float32))
    assert s.get_ret()[0].dim_in() == 0 and s.get_ret()[0].dim_out() == 0
    s.sample(np.asarray([0, 1, 2], np.int32), np.asarray([9.0, 9.0, 9.0], np.float32))
    blk = s.get_ret()[0]
    # a node's first edge is never emitted (strict k > first): node 1 yields nothing
    assert blk.row().tolist() == [2, 2] and blk.eid().tolist() == [13, 12]
    with pytest.raises(RuntimeError):
        s.sample(np.asarray([3], np.int32), np.asarray([1.0], np.float32))
    with pytest.raises(ValueError):
        sampler_core.ParallelSampler(indptr, indices, eid, ts, 1, 1, 1, [10], True, False, 0, 0.0)


def test_two_layers_expand_previous_block():
    rng = np.random.default_rng(2)
    n_nodes, n_edges = 20, 300
    owner = np.sort(rng.integers(0, n_nodes, n_edges))
    indptr = np.searchsorted(owner, np.arange(n_nodes + 1)).astype(np.int32)
    ts = np.concatenate([np.sort(rng.uniform(0, 100, indptr[v + 1] - indptr[v]))
                         for v in range(n_nodes)]).astype(np.float32)
    indices = rng.integers(0, n_nodes, n_edges).astype(np.int32)
    eid = np.arange(n_edges, dtype=np.int32)
    s = sampler_core.ParallelSampler(indptr, indices, eid, ts, 2, 1, 2, [3, 2], True, False, 1, 0.0)
    s.sample(np.asarray([1, 2, 3], np.int32), np.asarray([80.0, 85.0, 90.0], np.float32))
    b0, b1 = s.get_ret()
    assert b1.dim_out() == b0.dim_in()
    assert b1.nodes()[:b0.dim_in()].tolist() == b0.nodes().tolist()


def _load_ref():
    hits = glob.glob(os.path.join(ROOT, "oracle", "_ref", "sampler_core*.so"))
    if not hits:
        return None
    spec = importlib.util.spec_from_file_location("sampler_core", hits[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("seed", range(3))
def test_against_compiled_reference_live(seed):
    ref = _load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    rng = np.random.default_rng(100 + seed)
    n_nodes, n_edges = 500, 20000
    owner = np.sort((rng.zipf(1.3, n_edges) - 1) % n_nodes)
    indptr = np.searchsorted(owner, np.arange(n_nodes + 1)).astype(np.int32)
    ts = np.concatenate([np.sort(rng.uniform(0, 1e6, indptr[v + 1] - indptr[v]))
                         for v in range(n_nodes)]).astype(np.float32)
    indices = rng.integers(0, n_nodes, n_edges).astype(np.int32)
    eid = rng.permutation(n_edges).astype(np.int32)
    fan = [5, 20, 1][seed]
    mine = sampler_core.ParallelSampler(indptr, indices, eid, ts, 3, 1, 1, [fan], True, False, 1, 0.0)
    theirs = ref.ParallelSampler(indptr.tolist(), indices.tolist(), eid.tolist(), ts.tolist(), 3, 1,
                                 1, [fan], True, False, 1, 0.0)
    for b in range(6):
        roots = ((rng.zipf(1.3, 200) - 1) % n_nodes).astype(np.int32)
        rts = np.sort(rng.uniform(b * 1.5e5, (b + 1) * 1.5e5 + 1e5, 200)).astype(np.float32)
        mine.sample(roots, rts)
        theirs.sample(roots.tolist(), rts.tolist())
        g, w = mine.get_ret()[0], theirs.get_ret()[0]
        for f in FIELDS:
            assert np.array_equal(getattr(g, f)(), np.asarray(getattr(w, f)())), (seed, b, f)
        assert (g.dim_in(), g.dim_out()) == (w.dim_in(), w.dim_out())


@pytest.mark.parametrize("threads,layers,fans,recent,prop_time,hist,window", [
    (4, 1, [6], False, False, 1, 0.0),
    (3, 2, [4, 3], False, False, 1, 0.0),
    (2, 1, [5], True, False, 3, 5e4),
    (7, 2, [3, 3], False, False, 2, 8e4),
])
def test_other_modes_against_compiled_reference_live(threads, layers, fans, recent, prop_time,
                                                     hist, window):
    ref = _load_ref()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    rng = np.random.default_rng(7 * threads + layers)
    n_nodes, n_edges = 300, 12000
    owner = np.sort((rng.zipf(1.3, n_edges) - 1) % n_nodes)
    indptr = np.searchsorted(owner, np.arange(n_nodes + 1)).astype(np.int32)
    ts = np.concatenate([np.sort(rng.uniform(0, 1e6, indptr[v + 1] - indptr[v]))
                         for v in range(n_nodes)]).astype(np.float32)
    indices = rng.integers(0, n_nodes, n_edges).astype(np.int32)
    eid = rng.permutation(n_edges).astype(np.int32)
    mine = sampler_core.ParallelSampler(indptr, indices, eid, ts, threads, 1, layers, fans, recent,
                                        prop_time, hist, window)
    theirs = ref.ParallelSampler(indptr.tolist(), indices.tolist(), eid.tolist(), ts.tolist(),
                                 threads, 1, layers, fans, recent, prop_time, hist, window)
    for b in range(4):
        roots = ((rng.zipf(1.3, 150) - 1) % n_nodes).astype(np.int32)
        rts = np.sort(rng.uniform(b * 2e5, (b + 1) * 2e5 + 1e5, 150)).astype(np.float32)
        mine.sample(roots, rts)
        theirs.sample(roots.tolist(), rts.tolist())
        got, want = mine.get_ret(), theirs.get_ret()
        assert len(got) == len(want) == layers * hist
        for r, (g, w) in enumerate(zip(got, want)):
            for f in FIELDS:
                assert np.array_equal(getattr(g, f)(), np.asarray(getattr(w, f)())), (b, r, f)
            assert (g.dim_in(), g.dim_out()) == (w.dim_in(), w.dim_out())


@pytest.mark.parametrize("add_reverse", [True, False])
def test_build_tcsr_equals_per_node_lists_sorted_by_time(add_reverse):
    """gen_graph.py:40-95 restated with Python lists and a stable sort, on a stream whose
    timestamps repeat (ties keep stream order) and arrive unsorted."""
    import torch
    from yitu_amd.temporal import build_tcsr
    rng = np.random.default_rng(3)
    n, m = 40, 600
    src, dst = rng.integers(0, n, m), rng.integers(0, n, m)
    ts = rng.integers(0, 50, m).astype(np.float32)
    lists = [[] for _ in range(n)]
    for e in range(m):
        lists[src[e]].append((ts[e], dst[e], e))
        if add_reverse:
            lists[dst[e]].append((ts[e], src[e], e))
    indptr, indices, eid, tt = [0], [], [], []
    for l in lists:
        for t, d, e in sorted(l, key=lambda x: x[0]):  # stable
            indices.append(d), eid.append(e), tt.append(t)
        indptr.append(len(indices))
    got = build_tcsr(torch.from_numpy(src), torch.from_numpy(dst), torch.from_numpy(ts), n,
                     add_reverse)
    assert [g.dtype for g in got] == [torch.int32, torch.int32, torch.int32, torch.float32]
    assert np.array_equal(got[0].numpy(), indptr) and np.array_equal(got[1].numpy(), indices)
    assert np.array_equal(got[2].numpy(), eid) and np.array_equal(got[3].numpy(), tt)
    # and it is a valid input of the sampler
    s = sampler_core.ParallelSampler(*[g.numpy() for g in got], 1, 1, 1, [5], True, False, 1, 0.0)
    s.sample(src[-20:], np.full(20, 60.0, np.float32))
    assert s.get_ret()[0].dim_out() == 20


MODES = np.load(os.path.join(ROOT, "tests", "golden", "sampler_modes.npz"))


@pytest.mark.parametrize("case", range(int(MODES["n_cases"])))
def test_other_modes_match_reference_golden_vectors(case):
    """Uniform draws (the reference's per-thread rand_r streams, for 1 / 2 / 5 nominal
    threads), a second layer found by binary search, prop_time, and snapshots of a sliding
    window (num_history 2 and 3), every block of every batch bit for bit against what the
    compiled reference returned (tests/golden/make_sampler_golden.py: MODE_CASES)."""
    pre = "c%d_" % case
    threads, layers, recent, prop_time, hist = (int(v) for v in MODES[pre + "args"])
    s = sampler_core.ParallelSampler(MODES[pre + "indptr"], MODES[pre + "indices"], MODES[pre + "eid"],
                                     MODES[pre + "ts"], threads, 1, layers,
                                     [int(v) for v in MODES[pre + "fans"]], bool(recent),
                                     bool(prop_time), hist, float(MODES[pre + "window"]))
    for b in range(int(MODES[pre + "n_batches"])):
        bp = pre + "b%d_" % b
        s.sample(MODES[bp + "roots"], MODES[bp + "root_ts"])
        ret = s.get_ret()
        assert len(ret) == int(MODES[bp + "n_blocks"]) == layers * hist
        for r, blk in enumerate(ret):
            got = _block_arrays(blk)
            for f in FIELDS:
                want = MODES[bp + "r%d_" % r + f]
                assert got[f].dtype == want.dtype and got[f].shape == want.shape, (case, b, r, f)
                assert np.array_equal(got[f], want), (case, b, r, f)
            assert [blk.dim_in(), blk.dim_out()] == MODES[bp + "r%d_dims" % r].tolist()


def test_uniform_draws_do_not_depend_on_the_real_thread_count(monkeypatch):
    """The draws are a function of the nominal thread count; how many threads really run
    (OMP_NUM_THREADS of the host) must not matter: same blocks for the same arguments from
    two samplers, one of them built and run after the OpenMP pool was shrunk to one thread."""
    pre = "c2_"
    args = (MODES[pre + "indptr"], MODES[pre + "indices"], MODES[pre + "eid"], MODES[pre + "ts"],
            5, 1, 1, [10], False, False, 1, 0.0)
    a = sampler_core.ParallelSampler(*args)
    a.sample(MODES[pre + "b0_roots"], MODES[pre + "b0_root_ts"])
    import ctypes
    omp = ctypes.CDLL("libgomp.so.1")
    omp.omp_set_num_threads(1)
    try:
        b = sampler_core.ParallelSampler(*args)
        b.sample(MODES[pre + "b0_roots"], MODES[pre + "b0_root_ts"])
    finally:
        omp.omp_set_num_threads(os.cpu_count() or 1)
    for f in FIELDS:
        assert np.array_equal(_block_arrays(a.get_ret()[0])[f], _block_arrays(b.get_ret()[0])[f])
