"""Device-side most-recent-neighbour sampler (yitu_tsample_recent) against the
host sampler and against the golden vectors written by the reference's own
sampler (tests/golden/sampler_recent.npz). Integer and float32 compare work:
bit-exact, including the cursor quirks (state kept across batches, repeated
roots sharing a cursor, the first edge of a node never emitted)."""
import os

import numpy as np
import pytest
import torch

from yitu_amd import sampler_core

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "sampler_recent.npz"))
FIELDS = ("row", "col", "eid", "ts", "dts", "nodes")


def _same(dev_blk, host_blk, what):
    got = dev_blk.cpu_block()
    for f in FIELDS:
        a, b = getattr(got, f)(), getattr(host_blk, f)()
        assert a.dtype == b.dtype and a.shape == b.shape, (what, f, a.shape, b.shape)
        assert np.array_equal(a, b), (what, f)
    assert (got.dim_in(), got.dim_out()) == (host_blk.dim_in(), host_blk.dim_out())


@pytest.mark.parametrize("case", range(int(GOLD["n_cases"])))
def test_matches_reference_golden_vectors(dev, case):
    pre = "c%d_" % case
    s = sampler_core.GpuParallelSampler(GOLD[pre + "indptr"], GOLD[pre + "indices"],
                                        GOLD[pre + "eid"], GOLD[pre + "ts"], 2, 1, 1,
                                        [int(GOLD[pre + "fan"])], True,
                                        bool(GOLD[pre + "prop_time"]), 1, 0.0, device=dev)
    for b in range(int(GOLD[pre + "n_batches"])):
        bp = pre + "b%d_" % b
        s.sample(GOLD[bp + "roots"], GOLD[bp + "root_ts"])
        got = s.get_ret()[0].cpu_block()
        for f in FIELDS:
            want = GOLD[bp + f]
            assert getattr(got, f)().dtype == want.dtype, (case, b, f)
            assert np.array_equal(getattr(got, f)(), want), (case, b, f)
        assert [got.dim_in(), got.dim_out()] == GOLD[bp + "dims"].tolist()


def _tcsr(rng, n_nodes, n_events):
    src = (rng.zipf(1.3, n_events) - 1) % n_nodes
    dst = rng.integers(0, n_nodes, n_events)
    ts = np.sort(rng.uniform(0, 1000, n_events)).astype(np.float32)
    node = np.concatenate([src, dst])
    other = np.concatenate([dst, src])
    eid = np.concatenate([np.arange(n_events), np.arange(n_events)])
    tt = np.concatenate([ts, ts])
    order = np.lexsort((eid, tt, node))
    indptr = np.zeros(n_nodes + 1, np.int64)
    indptr[1:] = np.cumsum(np.bincount(node, minlength=n_nodes))
    return indptr, other[order], eid[order], tt[order], src, dst, ts


@pytest.mark.parametrize("layers,fans,prop", [(1, [20], False), (1, [3], True), (2, [5, 4], False)])
def test_equals_host_sampler_over_a_stream_of_batches(dev, layers, fans, prop):
    """Batches in time order, then repeated roots and queries that go back in time: the
    cursors are state, and both samplers must carry the same state."""
    rng = np.random.default_rng(5)
    indptr, indices, eid, tt, src, dst, ts = _tcsr(rng, 300, 8000)
    host = sampler_core.ParallelSampler(indptr, indices, eid, tt, 4, 1, layers, fans, True, prop,
                                        1, 0.0)
    gpu = sampler_core.GpuParallelSampler(indptr, indices, eid, tt, 4, 1, layers, fans, True, prop,
                                          1, 0.0, device=dev)
    batches = [np.arange(i, i + 200) for i in range(0, 8000, 1600)]
    batches += [rng.integers(0, 8000, 300), np.full(50, 4000), rng.integers(0, 500, 100)]
    for bi, ev in enumerate(batches):
        roots = np.concatenate([src[ev], dst[ev]])
        rts = np.concatenate([ts[ev], ts[ev]])
        host.sample(roots, rts)
        gpu.sample(roots, rts)
        hb, gb = host.get_ret(), gpu.get_ret()
        assert len(hb) == len(gb) == layers
        for l in range(layers):
            _same(gb[l], hb[l], (bi, l))
    host.reset()
    gpu.reset()
    ev = batches[-1]
    host.sample(src[ev], ts[ev])
    gpu.sample(src[ev], ts[ev])
    _same(gpu.get_ret()[0], host.get_ret()[0], "after reset")


def test_empty_batch_and_bad_root(dev):
    rng = np.random.default_rng(1)
    indptr, indices, eid, tt, *_ = _tcsr(rng, 50, 400)
    gpu = sampler_core.GpuParallelSampler(indptr, indices, eid, tt, 1, 1, 1, [4], True, False, 1,
                                          0.0, device=dev)
    gpu.sample(np.zeros(0, np.int32), np.zeros(0, np.float32))
    b = gpu.get_ret()[0]
    assert b.row().numel() == 0 and b.dim_in() == 0 and b.dim_out() == 0
    with pytest.raises(RuntimeError, match="out of range"):
        gpu.sample(np.array([3, 50]), np.array([10.0, 10.0]))


def test_device_block_feeds_the_attention_layer(dev):
    """The layer gives the same output from the device block as from the host block."""
    from yitu_amd.temporal import TemporalBlock, TransfomerAttentionLayer
    rng = np.random.default_rng(2)
    indptr, indices, eid, tt, src, dst, ts = _tcsr(rng, 400, 6000)
    host = sampler_core.ParallelSampler(indptr, indices, eid, tt, 4, 1, 1, [10], True, False, 1, 0.0)
    gpu = sampler_core.GpuParallelSampler(indptr, indices, eid, tt, 4, 1, 1, [10], True, False, 1,
                                          0.0, device=dev)
    ev = rng.integers(5000, 6000, 128)
    host.sample(src[ev], ts[ev])
    gpu.sample(src[ev], ts[ev])
    torch.manual_seed(0)
    memory = torch.randn(400, 24, device=dev)
    layer = TransfomerAttentionLayer(24, 0, 8, 2, 0.0, 0.0, 16).to(dev)
    a = layer(TemporalBlock.from_sampler(host.get_ret()[0], memory, device=dev))
    b = layer(TemporalBlock.from_device_block(gpu.get_ret()[0], memory))
    assert torch.equal(a, b)


MODES = np.load(os.path.join(ROOT, "tests", "golden", "sampler_modes.npz"))


@pytest.mark.parametrize("case", range(int(MODES["n_cases"])))
def test_other_modes_match_reference_golden_vectors(dev, case):
    """Uniform draws for 1 / 2 / 5 nominal threads, a second layer by binary search,
    prop_time, 2 and 3 window snapshots: every block of every batch bit for bit against
    what the compiled reference returned (tests/golden/make_sampler_golden.py)."""
    pre = "c%d_" % case
    threads, layers, recent, prop_time, hist = (int(v) for v in MODES[pre + "args"])
    s = sampler_core.GpuParallelSampler(MODES[pre + "indptr"], MODES[pre + "indices"],
                                        MODES[pre + "eid"], MODES[pre + "ts"], threads, 1, layers,
                                        [int(v) for v in MODES[pre + "fans"]], bool(recent),
                                        bool(prop_time), hist, float(MODES[pre + "window"]),
                                        device=dev)
    for b in range(int(MODES[pre + "n_batches"])):
        bp = pre + "b%d_" % b
        s.sample(MODES[bp + "roots"], MODES[bp + "root_ts"])
        ret = s.get_ret()
        assert len(ret) == int(MODES[bp + "n_blocks"]) == layers * hist
        for r, blk in enumerate(ret):
            got = blk.cpu_block()
            for f in FIELDS:
                want = MODES[bp + "r%d_" % r + f]
                assert getattr(got, f)().dtype == want.dtype, (case, b, r, f)
                assert np.array_equal(getattr(got, f)(), want), (case, b, r, f)
            assert [got.dim_in(), got.dim_out()] == MODES[bp + "r%d_dims" % r].tolist()


@pytest.mark.parametrize("threads,layers,fans,recent,prop,hist,window", [
    (16, 1, [20], False, False, 1, 0.0),      # uniform draws, many roots per chunk
    (3, 2, [6, 4], False, False, 1, 0.0),     # second layer by binary search
    (1, 1, [5], False, True, 1, 0.0),
    (4, 1, [8], True, False, 3, 40.0),        # most recent of three window snapshots
    (5, 2, [4, 3], False, False, 2, 60.0),    # uniform draws inside window snapshots, two layers
    (2, 2, [3, 3], True, False, 2, 50.0),     # cursors in both layers
])
def test_other_modes_equal_host_sampler_over_a_stream_of_batches(dev, threads, layers, fans, recent,
                                                                prop, hist, window):
    rng = np.random.default_rng(11 + threads)
    indptr, indices, eid, tt, src, dst, ts = _tcsr(rng, 300, 8000)
    args = (indptr, indices, eid, tt, threads, 1, layers, fans, recent, prop, hist, window)
    host = sampler_core.ParallelSampler(*args)
    gpu = sampler_core.GpuParallelSampler(*args, device=dev)
    batches = [np.arange(i, i + 200) for i in range(0, 8000, 1600)]
    batches += [rng.integers(0, 8000, 300), np.full(50, 4000), rng.integers(0, 500, 100),
                np.arange(7)]
    for bi, ev in enumerate(batches):
        roots = np.concatenate([src[ev], dst[ev]])
        rts = np.concatenate([ts[ev], ts[ev]])
        host.sample(roots, rts)
        gpu.sample(roots, rts)
        hb, gb = host.get_ret(), gpu.get_ret()
        assert len(hb) == len(gb) == layers * hist
        for l in range(len(hb)):
            _same(gb[l], hb[l], (bi, l))
    host.reset()
    gpu.reset()
    ev = batches[-2]
    host.sample(src[ev], ts[ev])
    gpu.sample(src[ev], ts[ev])
    for l in range(layers * hist):
        _same(gpu.get_ret()[l], host.get_ret()[l], ("after reset", l))


def test_uniform_mode_bad_root_and_empty_batch(dev):
    rng = np.random.default_rng(1)
    indptr, indices, eid, tt, *_ = _tcsr(rng, 50, 400)
    gpu = sampler_core.GpuParallelSampler(indptr, indices, eid, tt, 2, 1, 1, [4], False, False, 2,
                                          10.0, device=dev)
    gpu.sample(np.zeros(0, np.int32), np.zeros(0, np.float32))
    assert [b.dim_in() for b in gpu.get_ret()] == [0, 0]
    with pytest.raises(RuntimeError, match="out of range"):
        gpu.sample(np.array([3, 50]), np.array([10.0, 10.0]))
