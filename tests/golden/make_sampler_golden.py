"""Writes tests/golden/sampler_recent.npz and sampler_modes.npz: input/output vectors of the
reference's own temporal sampler (YiTu_GNN/YiTu_T/sampler_core.cpp compiled
as-is into oracle/_ref/ by oracle/Makefile) on small seeded event streams.

Run in the container that has the reference checkout mounted:
    make -C oracle ref && python tests/golden/make_sampler_golden.py
Only data is stored: the T-CSR inputs, the query batches and the COO blocks the
reference returns for them.
"""
import glob
import importlib.util
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)


def load_reference_sampler():
    hits = glob.glob(os.path.join(ROOT, "oracle", "_ref", "sampler_core*.so"))
    if not hits:
        raise SystemExit("oracle/_ref/sampler_core*.so missing: run `make -C oracle ref`")
    spec = importlib.util.spec_from_file_location("sampler_core", hits[0])
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def tcsr(n_nodes, src, dst, ts):
    """T-CSR with reverse edges, per-node lists sorted by time (gen_graph.py:79-95)."""
    lists = [[] for _ in range(n_nodes)]
    for e, (s, d, t) in enumerate(zip(src, dst, ts)):
        lists[s].append((t, d, e))
        lists[d].append((t, s, e))
    indptr, indices, eid, tss = [0], [], [], []
    for l in lists:
        l.sort(key=lambda x: x[0])
        for t, d, e in l:
            indices.append(d)
            eid.append(e)
            tss.append(t)
        indptr.append(len(indices))
    return (np.asarray(indptr, np.int32), np.asarray(indices, np.int32), np.asarray(eid, np.int32),
            np.asarray(tss, np.float32))


def make_case(seed, n_nodes, n_events, batch, fan, n_batches, prop_time):
    rng = np.random.default_rng(seed)
    src = (rng.zipf(1.2, n_events) - 1) % n_nodes
    dst = (rng.zipf(1.2, n_events) - 1) % n_nodes
    ts = np.sort(rng.uniform(0, 1e6, n_events)).astype(np.float32)
    indptr, indices, eid, tss = tcsr(n_nodes, src, dst, ts)
    batches = []
    lo = n_events // 2
    for b in range(n_batches):
        ev = np.sort(rng.integers(lo, n_events, batch))
        roots = np.concatenate([src[ev], dst[ev]]).astype(np.int32)
        rts = np.concatenate([ts[ev], ts[ev]]).astype(np.float32)
        batches.append((roots, rts))
        lo = min(n_events - 1, lo + (n_events - lo) // (n_batches + 1))
    return dict(indptr=indptr, indices=indices, eid=eid, ts=tss, fan=fan, prop_time=prop_time,
                batches=batches)


def main():
    ref = load_reference_sampler()
    out = {}
    cases = [make_case(1, 50, 600, 16, 5, 4, False), make_case(2, 300, 5000, 64, 20, 5, False),
             make_case(3, 40, 900, 32, 3, 3, True), make_case(4, 2000, 4000, 50, 10, 3, False)]
    out["n_cases"] = np.int64(len(cases))
    for ci, c in enumerate(cases):
        s = ref.ParallelSampler(c["indptr"].tolist(), c["indices"].tolist(), c["eid"].tolist(),
                                c["ts"].tolist(), 2, 1, 1, [c["fan"]], True, c["prop_time"], 1, 0.0)
        pre = "c%d_" % ci
        for k in ("indptr", "indices", "eid", "ts"):
            out[pre + k] = c[k]
        out[pre + "fan"] = np.int64(c["fan"])
        out[pre + "prop_time"] = np.int64(c["prop_time"])
        out[pre + "n_batches"] = np.int64(len(c["batches"]))
        for bi, (roots, rts) in enumerate(c["batches"]):
            s.sample(roots.tolist(), rts.tolist())
            blk = s.get_ret()[0]
            bp = pre + "b%d_" % bi
            out[bp + "roots"], out[bp + "root_ts"] = roots, rts
            out[bp + "row"] = np.asarray(blk.row(), np.int32)
            out[bp + "col"] = np.asarray(blk.col(), np.int32)
            out[bp + "eid"] = np.asarray(blk.eid(), np.int32)
            out[bp + "ts"] = np.asarray(blk.ts(), np.float32)
            out[bp + "dts"] = np.asarray(blk.dts(), np.float32)
            out[bp + "nodes"] = np.asarray(blk.nodes(), np.int32)
            out[bp + "dims"] = np.asarray([blk.dim_in(), blk.dim_out()], np.int64)
    path = os.path.join(ROOT, "tests", "golden", "sampler_recent.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")
    write_modes(ref)


# (seed, n_nodes, n_events, batch, n_batches, threads, layers, fans, recent, prop_time,
#  num_history, window): uniform draws with 1 / 2 / 5 nominal threads, two layers by binary
# search, prop_time cursors in the first layer, snapshots of a window (most recent and drawn)
MODE_CASES = [
    (11, 60, 3000, 24, 3, 1, 1, [5], False, False, 1, 0.0),
    (12, 60, 3000, 24, 3, 2, 1, [5], False, False, 1, 0.0),
    (13, 200, 8000, 40, 3, 5, 1, [10], False, False, 1, 0.0),
    (14, 80, 4000, 16, 2, 3, 2, [6, 4], False, False, 1, 0.0),
    (15, 80, 4000, 16, 2, 2, 1, [4], False, True, 1, 0.0),
    (16, 50, 4000, 20, 3, 2, 1, [5], True, False, 3, 50000.0),
    (17, 50, 4000, 20, 3, 4, 1, [3], False, False, 2, 100000.0),
    (18, 50, 4000, 12, 2, 2, 2, [4, 3], False, False, 2, 100000.0),
]


def write_modes(ref):
    out = {"n_cases": np.int64(len(MODE_CASES))}
    for ci, (seed, n_nodes, n_events, batch, n_batches, threads, layers, fans, recent, prop_time,
             hist, window) in enumerate(MODE_CASES):
        c = make_case(seed, n_nodes, n_events, batch, fans[0], n_batches, prop_time)
        s = ref.ParallelSampler(c["indptr"].tolist(), c["indices"].tolist(), c["eid"].tolist(),
                                c["ts"].tolist(), threads, 1, layers, list(fans), recent, prop_time,
                                hist, float(window))
        pre = "c%d_" % ci
        for k in ("indptr", "indices", "eid", "ts"):
            out[pre + k] = c[k]
        out[pre + "args"] = np.asarray([threads, layers, int(recent), int(prop_time), hist], np.int64)
        out[pre + "fans"] = np.asarray(fans, np.int64)
        out[pre + "window"] = np.float32(window)
        out[pre + "n_batches"] = np.int64(n_batches)
        for bi, (roots, rts) in enumerate(c["batches"]):
            s.sample(roots.tolist(), rts.tolist())
            ret = s.get_ret()
            bp = pre + "b%d_" % bi
            out[bp + "roots"], out[bp + "root_ts"] = roots, rts
            out[bp + "n_blocks"] = np.int64(len(ret))
            for ri, blk in enumerate(ret):
                rp = bp + "r%d_" % ri
                out[rp + "row"] = np.asarray(blk.row(), np.int32)
                out[rp + "col"] = np.asarray(blk.col(), np.int32)
                out[rp + "eid"] = np.asarray(blk.eid(), np.int32)
                out[rp + "ts"] = np.asarray(blk.ts(), np.float32)
                out[rp + "dts"] = np.asarray(blk.dts(), np.float32)
                out[rp + "nodes"] = np.asarray(blk.nodes(), np.int32)
                out[rp + "dims"] = np.asarray([blk.dim_in(), blk.dim_out()], np.int64)
    path = os.path.join(ROOT, "tests", "golden", "sampler_modes.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
