#!/usr/bin/env python3
"""Benchmark of the sparse message-passing hot path on one MI355X.

Default workload (``c3_spmm_f32``): the large GCN SpMM of the baseline's third
configuration -- R-MAT graph, 2^21 nodes, 63 M drawn edges (deduplicated, self
loops added), CSR by destination, features [N,128] fp32, edge weight
1/sqrt(d_i d_j). One step = forward aggregation of X plus backward aggregation
of dY (the reference's backward applies the same CSR, YiTu_GNN_kernel.cu:447-461),
both through the C ABI (yitu_agg_csr). ``value`` = edges / second with the
reference's definition: n_edges / (time of forward + backward)
(YiTu_GNN/YiTu_H/test/bench_macro.py:371-391). Inputs are resident in HBM before
the timed region.

Prints ONE JSON line on stdout. Other workloads: ``--workload c3_spmm_bf16``,
``c2_gat_f32``, ``c1_gcn_f32``.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

# HBM-side bytes per call (reads + writes leaving L2) measured with two rocprofv3 --pmc
# runs of this file, FETCH_SIZE then WRITE_SIZE, each scaled by what the same counter
# reads for the library's 1 GiB copy kernel (FETCH_SIZE x 2.0000, WRITE_SIZE x 1.0000):
# profiles/bench_c3_spmm_gat_rocprofv3.md. Per yitu_agg_csr call for the C3 workloads,
# per yitu_gat_forward call for C2.
MEASURED_TRAFFIC_BYTES = {
    "c3_spmm_f32": 21_803_805_752,
    "c3_spmm_bf16": 10_910_454_990,
    "c2_gat_f32": 6_556_746_400,
}


def _sync():
    torch.cuda.synchronize()


def build_c3(dev, scale=21, draws=63_000_000, seed=20242):
    from yitu_amd.data import graphgen
    src, dst = graphgen.rmat(scale, draws, seed, self_loops=True, device=dev)
    n = 1 << scale
    rp, ci = graphgen.csr_by_destination(src, dst, n)
    del src, dst
    return n, rp, ci, graphgen.gcn_norm(rp)


def agg_call(out, x, rp, ci, deg, plan, ws, maxdeg):
    from yitu_amd import _lib
    n, dim = x.shape
    rc = _lib.lib().yitu_agg_csr(
        _lib.ptr(out), _lib.ptr(x), _lib.c_int(1 if x.dtype == torch.bfloat16 else 0), _lib.ptr(rp),
        _lib.ptr(ci), _lib.ptr(deg), _lib.c_i64(rp.numel() - 1), _lib.c_i64(n),
        _lib.c_i64(ci.numel()), _lib.c_i64(dim), _lib.c_f32(1.0), _lib.c_i64(maxdeg), _lib.ptr(plan),
        _lib.ptr(ws), _lib.c_size(ws.numel()), _lib.stream_ptr(x.device))
    _lib.check(rc, "yitu_agg_csr")


def cpu_baseline_spmm(rp, ci, deg, x, dy):
    """The oracle's float/OpenMP restatement on the host cores, full workload."""
    import oracle
    rp_h, ci_h, deg_h = rp.cpu().numpy(), ci.cpu().numpy(), deg.cpu().numpy()
    x_h, dy_h = x.float().cpu().numpy(), dy.float().cpu().numpy()
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    oracle.row_agg(x_h[:1024], rp_h[:1025] - rp_h[0], ci_h[:rp_h[1024]], deg_h, oracle.MODE_GCN,
                   f64=False)  # warm-up: loads the library, spins up the team
    times = []
    for _ in range(2):
        t0 = time.perf_counter()
        oracle.row_agg(x_h, rp_h, ci_h, deg_h, oracle.MODE_GCN, f64=False)
        oracle.row_agg(dy_h, rp_h, ci_h, deg_h, oracle.MODE_GCN, f64=False)
        times.append(time.perf_counter() - t0)
    t = min(times)
    return {"value": ci_h.shape[0] / t, "unit": "edges/s", "cores": cores, "kind": "port",
            "sample": "full workload (2^21 nodes, %d edges, F=128), fwd+bwd, best of 2, "
                      "OpenMP float restatement oracle/yitu_oracle.c" % ci_h.shape[0],
            "seconds": t}


def run_spmm(args, dev, bf16):
    from yitu_amd import _lib
    n, rp, ci, deg = build_c3(dev)
    nnz = ci.numel()
    dim = 128
    g = torch.Generator(device=dev).manual_seed(20242)
    x = torch.randn(n, dim, generator=g, device=dev)
    dy = torch.randn(n, dim, generator=g, device=dev)
    if bf16:
        x, dy = x.to(torch.bfloat16), dy.to(torch.bfloat16)
    out = torch.empty(n, dim, device=dev)
    dx = torch.empty(n, dim, device=dev)
    maxdeg = int((rp[1:] - rp[:-1]).max().item())
    # per-graph preparation, outside the timed region like the reference's build_part
    plan = _lib.row_plan(rp, ci, n, 0x7FFFFFFF)
    ws = torch.empty(int(_lib.size_fn("yitu_spmm_workspace_bytes")(
        _lib.c_i64(nnz), _lib.c_i64(dim), _lib.c_int(1))), dtype=torch.uint8, device=dev)

    def step(events=None):
        for src_t, dst_t in ((x, out), (dy, dx)):
            if events is not None:
                e0 = torch.cuda.Event(enable_timing=True)
                e1 = torch.cuda.Event(enable_timing=True)
                e0.record()
            agg_call(dst_t, src_t, rp, ci, deg, plan, ws, maxdeg)
            if events is not None:
                e1.record()
                events.append((e0, e1))

    for _ in range(args.warmup):
        step()
    _sync()
    events = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(events)
    _sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    call_ms = sum(a.elapsed_time(b) for a, b in events) / len(events)

    b_in = 2 if bf16 else 4
    alg = 4 * (n + 1) + 4 * nnz + 4 * n + b_in * n * dim + 4 * n * dim  # per aggregation call
    achieved = alg / (call_ms * 1e-3) / 1e9
    name = "c3_spmm_bf16" if bf16 else "c3_spmm_f32"
    res = {
        "metric": "SpMM edges/sec (GCN aggregation fwd+bwd, n_edges / step time)",
        "value": nnz / (ms_per_step * 1e-3),
        "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16-in/f32-acc" if bf16 else "f32", "data": "synthetic",
        "config": {"workload": name, "graph": "R-MAT scale 21 (a,b,c,d)=(.57,.19,.19,.05), "
                   "63M draws dedup + self loops, CSR by destination", "n_nodes": n,
                   "n_edges": nnz, "max_in_degree": maxdeg, "feature_dim": dim,
                   "step": "aggregate(X) + aggregate(dY), same CSR, W = I"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(name),
                     "kernel": "one yitu_agg_csr call = spmm_rows_kernel + spmm_items_kernel + "
                               "spmm_reduce_kernel (row plan built once per graph, untimed)",
                     "kernel_ms": call_ms, "algorithmic_bytes": alg,
                     "gather_bytes_no_reuse": nnz * dim * b_in},
    }
    if not args.no_cpu:
        res["cpu_baseline"] = cpu_baseline_spmm(rp, ci, deg, x, dy)
    return res


def run_gat(args, dev):
    """Second configuration: GAT attention, 4 heads x 64, R-MAT 2^18 nodes, 13 M draws
    (deduplicated), fp32. One step = fused forward (SDDMM + LeakyReLU + edge softmax +
    aggregate, attn saved) + backward (grad of x', q, k), through the C ABI. The dense
    per-head projections q = <a_dst, x'>, k = <a_src, x'> are outside the timed step."""
    from yitu_amd import graph_ext
    from yitu_amd.data import graphgen
    scale, draws, h, f = 18, 13_000_000, 4, 64
    n = 1 << scale
    src, dst = graphgen.rmat(scale, draws, 20241, device=dev)
    rp, ci = graphgen.csr_by_destination(src, dst, n)
    del src, dst
    nnz = ci.numel()
    g = torch.Generator(device=dev).manual_seed(20241)
    x = torch.randn(n, h, f, generator=g, device=dev)
    a_src = torch.randn(h, f, generator=g, device=dev) * 0.1
    a_dst = torch.randn(h, f, generator=g, device=dev) * 0.1
    q = torch.einsum("nhf,hf->nh", x, a_dst).contiguous()
    k = torch.einsum("nhf,hf->nh", x, a_src).contiguous()
    gy = torch.randn(n, h, f, generator=g, device=dev)
    graph_ext.transposed(rp, ci, n)  # one-time graph preparation, outside the timed region
    from yitu_amd import _lib
    _lib.row_plan(rp, ci, n, 0xFFFFFF)

    ev = {"fwd": [], "bwd": []}

    def step(timed):
        es = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        es[0].record()
        out, attn = graph_ext.gat_forward(rp, ci, q, k, x)
        es[1].record()
        graph_ext.gat_backward(rp, ci, q, k, x, attn, gy)
        es[2].record()
        if timed:
            ev["fwd"].append((es[0], es[1]))
            ev["bwd"].append((es[1], es[2]))

    for _ in range(args.warmup):
        step(False)
    _sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(True)
    _sync()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    fwd_ms = sum(a.elapsed_time(b) for a, b in ev["fwd"]) / args.steps
    bwd_ms = sum(a.elapsed_time(b) for a, b in ev["bwd"]) / args.steps
    alg_fwd = 4 * (n + 1) + 4 * nnz + 8 * n * h + 4 * nnz * h + 8 * n * h * f
    alg_bwd = (2 * 4 * n * h * f + 4 * nnz * h + 8 * nnz + 8 * (n + 1) + 4 * nnz
               + 4 * n * h * f + 8 * n * h)
    return {
        "metric": "GAT attention fwd+bwd (fused SDDMM+LeakyReLU+softmax+aggregate), edges/sec",
        "value": nnz / (ms_per_step * 1e-3), "unit": "edges/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c2_gat_f32", "graph": "R-MAT scale 18, 13M draws dedup, CSR by "
                   "destination", "n_nodes": n, "n_edges": nnz, "heads": h, "head_dim": f},
        "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
        "roofline": {"bound": "hbm", "achieved": alg_fwd / (fwd_ms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg_fwd / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get("c2_gat_f32"),
                     "kernel": "yitu_gat_forward = gat_rows_kernel + gat_item_stats + "
                               "gat_row_combine + gat_item_apply + spmm_reduce",
                     "kernel_ms": fwd_ms, "algorithmic_bytes": alg_fwd,
                     "bwd_achieved": alg_bwd / (bwd_ms * 1e-3) / 1e9,
                     "bwd_algorithmic_bytes": alg_bwd},
    }


def calibration_copy(dev, n_bytes=1 << 30, reps=5):
    """1 GiB streaming copy through the library's copy kernel: the known-size
    launch that FETCH_SIZE / WRITE_SIZE are scaled by, and the achievable
    read+write bandwidth of this GPU."""
    from yitu_amd import _lib
    a = torch.empty(n_bytes, dtype=torch.uint8, device=dev)
    b = torch.empty(n_bytes, dtype=torch.uint8, device=dev)
    a.zero_()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(reps + 1):
        if i == 1:
            e0.record()
        rc = _lib.lib().yitu_stream_copy(_lib.ptr(b), _lib.ptr(a), _lib.c_i64(n_bytes),
                                         _lib.stream_ptr(dev))
        _lib.check(rc, "yitu_stream_copy")
    e1.record()
    _sync()
    ms = e0.elapsed_time(e1) / reps
    return {"bytes_read": n_bytes, "bytes_written": n_bytes, "ms": ms,
            "GBps_read_plus_write": 2 * n_bytes / (ms * 1e-3) / 1e9}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3_spmm_f32")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="default workload only")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus 1 only)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "c3_spmm_f32":
        res = run_spmm(args, dev, bf16=False)
        res["copy_calibration"] = calibration_copy(dev)
        if not args.no_extra:
            # the other single-GPU configurations ride along as extra fields
            args.no_cpu = True
            slim = lambda r: {k: r[k] for k in ("value", "unit", "ms_per_step", "dtype", "config",
                                                "roofline") if k in r}
            res["extra"] = {"c3_spmm_bf16": slim(run_spmm(args, dev, bf16=True)),
                            "c2_gat_f32": slim(run_gat(args, dev))}
    elif args.workload == "c3_spmm_bf16":
        res = run_spmm(args, dev, bf16=True)
    elif args.workload == "c2_gat_f32":
        res = run_gat(args, dev)
    else:
        sys.exit("unknown workload %s" % args.workload)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
