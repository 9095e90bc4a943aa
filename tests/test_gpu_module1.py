"""GPU parity of the module-1 drop-in (YiTu_GNN_kernel.forward / backward /
forward_gin / backward_gin / SAG) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from helpers import (ATOL_BF16, RTOL_BF16, assert_close, powerlaw_graph, random_csr,
                     scrambled_csr)
from yitu_amd import YiTu_GNN_kernel as K
from yitu_amd.data import graphgen

pytestmark = pytest.mark.gpu

PS, DW, WPB = 32, 32, 8  # tuning knobs of the reference signature (ignored by the kernels)


def _graph_args(indptr, indices, dev):
    pp, p2n = K.build_part(PS, indptr)
    return (indptr.to(dev), indices.to(dev), graphgen.gcn_norm(indptr).to(dev), pp.to(dev),
            p2n.to(dev))


@pytest.mark.parametrize("dim", [1, 2, 3, 4, 33, 64, 100, 128, 130, 256, 260, 512, 1030, 2052])
def test_sag_all_row_widths(dev, dim):
    n = 257
    indptr, indices = random_csr(n, n, 0.04, dim, hub_rows=(7,), hub_degree=150, empty_rows=(0, 5))
    x = torch.randn(n, dim, generator=torch.Generator().manual_seed(dim))
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    got = K.SAG(x.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert_close(got, oracle.sag(x.numpy(), indptr, indices), what="SAG dim=%d" % dim)
    assert torch.all(got[0] == 0) and torch.all(got[5] == 0)


@pytest.mark.parametrize("dim,bf16", [(64, False), (128, False), (128, True), (256, True), (33, False)])
def test_an_infinite_source_row_stays_infinite(dev, dim, bf16):
    """One source row holds +inf. Every destination that has it as a neighbour gets +inf (the
    IEEE sum, what a plain loop over the neighbours gives: never NaN, which 0 x inf from a
    padded lane would make of it), every other row is untouched. Rows of 1, 2, 3 ... edges
    and rows of several items are among the neighbours."""
    n = 600
    indptr, indices = random_csr(n, n, 0.01, 7, hub_rows=(3, 400), hub_degree=200, empty_rows=(9,))
    x = torch.rand(n, dim, generator=torch.Generator().manual_seed(dim)) + 0.5
    if bf16:
        x = x.to(torch.bfloat16).float()
    # the last neighbour of the first hub row: where the columns of a row ascend it is the
    # last edge of most rows that hold it, the edge that padded lanes load again
    src = int(indices[indptr[4] - 1])
    x_inf = x.clone()
    x_inf[src] = float("inf")
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    feed = (lambda t: t.to(torch.bfloat16)) if bf16 else (lambda t: t)
    base = K.SAG(feed(x).to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB).float().cpu()
    got = K.SAG(feed(x_inf).to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB).float().cpu()
    rows = torch.repeat_interleave(torch.arange(n), (indptr[1:] - indptr[:-1]).long())
    hit = torch.zeros(n, dtype=torch.bool)
    hit[rows[indices.long() == src]] = True
    assert hit.sum() >= 2 and not hit.all()
    assert torch.all(torch.isposinf(got[hit])), "a neighbour of the infinite row is not +inf"
    assert torch.equal(got[~hit], base[~hit])


@pytest.mark.parametrize("dim", [64, 128, 100])
def test_rows_with_unsorted_and_repeated_edges(dev, dim):
    """Edges of a row in any order, some of them twice: the sums are those of the loops
    over whatever the row holds, for short rows and for rows that the plan cuts at band
    crossings (which are then out of order)."""
    n = 1 << 13
    indptr, indices = random_csr(n, n, 0.001, dim, hub_rows=(5, 4000, 8191), hub_degree=3000,
                                 empty_rows=(2,))
    indptr, indices = scrambled_csr(indptr, indices, dim)
    g = torch.Generator().manual_seed(dim)
    x = torch.randn(n, dim, generator=g)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    got = K.SAG(x.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert_close(got, oracle.sag(x.numpy(), indptr, indices), what="SAG dim=%d" % dim)
    w = torch.eye(dim)
    got = K.forward(x.to(dev), w.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)[0]
    want = oracle.gcn_forward(x.numpy(), w.numpy(), indptr, indices, deg.cpu().numpy())
    assert_close(got, want, what="GCN dim=%d" % dim)


@pytest.mark.parametrize("hub_degree", [63, 64, 65, 127, 128, 129, 511, 1025, 3000])
@pytest.mark.parametrize("dim", [64, 128, 36])
def test_long_rows_take_the_planned_item_path(dev, hub_degree, dim):
    """Rows with >= 64 edges are cut into 64-edge items (one wave each, band order);
    single-item rows are written directly, the others through partial rows."""
    n = 4096
    indptr, indices = random_csr(n, n, 0.002, hub_degree, hub_rows=(1, 4000, 4095),
                                 hub_degree=hub_degree, empty_rows=(2,))
    x = torch.randn(n, dim, generator=torch.Generator().manual_seed(1))
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    w = torch.eye(dim)
    got = K.forward(x.to(dev), w.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)[0]
    want = oracle.gcn_forward(x.numpy(), w.numpy(), indptr, indices, deg.cpu().numpy())
    assert_close(got, want, what="hub=%d dim=%d" % (hub_degree, dim))


@pytest.mark.parametrize("fin,fout", [(16, 64), (64, 128), (50, 7)])
def test_gcn_forward_backward(dev, fin, fout):
    indptr, indices = powerlaw_graph(12, 60000, 3)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(fin)
    x = torch.randn(n, fin, generator=g)
    w = torch.randn(fin, fout, generator=g) / 8
    dy = torch.randn(n, fout, generator=g)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    out = K.forward(x.to(dev), w.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert isinstance(out, list) and len(out) == 1
    s = deg.cpu().numpy()
    assert_close(out[0], oracle.gcn_forward(x.numpy(), w.numpy(), indptr, indices, s))
    dx, dw = K.backward(dy.to(dev), x.to(dev), w.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)
    want_dx, want_dw = oracle.gcn_backward(dy.numpy(), x.numpy(), w.numpy(), indptr, indices, s)
    assert_close(dx, want_dx)
    # dW sums n = 4096 products per element: the allowance follows sum |x| |g|
    abs_dw = oracle.gcn_backward(dy.abs().numpy(), x.abs().numpy(), w.abs().numpy(), indptr, indices,
                                 s)[1]
    assert_close(dw, want_dw, abs_sum=abs_dw)


def test_gin_forward_backward(dev):
    indptr, indices = powerlaw_graph(11, 30000, 4)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(0)
    x = torch.randn(n, 48, generator=g)
    w = torch.randn(48, 20, generator=g) / 8
    dy = torch.randn(n, 20, generator=g)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    out, agg = K.forward_gin(x.to(dev), w.to(dev), rp, ci, 0.5, pp, p2n, PS, DW, WPB)
    want_out, want_agg = oracle.gin_forward(x.numpy(), w.numpy(), indptr, indices, 0.5)
    abs_agg = oracle.gin_forward(x.abs().numpy(), w.abs().numpy(), indptr, indices, 0.5)
    assert_close(agg, want_agg, abs_sum=abs_agg[1])
    assert_close(out, want_out, abs_sum=abs_agg[0])
    dx, dw = K.backward_gin(dy.to(dev), agg, w.to(dev), rp, ci, 0.5, pp, p2n, PS, DW, WPB)
    want_dx, want_dw = oracle.gin_backward(dy.numpy(), want_agg, w.numpy(), indptr, indices, 0.5)
    abs_dx, abs_dw = oracle.gin_backward(dy.abs().numpy(), np.abs(want_agg), w.abs().numpy(), indptr,
                                         indices, 0.5)
    assert_close(dx, want_dx, abs_sum=abs_dx)
    assert_close(dw, want_dw, abs_sum=abs_dw)


@pytest.mark.parametrize("dim", [8, 64, 128, 100, 256, 264])
def test_bf16_input_fp32_accumulate(dev, dim):
    indptr, indices = powerlaw_graph(12, 80000, 5)
    n = indptr.numel() - 1
    xb = torch.randn(n, dim, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    got = K._aggregate(xb.to(dev), rp, ci, deg, 1.0)
    bits = xb.view(torch.int16).numpy().view(np.uint16)
    want = oracle.row_agg_bf16(bits, indptr, indices, deg.cpu().numpy(), oracle.MODE_GCN)
    assert got.dtype == torch.float32
    assert_close(got, want, rtol=RTOL_BF16, atol=ATOL_BF16)
    # the inputs are exactly representable, so the fp32 bar holds as well
    assert_close(got, want)


def test_with_and_without_row_plan_agree(dev):
    """A call given no row plan builds a temporary one without slabs: its long rows are
    cut at other places than the per-graph plan cuts them, so the two results agree to
    rounding (and each of them is bitwise reproducible)."""
    from yitu_amd import _lib
    indptr, indices = powerlaw_graph(13, 200000, 8)
    n = indptr.numel() - 1
    x = torch.randn(n, 64, generator=torch.Generator().manual_seed(4)).to(dev)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    with_plan = K._aggregate(x, rp, ci, deg, 1.0)
    out = torch.empty_like(with_plan)
    ws = _lib.workspace(_lib.size_fn("yitu_spmm_workspace_bytes")(
        _lib.c_i64(ci.numel()), _lib.c_i64(64), _lib.c_int(0)), dev)
    rc = _lib.lib().yitu_agg_csr(_lib.ptr(out), _lib.ptr(x), 0, _lib.ptr(rp), _lib.ptr(ci),
                                 _lib.ptr(deg), _lib.c_i64(n), _lib.c_i64(n), _lib.c_i64(ci.numel()),
                                 _lib.c_i64(64), _lib.c_f32(1.0), _lib.c_i64(-1), _lib.ptr(None), _lib.ptr(None),
                                 _lib.ptr(ws), _lib.c_size(ws.numel()), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_agg_csr")
    first = out.clone()
    assert_close(first, with_plan)
    rc = _lib.lib().yitu_agg_csr(_lib.ptr(out), _lib.ptr(x), 0, _lib.ptr(rp), _lib.ptr(ci),
                                 _lib.ptr(deg), _lib.c_i64(n), _lib.c_i64(n), _lib.c_i64(ci.numel()),
                                 _lib.c_i64(64), _lib.c_f32(1.0), _lib.c_i64(-1), _lib.ptr(None), _lib.ptr(None),
                                 _lib.ptr(ws), _lib.c_size(ws.numel()), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_agg_csr")
    assert torch.equal(out, first)
    assert torch.equal(K._aggregate(x, rp, ci, deg, 1.0), with_plan)


def test_backward_transposed_is_the_true_gradient(dev):
    """On a directed graph the gradient of forward() aggregates dY over the transposed
    structure; checked against autograd through the dense normalised adjacency."""
    indptr, indices = random_csr(300, 300, 0.05, 11, hub_rows=(4,), hub_degree=200)
    n = 300
    g = torch.Generator().manual_seed(5)
    x = torch.randn(n, 24, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(24, 40, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(n, 40, generator=g, dtype=torch.float64)
    s = graphgen.gcn_norm(indptr).double()
    dense = torch.zeros(n, n, dtype=torch.float64)
    rows = torch.repeat_interleave(torch.arange(n), (indptr[1:] - indptr[:-1]).long())
    dense[rows, indices.long()] = s[rows] * s[indices.long()]
    ((dense @ (x @ w)) * dy).sum().backward()
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    dx, dw = K.backward_transposed(dy.float().to(dev), x.detach().float().to(dev),
                                   w.detach().float().to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert_close(dx, x.grad.float(), atol=2e-4)
    assert_close(dw, w.grad.float(), rtol=1e-4, atol=5e-4)


def test_results_are_bitwise_reproducible(dev):
    indptr, indices = powerlaw_graph(13, 200000, 6)
    n = indptr.numel() - 1
    x = torch.randn(n, 64, generator=torch.Generator().manual_seed(3)).to(dev)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    a = K.SAG(x, rp, ci, deg, pp, p2n, PS, DW, WPB)
    b = K.SAG(x, rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert torch.equal(a, b)


def test_linearity_and_row_block_invariance_at_scale(dev):
    """Size-independent properties on a 2^17-node power-law graph: linear in x,
    and a row's result does not depend on which other rows are in the launch."""
    src, dst = graphgen.rmat(17, 3_000_000, 7, self_loops=True, device=dev)
    n = 1 << 17
    rp, ci = graphgen.csr_by_destination(src, dst, n)
    deg = graphgen.gcn_norm(rp)
    g = torch.Generator(device=dev).manual_seed(1)
    x1 = torch.randn(n, 128, generator=g, device=dev)
    x2 = torch.randn(n, 128, generator=g, device=dev)
    f = lambda x: K._aggregate(x, rp, ci, deg, 1.0)
    y1, y2, y12 = f(x1), f(x2), f(x1 + 2 * x2)
    assert_close(y12, y1 + 2 * y2, atol=2e-4)
    lo, hi = 1000, 50000
    sub_rp = (rp[lo:hi + 1] - rp[lo]).contiguous()
    sub_ci = ci[rp[lo].item():rp[hi].item()].contiguous()
    out = torch.empty(hi - lo, 128, device=dev)
    from yitu_amd import _lib
    # no row plan is passed: the call builds a temporary one in its workspace
    ws = _lib.workspace(_lib.size_fn("yitu_spmm_workspace_bytes")(
        _lib.c_i64(sub_ci.numel()), _lib.c_i64(128), _lib.c_int(0)), dev)
    y_unscaled = K._aggregate(x1, rp, ci, None, 1.0)
    rc = _lib.lib().yitu_agg_csr(_lib.ptr(out), _lib.ptr(x1), 0, _lib.ptr(sub_rp), _lib.ptr(sub_ci),
                                 _lib.ptr(None), _lib.c_i64(hi - lo), _lib.c_i64(n),
                                 _lib.c_i64(sub_ci.numel()), _lib.c_i64(128), _lib.c_f32(1.0),
                                 _lib.c_i64(-1), _lib.ptr(None), _lib.ptr(None), _lib.ptr(ws),
                                 _lib.c_size(ws.numel()), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_agg_csr")
    # rows below 64 edges never depend on the launch they are in; longer rows are cut
    # into items at places that depend on the plan, so they agree to rounding
    short = (rp[lo + 1:hi + 1] - rp[lo:hi]) < 64
    assert torch.equal(out[short], y_unscaled[lo:hi][short])
    assert_close(out, y_unscaled[lo:hi], atol=5e-4)


def test_rejects_cpu_tensors_and_bad_dtypes(dev):
    indptr, indices = random_csr(10, 10, 0.3, 0)
    x = torch.randn(10, 4)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    with pytest.raises(RuntimeError):
        K.SAG(x, rp, ci, deg, pp, p2n, PS, DW, WPB)  # CPU features
    with pytest.raises(RuntimeError):
        K.SAG(x.to(dev), rp.long(), ci, deg, pp, p2n, PS, DW, WPB)
    with pytest.raises(RuntimeError):
        K.SAG(x.to(dev).t(), rp, ci, deg, pp, p2n, PS, DW, WPB)  # not contiguous


@pytest.mark.parametrize("n", [30, 0])
def test_graph_without_edges(dev, n):
    """Rows without any edge, and no rows at all: zeros of the right shape."""
    rp = torch.zeros(n + 1, dtype=torch.int32)
    ci = torch.zeros(0, dtype=torch.int32, device=dev)
    pp, p2n = K.build_part(PS, rp)
    assert pp.numel() == 1 and p2n.numel() == 0
    rp, pp, p2n = rp.to(dev), pp.to(dev), p2n.to(dev)
    x = torch.randn(n, 32, device=dev)
    w = torch.randn(32, 16, device=dev)
    dy = torch.randn(n, 16, device=dev)
    deg = torch.ones(n, device=dev)

    def zeros(t, *shape):
        return tuple(t.shape) == shape and not bool(t.any())

    (out,) = K.forward(x, w, rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert zeros(out, n, 16)
    dx, dw = K.backward(dy, x, w, rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert zeros(dx, n, 32) and zeros(dw, 32, 16)
    out, agg = K.forward_gin(x, w, rp, ci, 0.5, pp, p2n, PS, DW, WPB)
    assert zeros(out, n, 16) and zeros(agg, n, 32)
    assert zeros(K.SAG(x, rp, ci, deg, pp, p2n, PS, DW, WPB), n, 32)


@pytest.mark.parametrize("weight", ["identity", "uniform"])
def test_first_configuration_gcn_on_its_own_workload(dev, weight):
    """The GCN aggregation case as configured: Erdos-Renyi, 10,000 nodes, 100,000 directed
    draws plus a self loop per node, CSR by destination, edge weight 1 / sqrt(d_i d_j),
    features [N, 64] ~ N(0, 1), forward and backward through the drop-in signatures
    (YiTu_GNN.cpp:247-258), against the oracle at the plain bar rtol 1e-5 / atol 1e-4."""
    n, dim = 10_000, 64
    src, dst = graphgen.erdos_renyi(n, 100_000, seed=20241, self_loops=True)
    indptr, indices = graphgen.csr_by_destination(src, dst, n)
    g = torch.Generator().manual_seed(20241)
    x = torch.randn(n, dim, generator=g)
    dy = torch.randn(n, dim, generator=g)
    w = torch.eye(dim) if weight == "identity" else (torch.rand(dim, dim, generator=g) - 0.5) / 4
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    s = deg.cpu().numpy()
    out = K.forward(x.to(dev), w.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)[0]
    assert_close(out, oracle.gcn_forward(x.numpy(), w.numpy(), indptr, indices, s), what="forward")
    dx, dw = K.backward(dy.to(dev), x.to(dev), w.to(dev), rp, ci, deg, pp, p2n, PS, DW, WPB)
    want_dx, want_dw = oracle.gcn_backward(dy.numpy(), x.numpy(), w.numpy(), indptr, indices, s)
    assert_close(dx, want_dx, what="dX")
    # every element of dW adds 10,000 products
    abs_dw = oracle.gcn_backward(dy.abs().numpy(), x.abs().numpy(), w.abs().numpy(), indptr, indices,
                                 s)[1]
    assert_close(dw, want_dw, abs_sum=abs_dw, what="dW")
    # the aggregation alone, in the float order of the reference's neighbour groups
    agg = K._aggregate(x.to(dev), rp, ci, deg, 1.0)
    grouped = oracle.group_agg_f32(x.numpy(), indices, s, pp.cpu().numpy(), p2n.cpu().numpy(),
                                   oracle.MODE_GCN)
    assert_close(agg, grouped, what="aggregate vs neighbour-group order")


def test_edge_scale_is_the_same_aggregation(dev):
    """The per-edge column scales hold the very floats the kernel would gather from
    ``degrees``: results are bitwise equal with and without them, on short and on
    planned rows, and through forward / backward."""
    indptr, indices = powerlaw_graph(13, 200000, 11)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(6)
    x = torch.randn(n, 64, generator=g).to(dev)
    w = (torch.randn(64, 32, generator=g) / 8).to(dev)
    dy = torch.randn(n, 32, generator=g).to(dev)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    es = K.edge_scale(ci, deg)
    assert torch.equal(es, deg[ci.long()])
    plain = K._aggregate(x, rp, ci, deg, 1.0)
    assert torch.equal(K._aggregate(x, rp, ci, deg, 1.0, es), plain)
    assert_close(plain, oracle.row_agg(x.cpu().numpy(), indptr, indices, deg.cpu().numpy(),
                                       oracle.MODE_GCN))
    out = K.forward(x, w, rp, ci, deg, pp, p2n, PS, DW, WPB, edge_scale=es)[0]
    assert torch.equal(out, K.forward(x, w, rp, ci, deg, pp, p2n, PS, DW, WPB)[0])
    got = K.backward(dy, x, w, rp, ci, deg, pp, p2n, PS, DW, WPB, edge_scale=es)
    want = K.backward(dy, x, w, rp, ci, deg, pp, p2n, PS, DW, WPB)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    with pytest.raises(RuntimeError):
        K._aggregate(x, rp, ci, deg, 1.0, es[:-1].contiguous())


@pytest.mark.parametrize("per_row,dim", [(20, 64), (50, 128)])
def test_local_graph_rows_are_dealt_xcd_by_xcd(dev, per_row, dim):
    """A graph whose row plan says "local" (sources near the row's own id) has its short
    rows walked one eighth per XCD instead of round robin; the row count is no multiple of
    the launch's rounding, so surplus workgroups must find nothing. Same results, bit for
    bit on a second call, as for any graph; with 20 sources per row no row is long and the
    plan exists for its header alone (2^20 edges or more)."""
    from yitu_amd import _lib
    n, size = 70001, 500
    rng = np.random.default_rng(per_row)
    dst = np.repeat(np.arange(n), per_row)
    src = np.minimum(dst // size * size + rng.integers(0, size, dst.size), n - 1)
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(dst), torch.from_numpy(src), n, n)
    rp, ci, deg, pp, p2n = _graph_args(indptr, indices, dev)
    plan = _lib.row_plan(rp, ci, n, 0x7FFFFFFF)
    assert plan is not None
    header = plan[:1024].cpu().numpy().view(np.int32)
    assert 4 * int(header[66]) > 3 * int(header[67]) > 0
    x = torch.randn(n, dim, generator=torch.Generator().manual_seed(2))
    got = K._aggregate(x.to(dev), rp, ci, deg, 1.0)
    want = oracle.row_agg(x.numpy(), indptr, indices, deg.cpu().numpy(), oracle.MODE_GCN)
    assert_close(got, want)
    assert torch.equal(got, K._aggregate(x.to(dev), rp, ci, deg, 1.0))
