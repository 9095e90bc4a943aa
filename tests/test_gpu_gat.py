"""GPU parity of the fused GAT attention against the oracle's two-op composition
(sddmm_forward -> mh_spmm_forward and their backward), through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from helpers import (assert_close, powerlaw_graph, random_csr, scrambled_csr,
                     softmax_backward_abs_sums, spmm_abs_sums)
from yitu_amd import graph_ext
from yitu_amd.xgnn_h import block as xblock
from yitu_amd.xgnn_h import sparse

pytestmark = pytest.mark.gpu


def _oracle_gat(indptr, indices, q, k, x, gy):
    attn = oracle.sddmm_forward(indptr, indices, q[None], k)
    out = oracle.mh_spmm_forward(attn, indptr, indices, x)
    ga, gx = oracle.mh_spmm_backward(attn, indptr, indices, x, gy)
    gq, gk = oracle.sddmm_backward(indptr, indices, q[None], k, attn, ga)
    return attn, out, gq[0], gk, gx


def _run(dev, indptr, indices, n_dst, n_src, h, f, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n_dst, h, generator=g)
    k = torch.randn(n_src, h, generator=g)
    x = torch.randn(n_src, h, f, generator=g)
    gy = torch.randn(n_dst, h, f, generator=g)
    want_attn, want_out, want_gq, want_gk, want_gx = _oracle_gat(
        indptr, indices, q.numpy(), k.numpy(), x.numpy(), gy.numpy())
    # allowances of the long sums, from the data: the aggregate and grad_x are plain sums;
    # the softmax backward works on per-edge dots whose own absolute terms bound them
    abs_out, abs_ga, abs_gx = spmm_abs_sums(want_attn, indptr, indices, x, gy)
    abs_gq, abs_gk = softmax_backward_abs_sums(indptr, indices, want_attn, abs_ga, n_src)
    abs_gq = abs_gq[0]
    d = lambda t: t.to(dev)
    out, attn = graph_ext.gat_forward(d(indptr), d(indices), d(q), d(k), d(x))
    what = "H=%d F=%d" % (h, f)
    assert_close(attn, want_attn, what="attn " + what)
    assert_close(out, want_out, abs_sum=abs_out, what="out " + what)
    # without and with the forward output (the latter finishes the softmax backward
    # inside the one pass over the by-source edges when the rows are 256 floats)
    for fwd_out in (None, out):
        gq, gk, gx = graph_ext.gat_backward(d(indptr), d(indices), d(q), d(k), d(x), attn, d(gy),
                                            out=fwd_out)
        tag = what + (" (with out)" if fwd_out is not None else "")
        assert_close(gq, want_gq, abs_sum=abs_gq, what="grad_q " + tag)
        assert_close(gk, want_gk, abs_sum=abs_gk, what="grad_k " + tag)
        assert_close(gx, want_gx, abs_sum=abs_gx, what="grad_x " + tag)
    if graph_ext.gat_one_pass_shape(h, f):
        # the probabilities never stored: row statistics out of the forward, recomputed
        # per edge in the backward
        out2, none, stats = graph_ext.gat_forward(d(indptr), d(indices), d(q), d(k), d(x),
                                                  stats_only=True)
        assert none is None
        # long rows are summed from unnormalised item sums here: another rounding, same bar
        assert_close(out2, want_out, abs_sum=abs_out, what="out (stats) " + what)
        gq, gk, gx = graph_ext.gat_backward(d(indptr), d(indices), d(q), d(k), d(x), None, d(gy),
                                            out=out2, stats=stats)
        assert_close(gq, want_gq, abs_sum=abs_gq, what="grad_q (stats) " + what)
        assert_close(gk, want_gk, abs_sum=abs_gk, what="grad_k (stats) " + what)
        assert_close(gx, want_gx, abs_sum=abs_gx, what="grad_x (stats) " + what)
    return out


@pytest.mark.parametrize("h,f", [(4, 64), (1, 4), (1, 128), (2, 8), (3, 12), (8, 32), (5, 20),
                                 (16, 16), (33, 4), (64, 8), (4, 256), (2, 1000),
                                 (2, 128), (8, 64), (4, 128), (16, 64), (32, 32), (16, 32),
                                 (4, 6), (3, 5), (70, 4)])
def test_gat_shapes(dev, h, f):
    """The last three shapes take the unfused composition inside the same entry point."""
    n_dst, n_src = 203, 167
    indptr, indices = random_csr(n_dst, n_src, 0.08, h * 7 + f, hub_rows=(9,), hub_degree=160,
                                 empty_rows=(0, 202))
    out = _run(dev, indptr, indices, n_dst, n_src, h, f, seed=h + f)
    assert torch.all(out[0] == 0) and torch.all(out[202] == 0)


@pytest.mark.parametrize("h,f", [(4, 64), (2, 16), (8, 32)])
def test_gat_rows_with_unsorted_and_repeated_edges(dev, h, f):
    """The fused attention, forward and every gradient, on a multigraph whose rows hold
    their edges in random order (a repeated edge takes part in the softmax twice, as in
    the reference's loops, sddmm_cuda.cu:11-31)."""
    n = 1 << 12
    indptr, indices = random_csr(n, n, 0.002, 11 * h + f, hub_rows=(5, 2000, 4095),
                                 hub_degree=1500, empty_rows=(2,))
    indptr, indices = scrambled_csr(indptr, indices, h + f)
    _run(dev, indptr, indices, n, n, h, f, seed=h * f)


@pytest.mark.parametrize("h,f", [(4, 64), (2, 16), (4, 8), (1, 128), (8, 32)])
def test_gat_forward_of_an_infinite_source_row(dev, h, f):
    """One source's feature row is +inf. Destinations that have it as a neighbour come out
    +inf (probabilities here are far from underflow), every other row is bitwise untouched:
    a padded lane that loads the row again must not turn it into 0 x inf = NaN."""
    n = 600
    indptr, indices = random_csr(n, n, 0.01, h * 100 + f, hub_rows=(3, 400), hub_degree=200,
                                 empty_rows=(9,))
    g = torch.Generator().manual_seed(f)
    q = torch.randn(n, h, generator=g) * 0.3
    k = torch.randn(n, h, generator=g) * 0.3
    x = torch.rand(n, h, f, generator=g) + 0.5
    src = int(indices[indptr[4] - 1])  # the last neighbour of a hub row
    x_inf = x.clone()
    x_inf[src] = float("inf")
    d = lambda t: t.to(dev)
    base = graph_ext.gat_forward(d(indptr), d(indices), d(q), d(k), d(x))[0].cpu()
    got = graph_ext.gat_forward(d(indptr), d(indices), d(q), d(k), d(x_inf))[0].cpu()
    rows = torch.repeat_interleave(torch.arange(n), (indptr[1:] - indptr[:-1]).long())
    hit = torch.zeros(n, dtype=torch.bool)
    hit[rows[indices.long() == src]] = True
    assert hit.sum() >= 2 and not hit.all()
    assert torch.all(torch.isposinf(got[hit])), "a neighbour of the infinite row is not +inf"
    assert torch.equal(got[~hit], base[~hit])


@pytest.mark.parametrize("h,f", [(4, 64), (8, 8), (1, 32), (8, 64), (8, 128)])
def test_gat_power_law_hub_rows(dev, h, f):
    indptr, indices = powerlaw_graph(13, 150000, 11 * h + f)
    n = indptr.numel() - 1
    assert (indptr[1:] - indptr[:-1]).max() >= 1024
    assert ((indptr[1:] - indptr[:-1]) == 64).any() or True
    _run(dev, indptr, indices, n, n, h, f, seed=3)


def test_gat_autograd_equals_two_op_composition(dev):
    indptr, indices = powerlaw_graph(12, 60000, 5)
    n, h, f = indptr.numel() - 1, 4, 64
    blk = xblock.Block([n, n], [indptr, indices]).to(dev)
    g = torch.Generator().manual_seed(1)
    mk = lambda *s: torch.randn(*s, generator=g).to(dev).requires_grad_()
    q, k, x = mk(n, h), mk(n, h), mk(n, h, f)
    w = torch.randn(n, h, f, generator=g).to(dev)
    y1 = sparse.gspmm(blk, sparse.fused_gsddmm(blk, q, k), x)
    (y1 * w).sum().backward()
    g1 = [t.grad.clone() for t in (q, k, x)]
    for t in (q, k, x):
        t.grad = None
    y2 = sparse.fused_gat(blk, q, k, x)
    (y2 * w).sum().backward()
    assert_close(y2, y1, atol=2e-4)
    for a, t in zip(g1, (q, k, x)):
        assert_close(t.grad, a, atol=2e-4)


def test_gat_without_attn_buffer(dev):
    """attn may be NULL on the fused path (inference)."""
    from yitu_amd import _lib
    indptr, indices = random_csr(100, 100, 0.1, 1)
    g = torch.Generator().manual_seed(0)
    q, k, x = torch.randn(100, 4, generator=g), torch.randn(100, 4, generator=g), \
        torch.randn(100, 4, 16, generator=g)
    want = _oracle_gat(indptr, indices, q.numpy(), k.numpy(), x.numpy(),
                       np.zeros((100, 4, 16), np.float32))[1]
    d = lambda t: t.to(dev)
    ip, ix, qd, kd, xd = d(indptr), d(indices), d(q), d(k), d(x)
    out = torch.empty(100, 4, 16, device=dev)
    ws = _lib.workspace(256, dev)
    rc = _lib.lib().yitu_gat_forward(_lib.ptr(out), _lib.ptr(None), _lib.ptr(None), _lib.ptr(ip),
                                     _lib.ptr(ix),
                                     _lib.ptr(qd), _lib.ptr(kd), _lib.ptr(xd), _lib.c_i64(100),
                                     _lib.c_i64(100), _lib.c_i64(ix.numel()), _lib.c_i64(4),
                                     _lib.c_i64(16), _lib.c_i64(_lib.max_degree(ip)), _lib.ptr(None),
                                     _lib.ptr(ws), _lib.c_size(ws.numel()), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_gat_forward")
    assert_close(out, want)


@pytest.mark.parametrize("h,f", [(4, 64), (8, 32), (1, 256), (8, 64), (4, 256), (3, 12), (16, 16)])
def test_gat_head_mean_gradient(dev, h, f):
    """The layer's mean over heads taken inside the op: its gradient [n_dst, F] is handed
    to the backward as it is (gathered F floats per edge) and gives the same gradients as
    the explicit mean; the last two shapes fall outside the one-pass kernels and are
    expanded by the wrapper."""
    indptr, indices = powerlaw_graph(12, 60000, 3 * h + f)
    n = indptr.numel() - 1
    blk = xblock.Block([n, n], [indptr, indices]).to(dev)
    g = torch.Generator().manual_seed(h * f)
    mk = lambda *s: torch.randn(*s, generator=g).to(dev).requires_grad_()
    q, k, x = mk(n, h), mk(n, h), mk(n, h, f)
    w = torch.randn(n, f, generator=g).to(dev)
    y1 = sparse.fused_gat(blk, q, k, x).mean(dim=1)
    (y1 * w).sum().backward()
    want = [t.grad.clone() for t in (q, k, x)]
    for t in (q, k, x):
        t.grad = None
    y2 = sparse.fused_gat(blk, q, k, x, head_mean=True)
    (y2 * w).sum().backward()
    assert_close(y2, y1, atol=2e-4)
    for got, ref, name in zip((q.grad, k.grad, x.grad), want, "qkx"):
        assert_close(got, ref, atol=5e-4, what="grad_%s H=%d F=%d" % (name, h, f))


@pytest.mark.parametrize("n,h,f", [(1000, 4, 64), (37, 1, 4), (513, 8, 32), (300, 2, 256),
                                   (129, 16, 16), (64, 4, 256), (5, 3, 8)])
@pytest.mark.parametrize("two", [True, False])
def test_head_dot_forward_backward(dev, n, h, f, two):
    """Per-head projections against float64 torch algebra: outputs, grad_x written and
    accumulated, and the attention-vector gradients (sums over all rows)."""
    g = torch.Generator().manual_seed(n + h + f)
    x = torch.randn(n, h, f, generator=g)
    a, b = torch.randn(h, f, generator=g), torch.randn(h, f, generator=g)
    ga, gb = torch.randn(n, h, generator=g), torch.randn(n, h, generator=g)
    base = torch.randn(n, h, f, generator=g)
    d = lambda t: t.to(dev)
    oa, ob = graph_ext.head_dot(d(x), d(a), d(b) if two else None)
    xd = x.double()
    assert_close(oa, (xd * a.double()).sum(-1).float(), atol=1e-4 * f ** 0.5)
    if two:
        assert_close(ob, (xd * b.double()).sum(-1).float(), atol=1e-4 * f ** 0.5)
    else:
        assert ob is None
    want_gx = ga.double()[:, :, None] * a.double()
    want_gb = None
    if two:
        want_gx = want_gx + gb.double()[:, :, None] * b.double()
        want_gb = (gb.double()[:, :, None] * xd).sum(0).float()
    want_ga = (ga.double()[:, :, None] * xd).sum(0).float()
    gx, gva, gvb = graph_ext.head_dot_backward(d(x), d(a), d(b) if two else None, d(ga),
                                               d(gb) if two else None)
    assert_close(gx, want_gx.float())
    assert_close(gva, want_ga, atol=1e-4 * n ** 0.5)
    if two:
        assert_close(gvb, want_gb, atol=1e-4 * n ** 0.5)
    acc = d(base.clone())
    gx2, gva2, _ = graph_ext.head_dot_backward(d(x), d(a), d(b) if two else None, d(ga),
                                               d(gb) if two else None, grad_x=acc)
    assert gx2 is acc
    assert_close(gx2, (want_gx + base.double()).float())
    assert torch.equal(gva2, gva)  # fixed summation order


@pytest.mark.parametrize("h,f,bipartite", [(4, 64, False), (8, 32, True), (2, 24, False),
                                           (1, 256, True)])
def test_gat_head_layer_equals_torch_composition(dev, h, f, bipartite):
    """layers.GATHeadLayer (projections + attention + head mean as one op) against the same
    layer composed of torch ops and the two-op attention, outputs and every gradient.
    (2, 24) is a head width the projection kernels do not take: the wrapper composes."""
    from yitu_amd.xgnn_h import layers
    n_dst, n_src = (150, 220) if bipartite else (200, 200)
    indptr, indices = random_csr(n_dst, n_src, 0.1, 4 * h + f, hub_rows=(3,), hub_degree=n_src - 5,
                                 empty_rows=(0,))
    blk = xblock.Block([n_dst, n_src], [indptr, indices]).to(dev)
    torch.manual_seed(h * f)
    layer = layers.GATHeadLayer(20, f, h).to(dev)
    xs = torch.randn(n_src, 20, device=dev, requires_grad=True)
    xd = torch.randn(n_dst, 20, device=dev, requires_grad=True)
    w = torch.randn(n_dst, f, device=dev)
    inputs = (xs, xd) if bipartite else (xs,)

    y = layer(blk, [xs, xd] if bipartite else xs)
    (y * w).sum().backward()
    got = [y.detach()] + [t.grad.clone() for t in inputs] + [p.grad.clone() for p in layer.parameters()]
    for t in inputs:
        t.grad = None
    layer.zero_grad()

    h_src = layer.linear_v(xs).view(-1, h, f)
    h_dst = layer.linear_v(xd).view(-1, h, f) if bipartite else h_src
    q = (h_dst * layer.a_dst).sum(-1)
    k = (h_src * layer.a_src).sum(-1)
    y2 = sparse.gspmm(blk, sparse.fused_gsddmm(blk, q, k), h_src.contiguous()).mean(dim=1)
    (y2 * w).sum().backward()
    want = [y2.detach()] + [t.grad for t in inputs] + [p.grad for p in layer.parameters()]
    for a_, b_ in zip(got, want):
        assert_close(a_, b_, rtol=1e-4, atol=5e-4)


@pytest.mark.parametrize("n_dst", [12288 + 5, 30000, 50001])
def test_row_counts_between_the_rows_per_wave_steps(dev, n_dst):
    """A wave of the row kernels takes n_rows / 4096 rows (1 to 16): row counts that give
    3, 7 and 12 rows per wave, with a ragged last wave, a hub row and empty rows, through
    the fused attention (4 x 64: every one-pass kernel), the attention-only ops and the
    plain multi-head product."""
    n_src, h, f = 3000, 4, 64
    g = torch.Generator().manual_seed(n_dst)
    deg = torch.randint(0, 9, (n_dst,), generator=g)
    deg[n_dst // 2] = 300
    indptr = torch.zeros(n_dst + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(deg, 0)
    indices = torch.randint(0, n_src, (int(indptr[-1]),), generator=g, dtype=torch.int32)
    _run(dev, indptr, indices, n_dst, n_src, h, f, seed=1)
    d = lambda t: t.to(dev)
    values = torch.randn(indices.numel(), h, generator=g)
    x = torch.randn(n_src, h, 20, generator=g)
    gy = torch.randn(n_dst, h, 20, generator=g)
    got = graph_ext.spmm_forward(d(values), d(indptr), d(indices), d(x))
    assert_close(got, oracle.mh_spmm_forward(values, indptr, indices, x))
    ga, gx = graph_ext.spmm_backward(d(values), d(indptr), d(indices), d(x), d(gy))
    want_ga, want_gx = oracle.mh_spmm_backward(values, indptr, indices, x, gy)
    assert_close(ga, want_ga, atol=2e-4)
    assert_close(gx, want_gx, atol=5e-4)
