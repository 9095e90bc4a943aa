"""The allocation-free aggregation entry point (yitu_agg_csr_noalloc): its scratch
is a static device array inside the library. Checked against yitu_agg_csr given a
caller's workspace and no plan (the same temporary plan, hence the same bits) on
two calls in a row, the second on a smaller input, so that whatever the first call
left in the shared array must not matter."""
import ctypes

import pytest
import torch

import oracle
from helpers import assert_close, powerlaw_graph
from yitu_amd import _lib
from yitu_amd.data import graphgen

pytestmark = pytest.mark.gpu


def _with_workspace(x, rp, ci, deg, dev):
    n, dim = x.shape
    out = torch.empty(rp.numel() - 1, dim, device=dev)
    ws = _lib.workspace(_lib.size_fn("yitu_spmm_workspace_bytes")(
        _lib.c_i64(ci.numel()), _lib.c_i64(dim), _lib.c_int(0)), dev)
    rc = _lib.lib().yitu_agg_csr(_lib.ptr(out), _lib.ptr(x), 0, _lib.ptr(rp), _lib.ptr(ci),
                                 _lib.ptr(deg), _lib.c_i64(rp.numel() - 1), _lib.c_i64(n),
                                 _lib.c_i64(ci.numel()), _lib.c_i64(dim), _lib.c_f32(1.0),
                                 _lib.c_i64(-1), _lib.ptr(None), _lib.ptr(None), _lib.ptr(ws),
                                 _lib.c_size(ws.numel()), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_agg_csr")
    return out


def _no_alloc(x, rp, ci, deg, dev):
    n, dim = x.shape
    out = torch.empty(rp.numel() - 1, dim, device=dev)
    rc = _lib.lib().yitu_agg_csr_noalloc(_lib.ptr(out), _lib.ptr(x), 0, _lib.ptr(rp), _lib.ptr(ci),
                                         _lib.ptr(deg), _lib.c_i64(rp.numel() - 1), _lib.c_i64(n),
                                         _lib.c_i64(ci.numel()), _lib.c_i64(dim), _lib.c_f32(1.0),
                                         _lib.c_i64(-1), _lib.stream_ptr(dev))
    return rc, out


def test_two_calls_in_a_row_second_one_smaller(dev):
    for scale, draws, dim, seed in ((13, 120000, 64, 3), (11, 30000, 32, 4)):
        indptr, indices = powerlaw_graph(scale, draws, seed)
        n = indptr.numel() - 1
        assert (indptr[1:] - indptr[:-1]).max() >= 128  # long rows: plan and partial rows in use
        x = torch.randn(n, dim, generator=torch.Generator().manual_seed(seed))
        deg = graphgen.gcn_norm(indptr)
        args = (x.to(dev), indptr.to(dev), indices.to(dev), deg.to(dev), dev)
        rc, got = _no_alloc(*args)
        _lib.check(rc, "yitu_agg_csr_noalloc")
        assert torch.equal(got, _with_workspace(*args))
        assert_close(got, oracle.row_agg(x.numpy(), indptr, indices, deg.numpy(), oracle.MODE_GCN))


def test_rejects_what_does_not_fit_the_static_array(dev):
    fn = _lib.lib().yitu_agg_csr_noalloc_max_bytes
    fn.restype = ctypes.c_size_t
    assert fn() == 32 << 20
    # sizes only: the call must fail before it touches any pointer
    rc = _lib.lib().yitu_agg_csr_noalloc(_lib.ptr(None), _lib.ptr(None), 0, _lib.ptr(None),
                                         _lib.ptr(None), _lib.ptr(None), _lib.c_i64(1 << 20),
                                         _lib.c_i64(1 << 20), _lib.c_i64(1 << 26), _lib.c_i64(128),
                                         _lib.c_f32(1.0), _lib.c_i64(-1), _lib.stream_ptr(dev))
    assert rc < 0
    assert b"static array" in _lib.lib().yitu_last_error()


def test_large_graph_of_short_rows_needs_no_scratch(dev):
    """A graph beyond the static array's worst-case bound is accepted when the caller
    states that no row reaches the planning threshold: nothing is planned, nothing is
    staged. (2^17 rows x 12 edges, F = 64: the bound asks for about 37 MiB.)"""
    assert _lib.lib().yitu_agg_csr_noalloc_init() == 0
    n, per_row, dim = 1 << 17, 12, 64
    g = torch.Generator().manual_seed(11)
    indptr = (torch.arange(n + 1, dtype=torch.int64) * per_row).to(torch.int32)
    indices = torch.randint(0, n, (n * per_row,), generator=g).to(torch.int32)
    x = torch.randn(n, dim, generator=g)
    deg = graphgen.gcn_norm(indptr)
    need = _lib.size_fn("yitu_spmm_workspace_bytes")(_lib.c_i64(indices.numel()), _lib.c_i64(dim),
                                                     _lib.c_int(0))
    assert need > (32 << 20)
    xd, rp, ci, dg = x.to(dev), indptr.to(dev), indices.to(dev), deg.to(dev)
    out = torch.empty(n, dim, device=dev)
    args = (_lib.ptr(out), _lib.ptr(xd), 0, _lib.ptr(rp), _lib.ptr(ci), _lib.ptr(dg), _lib.c_i64(n),
            _lib.c_i64(n), _lib.c_i64(ci.numel()), _lib.c_i64(dim), _lib.c_f32(1.0))
    rc = _lib.lib().yitu_agg_csr_noalloc(*args, _lib.c_i64(-1), _lib.stream_ptr(dev))
    assert rc < 0  # without the hint the worst case does not fit
    rc = _lib.lib().yitu_agg_csr_noalloc(*args, _lib.c_i64(per_row), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_agg_csr_noalloc")
    assert_close(out, oracle.row_agg(x.numpy(), indptr, indices, deg.numpy(), oracle.MODE_GCN))
