"""Argument errors at the C ABI: every bad call returns a non-zero code with a message
in yitu_last_error() before anything is launched (the reference ends the process on a
kernel failure, YiTu_GNN_kernel.cu:309-314), and the library keeps working afterwards."""
import ctypes

import pytest
import torch

from yitu_amd import _lib, graph_ext

pytestmark = pytest.mark.gpu

P, I64, I32, F32, SZ = _lib.ptr, _lib.c_i64, _lib.c_int, _lib.c_f32, _lib.c_size


def _fails(rc, text):
    assert rc != 0
    msg = _lib.lib().yitu_last_error().decode()
    assert text in msg, msg


def test_bad_arguments_are_reported_not_launched(dev):
    L = _lib.lib()
    st = _lib.stream_ptr(dev)
    n, nnz, h, f = 40, 120, 2, 8
    indptr = torch.arange(0, nnz + 1, 3, dtype=torch.int32, device=dev)
    indices = torch.randint(0, n, (nnz,), dtype=torch.int32, device=dev)
    values = torch.rand(nnz, h, device=dev)
    x = torch.randn(n, h, f, device=dev)
    out = torch.empty(n, h, f, device=dev)
    ws = _lib.workspace(1 << 16, dev)
    none = P(None)

    def spmm(out_t=out, n_dst=n, n_src=n, edges=nnz, feats=x):
        return L.yitu_spmm_forward(P(out_t), P(values), P(indptr), P(indices), P(feats), I64(n_dst),
                                   I64(n_src), I64(edges), I64(h), I64(f), I64(3), none, P(ws),
                                   SZ(ws.numel()), st)

    _fails(spmm(n_dst=-1), "negative size")
    _fails(spmm(n_src=(1 << 24) + 1), "out of range")
    _fails(spmm(out_t=None), "null output")
    _fails(spmm(feats=None), "null input")
    assert spmm() == 0  # and a good call still works

    q = torch.randn(n, h, device=dev)
    gq, gk, gx = torch.empty(n, h, device=dev), torch.empty(n, h, device=dev), torch.empty_like(x)
    scratch = torch.empty(nnz, h, device=dev)
    tr = graph_ext.transposed(indptr, indices, n)
    rc = L.yitu_gat_backward(P(gq), P(gk), P(gx), P(scratch), P(scratch.clone()), P(indptr),
                             P(indices), P(q), P(q), P(x), none, none, none, P(out), P(tr.t_indptr),
                             P(tr.t_rows), P(tr.t_perm), I64(n), I64(n), I64(nnz), I64(h), I64(f), I64(3),
                             I64(64), none, none, I32(0), P(ws), SZ(ws.numel()), st)
    _fails(rc, "attn or the row statistics")

    a, b = torch.randn(16, 8, device=dev), torch.randn(8, 24, device=dev)
    c = torch.empty(16, 24, device=dev)

    def sgemm(ldc=24, lda=8):
        return L.yitu_sgemm(P(c), P(a), P(b), I64(16), I64(24), I64(8), I32(0), I32(0), I64(lda),
                            I64(24), I64(ldc), I32(0), none, SZ(0), st)

    _fails(sgemm(ldc=23), "out of range")
    _fails(sgemm(lda=7), "leading dimension")
    assert sgemm() == 0
    torch.cuda.synchronize()
    assert torch.allclose(c, a @ b, atol=1e-4)

    tables = (ctypes.c_void_p * 1)(c.data_ptr())
    rc = L.yitu_sgemm_typed(tables, None, None, None, None, I64(1), I64(24), I32(0), I32(0), I64(8),
                            I64(24), I64(24), I32(0), none, SZ(0), st)
    _fails(rc, "null problem table")

    colsum = torch.empty(24, device=dev)
    rc = L.yitu_column_sum(P(colsum), P(c), I64(16), I64(24), none, SZ(0), st)
    _fails(rc, "workspace too small")
    assert torch.equal(graph_ext.column_sum(c), graph_ext.column_sum(c))


def test_typed_bf16_products_report_bad_arguments(dev):
    """The typed bf16 entry points take host arrays of device pointers: null lists, null
    operands of a problem that has rows, unaligned widths and a short workspace are all
    reported; an empty list and a problem without rows are not errors."""
    L = _lib.lib()
    st = _lib.stream_ptr(dev)
    none = P(None)
    a = torch.randn(64, 64, device=dev).to(torch.bfloat16)
    w = torch.randn(32, 64, device=dev).to(torch.bfloat16)
    c = torch.empty(64, 32, device=dev)
    ws = _lib.workspace(1 << 20, dev)
    ptrs = lambda *ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() if t is not None else None
                                                      for t in ts])
    rows = lambda *v: (ctypes.c_int64 * len(v))(*v)

    def typed(cs=ptrs(c), as_=ptrs(a), bs=ptrs(w), m=rows(64), count=1, k=64, lda=64):
        return L.yitu_gemm_bf16_typed(cs, I32(0), as_, bs, m, I64(count), I64(32), I64(k), I32(1),
                                      I64(lda), I64(64), I64(32), P(ws), SZ(ws.numel()), st)

    assert typed() == 0
    assert typed(count=0) == 0
    _fails(typed(cs=None), "null pointer list")
    _fails(typed(as_=ptrs(None)), "null operand")
    _fails(typed(k=60, lda=60), "multiples of 8")
    _fails(typed(m=rows(-1)), "row count out of range")
    assert typed(as_=ptrs(None), m=rows(0)) == 0  # nothing to read for a type without rows

    g = torch.randn(64, 32, device=dev).to(torch.bfloat16)
    dw = torch.empty(64, 32, device=dev)

    def tn(cs=ptrs(dw), as_=ptrs(a), bs=ptrs(g), m=rows(64), ki=64, ws_bytes=ws.numel()):
        return L.yitu_gemm_bf16_tn_typed(cs, as_, bs, m, I64(1), I64(ki), I64(32), I64(64), I64(32),
                                         I64(32), I32(0), P(ws), SZ(ws_bytes), st)

    assert tn() == 0
    _fails(tn(ws_bytes=16), "workspace too small")
    _fails(tn(cs=ptrs(None)), "null operand")
    _fails(tn(ki=60), "multiples of 8")
    assert tn() == 0  # and a good call still works
    torch.cuda.synchronize()
    want = a.float().t() @ g.float()
    assert torch.allclose(dw, want, rtol=1e-4, atol=1e-3)


def test_typed_linear_forward_reports_bad_arguments(dev):
    """Host tables of device pointers: a null table, a null operand of a type that has rows
    and sizes out of range are reported; no types, a type without rows, a null bias table
    and null bias entries are not errors."""
    L = _lib.lib()
    st = _lib.stream_ptr(dev)
    x = torch.randn(64, 48, device=dev)
    w = torch.randn(32, 48, device=dev)
    b = torch.randn(32, device=dev)
    y = torch.empty(64, 32, device=dev)
    ws = _lib.workspace(1 << 20, dev)
    ptrs = lambda *ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() if t is not None else None
                                                      for t in ts])
    rows = lambda *v: (ctypes.c_int64 * len(v))(*v)

    def call(ys=ptrs(y), xs=ptrs(x), wts=ptrs(w), bs=ptrs(b), m=rows(64), count=1, n=32, k=48):
        return L.yitu_linear_forward_typed(ys, xs, wts, bs, m, I64(count), I64(n), I64(k), P(ws),
                                           SZ(ws.numel()), st)

    assert call() == 0
    torch.cuda.synchronize()
    assert torch.allclose(y, x @ w.t() + b, rtol=1e-4, atol=1e-4)
    assert call(count=0) == 0
    assert call(bs=None) == 0
    assert call(bs=ptrs(None)) == 0
    torch.cuda.synchronize()
    assert torch.allclose(y, x @ w.t(), rtol=1e-4, atol=1e-4)
    _fails(call(ys=None), "null problem table")
    _fails(call(xs=ptrs(None)), "null operand")
    _fails(call(m=rows(-1)), "size out of range")
    _fails(call(n=-1), "negative size")
    assert call(xs=ptrs(None), m=rows(0)) == 0
