"""CPU oracle for YiTu's sparse message-passing path (TEST INFRASTRUCTURE ONLY).

Thin ctypes front end over ``libyitu_oracle.so`` (built from ``yitu_oracle.c`` by
the Makefile beside it) plus the numpy glue that composes the reference's host
code (the dense ``torch::mm`` calls around the aggregation kernels). Only the
test-suite, the smoke check and the benchmark's ``cpu_baseline`` leg may import
this package; the shipped ``yitu_amd`` package never does.

Every function cites the reference lines it restates; paths are relative to the
reference checkout. Each is pinned in tests/test_oracle_module1.py and
tests/test_oracle_module2.py against an independent formulation (scipy's CSR
product, dense torch algebra with autograd, closed forms, brute-force loops).

Parity unpinned: the exact permutation of the Rabbit-Order reorder. Its reference
(rabbit_order.hpp) needs boost, which is absent, and holds no golden permutation,
so there is no function for it here; tests/test_rabbit.py pins the algorithm's
definition on small graphs and its invariants instead.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libyitu_oracle.so")
_lib = None


def build(force=False):
    """Compile the C restatement (and oracle/_ref when the reference is mounted)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libyitu_oracle.so"])
    subprocess.check_call(["make", "-C", _HERE, "ref"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_build_part_count.restype = ctypes.c_int64
        _lib.orc_stitch_csr.restype = ctypes.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


I64 = ctypes.c_int64

# --------------------------------------------------------------------------- #
# module 1: ccsrc/kernel
# --------------------------------------------------------------------------- #


def build_part(part_size, indptr):
    """YiTu_GNN.cpp:203-245. Returns int32 (partPtr[P+1], part2Node[P])."""
    indptr = _i32(indptr)
    n = indptr.shape[0] - 1
    cnt = lib().orc_build_part_count(ctypes.c_int(part_size), _p(indptr), I64(n))
    part_ptr = np.zeros(cnt + 1, dtype=np.int32)
    part2node = np.zeros(cnt, dtype=np.int32)
    lib().orc_build_part(ctypes.c_int(part_size), _p(indptr), I64(n), _p(part_ptr), _p(part2node))
    return part_ptr, part2node


MODE_GCN, MODE_SAG, MODE_GIN = 0, 1, 2


def group_agg_f32(x, col, deg, part_ptr, part2node, mode, eps=1.0):
    """Float aggregation in the kernel's neighbour-group order (cu:320-415, 180-257, 621-694)."""
    x = _f32(x)
    n, dim = x.shape
    out = np.empty_like(x)
    deg = _f32(deg if deg is not None else np.ones(n))
    col, part_ptr, part2node = _i32(col), _i32(part_ptr), _i32(part2node)
    lib().orc_group_agg_f32(_p(out), _p(x), _p(col), _p(deg), _p(part_ptr), _p(part2node),
                            I64(part2node.shape[0]), I64(n), I64(dim), ctypes.c_int(mode),
                            ctypes.c_float(eps))
    return out


def row_agg(x, indptr, col, deg, mode, eps=1.0, f64=True):
    """Row-wise closed form; f64=True is the double-accumulate referee, False the timed float build."""
    x = _f32(x)
    n_src, dim = x.shape
    indptr, col = _i32(indptr), _i32(col)
    n = indptr.shape[0] - 1
    out = np.empty((n, dim), dtype=np.float32)
    deg = _f32(deg if deg is not None else np.ones(max(n, n_src)))
    fn = lib().orc_row_agg_f64 if f64 else lib().orc_row_agg_f32_omp
    fn(_p(out), _p(x), _p(indptr), _p(col), _p(deg), I64(n), I64(dim), ctypes.c_int(mode),
       ctypes.c_float(eps))
    return out


def row_agg_bf16(x_bits, indptr, col, deg, mode, eps=1.0):
    """bf16 features given as uint16 bit patterns; double accumulate, float out."""
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    n_src, dim = x_bits.shape
    indptr, col = _i32(indptr), _i32(col)
    n = indptr.shape[0] - 1
    out = np.empty((n, dim), dtype=np.float32)
    deg = _f32(deg if deg is not None else np.ones(max(n, n_src)))
    lib().orc_row_agg_bf16_f64(_p(out), _p(x_bits), _p(indptr), _p(col), _p(deg), I64(n), I64(dim),
                               ctypes.c_int(mode), ctypes.c_float(eps))
    return out


def _mm(a, b):
    return (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)


def gcn_forward(x, w, indptr, col, deg):
    """spmm_forward_cuda, cu:264-317: T = X.W (cu:276), out = aggregate(T)."""
    return row_agg(_mm(_f32(x), _f32(w)), indptr, col, deg, MODE_GCN)


def gcn_backward(d_out, x, w, indptr, col, deg):
    """spmm_backward_cuda, cu:422-475: G = aggregate(dY) with the SAME CSR, dX = G.W^T, dW = X^T.G."""
    g = row_agg(d_out, indptr, col, deg, MODE_GCN)
    return _mm(g, _f32(w).T), _mm(_f32(x).T, g)


def gin_forward(x, w, indptr, col, eps):
    """spmm_forward_cuda_gin, cu:563-618: A = eps*sum_j X[j]; out = A.W; returns (out, A)."""
    agg = row_agg(x, indptr, col, None, MODE_GIN, eps)
    return _mm(agg, _f32(w)), agg


def gin_backward(d_out, x_agg, w, indptr, col, eps):
    """spmm_backward_cuda_gin, cu:701-751: dW = X^T.dY (X is the saved aggregate), dX = eps*sum_j (dY.W^T)[j]."""
    d_w = _mm(_f32(x_agg).T, _f32(d_out))
    g = _mm(_f32(d_out), _f32(w).T)
    return row_agg(g, indptr, col, None, MODE_GIN, eps), d_w


def sag(x, indptr, col):
    """SAG_cuda, cu:104-177: out[r] = sum_j X[j]."""
    return row_agg(x, indptr, col, None, MODE_SAG)


# --------------------------------------------------------------------------- #
# module 2: YiTu_GNN/YiTu_H/src (graph_ext)
# --------------------------------------------------------------------------- #


def mh_spmm_forward(values, indptr, indices, feat, f64=True):
    """spmm_cuda.cu:4-21,44-62."""
    values, feat = _f32(values), _f32(feat)
    indptr, indices = _i32(indptr), _i32(indices)
    n_dst = indptr.shape[0] - 1
    _, h, f = feat.shape
    out = np.zeros((n_dst, h, f), dtype=np.float32)
    lib().orc_mh_spmm_fwd(_p(out), _p(values), _p(indptr), _p(indices), _p(feat), I64(n_dst),
                          I64(h), I64(f), ctypes.c_int(1 if f64 else 0))
    return out


def mh_spmm_backward(values, indptr, indices, feat, grad_out):
    """spmm_cuda.cu:24-42,64-86. Returns (grad_a [E,H], grad_x [Ns,H,F])."""
    values, feat, grad_out = _f32(values), _f32(feat), _f32(grad_out)
    indptr, indices = _i32(indptr), _i32(indices)
    n_dst = indptr.shape[0] - 1
    n_src, h, f = feat.shape
    grad_a = np.zeros_like(values)
    grad_x = np.zeros_like(feat)
    lib().orc_mh_spmm_bwd(_p(grad_a), _p(grad_x), _p(values), _p(indptr), _p(indices), _p(feat),
                          _p(grad_out), I64(n_dst), I64(n_src), I64(h), I64(f))
    return grad_a, grad_x


def csr_transpose(indptr, indices, n_src):
    """By-source view (t_indptr, t_rows, t_perm) of a CSR: stable sort on the column."""
    indptr, indices = _i32(indptr), _i32(indices)
    n_dst = indptr.shape[0] - 1
    t_indptr = np.zeros(n_src + 1, dtype=np.int32)
    t_rows = np.zeros(indices.shape[0], dtype=np.int32)
    t_perm = np.zeros(indices.shape[0], dtype=np.int32)
    lib().orc_csr_transpose(_p(t_indptr), _p(t_rows), _p(t_perm), _p(indptr), _p(indices),
                            I64(n_dst), I64(n_src))
    return t_indptr, t_rows, t_perm


def mh_spmm_backward_omp(values, indptr, indices, feat, grad_out, transposed, need_grad_a=True,
                         need_grad_x=True):
    """Float, all cores, for timing: the gradients of mh_spmm_backward without atomics
    (grad_x over the by-source view ``transposed`` = csr_transpose(...))."""
    values, feat, grad_out = _f32(values), _f32(feat), _f32(grad_out)
    indptr, indices = _i32(indptr), _i32(indices)
    t_indptr, t_rows, t_perm = transposed
    n_dst = indptr.shape[0] - 1
    n_src, h, f = feat.shape
    grad_a = np.empty_like(values) if need_grad_a else None
    grad_x = np.empty_like(feat) if need_grad_x else None
    lib().orc_mh_spmm_bwd_omp(_p(grad_a) if need_grad_a else None,
                              _p(grad_x) if need_grad_x else None, _p(values), _p(indptr),
                              _p(indices), _p(feat), _p(grad_out), _p(t_indptr), _p(t_rows),
                              _p(t_perm), I64(n_dst), I64(n_src), I64(h), I64(f))
    return grad_a, grad_x


def sddmm_backward_omp(indptr, indices, query, key, attn, grad_out, transposed):
    """Float, all cores, for timing: sddmm_backward with grad_key summed by source."""
    query, key, attn, grad_out = _f32(query), _f32(key), _f32(attn), _f32(grad_out)
    indptr, indices = _i32(indptr), _i32(indices)
    t_indptr, _, t_perm = transposed
    gq = np.empty_like(query)
    gk = np.empty_like(key)
    scratch = np.empty_like(attn)
    lib().orc_sddmm_bwd_omp(_p(gq), _p(gk), _p(scratch), _p(indptr), _p(indices), _p(query),
                            _p(key), _p(attn), _p(grad_out), _p(t_indptr), _p(t_perm),
                            I64(indptr.shape[0] - 1), I64(key.shape[0]), I64(query.shape[-1]),
                            I64(query.shape[0]))
    return gq, gk


def gemm_omp(a, b, trans_a=False, trans_b=False):
    """Float, all cores, for timing: op(a) . op(b)."""
    a, b = _f32(a), _f32(b)
    n, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
    m = b.shape[0] if trans_b else b.shape[1]
    assert (b.shape[1] if trans_b else b.shape[0]) == k
    c = np.empty((n, m), dtype=np.float32)
    lib().orc_gemm_f32_omp(_p(c), _p(a), _p(b), I64(n), I64(m), I64(k),
                           ctypes.c_int(1 if trans_a else 0), ctypes.c_int(1 if trans_b else 0))
    return c


def sddmm_forward(indptr, indices, query, key):
    """sddmm_cuda.cu:5-33,69-89. query [n_bid,Nd,H], key [Ns,H] -> attn [E,H]."""
    query, key = _f32(query), _f32(key)
    indptr, indices = _i32(indptr), _i32(indices)
    assert query.ndim == 3 and key.ndim == 2 and query.shape[1] == indptr.shape[0] - 1
    h = query.shape[-1]
    attn = np.zeros((indices.shape[0], h), dtype=np.float32)
    lib().orc_sddmm_fwd(_p(attn), _p(indptr), _p(indices), _p(query), _p(key),
                        I64(indptr.shape[0] - 1), I64(h))
    return attn


def sddmm_backward(indptr, indices, query, key, attn, grad_out):
    """sddmm_cuda.cu:36-67,91-118. Returns (grad_query, grad_key)."""
    query, key, attn, grad_out = _f32(query), _f32(key), _f32(attn), _f32(grad_out)
    indptr, indices = _i32(indptr), _i32(indices)
    gq = np.zeros_like(query)
    gk = np.zeros_like(key)
    lib().orc_sddmm_bwd(_p(gq), _p(gk), _p(indptr), _p(indices), _p(query), _p(key), _p(attn),
                        _p(grad_out), I64(indptr.shape[0] - 1), I64(key.shape[0]),
                        I64(query.shape[-1]), I64(query.shape[0]))
    return gq, gk


def hfused_forward(spmm_values, spmm_indptr, spmm_indices, spmm_feat, sddmm_indptr, sddmm_indices,
                   sddmm_query, sddmm_key):
    """hfused_cuda.cu:5-45: the two independent ops of one launch."""
    return (mh_spmm_forward(spmm_values, spmm_indptr, spmm_indices, spmm_feat),
            sddmm_forward(sddmm_indptr, sddmm_indices, sddmm_query, sddmm_key))


def stitch_csr(blocks):
    """block.py:36-67. blocks = [(indptr, indices, n_src), ...] -> (indptr, indices, n_cols)."""
    n_blk = len(blocks)
    ptrs = [_i32(b[0]) for b in blocks]
    idxs = [_i32(b[1]) for b in blocks]
    n_rows = ptrs[0].shape[0] - 1
    assert all(p.shape[0] - 1 == n_rows for p in ptrs)
    total = int(sum(i.shape[0] for i in idxs))
    new_indptr = np.zeros(n_rows + 1, dtype=np.int32)
    new_indices = np.zeros(total, dtype=np.int32)
    arr_t = ctypes.c_void_p * n_blk
    n_srcs = np.asarray([b[2] for b in blocks], dtype=np.int64)
    rc = lib().orc_stitch_csr(ctypes.c_int(n_blk), I64(n_rows), arr_t(*[p.ctypes.data for p in ptrs]),
                              arr_t(*[i.ctypes.data for i in idxs]), _p(n_srcs), _p(new_indptr),
                              _p(new_indices))
    if rc != 0:
        raise AssertionError("stitch_csr: more than 16 blocks or column id above 2**24")
    return new_indptr, new_indices, int(n_srcs.sum())


def b2gemm(x, w_a, w_b):
    """fc_cuda.cu:4-75: y_a = x.w_a^T, y_b = x.w_b^T."""
    x, w_a, w_b = _f32(x), _f32(w_a), _f32(w_b)
    n, k = x.shape
    m = w_a.shape[0]
    ys = []
    for w in (w_a, w_b):
        y = np.empty((n, m), dtype=np.float32)
        lib().orc_gemm_nt_f64(_p(y), _p(x), _p(w), I64(n), I64(m), I64(k))
        ys.append(y)
    return ys


def b2gemm_backward(x, w_a, w_b, grad_a, grad_b):
    """fc_cuda.cu:77-215: dw_* = grad_*^T.x; dx = grad_a.w_a + grad_b.w_b. Returns (dx, dw_a, dw_b)."""
    x64 = _f32(x).astype(np.float64)
    ga, gb = _f32(grad_a).astype(np.float64), _f32(grad_b).astype(np.float64)
    dx = ga @ _f32(w_a).astype(np.float64) + gb @ _f32(w_b).astype(np.float64)
    return dx.astype(np.float32), (ga.T @ x64).astype(np.float32), (gb.T @ x64).astype(np.float32)
