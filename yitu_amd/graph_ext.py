"""Drop-in for the reference's ``graph_ext`` extension module
(YiTu_GNN/YiTu_H/src/entry.cpp:184-193): ``spmm_forward/backward``,
``sddmm_forward/backward``, ``hfused_forward/backward``, ``b2gemm`` and
``b2gemm_backward`` with the reference's argument order, dtype checks
(CHECK_INPUT: device + contiguous + exact dtype, common.h:6-12) and return
arity, backed by libyitu_hip.so.

Observable differences from the reference:
  * any number of destination rows works (the reference launches
    ``dim3(n_heads, n_nodes)`` and silently returns zeros above 65,535 rows,
    spmm_cuda.cu:57);
  * the edge softmax subtracts the row maximum (the reference does not,
    sddmm_cuda.cu:15-21); equal within tolerance wherever the reference does
    not overflow;
  * backward scatters are gathers over a transposed structure that is built on
    the device once per graph and cached on the ``indices`` tensor: results are
    bitwise reproducible, unlike the reference's float atomics;
  * ``hfused_backward`` returns ``[grad_a, grad_x, grad_query, grad_key]``; the
    reference version drops the first two and mis-indexes heads
    (hfused_cuda.cu:59,186) and is unreachable from its Python side.
"""
import weakref

import torch

from . import _lib
from ._lib import c_i64, c_int, c_size, check, ptr, stream_ptr

COL_MASK = 0xFFFFFF


def _check(t, dtype, name, dim=None):
    # CHECK_INPUT(x, dtype) of the reference (common.h:6-12)
    _lib.require_device(t)
    _lib.require_dtype(t, dtype, name)
    if dim is not None and t.dim() != dim:
        raise RuntimeError("%s must be %d-D, got %d-D" % (name, dim, t.dim()))


def _size_fn(name):
    fn = getattr(_lib.lib(), name)
    fn.restype = c_size
    return fn


# --------------------------------------------------------------------------- #
# transposed structure, cached per (indptr, indices) pair
# --------------------------------------------------------------------------- #
class _Transposed:
    __slots__ = ("t_indptr", "t_rows", "t_perm", "max_degree_t", "n_src", "plan_t")


_transposed = {}


def transposed(indptr, indices, n_src):
    """By-source view (t_indptr, t_rows, t_perm) of a packed CSR, built on the
    device on first use and kept for as long as ``indices`` is alive."""
    key = (id(indices), indices.data_ptr(), indices._version, id(indptr), indptr.data_ptr(),
           indptr._version, int(n_src))
    hit = _transposed.get(key)
    if hit is not None:
        return hit.get(indices.device)
    dev = indices.device
    n_rows = indptr.numel() - 1
    nnz = indices.numel()
    t = _Transposed()
    t.n_src = int(n_src)
    t.t_indptr = torch.empty(n_src + 1, dtype=torch.int32, device=dev)
    t.t_rows = torch.empty(nnz, dtype=torch.int32, device=dev)
    t.t_perm = torch.empty(nnz, dtype=torch.int32, device=dev)
    ws = _lib.workspace(_size_fn("yitu_csr_transpose_workspace_bytes")(c_i64(nnz), c_i64(n_src)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_csr_transpose(ptr(t.t_indptr), ptr(t.t_rows), ptr(t.t_perm), ptr(indptr),
                                           ptr(indices), c_i64(n_rows), c_i64(n_src), c_i64(nnz),
                                           c_int(COL_MASK), ptr(ws), c_size(ws.numel()),
                                           stream_ptr(dev))
    check(rc, "yitu_csr_transpose")
    t.max_degree_t = _lib.max_degree(t.t_indptr)
    t.plan_t = _lib.row_plan(t.t_indptr, t.t_rows, n_rows, 0x7FFFFFFF)
    _transposed[key] = _lib._Built(t, dev)
    weakref.finalize(indices, _transposed.pop, key, None)
    return t


def forget(*tensors):
    """Drops everything derived from the given index / weight tensors: widest row, row
    plan, by-source view, by-source weight copies. Needed after a tensor was refilled in
    place through its raw pointer (kernels of this library, DLPack consumers): torch's
    version counter, which the caches key on, does not see such writes."""
    idents = {id(t) for t in tensors if t is not None}
    derived = []
    for key in [k for k in _transposed if k[0] in idents or k[3] in idents]:
        t = _transposed.pop(key).value
        derived += [t.t_indptr, t.t_rows]
    _lib.forget(*tensors, *derived)
    for ident in list(_values_seen):
        state = _values_seen[ident]
        if ident in idents or state[2] in idents or state[4] in idents:
            _forget_values(ident)


# --------------------------------------------------------------------------- #
# SpMM
# --------------------------------------------------------------------------- #
def spmm_forward(values, indptr, indices, features, out_dtype=torch.float32):
    """out[r,h,k] = sum_i values[i,h] * features[col_i,h,k] (entry.cpp:80-90).
    ``features`` fp32 like the reference, or bf16 (fp32 accumulate; fp32 out, or bf16 rows
    with ``out_dtype=torch.bfloat16``: one rounding per output)."""
    _check(values, torch.float32, "values", 2)
    _check(indptr, torch.int32, "indptr", 1)
    _check(indices, torch.int32, "indices", 1)
    bf16 = features.dtype == torch.bfloat16
    _check(features, torch.bfloat16 if bf16 else torch.float32, "features", 3)
    dev = _lib.require_device(values, indptr, indices, features)
    n_dst = indptr.numel() - 1
    n_src, h, f = features.shape
    nnz = indices.numel()
    if values.shape[0] != nnz or values.shape[1] != h:
        raise RuntimeError("values must be [n_edges, n_heads]")
    if out_dtype not in (torch.float32, torch.bfloat16) or (out_dtype == torch.bfloat16
                                                            and not (bf16 and f % 8 == 0)):
        raise RuntimeError("out_dtype is float32, or bfloat16 for bf16 features whose head "
                           "width is a multiple of 8")
    out = torch.empty((n_dst, h, f), dtype=out_dtype, device=dev)
    maxdeg = _lib.max_degree(indptr)
    plan = _lib.row_plan(indptr, indices, n_src, COL_MASK)
    need = _size_fn("yitu_spmm_workspace_bytes")(c_i64(nnz), c_i64(h * f), c_int(1)) \
        if plan is not None and maxdeg >= 64 else 0
    ws = _lib.workspace(need, dev)
    entry = _lib.lib().yitu_spmm_forward
    if bf16:
        entry = _lib.lib().yitu_spmm_forward_bf16_rows if out_dtype == torch.bfloat16 \
            else _lib.lib().yitu_spmm_forward_bf16
    with torch.cuda.device(dev):
        rc = entry(ptr(out), ptr(values), ptr(indptr), ptr(indices), ptr(features), c_i64(n_dst),
                   c_i64(n_src), c_i64(nnz), c_i64(h), c_i64(f), c_i64(maxdeg), ptr(plan), ptr(ws),
                   c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_spmm_forward")
    return out


# Edge weights that take no gradient are usually constants of the graph (norms), passed
# again every step. The backward reads them through the edge permutation, a scattered
# 4-byte read per edge and head; the second time the same tensor (same version) comes
# by, a copy in by-source order is made and kept for as long as the tensor lives.
_values_seen = {}       # id(values) -> state of the tensor when it last came by
_values_by_source = {}  # id(values) -> (that state, the copy in by-source order)


def _by_source_values(values, indptr, indices, n_src, force=False):
    """The copy of ``values`` in by-source order once the same tensor has come by twice
    (``force``: at once), else None."""
    ident = id(values)
    state = (values.data_ptr(), values._version, id(indices), indices._version, id(indptr),
             indptr._version, int(n_src))
    hit = _values_by_source.get(ident)
    if hit is not None and hit[0] == state:
        return hit[1]
    if _values_seen.get(ident) != state:
        if ident not in _values_seen:
            weakref.finalize(values, _forget_values, ident)
        _values_seen[ident] = state
        _values_by_source.pop(ident, None)
        if not force:
            return None
    tr = transposed(indptr, indices, n_src)
    copy = values.index_select(0, tr.t_perm)
    _values_by_source[ident] = (state, copy)
    return copy


def _forget_values(ident):
    _values_seen.pop(ident, None)
    _values_by_source.pop(ident, None)


def spmm_backward(values, indptr, indices, features, grad_out, need_grad_a=True,
                  need_grad_x=True, grad_x_dtype=torch.float32):
    """Returns [grad_a [E,H], grad_x [Ns,H,F]] (entry.cpp:92-104). A gradient
    that the caller does not need is skipped and returned as None. ``grad_x_dtype``:
    bfloat16 with bf16 ``grad_out`` rows writes grad_x as bf16 rows (fp32 sums)."""
    _check(values, torch.float32, "values", 2)
    _check(indptr, torch.int32, "indptr", 1)
    _check(indices, torch.int32, "indices", 1)
    bf16 = grad_out.dtype == torch.bfloat16
    if bf16:
        # bf16 pipeline: gradient rows in bf16, fp32 sums and fp32 grad_x out. The edge
        # weights of such a pipeline are constants of the graph (norms): grad_a is not
        # offered, and the forward's features are not read at all.
        if need_grad_a:
            raise RuntimeError("spmm_backward with bf16 rows computes grad_x only "
                               "(need_grad_a=False): the reference's op is fp32")
        if features.dtype not in (torch.float32, torch.bfloat16) or features.dim() != 3:
            raise RuntimeError("features must be a [n_src, H, F] tensor")
        _check(grad_out, torch.bfloat16, "grad_out", 3)
    else:
        _check(features, torch.float32, "features", 3)
        _check(grad_out, torch.float32, "grad_out", 3)
    dev = _lib.require_device(values, indptr, indices, features, grad_out)
    n_dst = indptr.numel() - 1
    n_src, h, f = features.shape
    nnz = indices.numel()
    if grad_out.shape[0] != n_dst or grad_out.shape[1] != h or grad_out.shape[2] != f:
        raise RuntimeError("grad_out must be [n_dst, n_heads, n_features]")
    if not (need_grad_a or need_grad_x):
        return [None, None]
    if bf16:
        if n_dst > COL_MASK:
            raise RuntimeError("bf16 spmm_backward needs at most 2**24 destination rows")
        # grad_x[c] = sum over the edges of source c of values[e] * grad_out[row_e]: the
        # forward product over the by-source structure, weights copied into that order
        tr = transposed(indptr, indices, n_src)
        values_t = _by_source_values(values, indptr, indices, n_src, force=True)
        return [None, spmm_forward(values_t, tr.t_indptr, tr.t_rows, grad_out,
                                   out_dtype=grad_x_dtype)]
    if grad_x_dtype != torch.float32:
        raise RuntimeError("grad_x_dtype other than float32 needs bf16 grad_out rows")
    if not need_grad_a and nnz > 0 and n_dst <= COL_MASK:
        values_t = _by_source_values(values, indptr, indices, n_src)
        if values_t is not None:
            # constant edge weights, seen before: grad_x is a forward product over the
            # by-source structure, its weights already in that order
            tr = transposed(indptr, indices, n_src)
            return [None, spmm_forward(values_t, tr.t_indptr, tr.t_rows, grad_out)]
    grad_a = torch.empty_like(values) if need_grad_a else None
    grad_x = torch.empty_like(features) if need_grad_x else None
    tr = transposed(indptr, indices, n_src)
    maxdeg = _lib.max_degree(indptr)
    plan = _lib.row_plan(indptr, indices, n_src, COL_MASK)
    need = 0
    if max(maxdeg, tr.max_degree_t) >= 64:
        need = _size_fn("yitu_spmm_workspace_bytes")(c_i64(nnz), c_i64(h * f), c_int(1))
    ws = _lib.workspace(need, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_spmm_backward(ptr(grad_a), ptr(grad_x), ptr(values), ptr(indptr),
                                           ptr(indices), ptr(features), ptr(grad_out),
                                           ptr(tr.t_indptr), ptr(tr.t_rows), ptr(tr.t_perm),
                                           c_i64(n_dst), c_i64(n_src), c_i64(nnz), c_i64(h), c_i64(f),
                                           c_i64(maxdeg), c_i64(tr.max_degree_t), ptr(plan),
                                           ptr(tr.plan_t), ptr(ws), c_size(ws.numel()),
                                           stream_ptr(dev))
    check(rc, "yitu_spmm_backward")
    return [grad_a, grad_x]


def edge_dot(indptr, indices, dst_feat, src_feat):
    """e[i,h] = <dst_feat[row_i,h,:], src_feat[col_i,h,:]> for every edge i: the
    SDDMM-dot inside spmm_backward (spmm_cuda.cu:33-35) as an op of its own."""
    _check(indptr, torch.int32, "indptr", 1)
    _check(indices, torch.int32, "indices", 1)
    _check(dst_feat, torch.float32, "dst_feat", 3)
    _check(src_feat, torch.float32, "src_feat", 3)
    dev = _lib.require_device(indptr, indices, dst_feat, src_feat)
    n_dst = indptr.numel() - 1
    n_src, h, f = src_feat.shape
    nnz = indices.numel()
    if dst_feat.shape != (n_dst, h, f):
        raise RuntimeError("dst_feat must be [n_dst, H, F] matching src_feat's H and F")
    out = torch.empty((nnz, h), dtype=torch.float32, device=dev)
    maxdeg = _lib.max_degree(indptr)
    plan = _lib.row_plan(indptr, indices, n_src, COL_MASK)
    ws = _lib.workspace(0, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_spmm_backward(ptr(out), ptr(None), ptr(None), ptr(indptr), ptr(indices),
                                           ptr(src_feat), ptr(dst_feat), ptr(None), ptr(None),
                                           ptr(None), c_i64(n_dst), c_i64(n_src), c_i64(nnz),
                                           c_i64(h), c_i64(f), c_i64(maxdeg), c_i64(-1), ptr(plan),
                                           ptr(None), ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_spmm_backward")
    return out


# --------------------------------------------------------------------------- #
# SDDMM + LeakyReLU + edge softmax
# --------------------------------------------------------------------------- #
def _sddmm_shapes(indptr, indices, query, key):
    _check(indptr, torch.int32, "indptr", 1)
    _check(indices, torch.int32, "indices", 1)
    _check(query, torch.float32, "query", 3)
    _check(key, torch.float32, "key", 2)
    if query.size(-1) != key.size(-1):
        raise RuntimeError("query and key disagree on the number of heads")
    if query.size(1) != indptr.numel() - 1:
        raise RuntimeError("query.size(1) must equal the number of destination rows")
    if query.size(0) > 16:
        raise RuntimeError("at most 16 query blocks (the block tag is 4 bits wide)")
    return indptr.numel() - 1, key.size(0), indices.numel(), key.size(1), query.size(0)


def sddmm_forward(indptr, indices, query, key):
    """attn[i,h] = softmax_{row, bid}(leaky_relu(query[bid,r,h] + key[col,h], 0.2)) (entry.cpp:106-116)."""
    n_dst, n_src, nnz, h, n_bid = _sddmm_shapes(indptr, indices, query, key)
    dev = _lib.require_device(indptr, indices, query, key)
    attn = torch.empty((nnz, h), dtype=torch.float32, device=dev)
    maxdeg = _lib.max_degree(indptr)
    plan = _lib.row_plan(indptr, indices, n_src, COL_MASK) if n_bid == 1 else None
    need = 0
    if maxdeg >= 64:
        need = _size_fn("yitu_sddmm_workspace_bytes")(c_i64(n_dst), c_i64(nnz), c_i64(h),
                                                      c_i64(n_bid), c_int(1))
    ws = _lib.workspace(need, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_sddmm_forward(ptr(attn), ptr(indptr), ptr(indices), ptr(query), ptr(key),
                                           c_i64(n_dst), c_i64(n_src), c_i64(nnz), c_i64(h),
                                           c_i64(n_bid), c_i64(maxdeg), ptr(plan), ptr(ws),
                                           c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_sddmm_forward")
    return attn


def sddmm_backward(indptr, indices, query, key, attn_values, grad_out, deterministic=True):
    """Returns [grad_query, grad_key] (entry.cpp:118-134). ``deterministic=False``
    selects the float-atomic scatter for grad_key (the reference's form)."""
    n_dst, n_src, nnz, h, n_bid = _sddmm_shapes(indptr, indices, query, key)
    _check(attn_values, torch.float32, "attn_values", 2)
    _check(grad_out, torch.float32, "grad_out", 2)
    if attn_values.shape != (nnz, h) or grad_out.shape != attn_values.shape:
        raise RuntimeError("attn_values and grad_out must be [n_edges, n_heads]")
    dev = _lib.require_device(indptr, indices, query, key, attn_values, grad_out)
    grad_query = torch.empty_like(query)
    grad_key = torch.empty_like(key)
    maxdeg = _lib.max_degree(indptr)
    tr = transposed(indptr, indices, n_src) if deterministic else None
    grad_edge = torch.empty_like(attn_values) if deterministic else None
    plan = _lib.row_plan(indptr, indices, n_src, COL_MASK) if n_bid == 1 and deterministic else None
    need = 0
    if maxdeg >= 64 or (tr is not None and tr.max_degree_t >= 64):
        need = _size_fn("yitu_sddmm_workspace_bytes")(c_i64(n_dst), c_i64(nnz), c_i64(h),
                                                      c_i64(n_bid), c_int(1))
    ws = _lib.workspace(need, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_sddmm_backward(
            ptr(grad_query), ptr(grad_key), ptr(grad_edge), ptr(indptr), ptr(indices), ptr(query),
            ptr(key), ptr(attn_values), ptr(grad_out), ptr(tr.t_indptr if tr else None),
            ptr(tr.t_perm if tr else None), c_i64(n_dst), c_i64(n_src), c_i64(nnz), c_i64(h),
            c_i64(n_bid), c_i64(maxdeg), c_i64(tr.max_degree_t if tr else -1), ptr(plan),
            ptr(tr.plan_t if tr else None), ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_sddmm_backward")
    return [grad_query, grad_key]


# --------------------------------------------------------------------------- #
# horizontally fused SpMM || SDDMM
# --------------------------------------------------------------------------- #
def hfused_forward(spmm_values, spmm_indptr, spmm_indices, spmm_features, sddmm_indptr,
                   sddmm_indices, sddmm_query, sddmm_key):
    """An SpMM on graph A and an SDDMM+softmax on graph B with equal row counts
    (entry.cpp:136-155; hfused_cuda.cu:96-137) as one launch whose workgroups are split
    between the two ops (when neither graph has long rows; otherwise the two ops one
    after the other). Returns [spmm_out, attn]."""
    if spmm_indptr.numel() != sddmm_indptr.numel():
        raise RuntimeError("the two graphs must have the same number of rows")
    _check(spmm_values, torch.float32, "spmm_values", 2)
    _check(spmm_features, torch.float32, "spmm_features", 3)
    _check(sddmm_key, torch.float32, "sddmm_key", 2)
    if sddmm_query.dtype != torch.float32 or sddmm_query.dim() not in (2, 3):
        raise RuntimeError("sddmm_query must be float32 [n_dst, H] or [n_bid, n_dst, H]")
    for t, name in ((spmm_indptr, "spmm_indptr"), (spmm_indices, "spmm_indices"),
                    (sddmm_indptr, "sddmm_indptr"), (sddmm_indices, "sddmm_indices")):
        _check(t, torch.int32, name, 1)
    dev = _lib.require_device(spmm_values, spmm_indptr, spmm_indices, spmm_features, sddmm_indptr,
                              sddmm_indices, sddmm_query, sddmm_key)
    query = sddmm_query if sddmm_query.dim() == 3 else sddmm_query.unsqueeze(0)
    n_rows = spmm_indptr.numel() - 1
    n_src_a, h, f = spmm_features.shape
    n_bid = query.size(0)
    n_src_b = sddmm_key.size(0)
    nnz_a, nnz_b = spmm_indices.numel(), sddmm_indices.numel()
    if spmm_values.shape != (nnz_a, h):
        raise RuntimeError("spmm_values must be [n_edges, n_heads]")
    if query.size(1) != n_rows or query.size(2) != h or sddmm_key.size(1) != h:
        raise RuntimeError("query must be [n_bid, n_dst, H] and key [n_src, H] with the SpMM's H")
    if not 1 <= n_bid <= 16:
        raise RuntimeError("at most 16 query blocks (4-bit block tag)")
    out = torch.empty((n_rows, h, f), dtype=torch.float32, device=dev)
    attn = torch.zeros((nnz_b, h), dtype=torch.float32, device=dev)
    ws = _lib.workspace(_size_fn("yitu_hfused_forward_workspace_bytes")(
        c_i64(n_rows), c_i64(nnz_a), c_i64(h * f), c_i64(nnz_b), c_i64(h), c_i64(n_bid)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_hfused_forward(
            ptr(out), ptr(attn), ptr(spmm_values), ptr(spmm_indptr), ptr(spmm_indices),
            ptr(spmm_features), ptr(sddmm_indptr), ptr(sddmm_indices), ptr(query), ptr(sddmm_key),
            c_i64(n_rows), c_i64(n_src_a), c_i64(nnz_a), c_i64(h), c_i64(f), c_i64(n_src_b),
            c_i64(nnz_b), c_i64(n_bid), c_i64(_lib.max_degree(spmm_indptr)),
            c_i64(_lib.max_degree(sddmm_indptr)), ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_hfused_forward")
    return [out, attn]


def hfused_backward(spmm_values, spmm_indptr, spmm_indices, spmm_features, spmm_grad, sddmm_indptr,
                    sddmm_indices, sddmm_query, sddmm_key, sddmm_attn, sddmm_grad):
    """The two backward ops (entry.cpp:157-182) with the correct arithmetic, returning
    [grad_a, grad_x, grad_query, grad_key], in two launches shared by the two graphs: the
    per-row passes of both, then both by-source gathers (no atomics). Graphs with long rows
    run the two ops one after the other. The reference's fused backward kernel is
    unreachable (sparse.py:109-110) and indexes heads by threadIdx.x although they lie on
    threadIdx.y (hfused_cuda.cu:59,186)."""
    if spmm_indptr.numel() != sddmm_indptr.numel():
        raise RuntimeError("the two graphs must have the same number of rows")
    _check(spmm_values, torch.float32, "spmm_values", 2)
    _check(spmm_features, torch.float32, "spmm_features", 3)
    _check(spmm_grad, torch.float32, "spmm_grad", 3)
    _check(sddmm_attn, torch.float32, "sddmm_attn", 2)
    _check(sddmm_grad, torch.float32, "sddmm_grad", 2)
    n_rows, n_src_b, nnz_b, h, n_bid = _sddmm_shapes(sddmm_indptr, sddmm_indices, sddmm_query,
                                                     sddmm_key)
    dev = _lib.require_device(spmm_values, spmm_indptr, spmm_indices, spmm_features, spmm_grad,
                              sddmm_indptr, sddmm_indices, sddmm_query, sddmm_key, sddmm_attn,
                              sddmm_grad)
    n_src_a, h_a, f = spmm_features.shape
    nnz_a = spmm_indices.numel()
    if h_a != h or spmm_values.shape != (nnz_a, h) or spmm_grad.shape != (n_rows, h, f):
        raise RuntimeError("spmm_values must be [n_edges, H], spmm_grad [n_rows, H, F], with the "
                           "SDDMM's H")
    if sddmm_attn.shape != (nnz_b, h) or sddmm_grad.shape != (nnz_b, h):
        raise RuntimeError("sddmm_attn and sddmm_grad must be [n_edges, H]")
    ta = transposed(spmm_indptr, spmm_indices, n_src_a)
    tb = transposed(sddmm_indptr, sddmm_indices, n_src_b)
    grad_a = torch.empty_like(spmm_values)
    grad_x = torch.empty_like(spmm_features)
    grad_q = torch.empty_like(sddmm_query)
    grad_k = torch.empty_like(sddmm_key)
    grad_e = torch.empty_like(sddmm_attn)
    ws = _lib.workspace(_size_fn("yitu_hfused_backward_workspace_bytes")(
        c_i64(n_rows), c_i64(n_src_a), c_i64(nnz_a), c_i64(h * f), c_i64(n_src_b), c_i64(nnz_b),
        c_i64(h), c_i64(n_bid)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_hfused_backward(
            ptr(grad_a), ptr(grad_x), ptr(grad_q), ptr(grad_k), ptr(grad_e), ptr(spmm_values),
            ptr(spmm_indptr), ptr(spmm_indices), ptr(spmm_features), ptr(spmm_grad.contiguous()),
            ptr(ta.t_indptr), ptr(ta.t_rows), ptr(ta.t_perm), ptr(sddmm_indptr), ptr(sddmm_indices),
            ptr(sddmm_query), ptr(sddmm_key), ptr(sddmm_attn), ptr(sddmm_grad.contiguous()),
            ptr(tb.t_indptr), ptr(tb.t_perm), c_i64(n_rows), c_i64(n_src_a), c_i64(nnz_a), c_i64(h),
            c_i64(f), c_i64(n_src_b), c_i64(nnz_b), c_i64(n_bid),
            c_i64(_lib.max_degree(spmm_indptr)), c_i64(ta.max_degree_t),
            c_i64(_lib.max_degree(sddmm_indptr)), c_i64(tb.max_degree_t), ptr(ws),
            c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_hfused_backward")
    return [grad_a, grad_x, grad_q, grad_k]


# --------------------------------------------------------------------------- #
# two Linear layers sharing one input
# --------------------------------------------------------------------------- #
def b2gemm(x, w_a, w_b):
    """Returns [y_a, y_b] = [x . w_a^T, x . w_b^T] (entry.cpp:56-64) on the matrix cores."""
    _check(x, torch.float32, "x", 2)
    _check(w_a, torch.float32, "w_a", 2)
    _check(w_b, torch.float32, "w_b", 2)
    if w_a.shape != w_b.shape or w_a.size(1) != x.size(1):
        raise RuntimeError("w_a and w_b must both be [m, k] with k = x.size(1)")
    dev = _lib.require_device(x, w_a, w_b)
    n, k = x.shape
    m = w_a.size(0)
    y_a = torch.empty((n, m), dtype=torch.float32, device=dev)
    y_b = torch.empty((n, m), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_b2gemm(ptr(y_a), ptr(y_b), ptr(x), ptr(w_a), ptr(w_b), c_i64(n),
                                    c_i64(k), c_i64(m), stream_ptr(dev))
    check(rc, "yitu_b2gemm")
    return [y_a, y_b]


def b2gemm_backward(x, w_a, w_b, grad_a, grad_b):
    """Returns [dx, dw_a, dw_b] (entry.cpp:66-78)."""
    for t, name in ((x, "x"), (w_a, "w_a"), (w_b, "w_b"), (grad_a, "grad_a"), (grad_b, "grad_b")):
        _check(t, torch.float32, name, 2)
    if grad_a.shape != grad_b.shape or w_a.shape != w_b.shape:
        raise RuntimeError("the two halves of the bundle must have equal shapes")
    dev = _lib.require_device(x, w_a, w_b, grad_a, grad_b)
    n, k = x.shape
    m = w_a.size(0)
    if grad_a.shape != (n, m):
        raise RuntimeError("grad_* must be [n, m]")
    dx = torch.empty_like(x)
    dw_a = torch.empty_like(w_a)
    dw_b = torch.empty_like(w_b)
    ws = _lib.workspace(_size_fn("yitu_sgemm_workspace_bytes")(c_i64(m), c_i64(k), c_i64(n),
                                                               c_i64(2)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_b2gemm_backward(ptr(dx), ptr(dw_a), ptr(dw_b), ptr(x), ptr(w_a),
                                             ptr(w_b), ptr(grad_a), ptr(grad_b), c_i64(n), c_i64(k),
                                             c_i64(m), ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_b2gemm_backward")
    return [dx, dw_a, dw_b]


def linear_forward(x, weight, bias=None):
    """x . weight^T + bias in fp32 on the matrix cores (``weight`` [n, k] as nn.Linear keeps
    it, ``bias`` [n] or None), the bias added inside the product where the kernel allows."""
    _check(x, torch.float32, "x", 2)
    _check(weight, torch.float32, "weight", 2)
    if bias is not None:
        _check(bias, torch.float32, "bias", 1)
    dev = _lib.require_device(x, weight) if bias is None else _lib.require_device(x, weight, bias)
    m, k = x.shape
    n = weight.size(0)
    if weight.size(1) != k or (bias is not None and bias.numel() != n):
        raise RuntimeError("linear_forward: x [m, k], weight [n, k], bias [n]")
    y = torch.empty((m, n), dtype=torch.float32, device=dev)
    ws = _lib.workspace(_size_fn("yitu_sgemm_workspace_bytes")(c_i64(m), c_i64(n), c_i64(k),
                                                               c_i64(1)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_linear_forward(ptr(y), ptr(x), ptr(weight), ptr(bias), c_i64(m),
                                            c_i64(n), c_i64(k), ptr(ws), c_size(ws.numel()),
                                            stream_ptr(dev))
    check(rc, "yitu_linear_forward")
    return y


def linear_forward_typed(x_list, weight_list, bias_list, out_list=None):
    """[x_i . weight_i^T + bias_i] for Linear layers that share both widths (the per-type
    layers of a heterogeneous model), up to 32 layers per launch. ``bias_list`` entries may be
    None. ``out_list``: contiguous [m_i, n] tensors to write (e.g. row slices of one buffer)."""
    import ctypes
    count = len(x_list)
    if count == 0 or len(weight_list) != count or len(bias_list) != count:
        raise RuntimeError("linear_forward_typed needs as many weights and biases as inputs")
    n, k = weight_list[0].shape
    for x, w, b in zip(x_list, weight_list, bias_list):
        _check(x, torch.float32, "x", 2)
        _check(w, torch.float32, "weight", 2)
        if tuple(w.shape) != (n, k) or x.size(1) != k:
            raise RuntimeError("linear_forward_typed: x_i [m_i, k], weight_i [n, k]")
        if b is not None:
            _check(b, torch.float32, "bias", 1)
            if b.numel() != n:
                raise RuntimeError("linear_forward_typed: bias_i [n]")
    dev = _lib.require_device(*x_list, *weight_list, *[b for b in bias_list if b is not None])
    ms = [x.size(0) for x in x_list]
    if out_list is None:
        out_list = [torch.empty((m, n), dtype=torch.float32, device=dev) for m in ms]
    else:
        for c, m in zip(out_list, ms):
            _check(c, torch.float32, "out", 2)
            if tuple(c.shape) != (m, n) or c.device != dev:
                raise RuntimeError("out must be [%d, %d] on the operands' device" % (m, n))
    ws = _lib.workspace(_size_fn("yitu_sgemm_workspace_bytes")(
        c_i64(max(ms)), c_i64(n), c_i64(k), c_i64(count)), dev)
    pointers = lambda ts: (ctypes.c_void_p * count)(
        *[(t.data_ptr() or None) if t is not None else None for t in ts])
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_linear_forward_typed(
            pointers(out_list), pointers(x_list), pointers(weight_list), pointers(bias_list),
            (ctypes.c_int64 * count)(*ms), c_i64(count), c_i64(n), c_i64(k), ptr(ws),
            c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_linear_forward_typed")
    return list(out_list)


def sgemm(a, b, trans_a=False, trans_b=False, out=None):
    """op(a) . op(b) in fp32 on the matrix cores; a, b contiguous 2-D. ``out``:
    a contiguous [m, n] tensor (e.g. a row slice of a larger buffer) to write."""
    _check(a, torch.float32, "a", 2)
    _check(b, torch.float32, "b", 2)
    dev = _lib.require_device(a, b)
    m, k = (a.size(1), a.size(0)) if trans_a else (a.size(0), a.size(1))
    kb, n = (b.size(1), b.size(0)) if trans_b else (b.size(0), b.size(1))
    if k != kb:
        raise RuntimeError("inner dimensions differ: %d vs %d" % (k, kb))
    if out is None:
        c = torch.empty((m, n), dtype=torch.float32, device=dev)
    else:
        _check(out, torch.float32, "out", 2)
        if tuple(out.shape) != (m, n) or out.device != dev:
            raise RuntimeError("out must be [%d, %d] on the operands' device" % (m, n))
        c = out
    ws = _lib.workspace(_size_fn("yitu_sgemm_workspace_bytes")(c_i64(m), c_i64(n), c_i64(k),
                                                               c_i64(1)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_sgemm(ptr(c), ptr(a), ptr(b), c_i64(m), c_i64(n), c_i64(k),
                                   c_int(int(trans_a)), c_int(int(trans_b)), c_i64(a.size(1)),
                                   c_i64(b.size(1)), c_i64(n), c_int(0), ptr(ws), c_size(ws.numel()),
                                   stream_ptr(dev))
    check(rc, "yitu_sgemm")
    return c


def sgemm_typed(a_list, b_list, trans_a=False, trans_b=False, out_list=None):
    """[op(a_i) . op(b_i)] for operand pairs that share the output width, the
    transposes and the row strides (the per-type Linear layers of a heterogeneous
    model and their gradient products), up to 32 products per launch so that the
    row tiles of all types fill the chip together. ``out_list``: contiguous
    [m_i, n] tensors to write (e.g. row slices of one buffer)."""
    import ctypes
    if len(a_list) != len(b_list) or not a_list:
        raise RuntimeError("sgemm_typed needs as many a as b operands, at least one")
    for a, b in zip(a_list, b_list):
        _check(a, torch.float32, "a", 2)
        _check(b, torch.float32, "b", 2)
    dev = _lib.require_device(*a_list, *b_list)
    ms = [a.size(1) if trans_a else a.size(0) for a in a_list]
    ks = [a.size(0) if trans_a else a.size(1) for a in a_list]
    n = b_list[0].size(0) if trans_b else b_list[0].size(1)
    lda, ldb = a_list[0].size(1), b_list[0].size(1)
    shared = True
    for a, b, k in zip(a_list, b_list, ks):
        kb, nb = (b.size(1), b.size(0)) if trans_b else (b.size(0), b.size(1))
        if kb != k:
            raise RuntimeError("inner dimensions differ: %d vs %d" % (k, kb))
        shared = shared and nb == n and a.size(1) == lda and b.size(1) == ldb
    if not shared:  # widths differ between the types: one product at a time
        outs = out_list if out_list is not None else [None] * len(a_list)
        return [sgemm(a, b, trans_a, trans_b, out=c) for a, b, c in zip(a_list, b_list, outs)]
    if out_list is None:
        out_list = [torch.empty((m, n), dtype=torch.float32, device=dev) for m in ms]
    else:
        for c, m in zip(out_list, ms):
            _check(c, torch.float32, "out", 2)
            if tuple(c.shape) != (m, n) or c.device != dev:
                raise RuntimeError("out must be [%d, %d] on the operands' device" % (m, n))
    count = len(a_list)
    ws = _lib.workspace(_size_fn("yitu_sgemm_workspace_bytes")(
        c_i64(max(ms)), c_i64(n), c_i64(max(ks)), c_i64(count)), dev)
    pointers = lambda ts: (ctypes.c_void_p * count)(*[t.data_ptr() or None for t in ts])
    sizes = lambda v: (ctypes.c_int64 * count)(*v)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_sgemm_typed(pointers(out_list), pointers(a_list), pointers(b_list),
                                         sizes(ms), sizes(ks), c_i64(count), c_i64(n),
                                         c_int(int(trans_a)), c_int(int(trans_b)), c_i64(lda),
                                         c_i64(ldb), c_i64(n), c_int(0), ptr(ws),
                                         c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_sgemm_typed")
    return list(out_list)


def gemm_bf16(a, b, trans_b=False, out_dtype=torch.float32, out=None):
    """a . op(b) with bf16 operands and fp32 accumulation on the matrix cores.
    ``a`` [m, k]; ``b`` [k, n], or [n, k] with ``trans_b`` (a Linear weight).
    ``out``: a contiguous [m, n] fp32 or bf16 tensor to write (sets ``out_dtype``)."""
    _check(a, torch.bfloat16, "a", 2)
    _check(b, torch.bfloat16, "b", 2)
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise RuntimeError("out_dtype must be float32 or bfloat16")
    dev = _lib.require_device(a, b)
    m, k = a.shape
    n, kb = (b.size(0), b.size(1)) if trans_b else (b.size(1), b.size(0))
    if k != kb:
        raise RuntimeError("inner dimensions differ: %d vs %d" % (k, kb))
    if out is None:
        c = torch.empty((m, n), dtype=out_dtype, device=dev)
    else:
        out_dtype = out.dtype
        if out_dtype not in (torch.float32, torch.bfloat16) or tuple(out.shape) != (m, n) \
                or out.device != dev or not out.is_contiguous():
            raise RuntimeError("out must be a contiguous [%d, %d] fp32 or bf16 tensor" % (m, n))
        c = out
    ws = _lib.workspace(_size_fn("yitu_gemm_bf16_workspace_bytes")(c_i64(n), c_i64(k),
                                                                  c_int(int(trans_b))), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_gemm_bf16(ptr(c), c_int(int(out_dtype == torch.bfloat16)), ptr(a),
                                       ptr(b), c_i64(m), c_i64(n), c_i64(k), c_int(int(trans_b)),
                                       c_i64(a.size(1)), c_i64(b.size(1)), c_i64(n), ptr(ws),
                                       c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_gemm_bf16")
    return c


def gemm_bf16_typed(a_list, b_list, trans_b=False, out_dtype=torch.float32, out_list=None):
    """[a_i . op(b_i)] with bf16 operands for pairs that share the widths (the per-type
    Linear layers of a heterogeneous model in bf16), eight products per launch.
    ``out_list``: contiguous [m_i, n] fp32 or bf16 tensors to write (e.g. row slices of
    one buffer; sets ``out_dtype``)."""
    import ctypes
    if len(a_list) != len(b_list) or not a_list:
        raise RuntimeError("gemm_bf16_typed needs as many a as b operands, at least one")
    for a, b in zip(a_list, b_list):
        _check(a, torch.bfloat16, "a", 2)
        _check(b, torch.bfloat16, "b", 2)
    dev = _lib.require_device(*a_list, *b_list)
    k = a_list[0].size(1)
    n = b_list[0].size(0) if trans_b else b_list[0].size(1)
    for a, b in zip(a_list, b_list):
        if a.size(1) != k or tuple(b.shape) != ((n, k) if trans_b else (k, n)):
            raise RuntimeError("gemm_bf16_typed: every pair must be [m_i, %d] x %s"
                               % (k, "[%d, %d]" % ((n, k) if trans_b else (k, n))))
    ms = [a.size(0) for a in a_list]
    if out_list is None:
        if out_dtype not in (torch.float32, torch.bfloat16):
            raise RuntimeError("out_dtype must be float32 or bfloat16")
        out_list = [torch.empty((m, n), dtype=out_dtype, device=dev) for m in ms]
    else:
        out_dtype = out_list[0].dtype
        for c, m in zip(out_list, ms):
            if c.dtype != out_dtype or out_dtype not in (torch.float32, torch.bfloat16) \
                    or tuple(c.shape) != (m, n) or c.device != dev or not c.is_contiguous():
                raise RuntimeError("out must be contiguous [%d, %d] fp32 or bf16 tensors of one "
                                   "type" % (m, n))
    count = len(a_list)
    ws = _lib.workspace(_size_fn("yitu_gemm_bf16_typed_workspace_bytes")(
        c_i64(count), c_i64(n), c_i64(k), c_int(int(trans_b))), dev)
    pointers = lambda ts: (ctypes.c_void_p * count)(*[t.data_ptr() or None for t in ts])
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_gemm_bf16_typed(
            pointers(out_list), c_int(int(out_dtype == torch.bfloat16)), pointers(a_list),
            pointers(b_list), (ctypes.c_int64 * count)(*ms), c_i64(count), c_i64(n), c_i64(k),
            c_int(int(trans_b)), c_i64(k), c_i64(b_list[0].size(1)), c_i64(n), ptr(ws),
            c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_gemm_bf16_typed")
    return list(out_list)


def gemm_bf16_tn(a, b, out=None, accumulate=False):
    """a^T . b for bf16 ``a`` [m, ki] and ``b`` [m, no] (rows may be strided slices of a
    wider buffer), fp32 accumulation on the matrix cores, fp32 [ki, no] out: the weight
    gradient X^T . dY of a bf16 layer. ``accumulate`` adds to ``out``."""
    for t, name in ((a, "a"), (b, "b")):
        if t.dtype != torch.bfloat16 or t.dim() != 2 or t.stride(1) != 1 or not t.is_cuda:
            raise RuntimeError("%s must be a 2-D bf16 GPU tensor with contiguous rows" % name)
    if a.device != b.device or a.size(0) != b.size(0):
        raise RuntimeError("a and b must have the same number of rows on one device")
    dev = a.device
    m, ki = a.shape
    no = b.size(1)
    if out is None:
        if accumulate:
            raise RuntimeError("accumulate needs an output to add to")
        out = torch.empty((ki, no), dtype=torch.float32, device=dev)
    elif out.dtype != torch.float32 or tuple(out.shape) != (ki, no) or not out.is_contiguous() \
            or out.device != dev:
        raise RuntimeError("out must be a contiguous fp32 [%d, %d] tensor" % (ki, no))
    ws = _lib.workspace(_size_fn("yitu_gemm_bf16_tn_workspace_bytes")(c_i64(m), c_i64(ki), c_i64(no)),
                        dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_gemm_bf16_tn(ptr(out), ptr(a), ptr(b), c_i64(m), c_i64(ki), c_i64(no),
                                          c_i64(a.stride(0)), c_i64(b.stride(0)), c_i64(no),
                                          c_int(int(accumulate)), ptr(ws), c_size(ws.numel()),
                                          stream_ptr(dev))
    check(rc, "yitu_gemm_bf16_tn")
    return out


def gemm_bf16_tn_typed(a_list, b_list, out_list=None, accumulate=False):
    """[a_i^T . b_i] for bf16 pairs [m_i, ki], [m_i, no] of one shape (rows may be strided
    slices of wider buffers with a common row stride): the weight gradients of a
    heterogeneous bf16 layer, eight products per launch. fp32 [ki, no] outputs."""
    import ctypes
    if len(a_list) != len(b_list) or not a_list:
        raise RuntimeError("gemm_bf16_tn_typed needs as many a as b operands, at least one")
    for t in list(a_list) + list(b_list):
        if t.dtype != torch.bfloat16 or t.dim() != 2 or t.stride(1) != 1 or not t.is_cuda:
            raise RuntimeError("operands must be 2-D bf16 GPU tensors with contiguous rows")
    dev = a_list[0].device
    ki, no = a_list[0].size(1), b_list[0].size(1)
    lda, ldb = a_list[0].stride(0), b_list[0].stride(0)
    for a, b in zip(a_list, b_list):
        if a.device != dev or b.device != dev or a.size(0) != b.size(0) or a.size(1) != ki \
                or b.size(1) != no or (a.size(0) > 1 and a.stride(0) != lda) \
                or (b.size(0) > 1 and b.stride(0) != ldb):
            raise RuntimeError("gemm_bf16_tn_typed: every pair must be [m_i, %d], [m_i, %d] with "
                               "common row strides on one device" % (ki, no))
    ms = [a.size(0) for a in a_list]
    if out_list is None:
        if accumulate:
            raise RuntimeError("accumulate needs outputs to add to")
        out_list = [torch.empty((ki, no), dtype=torch.float32, device=dev) for _ in ms]
    else:
        for c in out_list:
            if c.dtype != torch.float32 or tuple(c.shape) != (ki, no) or not c.is_contiguous() \
                    or c.device != dev:
                raise RuntimeError("out must be contiguous fp32 [%d, %d] tensors" % (ki, no))
    count = len(a_list)
    m_arr = (ctypes.c_int64 * count)(*ms)
    ws = _lib.workspace(_size_fn("yitu_gemm_bf16_tn_typed_workspace_bytes")(
        m_arr, c_i64(count), c_i64(ki), c_i64(no)), dev)
    pointers = lambda ts: (ctypes.c_void_p * count)(*[t.data_ptr() or None for t in ts])
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_gemm_bf16_tn_typed(
            pointers(out_list), pointers(a_list), pointers(b_list), m_arr, c_i64(count), c_i64(ki),
            c_i64(no), c_i64(max(lda, ki)), c_i64(max(ldb, no)), c_i64(no), c_int(int(accumulate)),
            ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_gemm_bf16_tn_typed")
    return list(out_list)


# --------------------------------------------------------------------------- #
# fused GAT attention (extension: the composition sddmm_forward -> spmm_forward)
# --------------------------------------------------------------------------- #
def gat_forward(indptr, indices, query, key, features, stats_only=False):
    """Returns [out [Nd,H,F], attn [E,H]] = the reference's two-op GAT lowering
    (sddmm_forward then spmm_forward, n_bid = 1) in one pass per destination row.
    ``stats_only``: returns [out, None, stats] instead, stats [Nd,H,2] = each row's
    softmax (max, 1 / sum): all that ``gat_backward`` needs of the attention for the
    one-pass shapes (``gat_one_pass_shape``); the probabilities are then never stored."""
    _check(indptr, torch.int32, "indptr", 1)
    _check(indices, torch.int32, "indices", 1)
    _check(query, torch.float32, "query", 2)
    _check(key, torch.float32, "key", 2)
    _check(features, torch.float32, "features", 3)
    dev = _lib.require_device(indptr, indices, query, key, features)
    n_dst = indptr.numel() - 1
    n_src, h, f = features.shape
    nnz = indices.numel()
    if query.shape != (n_dst, h) or key.shape != (n_src, h):
        raise RuntimeError("query must be [n_dst, H] and key [n_src, H]")
    if stats_only and not gat_one_pass_shape(h, f):
        raise RuntimeError("stats_only needs a one-pass shape (see gat_one_pass_shape)")
    out = torch.empty((n_dst, h, f), dtype=torch.float32, device=dev)
    attn = None if stats_only else torch.empty((nnz, h), dtype=torch.float32, device=dev)
    stats = torch.empty((n_dst, h, 2), dtype=torch.float32, device=dev) if stats_only else None
    maxdeg = _lib.max_degree(indptr)
    plan = _lib.row_plan(indptr, indices, n_src, COL_MASK)
    need = 0
    if maxdeg >= 64:
        need = _size_fn("yitu_gat_workspace_bytes")(c_i64(n_dst), c_i64(nnz), c_i64(h), c_i64(f),
                                                    c_int(1))
    ws = _lib.workspace(need, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_gat_forward(ptr(out), ptr(attn), ptr(stats), ptr(indptr), ptr(indices),
                                         ptr(query), ptr(key), ptr(features), c_i64(n_dst),
                                         c_i64(n_src), c_i64(nnz), c_i64(h), c_i64(f), c_i64(maxdeg),
                                         ptr(plan), ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_gat_forward")
    return [out, None, stats] if stats_only else [out, attn]


def gat_one_pass_shape(n_heads, n_features, with_out=True):
    """Whether ``yitu_gat_backward`` takes its one-pass path for [*, H, F] rows (the
    shapes for which a head-mean gradient can be passed as it is)."""
    row = n_heads * n_features
    lph = n_features // 4
    return (n_features % 4 == 0 and 8 <= lph <= 64 and lph & (lph - 1) == 0 and
            row in (256, 512, 1024))


def gat_backward(indptr, indices, query, key, features, attn, grad_out, out=None,
                 head_mean=False, stats=None):
    """Returns [grad_query, grad_key, grad_features] of gat_forward's ``out``.
    Passing the forward output ``out`` [n_dst, H, F] lets the softmax backward use
    sum_e a d_attn = <grad_out[row], out[row]> and finish in the same pass over
    the edges that computes grad_features (rows of 256, 512, 1024 floats); without
    it the attention gradient takes passes of its own.
    ``head_mean``: ``grad_out`` is [n_dst, F], the gradient of ``out.mean(dim=1)``
    (the layer's result, model.py:106); the pass then gathers F floats per edge.
    ``stats``: the row statistics of ``gat_forward(stats_only=True)``; ``attn`` may then
    be None (needs ``out`` and a one-pass shape)."""
    if attn is not None:
        _check(attn, torch.float32, "attn", 2)
    elif stats is None or out is None:
        raise RuntimeError("without attn the backward needs stats and out")
    if stats is not None:
        _check(stats, torch.float32, "stats", 3)
    dev = _lib.require_device(indptr, indices, query, key, features, grad_out)
    n_dst = indptr.numel() - 1
    n_src, h, f = features.shape
    nnz = indices.numel()
    if head_mean:
        _check(grad_out, torch.float32, "grad_out", 2)
        if tuple(grad_out.shape) != (n_dst, f):
            raise RuntimeError("a head-mean grad_out must be [n_dst, n_features]")
        if not (gat_one_pass_shape(h, f, out is not None) and n_dst > 0 and nnz > 0):
            # shapes outside the one-pass kernels: spell the gradient out per head
            grad_out = (grad_out / h).unsqueeze(1).expand(n_dst, h, f).contiguous()
            head_mean = False
    if not head_mean:
        _check(grad_out, torch.float32, "grad_out", 3)
    if out is not None:
        _check(out, torch.float32, "out", 3)
        if tuple(out.shape) != (n_dst, h, f):
            raise RuntimeError("out must be [n_dst, n_heads, n_features]")
    tr = transposed(indptr, indices, n_src)
    grad_q = torch.empty_like(query)
    grad_k = torch.empty_like(key)
    grad_x = torch.empty_like(features)
    s1 = torch.empty((nnz, h), dtype=torch.float32, device=dev)
    s2 = s1 if attn is None else torch.empty_like(s1)  # unused by the one-pass path
    maxdeg = _lib.max_degree(indptr)
    plan = _lib.row_plan(indptr, indices, n_src, COL_MASK)
    need = 0
    if max(maxdeg, tr.max_degree_t) >= 64 or out is not None:
        need = _size_fn("yitu_gat_workspace_bytes")(c_i64(max(n_dst, n_src)), c_i64(nnz), c_i64(h),
                                                    c_i64(f), c_int(1))
    ws = _lib.workspace(need, dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_gat_backward(
            ptr(grad_q), ptr(grad_k), ptr(grad_x), ptr(s1), ptr(s2), ptr(indptr), ptr(indices),
            ptr(query), ptr(key), ptr(features), ptr(attn), ptr(stats), ptr(out), ptr(grad_out),
            ptr(tr.t_indptr), ptr(tr.t_rows), ptr(tr.t_perm), c_i64(n_dst), c_i64(n_src),
            c_i64(nnz), c_i64(h), c_i64(f), c_i64(maxdeg), c_i64(tr.max_degree_t), ptr(plan),
            ptr(tr.plan_t), c_int(int(head_mean)), ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_gat_backward")
    return [grad_q, grad_k, grad_x]


# --------------------------------------------------------------------------- #
# per-head projections (attention vectors)
# --------------------------------------------------------------------------- #
def head_dot_shape(n_heads, n_features):
    """Shapes the projection kernels take: head width 4 * a power of two up to 256,
    rows of at most 1024 floats."""
    lph = n_features // 4
    return (n_features % 4 == 0 and 1 <= lph <= 64 and lph & (lph - 1) == 0 and
            n_heads * n_features <= 1024)


def head_dot(x, vec_a, vec_b=None):
    """out_a[n,h] = <vec_a[h,:], x[n,h,:]> (and out_b with ``vec_b``): x [n,H,F],
    vec_* [H,F]. Returns (out_a, out_b or None)."""
    _check(x, torch.float32, "x", 3)
    _check(vec_a, torch.float32, "vec_a", 2)
    if vec_b is not None:
        _check(vec_b, torch.float32, "vec_b", 2)
    dev = _lib.require_device(x, vec_a)
    n, h, f = x.shape
    if tuple(vec_a.shape) != (h, f) or (vec_b is not None and tuple(vec_b.shape) != (h, f)):
        raise RuntimeError("attention vectors must be [n_heads, n_features]")
    out_a = torch.empty((n, h), dtype=torch.float32, device=dev)
    out_b = torch.empty((n, h), dtype=torch.float32, device=dev) if vec_b is not None else None
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_head_dot(ptr(out_a), ptr(out_b), ptr(x), ptr(vec_a), ptr(vec_b),
                                      c_i64(n), c_i64(h), c_i64(f), stream_ptr(dev))
    check(rc, "yitu_head_dot")
    return out_a, out_b


def head_dot_backward(x, vec_a, vec_b, grad_a, grad_b, grad_x=None):
    """Returns (grad_x, grad_vec_a, grad_vec_b). ``grad_x`` given: the projections'
    share is added to it in place (it holds the gradient that reached x by other
    paths); otherwise a new tensor is written."""
    _check(x, torch.float32, "x", 3)
    _check(grad_a, torch.float32, "grad_a", 2)
    dev = _lib.require_device(x, vec_a, grad_a)
    n, h, f = x.shape
    accumulate = grad_x is not None
    if accumulate:
        _check(grad_x, torch.float32, "grad_x", 3)
        if grad_x.shape != x.shape:
            raise RuntimeError("grad_x must have the shape of x")
    else:
        grad_x = torch.empty_like(x)
    gva = torch.empty_like(vec_a)
    gvb = torch.empty_like(vec_b) if vec_b is not None else None
    ws = _lib.workspace(_size_fn("yitu_head_dot_workspace_bytes")(c_i64(n), c_i64(h), c_i64(f)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_head_dot_backward(
            ptr(grad_x), c_int(int(accumulate)), ptr(gva), ptr(gvb), ptr(x), ptr(vec_a), ptr(vec_b),
            ptr(grad_a), ptr(grad_b), c_i64(n), c_i64(h), c_i64(f), ptr(ws), c_size(ws.numel()),
            stream_ptr(dev))
    check(rc, "yitu_head_dot_backward")
    return grad_x, gva, gvb


# --------------------------------------------------------------------------- #
# Linear layers with few outputs
# --------------------------------------------------------------------------- #
def skinny_linear_shape(in_features, out_features):
    tiles = 1 if in_features <= 256 else (2 if in_features <= 512 else 4)
    return (in_features % 4 == 0 and 0 < in_features <= 1024 and 0 < out_features <= 16 and
            out_features * tiles <= 16)


def skinny_linear(x, weight, bias=None):
    """x [n, K] . weight [J, K]^T + bias [J] for a handful of outputs J."""
    _check(x, torch.float32, "x", 2)
    _check(weight, torch.float32, "weight", 2)
    if bias is not None:
        _check(bias, torch.float32, "bias", 1)
    dev = _lib.require_device(x, weight)
    n, k = x.shape
    j = weight.size(0)
    if weight.size(1) != k or (bias is not None and bias.numel() != j):
        raise RuntimeError("weight must be [out, in] and bias [out]")
    y = torch.empty((n, j), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_skinny_linear(ptr(y), ptr(x), ptr(weight), ptr(bias), c_i64(n), c_i64(k),
                                           c_i64(j), stream_ptr(dev))
    check(rc, "yitu_skinny_linear")
    return y


def skinny_linear_backward(x, weight, grad_y, grad_x=None, need_bias=True):
    """Returns (grad_x, grad_weight, grad_bias or None); a given ``grad_x`` is added to in place."""
    _check(grad_y, torch.float32, "grad_y", 2)
    dev = _lib.require_device(x, weight, grad_y)
    n, k = x.shape
    j = weight.size(0)
    accumulate = grad_x is not None
    if not accumulate:
        grad_x = torch.empty_like(x)
    else:
        _check(grad_x, torch.float32, "grad_x", 2)
    gw = torch.empty_like(weight)
    gb = torch.empty(j, dtype=torch.float32, device=dev) if need_bias else None
    ws = _lib.workspace(_size_fn("yitu_skinny_linear_workspace_bytes")(c_i64(n), c_i64(k), c_i64(j)),
                        dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_skinny_linear_backward(
            ptr(grad_x), c_int(int(accumulate)), ptr(gw), ptr(gb), ptr(x), ptr(weight), ptr(grad_y),
            c_i64(n), c_i64(k), c_i64(j), ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_skinny_linear_backward")
    return grad_x, gw, gb


def column_sum(x):
    """Sum over the rows of a 2-D fp32 tensor (a Linear's bias gradient), in a fixed order and
    without a cleared accumulator: safe to record into a HIP graph."""
    _check(x, torch.float32, "x", 2)
    dev = _lib.require_device(x)
    m, n = x.shape
    out = torch.empty(n, dtype=torch.float32, device=dev)
    ws = _lib.workspace(_size_fn("yitu_column_sum_workspace_bytes")(c_i64(m), c_i64(n)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_column_sum(ptr(out), ptr(x), c_i64(m), c_i64(n), ptr(ws),
                                        c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_column_sum")
    return out


COLUMN_SUM_TYPED_MAX_ROWS = 4096  # above this a matrix takes column_sum's two-stage form


def column_sum_typed(x_list):
    """``[x_i.sum(0)]`` for 2-D fp32 tensors of one width whose rows are one common stride
    apart (row slices of one buffer): one launch per 32 of them when they are short (the bias
    gradients of the per-relation Linears of a small heterogeneous graph), otherwise
    ``column_sum`` each. Fixed summation order, no cleared accumulator."""
    import ctypes
    if not x_list:
        return []
    n = x_list[0].size(1)
    ld = x_list[0].stride(0) if x_list[0].size(0) > 1 else n
    short = True
    for x in x_list:
        if x.dtype != torch.float32 or x.dim() != 2 or not x.is_cuda or x.size(1) != n or \
                (x.size(1) > 1 and x.stride(1) != 1):
            raise RuntimeError("column_sum_typed takes 2-D fp32 GPU tensors of one width")
        short = short and x.size(0) <= COLUMN_SUM_TYPED_MAX_ROWS and \
            (x.size(0) <= 1 or x.stride(0) == ld)
    if not short or ld < n:
        return [column_sum(x.contiguous()) for x in x_list]
    dev = x_list[0].device
    count = len(x_list)
    out = torch.empty((count, n), dtype=torch.float32, device=dev)
    pointers = lambda ts: (ctypes.c_void_p * count)(*[t.data_ptr() or None for t in ts])
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_column_sum_typed(
            pointers([out[i] for i in range(count)]), pointers(x_list),
            (ctypes.c_int64 * count)(*[x.size(0) for x in x_list]), c_i64(count), c_i64(n),
            c_i64(ld), stream_ptr(dev))
    check(rc, "yitu_column_sum_typed")
    return list(out.unbind(0))
