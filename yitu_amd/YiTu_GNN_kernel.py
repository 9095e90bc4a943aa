"""Drop-in for the reference's ``YiTu_GNN.YiTu_GNN_kernel`` extension module
(ccsrc/kernel/YiTu_GNN.cpp:247-258): same function names, positional order and
return arity, backed by the gfx950 kernels of libyitu_hip.so.

Differences from the reference that callers can observe:
  * the neighbour-group arguments (part_pointers, part2Node, partSize,
    dimWorker, warpPerBlock) are accepted and validated for device/contiguity
    like the others but do not steer the kernels: their role is played by a row
    plan that is built on the device on first use of a graph and cached;
  * outputs live on the input's device (the reference allocates ``forward``'s
    output on the default CUDA device, YiTu_GNN_kernel.cu:278);
  * failures raise ``RuntimeError`` instead of ``exit(-1)`` (cu:309-314);
  * results are bitwise reproducible (no atomics);
  * ``build_part`` returns int32 tensors holding the exact integers; the
    reference stores them in float32 (YiTu_GNN.cpp:222-223), which callers cast
    back with ``.int()`` -- a no-op here.
"""
import torch

from . import _lib
from ._lib import c_f32, c_i64, c_int, c_size, check, ptr, stream_ptr


def _mm(a, b, trans_a=False, trans_b=False):
    """Dense fp32 product on the matrix cores (the reference calls torch::mm)."""
    from .graph_ext import sgemm
    return sgemm(a.contiguous(), b.contiguous(), trans_a, trans_b)


def _check_inputs(*tensors):
    # CHECK_INPUT of the reference: CUDA + contiguous (YiTu_GNN.cpp:65-69)
    return _lib.require_device(*tensors)


def edge_scale(column_index, degrees):
    """Per-edge column scales ``degrees[column_index[e]]`` of a graph (float32 [nnz]):
    per-graph preparation, like ``build_part``. Passed as ``edge_scale=`` to ``forward`` /
    ``backward`` the aggregation reads them in edge order instead of gathering ``degrees``
    once per edge. The caller owns the tensor: it must be rebuilt when ``column_index`` or
    ``degrees`` change."""
    _lib.require_device(column_index, degrees)
    _lib.require_dtype(column_index, torch.int32, "column_index")
    _lib.require_dtype(degrees, torch.float32, "degrees")
    out = torch.empty(column_index.numel(), dtype=torch.float32, device=column_index.device)
    with torch.cuda.device(column_index.device):
        rc = _lib.lib().yitu_edge_scale(ptr(out), ptr(column_index), ptr(degrees),
                                        c_i64(column_index.numel()), c_i64(degrees.numel()),
                                        stream_ptr(column_index.device))
    check(rc, "yitu_edge_scale")
    return out


def _aggregate(x, row_pointers, column_index, degrees, alpha, edge_scale=None):
    """out[r] = alpha * s_r * sum_j s_j x[j] over the CSR row r (s = degrees or 1)."""
    _lib.require_dtype(row_pointers, torch.int32, "row_pointers")
    _lib.require_dtype(column_index, torch.int32, "column_index")
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise RuntimeError("features must be float32 or bfloat16, got %s" % x.dtype)
    if x.dim() != 2:
        raise RuntimeError("features must be 2-D [n_nodes, dim]")
    if degrees is not None:
        _lib.require_dtype(degrees, torch.float32, "degrees")
    n_rows = row_pointers.numel() - 1
    n_src, dim = x.shape
    nnz = column_index.numel()
    if degrees is not None and degrees.numel() < max(n_rows, n_src):
        raise RuntimeError("degrees is shorter than the number of nodes")
    if edge_scale is not None:
        _lib.require_device(edge_scale)
        _lib.require_dtype(edge_scale, torch.float32, "edge_scale")
        if edge_scale.numel() != nnz:
            raise RuntimeError("edge_scale must hold one value per edge")
    out = torch.empty((n_rows, dim), dtype=torch.float32, device=x.device)
    maxdeg = _lib.max_degree(row_pointers)
    plan = _lib.row_plan(row_pointers, column_index, n_src, 0x7FFFFFFF)
    need = _lib.size_fn("yitu_spmm_workspace_bytes")(c_i64(nnz), c_i64(dim), c_int(1)) \
        if plan is not None and maxdeg >= 64 else 0
    ws = _lib.workspace(need, x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().yitu_agg_csr(
            ptr(out), ptr(x), c_int(1 if x.dtype == torch.bfloat16 else 0), ptr(row_pointers),
            ptr(column_index), ptr(degrees), c_i64(n_rows), c_i64(n_src), c_i64(nnz), c_i64(dim),
            c_f32(alpha), c_i64(maxdeg), ptr(plan), ptr(edge_scale), ptr(ws), c_size(ws.numel()),
            stream_ptr(x.device))
    check(rc, "yitu_agg_csr")
    return out


def SAG(input, row_pointers, column_index, degrees, part_pointers, part2Node, partSize, dimWorker,
        warpPerBlock):
    """Unweighted neighbour sum (YiTu_GNN.cpp:71-92; YiTu_GNN_kernel.cu:104-257)."""
    _check_inputs(input, row_pointers, column_index, degrees, part_pointers, part2Node)
    return _aggregate(input, row_pointers, column_index, None, 1.0)


def forward(input, weight, row_pointers, column_index, degrees, part_pointers, part2Node, partSize,
            dimWorker, warpPerBlock, edge_scale=None):
    """GCN: out = aggregate_{s_i s_j}(X.W) (YiTu_GNN.cpp:94-117; cu:264-317). Returns [out].
    ``edge_scale`` (optional, not in the reference): see ``edge_scale()``."""
    _check_inputs(input, weight, row_pointers, column_index, degrees, part_pointers, part2Node)
    tmp = _mm(input, weight)
    return [_aggregate(tmp, row_pointers, column_index, degrees, 1.0, edge_scale)]


def backward(d_output, X, W, row_pointers, column_index, degrees, part_pointers, part2Node,
             partSize, dimWorker, warpPerBlock, edge_scale=None):
    """GCN backward with the reference's semantics: the SAME CSR aggregates dY
    (not its transpose), then dX = G.W^T, dW = X^T.G (YiTu_GNN.cpp:119-145;
    cu:422-475). Returns [d_input, d_weight]."""
    _check_inputs(d_output, X, W, row_pointers, column_index, degrees, part_pointers, part2Node)
    g = _aggregate(d_output, row_pointers, column_index, degrees, 1.0, edge_scale)
    return [_mm(g, W, trans_b=True), _mm(X, g, trans_a=True)]


def backward_transposed(d_output, X, W, row_pointers, column_index, degrees, part_pointers,
                        part2Node, partSize, dimWorker, warpPerBlock):
    """The gradient of ``forward`` for graphs that are not symmetric: dY is
    aggregated over the TRANSPOSED structure (G = A^T.dY), then dX = G.W^T,
    dW = X^T.G. Not in the reference, whose ``backward`` reuses the forward CSR
    (cu:447-461) and is therefore exact for symmetric graphs only. Same
    arguments as ``backward``; the by-source structure is built on the device on
    first use and cached. Node ids must fit 24 bits."""
    _check_inputs(d_output, X, W, row_pointers, column_index, degrees, part_pointers, part2Node)
    from . import graph_ext
    t = graph_ext.transposed(row_pointers, column_index, X.shape[0])
    g = _aggregate(d_output, t.t_indptr, t.t_rows, degrees, 1.0)
    return [_mm(g, W, trans_b=True), _mm(X, g, trans_a=True)]


def forward_gin(input, weight, row_pointers, column_index, epsilon, part_pointers, part2Node,
                partSize, dimWorker, warpPerBlock):
    """GIN: A = eps * sum_j X[j]; out = A.W (YiTu_GNN.cpp:150-172; cu:563-618). Returns [out, A]."""
    _check_inputs(input, weight, row_pointers, column_index, part_pointers, part2Node)
    agg = _aggregate(input, row_pointers, column_index, None, float(epsilon))
    return [_mm(agg, weight), agg]


def backward_gin(d_output, X, W, row_pointers, column_index, epsilon, part_pointers, part2Node,
                 partSize, dimWorker, warpPerBlock):
    """GIN backward: dW = X^T.dY (X is the saved aggregate), dX = eps * sum_j (dY.W^T)[j]
    (YiTu_GNN.cpp:177-201; cu:701-751). Returns [d_input, d_weight]."""
    _check_inputs(d_output, X, W, row_pointers, column_index, part_pointers, part2Node)
    d_weight = _mm(X, d_output, trans_a=True)
    g = _mm(d_output, W, trans_b=True)
    return [_aggregate(g, row_pointers, column_index, None, float(epsilon)), d_weight]


def _build_part_device(part_size, indptr):
    _lib.require_dtype(indptr, torch.int32, "indptr")
    if part_size <= 0:
        raise RuntimeError("partSize must be positive")
    dev = indptr.device
    indptr = indptr.contiguous()
    n_rows = indptr.numel() - 1
    nnz = int(indptr[-1].item()) if n_rows > 0 else 0
    capacity = nnz // part_size + n_rows
    part_ptr = torch.zeros(capacity + 1, dtype=torch.int32, device=dev)
    part2node = torch.empty(capacity, dtype=torch.int32, device=dev)
    n_parts = torch.zeros(1, dtype=torch.int64, device=dev)
    ws = _lib.workspace(_lib.size_fn("yitu_build_part_workspace_bytes")(c_i64(n_rows)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_build_part(ptr(part_ptr), ptr(part2node), ptr(n_parts), ptr(indptr),
                                        c_i64(n_rows), c_i64(part_size), c_i64(capacity), ptr(ws),
                                        c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_build_part")
    n = int(n_parts.item())
    return [part_ptr[:n + 1], part2node[:n]]


def build_part(partSize, indptr):
    """Neighbour-group partition of a CSR (YiTu_GNN.cpp:203-245): group p covers
    edges [partPtr[p], partPtr[p+1]) of row part2Node[p], at most partSize of
    them. ``indptr`` is an int32 tensor: on the CPU like the reference's
    (accessor<int,1>), or on the GPU, where the partition is built by
    ``yitu_build_part`` and stays there; returns [partPtr, part2Node] (int32, on
    indptr's device). As in the reference the sentinel partPtr[P] is only written
    when the last row is non-empty, otherwise it stays 0."""
    if indptr.is_cuda:
        return _build_part_device(int(partSize), indptr)
    _lib.require_dtype(indptr, torch.int32, "indptr")
    partSize = int(partSize)
    if partSize <= 0:
        raise RuntimeError("partSize must be positive")
    ip = indptr.contiguous().to(torch.int64)
    deg = ip[1:] - ip[:-1]
    cnt = (deg + partSize - 1) // partSize
    n_parts = int(cnt.sum())
    rows = torch.repeat_interleave(torch.arange(deg.numel(), dtype=torch.int64), cnt)
    first = torch.cumsum(cnt, 0) - cnt
    within = torch.arange(n_parts, dtype=torch.int64) - first[rows]
    part_ptr = torch.zeros(n_parts + 1, dtype=torch.int32)
    part_ptr[:n_parts] = (ip[:-1][rows] + within * partSize).to(torch.int32)
    if deg.numel() > 0 and deg[-1] > 0:
        part_ptr[n_parts] = int(ip[-1])
    return [part_ptr, rows.to(torch.int32)]
