"""Edge list -> canonical CSR on the GPU through the C ABI (yitu_coo_to_csr):
rows ascending, columns ascending inside a row, duplicates merged, int32 -- what
``scipy.sparse.coo_matrix(...).tocsr()`` gives the reference
(YiTu_GNN/data/dataset.py:116-129)."""
import torch

from .. import _lib


def coo_to_csr(rows, cols, n_rows, n_cols=None):
    """``rows``, ``cols``: integer device tensors [E]. Returns (indptr int32
    [n_rows + 1], indices int32 [nnz]) on the same device."""
    n_cols = n_rows if n_cols is None else n_cols
    dev = _lib.require_device(rows, cols)
    if rows.shape != cols.shape or rows.dim() != 1:
        raise RuntimeError("rows and cols must be 1-D and equally long")
    rows = rows.to(torch.int32).contiguous()
    cols = cols.to(torch.int32).contiguous()
    n_edges = rows.numel()
    indptr = torch.empty(n_rows + 1, dtype=torch.int32, device=dev)
    indices = torch.empty(max(n_edges, 1), dtype=torch.int32, device=dev)
    nnz = torch.empty(1, dtype=torch.int64, device=dev)
    ws = _lib.workspace(_lib.size_fn("yitu_coo_to_csr_workspace_bytes")(
        _lib.c_i64(n_edges), _lib.c_i64(n_rows)), dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().yitu_coo_to_csr(
            _lib.ptr(indptr), _lib.ptr(indices), _lib.ptr(nnz), _lib.ptr(rows), _lib.ptr(cols),
            _lib.c_i64(n_edges), _lib.c_i64(n_rows), _lib.c_i64(n_cols), _lib.ptr(ws),
            _lib.c_size(ws.numel()), _lib.stream_ptr(dev))
    _lib.check(rc, "yitu_coo_to_csr")
    count = int(nnz.item())
    if count < 0:
        raise RuntimeError("edge list holds a node id outside [0, n_rows) x [0, n_cols)")
    return indptr, indices[:count].clone()
