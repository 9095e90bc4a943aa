"""Dense <-> CSR helpers used by the parity tests (xgnn_h/convert.py), vectorised."""
import torch


def to_dense(n_rows, n_cols, sparse, values):
    indptr, indices = sparse
    assert values.dim() == 1 and values.size(0) == indices.size(0)
    deg = (indptr[1:] - indptr[:-1]).long()
    rows = torch.repeat_interleave(torch.arange(n_rows, device=indptr.device), deg)
    dense = torch.zeros(n_rows, n_cols, device=values.device)
    dense[rows.to(values.device), (indices.long() & 0xFFFFFF).to(values.device)] = values
    return dense


def to_dense_mha(n_rows, n_cols, sparse, values):
    assert values.dim() == 2
    return torch.stack([to_dense(n_rows, n_cols, sparse, values[:, h].contiguous())
                        for h in range(values.size(1))])


def to_csr(dense):
    assert dense.dim() == 2
    rows, cols = torch.nonzero(dense, as_tuple=True)
    counts = torch.bincount(rows, minlength=dense.size(0))
    indptr = torch.zeros(dense.size(0) + 1, dtype=torch.int64)
    indptr[1:] = torch.cumsum(counts, 0)
    return [indptr.to(torch.int32), cols.to(torch.int32)], dense[rows, cols].float()
