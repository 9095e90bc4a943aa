"""Seeded synthetic graphs for tests and benchmarks, and the canonical CSR
build shared by them.

The CSR convention is the one the reference obtains from
``scipy.sparse.coo_matrix(...).tocsr()`` (YiTu_GNN/data/dataset.py:116-129):
rows sorted, columns sorted inside each row, duplicate edges merged, int32.
All functions run on whichever torch device they are given (CPU by default) so
the large benchmark graphs can be produced on the GPU in a second or two.
"""
import torch


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def csr_from_edges(rows, cols, n_rows, n_cols=None):
    """Canonical CSR of the edge set {(rows[i], cols[i])}: (indptr, indices) int32."""
    n_cols = n_rows if n_cols is None else n_cols
    key = rows.to(torch.int64) * n_cols + cols.to(torch.int64)
    key = torch.unique(key)  # sorted, duplicates merged
    r = torch.div(key, n_cols, rounding_mode="floor")
    c = key - r * n_cols
    counts = torch.bincount(r, minlength=n_rows)
    indptr = torch.zeros(n_rows + 1, dtype=torch.int64, device=key.device)
    indptr[1:] = torch.cumsum(counts, 0)
    return indptr.to(torch.int32), c.to(torch.int32)


def erdos_renyi(n, m, seed, self_loops=True, device="cpu"):
    """m directed (src, dst) pairs drawn uniformly, plus (i, i) for every i."""
    g = _gen(seed, device)
    src = torch.randint(0, n, (m,), generator=g, device=device)
    dst = torch.randint(0, n, (m,), generator=g, device=device)
    if self_loops:
        loop = torch.arange(n, device=device)
        src = torch.cat([src, loop])
        dst = torch.cat([dst, loop])
    return src, dst


def rmat(scale, m, seed, a=0.57, b=0.19, c=0.19, d=0.05, self_loops=False, device="cpu",
         chunk=1 << 24):
    """R-MAT edge list on 2**scale vertices: m draws, one quadrant per level."""
    g = _gen(seed, device)
    srcs, dsts = [], []
    for s0 in range(0, m, chunk):
        mm = min(chunk, m - s0)
        src = torch.zeros(mm, dtype=torch.int64, device=device)
        dst = torch.zeros(mm, dtype=torch.int64, device=device)
        for _ in range(scale):
            u = torch.rand(mm, generator=g, device=device)
            sbit = (u >= a + b)
            dbit = ((u >= a) & (u < a + b)) | (u >= a + b + c)
            src = (src << 1) | sbit.to(torch.int64)
            dst = (dst << 1) | dbit.to(torch.int64)
        srcs.append(src)
        dsts.append(dst)
    src = torch.cat(srcs)
    dst = torch.cat(dsts)
    if self_loops:
        loop = torch.arange(1 << scale, device=device)
        src = torch.cat([src, loop])
        dst = torch.cat([dst, loop])
    return src, dst


def csr_by_destination(src, dst, n):
    """CSR whose row r lists the sources of r's in-edges."""
    return csr_from_edges(dst, src, n, n)


def gcn_norm(indptr, power=-0.5):
    """Per-node scale s with s_i * s_j = 1 / sqrt(d_i d_j); empty rows count as degree 1."""
    deg = (indptr[1:] - indptr[:-1]).to(torch.float32).clamp_(min=1.0)
    return deg.pow(power)


def bipartite_uniform(n_dst, n_src, avg_degree, seed, device="cpu"):
    """Each destination row draws Poisson(avg_degree) uniform sources; duplicates merged."""
    g = _gen(seed, device)
    lam = torch.full((n_dst,), float(avg_degree), device=device)
    cnt = torch.poisson(lam, generator=g).to(torch.int64)
    rows = torch.repeat_interleave(torch.arange(n_dst, device=device), cnt)
    cols = torch.randint(0, n_src, (int(cnt.sum()),), generator=g, device=device)
    return csr_from_edges(rows, cols, n_dst, n_src)


def planted_partition(n_comm, size, intra, inter, seed, device="cpu"):
    """Planted-partition graph: n_comm communities of `size` vertices; every vertex draws
    `intra` sources inside its community and `inter` anywhere. Ids as planted (a
    community is a contiguous id block). Returns (src, dst) int64 on `device`, self loops
    included once per vertex."""
    g = torch.Generator(device=device).manual_seed(seed)
    n = n_comm * size
    dst = torch.arange(n, device=device).repeat_interleave(intra)
    base = dst // size * size
    src = base + torch.randint(0, size, (n * intra,), generator=g, device=device)
    dst2 = torch.arange(n, device=device).repeat_interleave(inter)
    src2 = torch.randint(0, n, (n * inter,), generator=g, device=device)
    loop = torch.arange(n, device=device)
    return torch.cat([src, src2, loop]), torch.cat([dst, dst2, loop])
