"""Pins the CPU oracle's module-1 functions (GCN / GIN / SAG aggregation,
build_part, CSR build) against independent formulations: scipy's CSR product,
dense torch algebra with autograd, closed forms and brute force."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

import oracle
from helpers import assert_close, random_csr
from yitu_amd.data import graphgen


def _scipy_adj(indptr, indices, n_src, weights=None):
    data = np.ones(indices.shape[0], dtype=np.float64) if weights is None else weights
    return sp.csr_matrix((data, indices.numpy(), indptr.numpy()),
                         shape=(indptr.numel() - 1, n_src))


@pytest.mark.parametrize("n,dim,seed", [(1, 1, 0), (37, 5, 1), (300, 64, 2), (513, 33, 3)])
def test_sag_equals_scipy_product(n, dim, seed):
    indptr, indices = random_csr(n, n, 0.05, seed, hub_rows=(0,), hub_degree=n // 2,
                                 empty_rows=(n - 1,))
    x = np.random.default_rng(seed).standard_normal((n, dim)).astype(np.float32)
    want = _scipy_adj(indptr, indices, n) @ x.astype(np.float64)
    assert_close(oracle.sag(x, indptr, indices), want.astype(np.float32))


@pytest.mark.parametrize("mode", [oracle.MODE_GCN, oracle.MODE_SAG, oracle.MODE_GIN])
def test_group_ordered_float_variant_agrees_with_row_referee(mode):
    """The kernel-order float restatement (one partial per neighbour group) and
    the double-accumulate row form differ only by float summation error."""
    n, dim = 300, 24
    indptr, indices = random_csr(n, n, 0.05, 11, hub_rows=(5,), hub_degree=200, empty_rows=(0,))
    x = np.random.default_rng(3).standard_normal((n, dim)).astype(np.float32)
    s = graphgen.gcn_norm(indptr).numpy()
    pp, p2n = oracle.build_part(7, indptr)
    got = oracle.group_agg_f32(x, indices, s, pp, p2n, mode, 0.5)
    assert_close(got, oracle.row_agg(x, indptr, indices, s, mode, 0.5))


def test_group_variant_reproduces_missing_sentinel_quirk():
    """With an empty LAST row build_part leaves partPtr[P] = 0, so the kernel sees
    an empty range for the final group and drops its edges (YiTu_GNN.cpp:240-241,
    YiTu_GNN_kernel.cu:352). The row-form referee (and the HIP op) do not."""
    n, dim = 37, 5
    indptr, indices = random_csr(n, n, 0.2, 1, empty_rows=(n - 1,))
    x = np.random.default_rng(1).standard_normal((n, dim)).astype(np.float32)
    pp, p2n = oracle.build_part(64, indptr)
    assert pp[-1] == 0
    got = oracle.group_agg_f32(x, indices, None, pp, p2n, oracle.MODE_SAG)
    want = oracle.sag(x, indptr, indices)
    last = int(p2n[-1])
    assert np.all(got[last] == 0) and np.abs(want[last]).max() > 0
    keep = np.arange(n) != last
    assert_close(got[keep], want[keep])


@pytest.mark.parametrize("n,fin,fout,seed", [(64, 8, 4, 0), (257, 16, 32, 1)])
def test_gcn_forward_backward_equal_dense_autograd(n, fin, fout, seed):
    """out = diag(s) A diag(s) (X W); the reference backward applies the SAME
    operator to dY (YiTu_GNN_kernel.cu:447-461), which is autograd's answer only
    for a symmetric A, so the graph here is symmetrised."""
    rng = np.random.default_rng(seed)
    a = rng.random((n, n)) < 0.06
    a = a | a.T
    rows, cols = np.nonzero(a)
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(rows), torch.from_numpy(cols), n)
    s = graphgen.gcn_norm(indptr)
    x = torch.randn(n, fin, dtype=torch.float64, requires_grad=True)
    w = torch.randn(fin, fout, dtype=torch.float64, requires_grad=True)
    ahat = torch.from_numpy(a.astype(np.float64)) * s.double()[:, None] * s.double()[None, :]
    y = ahat @ (x @ w)
    dy = torch.randn(n, fout, dtype=torch.float64)
    y.backward(dy)
    got = oracle.gcn_forward(x.detach().float().numpy(), w.detach().float().numpy(), indptr,
                             indices, s.numpy())
    assert_close(got, y.detach().float())
    dx, dw = oracle.gcn_backward(dy.float().numpy(), x.detach().float().numpy(),
                                 w.detach().float().numpy(), indptr, indices, s.numpy())
    assert_close(dx, x.grad.float(), atol=2e-4)
    assert_close(dw, w.grad.float(), atol=2e-4)


def test_gcn_backward_uses_forward_csr_on_directed_graph():
    """On a directed graph the reference's backward is A_hat dY, NOT A_hat^T dY."""
    n = 50
    indptr, indices = random_csr(n, n, 0.1, 5)
    s = graphgen.gcn_norm(indptr).numpy()
    dy = np.random.default_rng(0).standard_normal((n, 3)).astype(np.float32)
    x = np.zeros((n, 3), np.float32)
    w = np.eye(3, dtype=np.float32)
    dx, _ = oracle.gcn_backward(dy, x, w, indptr, indices, s)
    adj = _scipy_adj(indptr, indices, n).toarray() * s[:, None] * s[None, :]
    assert_close(dx, adj @ dy)
    assert np.abs(dx - adj.T @ dy).max() > 1e-2


@pytest.mark.parametrize("seed", [0, 1])
def test_gin_forward_backward(seed):
    n, fin, fout, eps = 120, 6, 9, 0.5
    rng = np.random.default_rng(seed)
    a = rng.random((n, n)) < 0.05
    a = a | a.T
    rows, cols = np.nonzero(a)
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(rows), torch.from_numpy(cols), n)
    x = torch.randn(n, fin, dtype=torch.float64, requires_grad=True)
    w = torch.randn(fin, fout, dtype=torch.float64, requires_grad=True)
    ad = torch.from_numpy(a.astype(np.float64))
    y = (eps * (ad @ x)) @ w
    dy = torch.randn(n, fout, dtype=torch.float64)
    y.backward(dy)
    out, agg = oracle.gin_forward(x.detach().float().numpy(), w.detach().float().numpy(), indptr,
                                  indices, eps)
    assert_close(out, y.detach().float())
    assert_close(agg, (eps * (ad @ x)).detach().float())
    dx, dw = oracle.gin_backward(dy.float().numpy(), agg, w.detach().float().numpy(), indptr,
                                 indices, eps)
    assert_close(dx, x.grad.float(), atol=2e-4)
    assert_close(dw, w.grad.float(), atol=2e-4)


def test_special_cases_reduce_to_each_other():
    """s == 1 and W == I reduce the GCN op to SAG; eps == 1 reduces GIN to SAG."""
    n, dim = 90, 12
    indptr, indices = random_csr(n, n, 0.08, 9)
    x = np.random.default_rng(1).standard_normal((n, dim)).astype(np.float32)
    base = oracle.sag(x, indptr, indices)
    ones = np.ones(n, np.float32)
    assert np.array_equal(oracle.gcn_forward(x, np.eye(dim, dtype=np.float32), indptr, indices,
                                             ones), base)
    assert np.array_equal(oracle.gin_forward(x, np.eye(dim, dtype=np.float32), indptr, indices,
                                             1.0)[1], base)


def test_bf16_variant_matches_f32_on_bf16_representable_input():
    n, dim = 70, 16
    indptr, indices = random_csr(n, n, 0.1, 4)
    xb = torch.randn(n, dim).to(torch.bfloat16)
    s = graphgen.gcn_norm(indptr).numpy()
    bits = xb.view(torch.int16).numpy().view(np.uint16)
    got = oracle.row_agg_bf16(bits, indptr, indices, s, oracle.MODE_GCN)
    want = oracle.row_agg(xb.float().numpy(), indptr, indices, s, oracle.MODE_GCN)
    assert np.array_equal(got, want)


# ---- build_part -------------------------------------------------------------

def _build_part_bruteforce(ps, indptr):
    pp, p2n = [], []
    for r in range(len(indptr) - 1):
        for b in range(indptr[r], indptr[r + 1], ps):
            pp.append(b)
            p2n.append(r)
    return pp, p2n


@pytest.mark.parametrize("ps", [1, 3, 32])
@pytest.mark.parametrize("last_empty", [False, True])
def test_build_part_closed_form(ps, last_empty):
    indptr, _ = random_csr(40, 40, 0.2, ps, hub_rows=(3,), hub_degree=39,
                           empty_rows=(0, 39) if last_empty else (0,))
    pp, p2n = oracle.build_part(ps, indptr.numpy())
    bpp, bp2n = _build_part_bruteforce(ps, indptr.tolist())
    deg = np.diff(indptr.numpy())
    assert len(p2n) == int(np.ceil(deg / ps).sum())
    assert p2n.tolist() == bp2n and pp[:-1].tolist() == bpp
    # sentinel only written when the last row is non-empty (YiTu_GNN.cpp:240-241)
    assert pp[-1] == (0 if last_empty else indptr[-1].item())
    assert np.all(np.diff(p2n) >= 0)


# ---- canonical CSR ----------------------------------------------------------

@pytest.mark.parametrize("seed", [0, 1, 2])
def test_csr_build_is_scipy_canonical(seed):
    """The reference builds its CSR with scipy coo -> csr (dataset.py:116-129)."""
    rng = np.random.default_rng(seed)
    n, m = 200, 3000
    src = rng.integers(0, n, m)
    dst = rng.integers(0, n, m)
    ref = sp.coo_matrix((np.ones(m), (src, dst)), shape=(n, n)).tocsr()
    ref.sum_duplicates()
    ref.sort_indices()
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(src), torch.from_numpy(dst), n)
    assert indptr.dtype == torch.int32 and indices.dtype == torch.int32
    assert np.array_equal(indptr.numpy(), ref.indptr)
    assert np.array_equal(indices.numpy(), ref.indices)
