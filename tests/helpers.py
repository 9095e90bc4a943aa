"""Shared test helpers: small seeded graphs and the tolerances of the parity bar."""
import numpy as np
import torch

from yitu_amd.data import graphgen

# fp32 outputs and gradients: rtol 1e-5 / atol 1e-4; bf16-in / fp32-accumulate: rtol 1e-2
RTOL_F32, ATOL_F32 = 1e-5, 1e-4
RTOL_BF16, ATOL_BF16 = 1e-2, 1e-4


# Error model of a long fp32 sum. An output element y = sum_i t_i added in fp32 in an
# order other than the oracle's differs from it by rounding noise proportional to
# sum_i |t_i|, not to |y| (cancellation) and not to a constant (hub rows add 10^3..10^5
# terms). With unit roundoff u = 2^-24 a sequential sum of n terms of random sign has a
# standard error of about 0.35 u sum|t|, a tree sum less; SUM_ULPS * u * sum|t| with
# SUM_ULPS = 4 is beyond ten standard errors of either and still 25 times below the
# worst case of a 100-deep order. Tests pass ``abs_sum`` (the same reduction evaluated
# on absolute values, usually by the oracle itself) and the bound becomes
#     atol 1e-4 + rtol 1e-5 |want| + SUM_ULPS * 2^-24 * abs_sum,
# so that rows of a few dozen terms keep the plain bar and long rows get exactly the
# allowance their own data justifies. ``ulps`` raises the factor for quantities that
# carry the relative error of expf of a softmax argument (|argument| * u each).
UNIT_ROUNDOFF = 2.0 ** -24
SUM_ULPS = 4.0


def _np(a):
    return a.detach().cpu().numpy() if isinstance(a, torch.Tensor) else np.asarray(a)


def assert_close(got, want, rtol=RTOL_F32, atol=ATOL_F32, what="", abs_sum=None, ulps=SUM_ULPS):
    got, want = _np(got), _np(want)
    assert got.shape == want.shape, "%s shape %s vs %s" % (what, got.shape, want.shape)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = atol + rtol * np.abs(want.astype(np.float64))
    if abs_sum is not None:
        bound = bound + ulps * UNIT_ROUNDOFF * np.abs(_np(abs_sum).astype(np.float64))
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError("%s: %d / %d elements off; worst at %s got %r want %r" %
                             (what, bad.sum(), bad.size, i, got[i], want[i]))


def spmm_abs_sums(values, indptr, indices, x, gy=None):
    """Sums of absolute terms of the multi-head SpMM's three reductions (``abs_sum`` of
    ``assert_close``): out = sum a x, and with ``gy`` also grad_a = sum_f gy x and
    grad_x = sum_e a gy, each evaluated by the oracle on the absolute inputs."""
    import oracle
    a, xa = np.abs(_np(values)), np.abs(_np(x))
    out = oracle.mh_spmm_forward(a, indptr, indices, xa)
    if gy is None:
        return out
    ga, gx = oracle.mh_spmm_backward(a, indptr, indices, xa, np.abs(_np(gy)))
    return out, ga, gx


def softmax_backward_abs_sums(indptr, indices, attn, grad_abs, n_src):
    """Bounds on the absolute terms behind the edge-softmax backward (sddmm_cuda.cu:36-66):
    with T[r,b,h] = sum_e a_e |g_e| over the edges of destination r that carry block tag b,
    grad_query[b,r,h] = sum_e a_e (g_e - S) d_e has absolute terms below 2 T, and the
    per-edge logit gradient is below a_e (|g_e| + T), summed per source for grad_key.
    ``grad_abs``: |g| per edge and head, or a bound on it (for the fused op, whose g is
    itself a dot product, the dot of the absolute operands). Returns (query, key) bounds
    shaped [n_bid, n_dst, H] and [n_src, H]."""
    indptr, indices = _np(indptr).astype(np.int64), _np(indices).astype(np.int64)
    a, g = _np(attn).astype(np.float64), np.abs(_np(grad_abs)).astype(np.float64)
    n_dst, h = indptr.size - 1, a.shape[1]
    rows = np.repeat(np.arange(n_dst), np.diff(indptr))
    bid, col = indices >> 24, indices & 0xffffff
    n_bid = int(bid.max()) + 1 if bid.size else 1
    t = np.zeros((n_bid * n_dst, h))
    np.add.at(t, bid * n_dst + rows, a * g)
    key_bound = np.zeros((n_src, h))
    np.add.at(key_bound, col, a * (g + t[bid * n_dst + rows]))
    return 2.0 * t.reshape(n_bid, n_dst, h), key_bound


def random_csr(n_dst, n_src, density, seed, hub_rows=(), hub_degree=0, empty_rows=()):
    """Canonical CSR with a given density plus optional hub / empty rows."""
    rng = np.random.default_rng(seed)
    rows, cols = np.nonzero(rng.random((n_dst, n_src)) < density)
    keep = ~np.isin(rows, np.asarray(list(empty_rows), dtype=np.int64))
    rows, cols = rows[keep], cols[keep]
    for r in hub_rows:
        c = rng.choice(n_src, size=min(hub_degree, n_src), replace=False)
        rows = np.concatenate([rows, np.full(c.shape, r)])
        cols = np.concatenate([cols, c])
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(rows), torch.from_numpy(cols),
                                              n_dst, n_src)
    return indptr, indices


def scrambled_csr(indptr, indices, seed, repeat=0.15):
    """The same rows with their edges in random order and a share of them repeated (a
    multigraph): what the reference's loops accept (YiTu_GNN_kernel.cu:186-199 walks
    whatever the row holds), though most builders emit sorted, unique columns."""
    rng = np.random.default_rng(seed)
    ip = indptr.numpy().astype(np.int64)
    ix = indices.numpy()
    rows = np.repeat(np.arange(len(ip) - 1), np.diff(ip))
    extra = rng.random(len(ix)) < repeat
    rows = np.concatenate([rows, rows[extra]])
    cols = np.concatenate([ix, ix[extra]])
    order = np.lexsort((rng.random(len(rows)), rows))  # rows together, edges shuffled inside
    rows, cols = rows[order], cols[order]
    new_ip = np.zeros(len(ip), dtype=np.int64)
    np.cumsum(np.bincount(rows, minlength=len(ip) - 1), out=new_ip[1:])
    return torch.from_numpy(new_ip.astype(np.int32)), torch.from_numpy(cols.astype(np.int32))


def powerlaw_graph(scale, m, seed):
    src, dst = graphgen.rmat(scale, m, seed, self_loops=True)
    return graphgen.csr_by_destination(src, dst, 1 << scale)


from oracle.temporal import dense_temporal_attention  # noqa: E402,F401  (dense masked attention)
