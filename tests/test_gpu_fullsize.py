"""Size-independent properties at the full sizes of the second to fifth
configurations (R-MAT 2^18 nodes / 13 M draws, 4 heads x 64; R-MAT 2^21 nodes /
63 M draws, 128 features; 4 node types with 8 relations at 256 features; 2^20
temporal events with 2,048 roots x 20 neighbours), where the CPU oracle would
take minutes: exact row counts, column-sum checksums in float64, the adjoint
identity between forward and backward, softmax rows that sum to one, closed
forms, host and device sampler bit for bit, reproducibility; and values: thousands
of sampled output and gradient rows (the widest rows and the rows either side of the
planning threshold among them) against float64 index algebra in torch."""
import pytest
import torch

from yitu_amd import YiTu_GNN_kernel as K, graph_ext
from yitu_amd.data import graphgen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def c3(dev):
    src, dst = graphgen.rmat(21, 63_000_000, 20242, self_loops=True, device=dev)
    n = 1 << 21
    rp, ci = graphgen.csr_by_destination(src, dst, n)
    del src, dst
    return n, rp, ci, graphgen.gcn_norm(rp)


def test_c3_neighbour_counts_are_exact(dev, c3):
    """Unweighted aggregation of all-ones features is the in-degree, an integer below
    2^24: every sum order gives the same bits."""
    n, rp, ci, _ = c3
    deg = (rp[1:] - rp[:-1]).to(torch.float32)
    assert int(deg.max()) > 10_000
    for dtype in (torch.float32, torch.bfloat16):
        out = K._aggregate(torch.ones(n, 128, dtype=dtype, device=dev), rp, ci, None, 1.0)
        assert torch.equal(out, deg[:, None].expand(-1, 128))


def test_c3_column_sum_checksum_and_reproducibility(dev, c3):
    """1^T (A X) = (A^T 1)^T X, the right side in float64 with torch index ops."""
    n, rp, ci, s = c3
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(n, 128, generator=g, device=dev)
    out = K._aggregate(x, rp, ci, s, 1.0)
    assert torch.equal(out, K._aggregate(x, rp, ci, s, 1.0))
    rows = torch.repeat_interleave(torch.arange(n, device=dev), (rp[1:] - rp[:-1]).long())
    w = s.double()[rows] * s.double()[ci.long()]
    colw = torch.zeros(n, dtype=torch.float64, device=dev).index_add_(0, ci.long(), w)
    want = colw @ x.double()
    got = out.double().sum(0)
    scale = (colw.abs() @ x.double().abs()).max()
    assert float((got - want).abs().max()) < 1e-6 * float(scale)
    # bf16 inputs that are exactly representable give the fp32 result up to summation order
    xb = x.to(torch.bfloat16)
    ob = K._aggregate(xb, rp, ci, s, 1.0)
    of = K._aggregate(xb.float(), rp, ci, s, 1.0)
    assert torch.allclose(ob, of, rtol=1e-5, atol=1e-4)


@pytest.fixture(scope="module")
def c3_reordered(dev):
    """The same draws with the vertex ids renamed by the host library's Rabbit-Order
    reorder (one thread: the reproducible order), as the benchmark runs them."""
    from yitu_amd import rabbit
    src, dst = graphgen.rmat(21, 63_000_000, 20242, self_loops=True, device=dev)
    n = 1 << 21
    ei = rabbit.reorder(torch.stack([src, dst]).to(torch.int32).cpu())
    del src, dst
    rp, ci = graphgen.csr_by_destination(ei[0].to(dev).long(), ei[1].to(dev).long(), n)
    del ei
    return n, rp, ci, graphgen.gcn_norm(rp)


def _sample_rows(rp, count, seed, dev):
    """Random rows plus the ones a row-split kernel treats differently: the widest row,
    rows of 63 / 64 / 65 edges (either side of the planning threshold), a few rows of
    several items, an empty row if there is one."""
    deg = (rp[1:] - rp[:-1]).long()
    g = torch.Generator(device=dev).manual_seed(seed)
    picks = [torch.randint(0, deg.numel(), (count,), generator=g, device=dev), deg.argmax()[None]]
    for d in (0, 1, 63, 64, 65, 127, 128, 129):
        picks.append(torch.nonzero(deg == d).flatten()[:8])
    picks.append(torch.topk(deg, 32).indices)
    return torch.unique(torch.cat(picks))


def _edges_of(rp, rows):
    """(edge ids, position of the edge's row in ``rows``) for the CSR rows ``rows``."""
    beg, cnt = rp[rows].long(), (rp[rows + 1] - rp[rows]).long()
    which = torch.repeat_interleave(torch.arange(rows.numel(), device=rows.device), cnt)
    first = torch.cumsum(cnt, 0) - cnt
    e = beg[which] + torch.arange(which.numel(), device=rows.device) - first[which]
    return e, which


def test_c3_reordered_graph_sampled_rows_against_float64(dev, c3_reordered):
    """Values, not only checksums: about 4,000 output rows of the reordered graph, among
    them the widest row (about 10^5 edges) and rows of 63 / 64 / 65 edges, against
    float64 index algebra in torch; fp32 rows and bf16 rows, through the row plan, with and
    without the per-edge column scales that the benchmark passes, weighted and unweighted."""
    from helpers import assert_close
    n, rp, ci, s = c3_reordered
    rows = _sample_rows(rp, 4096, 41, dev)
    deg = (rp[1:] - rp[:-1]).long()
    assert int(deg[rows].max()) == int(deg.max()) > 10_000
    assert all(int((deg[rows] == d).sum()) > 0 for d in (63, 64, 65))
    e, which = _edges_of(rp, rows)
    col = ci[e].long()
    w = s.double()[rows][which] * s.double()[col]
    g = torch.Generator(device=dev).manual_seed(42)
    x = torch.randn(n, 128, generator=g, device=dev)
    es = K.edge_scale(ci, s)
    for xin in (x, x.to(torch.bfloat16)):
        xd = xin.double()
        want = torch.zeros(rows.numel(), 128, dtype=torch.float64, device=dev)
        abs_sum = torch.zeros_like(want)
        for lo in range(0, e.numel(), 1 << 20):
            sl = slice(lo, lo + (1 << 20))
            t = w[sl, None] * xd[col[sl]]
            want.index_add_(0, which[sl], t)
            abs_sum.index_add_(0, which[sl], t.abs())
        for scales in (None, es):
            got = K._aggregate(xin, rp, ci, s, 1.0, edge_scale=scales)
            assert got.dtype == torch.float32
            assert_close(got[rows], want, abs_sum=abs_sum,
                         what="%s rows, edge scales %s" % (xin.dtype, scales is not None))
        # unweighted sums (SAG / GIN) on the same rows
        got = K._aggregate(xin, rp, ci, None, 0.5)
        ones = torch.zeros_like(want)
        ones_abs = torch.zeros_like(want)
        for lo in range(0, e.numel(), 1 << 20):
            sl = slice(lo, lo + (1 << 20))
            ones.index_add_(0, which[sl], 0.5 * xd[col[sl]])
            ones_abs.index_add_(0, which[sl], 0.5 * xd[col[sl]].abs())
        assert_close(got[rows], ones, abs_sum=ones_abs, what="%s rows, unweighted" % xin.dtype)


@pytest.fixture(scope="module")
def c2(dev):
    src, dst = graphgen.rmat(18, 13_000_000, 20241, device=dev)
    n = 1 << 18
    rp, ci = graphgen.csr_by_destination(src, dst, n)
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(n, 4, 64, generator=g, device=dev)
    q = torch.randn(n, 4, generator=g, device=dev)
    k = torch.randn(n, 4, generator=g, device=dev)
    return n, rp, ci, x, q, k


def _row_sums(rp, v):
    c = torch.cat([torch.zeros(1, v.size(1), dtype=torch.float64, device=v.device),
                   v.double().cumsum(0)])
    return c[rp[1:].long()] - c[rp[:-1].long()]


def test_c2_attention_rows_sum_to_one_and_fused_equals_two_ops(dev, c2):
    n, rp, ci, x, q, k = c2
    out, attn = graph_ext.gat_forward(rp, ci, q, k, x)
    nonempty = (rp[1:] > rp[:-1])
    sums = _row_sums(rp, attn)
    assert float((sums[nonempty] - 1.0).abs().max()) < 1e-5
    assert torch.all(attn >= 0)
    attn2 = graph_ext.sddmm_forward(rp, ci, q.unsqueeze(0).contiguous(), k)
    assert torch.allclose(attn, attn2, rtol=1e-5, atol=1e-7)
    out2 = graph_ext.spmm_forward(attn2, rp, ci, x)
    assert torch.allclose(out, out2, rtol=1e-5, atol=1e-4)
    # all-ones features: a convex combination of ones
    ones, _ = graph_ext.gat_forward(rp, ci, q, k, torch.ones_like(x))
    assert float((ones[nonempty] - 1.0).abs().max()) < 1e-5 and torch.all(ones[~nonempty] == 0)


def test_c2_backward_is_the_adjoint_of_forward(dev, c2):
    """out is linear in x: <gy, F(d)> = <grad_x, d>; and a central difference along a
    random direction of (q, k) matches <grad_q, dq> + <grad_k, dk>."""
    n, rp, ci, x, q, k = c2
    g = torch.Generator(device=dev).manual_seed(6)
    gy = torch.randn(n, 4, 64, generator=g, device=dev)
    d = torch.randn(n, 4, 64, generator=g, device=dev)
    out, attn = graph_ext.gat_forward(rp, ci, q, k, x)
    gq, gk, gx = graph_ext.gat_backward(rp, ci, q, k, x, attn, gy)
    fd, _ = graph_ext.gat_forward(rp, ci, q, k, d)
    lhs = float((gy.double() * fd.double()).sum())
    rhs = float((gx.double() * d.double()).sum())
    assert abs(lhs - rhs) < 1e-6 * float((gy.double().abs() * fd.double().abs()).sum())
    dq = torch.randn(n, 4, generator=g, device=dev)
    dk = torch.randn(n, 4, generator=g, device=dev)
    eps = 3e-3
    fp, _ = graph_ext.gat_forward(rp, ci, q + eps * dq, k + eps * dk, x)
    fm, _ = graph_ext.gat_forward(rp, ci, q - eps * dq, k - eps * dk, x)
    num = float((gy.double() * (fp.double() - fm.double())).sum()) / (2 * eps)
    ana = float((gq.double() * dq.double()).sum() + (gk.double() * dk.double()).sum())
    # measured against |grad| |direction|: the inner product itself nearly cancels
    scale = float(((gq.double().pow(2).sum() + gk.double().pow(2).sum()) *
                   (dq.double().pow(2).sum() + dk.double().pow(2).sum())).sqrt())
    assert abs(num - ana) < 5e-5 * scale, (num, ana, scale)
    again = graph_ext.gat_backward(rp, ci, q, k, x, attn, gy)
    assert all(torch.equal(a, b) for a, b in zip((gq, gk, gx), again))
    # with the forward output: the one-pass backward; same gradients, reproducible
    full = graph_ext.gat_backward(rp, ci, q, k, x, attn, gy, out=out)
    assert torch.equal(full[2], gx)
    for got, want in zip(full[:2], (gq, gk)):
        scale_g = float(want.abs().max())
        assert float((got - want).abs().max()) < 1e-4 * max(scale_g, 1.0)
    again = graph_ext.gat_backward(rp, ci, q, k, x, attn, gy, out=out)
    assert all(torch.equal(a, b) for a, b in zip(full, again))
    # probabilities never stored: row statistics from the forward, recomputed per edge
    out2, _, stats = graph_ext.gat_forward(rp, ci, q, k, x, stats_only=True)
    assert float((out2 - out).abs().max()) < 1e-5 * max(float(out.abs().max()), 1.0)
    again, _, _ = graph_ext.gat_forward(rp, ci, q, k, x, stats_only=True)
    assert torch.equal(again, out2)  # fixed summation order
    lean = graph_ext.gat_backward(rp, ci, q, k, x, None, gy, out=out2, stats=stats)
    for got, want in zip(lean, full):
        assert float((got - want).abs().max()) < 1e-5 * max(float(want.abs().max()), 1.0)


def test_c2_fused_gat_values_against_float64(dev, c2):
    """The fused forward and every gradient against a float64 statement of the reference's
    two ops in torch index algebra (LeakyReLU 0.2, softmax over each destination's edges,
    weighted sum; sddmm_cuda.cu:5-67, spmm_cuda.cu:4-42): grad_query and grad_key on every
    node, the output on about 4,000 destination rows and grad_features on about 4,000
    sources, the widest row and the most popular source among them."""
    from helpers import assert_close
    n, rp, ci, x, q, k = c2
    h, f = 4, 64
    nnz = ci.numel()
    deg = (rp[1:] - rp[:-1]).long()
    row = torch.repeat_interleave(torch.arange(n, device=dev), deg)
    col = ci.long()
    g = torch.Generator(device=dev).manual_seed(61)
    gy = torch.randn(n, h, f, generator=g, device=dev)
    # softmax in float64 over all edges
    z = q.double()[row] + k.double()[col]
    slope = torch.where(z > 0, torch.ones_like(z), torch.full_like(z, 0.2))
    z = z * slope
    zmax = torch.full((n, h), -1e300, dtype=torch.float64, device=dev).scatter_reduce_(
        0, row[:, None].expand(-1, h), z, "amax")
    p = torch.exp(z - zmax[row])
    a = p / torch.zeros(n, h, dtype=torch.float64, device=dev).index_add_(0, row, p)[row]
    # per-edge dots <gy[row], x[col]> and their absolute terms, in chunks
    d_attn = torch.empty(nnz, h, dtype=torch.float64, device=dev)
    d_abs = torch.empty_like(d_attn)
    for lo in range(0, nnz, 1 << 19):
        sl = slice(lo, lo + (1 << 19))
        gr, xc = gy[row[sl]].double(), x[col[sl]].double()
        d_attn[sl] = (gr * xc).sum(-1)
        d_abs[sl] = (gr.abs() * xc.abs()).sum(-1)
    ssum = torch.zeros(n, h, dtype=torch.float64, device=dev).index_add_(0, row, a * d_attn)
    dz = a * (d_attn - ssum[row]) * slope
    want_gq = torch.zeros(n, h, dtype=torch.float64, device=dev).index_add_(0, row, dz)
    want_gk = torch.zeros(n, h, dtype=torch.float64, device=dev).index_add_(0, col, dz)
    # allowances: absolute terms behind the two segmented sums (helpers.softmax_backward_abs_sums)
    t_abs = torch.zeros(n, h, dtype=torch.float64, device=dev).index_add_(0, row, a * d_abs)
    abs_gq = 2.0 * t_abs
    abs_gk = torch.zeros(n, h, dtype=torch.float64, device=dev).index_add_(
        0, col, a * (d_abs + t_abs[row]))
    # sampled destination rows: out; sampled sources: grad_features
    rows = _sample_rows(rp, 4096, 62, dev)
    e, which = _edges_of(rp, rows)
    want_out = torch.zeros(rows.numel(), h, f, dtype=torch.float64, device=dev)
    abs_out = torch.zeros_like(want_out)
    for lo in range(0, e.numel(), 1 << 19):
        sl = slice(lo, lo + (1 << 19))
        t = a[e[sl]][:, :, None] * x[col[e[sl]]].double()
        want_out.index_add_(0, which[sl], t)
        abs_out.index_add_(0, which[sl], t.abs())
    # sources sampled by out-degree, their edges found by column (independent of the
    # library's own by-source arrays)
    t_indptr = torch.zeros(n + 1, dtype=torch.long, device=dev)
    t_indptr[1:] = torch.cumsum(torch.bincount(col, minlength=n), 0)
    srcs = _sample_rows(t_indptr, 4096, 63, dev)
    pos = torch.full((n,), -1, dtype=torch.long, device=dev)
    pos[srcs] = torch.arange(srcs.numel(), device=dev)
    mine = torch.nonzero(pos[col] >= 0).flatten()
    assert mine.numel() == int((t_indptr[srcs + 1] - t_indptr[srcs]).sum())
    want_gx = torch.zeros(srcs.numel(), h, f, dtype=torch.float64, device=dev)
    abs_gx = torch.zeros_like(want_gx)
    for lo in range(0, mine.numel(), 1 << 19):
        ed = mine[lo:lo + (1 << 19)]
        t = a[ed][:, :, None] * gy[row[ed]].double()
        want_gx.index_add_(0, pos[col[ed]], t)
        abs_gx.index_add_(0, pos[col[ed]], t.abs())
    del d_abs, t_abs, p, z
    # the library: probabilities stored, and the statistics-only form the benchmark times
    out, attn = graph_ext.gat_forward(rp, ci, q, k, x)
    assert_close(attn, a, what="attn")
    assert_close(out[rows], want_out, abs_sum=abs_out, what="out")
    out2, _, stats = graph_ext.gat_forward(rp, ci, q, k, x, stats_only=True)
    assert_close(out2[rows], want_out, abs_sum=abs_out, what="out (statistics only)")
    for name, grads in (("attn", graph_ext.gat_backward(rp, ci, q, k, x, attn, gy)),
                        ("attn + out", graph_ext.gat_backward(rp, ci, q, k, x, attn, gy, out=out)),
                        ("statistics", graph_ext.gat_backward(rp, ci, q, k, x, None, gy, out=out2,
                                                              stats=stats))):
        gq, gk, gx = grads
        assert_close(gq, want_gq, abs_sum=abs_gq, what="grad_query from " + name)
        assert_close(gk, want_gk, abs_sum=abs_gk, what="grad_key from " + name)
        assert_close(gx[srcs], want_gx, abs_sum=abs_gx, what="grad_features from " + name)


# ---- fourth configuration: 4 node types, 8 relations, 256 features --------------------

@pytest.fixture(scope="module")
def c4(dev):
    from yitu_amd.xgnn_h import block as xblock
    sizes = [1 << 18, 1 << 17, 1 << 16, 1 << 15]
    off = [0]
    for n in sizes:
        off.append(off[-1] + n)
    rels = []
    for r in range(8):
        s_t, d_t = r % 4, (r + 1 + r // 4) % 4
        rp, ci = graphgen.bipartite_uniform(sizes[d_t], sizes[s_t], 8, 20243 + r, device=dev)
        indeg = (rp[1:] - rp[:-1]).float()
        norm = torch.where(indeg > 0, 1.0 / indeg.clamp(min=1), torch.zeros_like(indeg))[:, None]
        rels.append((s_t, d_t, rp, ci, norm))
    per_dst = [sum(1 for r in rels if r[1] == t) for t in range(4)]
    stacked, values = xblock.stack_blocks(
        [xblock.Block([sizes[d], sizes[s]], [rp, ci]) for s, d, rp, ci, _ in rels],
        [off[d] for _, d, _, _, _ in rels], [off[s] for s, _, _, _, _ in rels], off[-1], off[-1],
        [norm / per_dst[d] for _, d, _, _, norm in rels])
    return sizes, off, rels, per_dst, stacked.adj_sparse, values


def test_c4_stacked_relations_closed_form_and_adjoint(dev, c4):
    """Mean over each relation's neighbours, then mean over the relations of the
    destination type, as one edge-weighted product over the stacked structure:
    constant features give (relations with at least one edge into the row) /
    (relations of the type) exactly up to rounding; the result equals the
    relation-by-relation composition; <A x, y> = <x, A^T y> in float64."""
    sizes, off, rels, per_dst, (indptr, indices), values = c4
    n_all, dim = off[-1], 256
    assert indices.numel() == sum(int(r[3].numel()) for r in rels) > 7_000_000
    ones = torch.ones(n_all, 1, dim, device=dev)
    got = graph_ext.spmm_forward(values, indptr, indices, ones).view(n_all, dim)
    want = torch.zeros(n_all, device=dev)
    for _, d, rp, _, _ in rels:
        want[off[d]:off[d + 1]] += (rp[1:] > rp[:-1]).float() / per_dst[d]
    assert float((got - want[:, None]).abs().max()) < 1e-6
    g = torch.Generator(device=dev).manual_seed(9)
    x = torch.randn(n_all, dim, generator=g, device=dev)
    y = torch.randn(n_all, dim, generator=g, device=dev)
    ax = graph_ext.spmm_forward(values, indptr, indices, x.view(n_all, 1, dim)).view(n_all, dim)
    by_rel = torch.zeros(n_all, dim, device=dev)
    for s, d, rp, ci, norm in rels:
        by_rel[off[d]:off[d + 1]] += K._aggregate(x[off[s]:off[s + 1]], rp, ci, None, 1.0) * \
            (norm / per_dst[d])
    assert torch.allclose(ax, by_rel, rtol=1e-5, atol=1e-4)
    aty = graph_ext.spmm_backward(values, indptr, indices, x.view(n_all, 1, dim),
                                  y.view(n_all, 1, dim), need_grad_a=False)[1].view(n_all, dim)
    lhs = float((ax.double() * y.double()).sum())
    rhs = float((x.double() * aty.double()).sum())
    scale = float((ax.double().abs() * y.double().abs()).sum())
    assert abs(lhs - rhs) < 1e-6 * scale, (lhs, rhs, scale)
    # bf16 rows: exactly representable inputs give the fp32 result up to summation order
    xb = x.to(torch.bfloat16)
    ab = graph_ext.spmm_forward(values, indptr, indices, xb.view(n_all, 1, dim))
    af = graph_ext.spmm_forward(values, indptr, indices, xb.float().view(n_all, 1, dim))
    assert torch.allclose(ab, af, rtol=1e-5, atol=1e-4)


def test_c4_typed_gemms_against_float64(dev, c4):
    """[n_t, 256] x [256, 256] per node type, forward and both gradients, on a
    sample of rows against float64 (dW over all rows)."""
    sizes = c4[0]
    dim = 256
    g = torch.Generator(device=dev).manual_seed(11)
    for n in sizes:
        x = torch.randn(n, dim, generator=g, device=dev)
        w = torch.randn(dim, dim, generator=g, device=dev) * 0.02
        dy = torch.randn(n, dim, generator=g, device=dev)
        rows = torch.randint(0, n, (4096,), generator=g, device=dev)
        y = graph_ext.sgemm(x, w)
        assert torch.allclose(y[rows].double(), x[rows].double() @ w.double(), rtol=1e-5, atol=1e-5)
        dx = graph_ext.sgemm(dy, w, trans_b=True)
        assert torch.allclose(dx[rows].double(), dy[rows].double() @ w.double().t(), rtol=1e-5,
                              atol=1e-5)
        dw = graph_ext.sgemm(x, dy, trans_a=True)
        want = x.double().t() @ dy.double()
        # n products per element: the bar scales with sqrt(n)
        assert float((dw.double() - want).abs().max()) < 2e-6 * (n ** 0.5) * 4
        y16 = graph_ext.gemm_bf16(x.bfloat16(), w.bfloat16())
        want16 = x.bfloat16()[rows].double() @ w.bfloat16().double()
        assert torch.allclose(y16[rows].double(), want16, rtol=1e-2, atol=1e-2)


def test_c4_bf16_backward_at_full_size(dev, c4):
    """The backward of the heterogeneous layer in bf16 at the configured sizes: bf16 rows
    out of the by-source aggregation over the stacked 7.9 M-edge structure (sampled rows
    against float64, one bf16 rounding allowed on top of the fp32 bar) and the four weight
    gradients X^T . G of the real node-type heights in one grouped call (every element
    against float64, allowance from the absolute terms)."""
    from helpers import assert_close
    sizes, off, rels, per_dst, (indptr, indices), values = c4
    n_all, dim = off[-1], 256
    g = torch.Generator(device=dev).manual_seed(13)
    x16 = torch.randn(n_all, dim, generator=g, device=dev).to(torch.bfloat16)
    gy16 = torch.randn(n_all, dim, generator=g, device=dev).to(torch.bfloat16)
    # grad_x = A^T gy with bf16 gradient rows in and bf16 rows out
    got = graph_ext.spmm_backward(values, indptr, indices, x16.view(n_all, 1, dim),
                                  gy16.view(n_all, 1, dim), need_grad_a=False,
                                  grad_x_dtype=torch.bfloat16)[1].view(n_all, dim)
    assert got.dtype == torch.bfloat16
    col = indices.long() & 0xffffff
    t_indptr = torch.zeros(n_all + 1, dtype=torch.long, device=dev)
    t_indptr[1:] = torch.cumsum(torch.bincount(col, minlength=n_all), 0)
    srcs = _sample_rows(t_indptr, 4096, 14, dev)
    pos = torch.full((n_all,), -1, dtype=torch.long, device=dev)
    pos[srcs] = torch.arange(srcs.numel(), device=dev)
    row = torch.repeat_interleave(torch.arange(n_all, device=dev), (indptr[1:] - indptr[:-1]).long())
    mine = torch.nonzero(pos[col] >= 0).flatten()
    t = values[mine].double() * gy16[row[mine]].double()
    want = torch.zeros(srcs.numel(), dim, dtype=torch.float64, device=dev).index_add_(0, pos[col[mine]], t)
    abs_sum = torch.zeros_like(want).index_add_(0, pos[col[mine]], t.abs())
    # fp32 sums, then one rounding to bf16 (relative 2^-9)
    assert_close(got[srcs].float(), want, rtol=2.0 ** -8, abs_sum=abs_sum, what="bf16 grad rows")
    fp32 = graph_ext.spmm_backward(values, indptr, indices, x16.view(n_all, 1, dim),
                                   gy16.view(n_all, 1, dim), need_grad_a=False)[1].view(n_all, dim)
    assert_close(fp32[srcs], want, abs_sum=abs_sum, what="fp32 grad rows from bf16 gradients")
    assert torch.equal(got, fp32.to(torch.bfloat16))  # the same sums, rounded once
    # weight gradients of the four node types, one grouped launch
    xs = [x16[off[t]:off[t + 1]] for t in range(4)]
    gs = [got[off[t]:off[t + 1]] for t in range(4)]
    dws = graph_ext.gemm_bf16_tn_typed(xs, gs)
    for xt, gt, dw in zip(xs, gs, dws):
        want_w = xt.double().t() @ gt.double()
        abs_w = xt.double().abs().t() @ gt.double().abs()
        assert dw.dtype == torch.float32 and dw.shape == (dim, dim)
        assert_close(dw, want_w, abs_sum=abs_w, what="dW of %d rows" % xt.size(0))
    again = graph_ext.gemm_bf16_tn_typed(xs, gs)
    assert all(torch.equal(a, b) for a, b in zip(dws, again))
    # and the input gradients G . W^T through the grouped bf16 product, on sampled rows
    ws = [(torch.randn(dim, dim, generator=g, device=dev) * 0.02).to(torch.bfloat16) for _ in range(4)]
    dxs = graph_ext.gemm_bf16_typed(gs, ws, trans_b=True)
    for gt, w, dx in zip(gs, ws, dxs):
        pick = torch.randint(0, gt.size(0), (2048,), generator=g, device=dev)
        want_x = gt[pick].double() @ w.double().t()
        abs_x = gt[pick].double().abs() @ w.double().abs().t()
        assert_close(dx[pick], want_x, abs_sum=abs_x, what="dX of %d rows" % gt.size(0))


# ---- fifth configuration: 2^20 events, 2^17 nodes, 2,048 roots x 20 neighbours --------

def test_c5_device_sampler_equals_host_and_layer_equals_dense_attention(dev):
    import numpy as np
    from helpers import assert_close, dense_temporal_attention
    from yitu_amd import sampler_core
    from yitu_amd.temporal import TemporalBlock, TransfomerAttentionLayer
    rng = np.random.default_rng(20244)
    n_nodes, n_events, k, batch = 1 << 17, 1 << 20, 20, 2048
    src = ((rng.zipf(1.2, n_events) - 1) % n_nodes).astype(np.int64)
    dst = ((rng.zipf(1.2, n_events) - 1) % n_nodes).astype(np.int64)
    ts = np.sort(rng.uniform(0, 1e6, n_events)).astype(np.float32)
    node = np.concatenate([src, dst])
    other = np.concatenate([dst, src])
    eid = np.concatenate([np.arange(n_events), np.arange(n_events)])
    tt = np.concatenate([ts, ts])
    order = np.lexsort((eid, tt, node))
    indptr = np.zeros(n_nodes + 1, np.int64)
    indptr[1:] = np.cumsum(np.bincount(node, minlength=n_nodes))
    args = (indptr, other[order], eid[order], tt[order], 16, 1, 1, [k], True, False, 1, 0.0)
    host = sampler_core.ParallelSampler(*args)
    device = sampler_core.GpuParallelSampler(*args, device=dev)
    # three consecutive batches in time order: the cursors carry over between them
    for lo in (0.90, 0.93, 0.96):
        ev = np.sort(rng.integers(int(n_events * lo), int(n_events * (lo + 0.03)), batch // 2))
        roots = np.concatenate([src[ev], dst[ev]])
        root_ts = np.concatenate([ts[ev], ts[ev]])
        host.sample(roots, root_ts)
        device.sample(torch.as_tensor(roots, dtype=torch.int32, device=dev),
                      torch.as_tensor(root_ts, dtype=torch.float32, device=dev))
        tgb, dblk = host.get_ret()[0], device.get_ret()[0].cpu_block()
        for f in ("row", "col", "eid", "ts", "dts", "nodes"):
            assert np.array_equal(getattr(dblk, f)(), getattr(tgb, f)()), f
    # every root's neighbours are its k most recent events before its time
    row, dts = tgb.row(), tgb.dts()
    assert np.bincount(row, minlength=batch).max() <= k and (dts[batch:] >= 0).all()
    torch.manual_seed(20244)
    memory = torch.randn(n_nodes, 172, device=dev)
    layer = TransfomerAttentionLayer(172, 0, 100, 1, 0.0, 0.0, 100).to(dev)
    blk = TemporalBlock.from_sampler(tgb, memory, device=dev)
    assert blk.n_dst == batch and blk.num_edges() > batch
    blk.h.requires_grad_()
    out = layer(blk)
    w = torch.randn_like(out)
    (out * w).sum().backward()
    grads = [blk.h.grad.clone()] + [p.grad.clone() for p in layer.parameters()]
    blk.h.grad = None
    layer.zero_grad()
    want = dense_temporal_attention(layer, blk.h, blk.row, blk.dt, blk.n_dst, k)
    (want * w).sum().backward()
    assert_close(out, want, atol=2e-4)
    names = ["h"] + [n for n, _ in layer.named_parameters()]
    for got, ref, name in zip(grads, [blk.h.grad] + [p.grad for p in layer.parameters()], names):
        # parameter gradients sum over 2,048 roots (and up to 40,960 edges)
        rtol = 1e-3 if name == "time_enc.w.weight" else 1e-4  # products with dt up to 10^6
        assert_close(got, ref, rtol=rtol, atol=5e-3 if name != "h" else 5e-4, what=name)
