"""Size-independent properties at the full sizes of the second and third
configurations (R-MAT 2^18 nodes / 13 M draws, 4 heads x 64; R-MAT 2^21 nodes /
63 M draws, 128 features), where the CPU oracle would take minutes: exact row
counts, column-sum checksums in float64, the adjoint identity between forward
and backward, softmax rows that sum to one, reproducibility."""
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
