"""GPU parity of the graph_ext drop-in (multi-head SpMM, SDDMM + LeakyReLU +
edge softmax, hfused, the transposed-structure builder) against the CPU oracle,
through the C ABI, plus the reference's own dense-torch checks run end to end
through the autograd wrappers."""
import numpy as np
import pytest
import torch
from torch import nn

import oracle
from helpers import softmax_backward_abs_sums, spmm_abs_sums, assert_close, powerlaw_graph, random_csr
from yitu_amd import graph_ext
from yitu_amd.xgnn_h import block as xblock
from yitu_amd.xgnn_h import sparse

pytestmark = pytest.mark.gpu


def _rng_shapes(seed):
    rng = np.random.default_rng(seed)
    return (int(rng.integers(1, 300)), int(rng.integers(1, 300)), int(rng.integers(1, 33)),
            int(rng.integers(1, 257)))


# ---- transposed structure (integer work: bit exact) ---------------------------

@pytest.mark.parametrize("n_dst,n_src,density,seed", [(1, 1, 1.0, 0), (50, 70, 0.1, 1),
                                                      (3000, 2000, 0.01, 2), (10, 5000, 0.3, 3)])
def test_csr_transpose_bit_exact(dev, n_dst, n_src, density, seed):
    indptr, indices = random_csr(n_dst, n_src, density, seed, empty_rows=(0,) if n_dst > 1 else ())
    tag = (torch.arange(indices.numel()) % 3).to(torch.int32) << 24  # block tags must be ignored
    packed = indices | tag
    tr = graph_ext.transposed(indptr.to(dev), packed.to(dev), n_src)
    deg = np.diff(indptr.numpy())
    rows = np.repeat(np.arange(n_dst), deg)
    order = np.argsort(indices.numpy(), kind="stable")
    want_ptr = np.zeros(n_src + 1, np.int64)
    np.add.at(want_ptr, indices.numpy().astype(np.int64) + 1, 1)
    want_ptr = np.cumsum(want_ptr)
    assert np.array_equal(tr.t_indptr.cpu().numpy(), want_ptr)
    assert np.array_equal(tr.t_perm.cpu().numpy(), order)
    assert np.array_equal(tr.t_rows.cpu().numpy(), rows[order])


# ---- SpMM -----------------------------------------------------------------------

@pytest.mark.parametrize("seed", range(8))
def test_spmm_random_shapes(dev, seed):
    """Shape ranges of check_gspmm (test_kernel.py:25-29)."""
    n_src, n_dst, h, f = _rng_shapes(seed)
    indptr, indices = random_csr(n_dst, n_src, 0.05, seed)
    g = torch.Generator().manual_seed(seed)
    values = torch.randn(indices.numel(), h, generator=g)
    x = torch.randn(n_src, h, f, generator=g)
    gy = torch.randn(n_dst, h, f, generator=g)
    args = (values.to(dev), indptr.to(dev), indices.to(dev), x.to(dev))
    what = "n_dst=%d n_src=%d H=%d F=%d" % (n_dst, n_src, h, f)
    abs_out, abs_ga, abs_gx = spmm_abs_sums(values, indptr, indices, x, gy)
    assert_close(graph_ext.spmm_forward(*args), oracle.mh_spmm_forward(values, indptr, indices, x),
                 abs_sum=abs_out, what=what)
    ga, gx = graph_ext.spmm_backward(*args, gy.to(dev))
    want_ga, want_gx = oracle.mh_spmm_backward(values, indptr, indices, x, gy)
    assert_close(ga, want_ga, abs_sum=abs_ga, what="grad_a " + what)
    assert_close(gx, want_gx, abs_sum=abs_gx, what="grad_x " + what)


@pytest.mark.parametrize("h,f", [(4, 64), (1, 128), (8, 8), (2, 600), (3, 5)])
def test_spmm_power_law_with_hub_rows_and_columns(dev, h, f):
    indptr, indices = powerlaw_graph(13, 150000, h * 100 + f)
    n = indptr.numel() - 1
    assert (indptr[1:] - indptr[:-1]).max() >= 512
    g = torch.Generator().manual_seed(1)
    values = torch.randn(indices.numel(), h, generator=g)
    x = torch.randn(n, h, f, generator=g)
    gy = torch.randn(n, h, f, generator=g)
    args = (values.to(dev), indptr.to(dev), indices.to(dev), x.to(dev))
    abs_out, abs_ga, abs_gx = spmm_abs_sums(values, indptr, indices, x, gy)
    assert_close(graph_ext.spmm_forward(*args), oracle.mh_spmm_forward(values, indptr, indices, x),
                 abs_sum=abs_out)
    ga, gx = graph_ext.spmm_backward(*args, gy.to(dev))
    want_ga, want_gx = oracle.mh_spmm_backward(values, indptr, indices, x, gy)
    assert_close(ga, want_ga, abs_sum=abs_ga)
    assert_close(gx, want_gx, abs_sum=abs_gx)
    ga2, gx2 = graph_ext.spmm_backward(*args, gy.to(dev))
    assert torch.equal(ga, ga2) and torch.equal(gx, gx2)  # no atomics: reproducible


@pytest.mark.parametrize("h,f", [(1, 256), (4, 64), (2, 64), (1, 64), (2, 24), (3, 5), (1, 8)])
def test_spmm_bf16_features(dev, h, f):
    """bf16 feature rows, fp32 edge values and accumulation: equal to the fp32 op on the
    rounded features (tolerance of the bf16 bar; in fact only the order of the fp32 sums
    differs), on a power-law graph so that planned rows are covered."""
    indptr, indices = powerlaw_graph(12, 50000, 9 * h + f)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(h + f)
    values = torch.rand(indices.numel(), h, generator=g)
    x16 = torch.randn(n, h, f, generator=g).to(torch.bfloat16)
    want = oracle.mh_spmm_forward(values, indptr, indices, x16.float())
    got = graph_ext.spmm_forward(values.to(dev), indptr.to(dev), indices.to(dev), x16.to(dev))
    assert got.dtype == torch.float32
    assert_close(got, want, rtol=1e-2, atol=1e-4, what="H=%d F=%d" % (h, f))
    same = graph_ext.spmm_forward(values.to(dev), indptr.to(dev), indices.to(dev),
                                  x16.float().to(dev))
    assert_close(got, same, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("h,f", [(1, 256), (4, 64), (2, 64), (1, 64), (2, 24)])
def test_spmm_backward_bf16_rows(dev, h, f):
    """grad_x of the product from bf16 gradient rows (fp32 weights, fp32 sums, fp32 out):
    equal to the fp32 op on the same (exactly representable) rows, hence to the oracle,
    on a power-law graph so that the by-source structure has planned rows."""
    indptr, indices = powerlaw_graph(12, 50000, 7 * h + f)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(h * f)
    values = torch.rand(indices.numel(), h, generator=g)
    x = torch.randn(n, h, f, generator=g)
    gy16 = torch.randn(n, h, f, generator=g).to(torch.bfloat16)
    args = (values.to(dev), indptr.to(dev), indices.to(dev))
    ga, gx = graph_ext.spmm_backward(*args, x.to(dev).to(torch.bfloat16), gy16.to(dev),
                                     need_grad_a=False)
    assert ga is None and gx.dtype == torch.float32
    want = oracle.mh_spmm_backward(values, indptr, indices, x, gy16.float())[1]
    abs_sum = oracle.mh_spmm_backward(values.abs(), indptr, indices, x.abs(), gy16.float().abs())[1]
    assert_close(gx, want, rtol=1e-2, atol=1e-4, what="bf16 bar")
    assert_close(gx, want, abs_sum=abs_sum, what="fp32 bar")
    with pytest.raises(RuntimeError, match="grad_x only"):
        graph_ext.spmm_backward(*args, x.to(dev), gy16.to(dev))


@pytest.mark.parametrize("h,f", [(1, 256), (4, 64), (2, 64), (1, 64), (1, 32), (2, 24), (1, 8)])
def test_spmm_bf16_rows_in_and_out(dev, h, f):
    """bf16 rows out: exactly the fp32-out result of the same call rounded once to nearest
    even (short rows, single-item rows and reduced rows all take the same store), forward
    and as the grad_x of the backward."""
    indptr, indices = powerlaw_graph(12, 50000, 5 * h + f)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(3 * h + f)
    values = torch.rand(indices.numel(), h, generator=g).to(dev)
    x16 = torch.randn(n, h, f, generator=g).to(torch.bfloat16).to(dev)
    args = (values, indptr.to(dev), indices.to(dev))
    full = graph_ext.spmm_forward(*args, x16)
    got = graph_ext.spmm_forward(*args, x16, out_dtype=torch.bfloat16)
    assert got.dtype == torch.bfloat16 and torch.equal(got, full.to(torch.bfloat16))
    gx32 = graph_ext.spmm_backward(*args, x16, x16, need_grad_a=False)[1]
    gx16 = graph_ext.spmm_backward(*args, x16, x16, need_grad_a=False,
                                   grad_x_dtype=torch.bfloat16)[1]
    assert gx16.dtype == torch.bfloat16 and torch.equal(gx16, gx32.to(torch.bfloat16))
    with pytest.raises(RuntimeError, match="out_dtype"):
        graph_ext.spmm_forward(*args, x16.float(), out_dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="grad_x_dtype"):
        graph_ext.spmm_backward(*args, x16.float(), x16.float(), need_grad_a=False,
                                grad_x_dtype=torch.bfloat16)


def test_spmm_bf16_rows_out_rejects_odd_head_width(dev):
    indptr, indices = powerlaw_graph(8, 2000, 1)
    n = indptr.numel() - 1
    x16 = torch.zeros(n, 3, 5, dtype=torch.bfloat16, device=dev)
    values = torch.ones(indices.numel(), 3, device=dev)
    with pytest.raises(RuntimeError, match="out_dtype"):
        graph_ext.spmm_forward(values, indptr.to(dev), indices.to(dev), x16,
                               out_dtype=torch.bfloat16)


def test_spmm_more_than_65535_rows(dev):
    """The reference's dim3(n_heads, n_nodes) launch is invalid above 65,535 rows."""
    n_dst, n_src, h, f = 70000, 1000, 2, 8
    g = torch.Generator().manual_seed(0)
    deg = torch.randint(0, 6, (n_dst,), generator=g)
    indptr = torch.zeros(n_dst + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(deg, 0)
    indices = torch.randint(0, n_src, (int(indptr[-1]),), generator=g, dtype=torch.int32)
    values = torch.randn(indices.numel(), h, generator=g)
    x = torch.randn(n_src, h, f, generator=g)
    got = graph_ext.spmm_forward(values.to(dev), indptr.to(dev), indices.to(dev), x.to(dev))
    assert_close(got, oracle.mh_spmm_forward(values, indptr, indices, x))


# ---- SDDMM + softmax --------------------------------------------------------------

@pytest.mark.parametrize("h", [1, 2, 3, 4, 7, 8, 16, 33, 70])
@pytest.mark.parametrize("deterministic", [True, False])
def test_sddmm_head_counts(dev, h, deterministic):
    n_dst, n_src = 211, 157
    indptr, indices = random_csr(n_dst, n_src, 0.1, h, hub_rows=(5,), hub_degree=150,
                                 empty_rows=(0, 210))
    g = torch.Generator().manual_seed(h)
    q = torch.randn(1, n_dst, h, generator=g)
    k = torch.randn(n_src, h, generator=g)
    ge = torch.randn(indices.numel(), h, generator=g)
    dargs = (indptr.to(dev), indices.to(dev), q.to(dev), k.to(dev))
    attn = graph_ext.sddmm_forward(*dargs)
    want = oracle.sddmm_forward(indptr, indices, q, k)
    assert_close(attn, want, what="attn H=%d" % h)
    gq, gk = graph_ext.sddmm_backward(*dargs, attn, ge.to(dev), deterministic=deterministic)
    want_gq, want_gk = oracle.sddmm_backward(indptr, indices, q, k, want, ge)
    assert_close(gq, want_gq, what="grad_q H=%d" % h)
    assert_close(gk, want_gk, what="grad_k H=%d" % h)
    assert torch.all(gq[0, 0] == 0) and torch.all(gq[0, 210] == 0)  # empty rows


@pytest.mark.parametrize("pattern", ["boundaries", "tiny", "mixed", "sparse"])
@pytest.mark.parametrize("h", [1, 2, 4, 8, 3])
def test_packed_rows_at_chunk_boundaries(dev, pattern, h):
    """Row lengths chosen against the one-lane-per-edge kernels: a wave packs whole rows
    into chunks of at most 64 edges and owns up to 63 rows, so rows of 63 / 64 / 65 edges
    next to each other, runs of empty rows, rows of one edge and rows that the plan takes
    (64 and more) between short ones all have to land in the right chunk. Attention forward
    and backward, the fused forward with row statistics, and grad_key's segmented sum."""
    g = torch.Generator().manual_seed(len(pattern) * 10 + h)
    n_dst, n_src = 20000, 3000  # more than 16,384 rows: several rows per wave
    if pattern == "boundaries":
        choice = torch.tensor([0, 1, 62, 63, 64, 65, 31, 32, 33, 2, 127, 128, 129])
    elif pattern == "tiny":
        choice = torch.tensor([0, 0, 0, 1, 1, 2, 3])
    elif pattern == "mixed":
        choice = torch.tensor([0, 5, 9, 17, 40, 63, 64, 200, 1, 1, 700])
    else:
        choice = torch.tensor([0] * 30 + [7, 63])
    deg = choice[torch.randint(0, choice.numel(), (n_dst,), generator=g)]
    indptr = torch.zeros(n_dst + 1, dtype=torch.int32)
    indptr[1:] = torch.cumsum(deg, 0)
    nnz = int(indptr[-1])
    indices = torch.randint(0, n_src, (nnz,), generator=g, dtype=torch.int32)
    q = torch.randn(1, n_dst, h, generator=g)
    k = torch.randn(n_src, h, generator=g)
    ge = torch.randn(nnz, h, generator=g)
    dargs = (indptr.to(dev), indices.to(dev), q.to(dev), k.to(dev))
    attn = graph_ext.sddmm_forward(*dargs)
    want = oracle.sddmm_forward(indptr, indices, q, k)
    assert_close(attn, want, what="attn")
    gq, gk = graph_ext.sddmm_backward(*dargs, attn, ge.to(dev))
    want_gq, want_gk = oracle.sddmm_backward(indptr, indices, q, k, want, ge)
    abs_gq, abs_gk = softmax_backward_abs_sums(indptr, indices, want, ge.abs(), n_src)
    assert_close(gq, want_gq, abs_sum=abs_gq, what="grad_q")
    assert_close(gk, want_gk, abs_sum=abs_gk, what="grad_k")
    assert torch.all(gq[0][deg == 0] == 0)
    if h in (1, 2, 4):  # rows of 256 floats: the fused forward's whole-wave layout
        f = 256 // h
        x = torch.randn(n_src, h, f, generator=g)
        out, _, stats = graph_ext.gat_forward(indptr.to(dev), indices.to(dev), q[0].to(dev),
                                              k.to(dev), x.to(dev), stats_only=True)
        want_out = oracle.mh_spmm_forward(want, indptr, indices, x)
        assert_close(out, want_out, abs_sum=spmm_abs_sums(want, indptr, indices, x),
                     what="fused out")
        assert torch.all(out[deg == 0] == 0)
        # (max, 1 / sum) of every non-empty row reproduce the probabilities
        rows = torch.repeat_interleave(torch.arange(n_dst), deg.long())
        logit = torch.nn.functional.leaky_relu(q[0][rows] + k[indices.long()], 0.2)
        st = stats.cpu()
        again = torch.exp(logit - st[rows, :, 0]) * st[rows, :, 1]
        assert_close(again, want, rtol=1e-4, atol=1e-6, what="row statistics")


@pytest.mark.parametrize("h", [4, 8, 5])
def test_sddmm_power_law_hub_rows(dev, h):
    indptr, indices = powerlaw_graph(13, 150000, 40 + h)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(2)
    q = torch.randn(1, n, h, generator=g)
    k = torch.randn(n, h, generator=g)
    ge = torch.randn(indices.numel(), h, generator=g)
    dargs = (indptr.to(dev), indices.to(dev), q.to(dev), k.to(dev))
    attn = graph_ext.sddmm_forward(*dargs)
    want = oracle.sddmm_forward(indptr, indices, q, k)
    assert_close(attn, want)
    for det in (True, False):
        gq, gk = graph_ext.sddmm_backward(*dargs, attn, ge.to(dev), deterministic=det)
        want_gq, want_gk = oracle.sddmm_backward(indptr, indices, q, k, want, ge)
        abs_gq, abs_gk = softmax_backward_abs_sums(indptr, indices, want, ge, n)
        assert_close(gq, want_gq, abs_sum=abs_gq)
        assert_close(gk, want_gk, abs_sum=abs_gk)


def test_sddmm_large_logits_do_not_overflow(dev):
    """Logits near 100 overflow the reference's un-shifted expf; the shifted form stays finite
    and still sums to one."""
    indptr, indices = random_csr(50, 50, 0.2, 3)
    q = torch.full((1, 50, 2), 60.0)
    k = torch.rand(50, 2) * 40
    attn = graph_ext.sddmm_forward(indptr.to(dev), indices.to(dev), q.to(dev), k.to(dev)).cpu()
    assert torch.isfinite(attn).all()
    rows = torch.repeat_interleave(torch.arange(50), (indptr[1:] - indptr[:-1]).long())
    sums = torch.zeros(50, 2).index_add_(0, rows, attn)
    assert torch.allclose(sums[(indptr[1:] - indptr[:-1]) > 0], torch.ones(1), atol=1e-5)


@pytest.mark.parametrize("n_blk", [2, 5, 16])
def test_stitched_blocks_multi_bid(dev, n_blk):
    rng = np.random.default_rng(n_blk)
    n_dst, h, f = 300, 4, 16
    blocks, xs, qs, ks = [], [], [], []
    for b in range(n_blk):
        n_src = int(rng.integers(5, 200))
        ip, ix = random_csr(n_dst, n_src, 0.05, 10 * n_blk + b, hub_rows=(b,) if b < 2 else (),
                            hub_degree=n_src)
        blocks.append(xblock.Block([n_dst, n_src], [ip, ix]))
        xs.append(torch.from_numpy(rng.standard_normal((n_src, h, f)).astype(np.float32)))
        qs.append(torch.from_numpy(rng.standard_normal((n_dst, h)).astype(np.float32)))
        ks.append(torch.from_numpy(rng.standard_normal((n_src, h)).astype(np.float32)))
    st = xblock.stitch_csr(blocks)
    sp, si = st.adj_sparse
    q, k, x = torch.stack(qs), torch.cat(ks), torch.cat(xs)
    ge = torch.from_numpy(rng.standard_normal((si.numel(), h)).astype(np.float32))
    dargs = (sp.to(dev), si.to(dev), q.to(dev), k.to(dev))
    attn = graph_ext.sddmm_forward(*dargs)
    want = oracle.sddmm_forward(sp, si, q, k)
    assert_close(attn, want)
    out = graph_ext.spmm_forward(attn, sp.to(dev), si.to(dev), x.to(dev))
    assert_close(out, oracle.mh_spmm_forward(want, sp, si, x))
    gq, gk = graph_ext.sddmm_backward(*dargs, attn, ge.to(dev))
    want_gq, want_gk = oracle.sddmm_backward(sp, si, q, k, want, ge)
    assert_close(gq, want_gq)
    assert_close(gk, want_gk)


@pytest.mark.parametrize("n_blk,h,f,head_mean", [(2, 4, 16, False), (5, 4, 64, True),
                                                 (16, 2, 8, False), (3, 1, 256, False)])
def test_stitched_blocks_fused_attention(dev, n_blk, h, f, head_mean):
    """The fused attention op on a stitched block (one query block per relation, softmax per
    (destination, block tag), sddmm_cuda.cu:11-31 followed by spmm_cuda.cu:4-21) against
    the oracle's two functions, forward and every gradient; hub rows included, and
    (4 x 64, 1 x 256) the shapes whose backward is the single by-source pass."""
    from yitu_amd.xgnn_h import sparse
    rng = np.random.default_rng(n_blk)
    n_dst = 300
    blocks, xs, qs, ks = [], [], [], []
    for b in range(n_blk):
        n_src = int(rng.integers(5, 200))
        ip, ix = random_csr(n_dst, n_src, 0.05, 10 * n_blk + b, hub_rows=(b,) if b < 2 else (),
                            hub_degree=n_src, empty_rows=(7 + b,))
        blocks.append(xblock.Block([n_dst, n_src], [ip, ix]))
        xs.append(torch.from_numpy(rng.standard_normal((n_src, h, f)).astype(np.float32)))
        qs.append(torch.from_numpy(rng.standard_normal((n_dst, h)).astype(np.float32)))
        ks.append(torch.from_numpy(rng.standard_normal((n_src, h)).astype(np.float32)))
    st = xblock.stitch_csr(blocks)
    sp, si = st.adj_sparse
    q, k, x = torch.stack(qs), torch.cat(ks), torch.cat(xs)
    dq, dk, dx = (t.to(dev).requires_grad_() for t in (q, k, x))
    out = sparse.fused_gat(st.to(dev), dq, dk, dx, head_mean=head_mean)
    want_attn = oracle.sddmm_forward(sp, si, q, k)
    want = oracle.mh_spmm_forward(want_attn, sp, si, x)
    g_out = torch.from_numpy(rng.standard_normal(out.shape).astype(np.float32))
    out.backward(g_out.to(dev))
    g_full = g_out.unsqueeze(1).expand(-1, h, -1) / h if head_mean else g_out
    g_full = np.ascontiguousarray(g_full.numpy())
    abs_out, abs_ga, abs_gx = spmm_abs_sums(want_attn, sp, si, x, g_full)
    assert_close(out, want.mean(axis=1) if head_mean else want,
                 abs_sum=abs_out.mean(axis=1) if head_mean else abs_out)
    want_ga, want_gx = oracle.mh_spmm_backward(want_attn, sp, si, x.numpy(), g_full)
    want_gq, want_gk = oracle.sddmm_backward(sp, si, q.numpy(), k.numpy(), want_attn, want_ga)
    abs_gq, abs_gk = softmax_backward_abs_sums(sp, si, want_attn, abs_ga, k.shape[0])
    assert_close(dx.grad, want_gx, abs_sum=abs_gx, what="grad_x")
    assert_close(dq.grad, want_gq, abs_sum=abs_gq, what="grad_query")
    assert_close(dk.grad, want_gk, abs_sum=abs_gk, what="grad_key")
    # one query block: the same entry point, the plain block
    ip0, ix0 = blocks[0].adj_sparse
    want_one = oracle.mh_spmm_forward(oracle.sddmm_forward(ip0, ix0, qs[0].unsqueeze(0), ks[0]),
                                      ip0, ix0, xs[0])
    one = sparse.fused_gat(xblock.Block(blocks[0].size, [ip0.to(dev), ix0.to(dev)]),
                           qs[0].to(dev).unsqueeze(0), ks[0].to(dev), xs[0].to(dev))
    assert_close(one, want_one)


# ---- the reference's own checks, end to end through autograd -----------------------

@pytest.mark.parametrize("seed", range(4))
def test_check_gsddmm_dense_reference(dev, seed):
    """test_kernel.py:97-184 with seeded inputs: fused_gsddmm -> gspmm against
    dense LeakyReLU / -1e38 mask / softmax / bmm, forward and Linear weight grads."""
    rng = np.random.default_rng(seed)
    n_src, n_dst = int(rng.integers(1, 512)), int(rng.integers(1, 512))
    h, f = int(rng.integers(1, 17)), int(rng.integers(1, 257))
    torch.manual_seed(seed)
    adj = (torch.rand(n_dst, n_src) < 0.02).float()
    if adj.max() == 0:
        adj[0, 0] = 1.0
    from yitu_amd.xgnn_h import convert
    (indptr, indices), _ = convert.to_csr(adj)
    x_dst = torch.randn(n_dst, h, f, device=dev)
    x_src = torch.randn(n_src, h, f, device=dev)
    lq, lk = nn.Linear(f, 1).to(dev), nn.Linear(f, 1).to(dev)
    blk = xblock.Block([n_dst, n_src], [indptr, indices]).to(dev)
    adj = adj.to(dev)
    q, k = lq(x_dst).squeeze(-1), lk(x_src).squeeze(-1)
    e = nn.functional.leaky_relu(q[:, None, :] + k[None, :, :], 0.2)
    e = torch.where(adj[:, :, None] > 0, e, torch.full_like(e, -1e38))
    a1 = torch.softmax(e.permute(2, 0, 1), dim=-1) * adj[None]
    y1 = torch.bmm(a1, x_src.transpose(0, 1)).transpose(0, 1)
    y1.sum().backward()
    gq1, gk1 = lq.weight.grad.clone(), lk.weight.grad.clone()
    lq.zero_grad()
    lk.zero_grad()
    q, k = lq(x_dst).squeeze(-1), lk(x_src).squeeze(-1)
    a2 = sparse.fused_gsddmm(blk, q, k)
    y2 = sparse.gspmm(blk, a2, x_src)
    y2.sum().backward()
    assert torch.allclose(y1, y2, atol=1e-3)
    assert torch.allclose(gq1, lq.weight.grad, atol=1e-3)
    assert torch.allclose(gk1, lk.weight.grad, atol=1e-3)


def test_check_hfuse(dev):
    """test_kernel.py:362-433: hfused == the two separate ops (its fixed shape)."""
    n_dst, n_src, h, f = 4096, 2048, 8, 4
    a_ptr, a_idx = random_csr(n_dst, n_src, 0.02, 1)
    b_ptr, b_idx = random_csr(n_dst, n_src, 0.02, 2)
    g = torch.Generator().manual_seed(0)
    vals = torch.randn(a_idx.numel(), h, generator=g).to(dev)
    x_src = torch.randn(n_src, h, f, generator=g).to(dev).requires_grad_()
    q = torch.randn(n_dst, h, generator=g).to(dev).requires_grad_()
    k = torch.randn(n_src, h, generator=g).to(dev).requires_grad_()
    ba = xblock.Block([n_dst, n_src], [a_ptr, a_idx]).to(dev)
    bb = xblock.Block([n_dst, n_src], [b_ptr, b_idx]).to(dev)
    y1 = sparse.gspmm(ba, vals, x_src)
    y2 = sparse.fused_gsddmm(bb, q, k)
    y3, y4 = sparse.hfused_spddmm(ba, vals, x_src, bb, q, k)
    assert torch.allclose(y1, y3, atol=1e-3) and torch.allclose(y2, y4, atol=1e-3)
    w = torch.randn_like(y4)
    (y1.sum() + (y2 * w).sum()).backward()
    g1 = [t.grad.clone() for t in (x_src, q, k)]
    for t in (x_src, q, k):
        t.grad = None
    (y3.sum() + (y4 * w).sum()).backward()
    for a, b in zip(g1, (x_src, q, k)):
        assert torch.allclose(a, b.grad, atol=1e-3)


@pytest.mark.parametrize("n_dst,n_src,h,f,n_bid,long_rows", [
    (4096, 2048, 8, 4, 1, False), (300, 500, 1, 4, 1, False), (1000, 700, 3, 16, 2, False),
    (513, 129, 16, 64, 5, False), (64, 64, 4, 256, 1, False), (2000, 900, 4, 8, 1, True),
    (400, 300, 2, 6, 1, False), (400, 300, 20, 4, 1, False)])
def test_hfused_forward_against_the_oracle_ops(dev, n_dst, n_src, h, f, n_bid, long_rows):
    """The one-launch form (and its two-op fallback for long rows, unvectorised widths or
    more than 16 heads) against the oracle's two functions, not against the ops it is
    built from (hfused_cuda.cu:5-45)."""
    hubs = dict(hub_rows=(3,), hub_degree=600) if long_rows else {}
    a_ptr, a_idx = random_csr(n_dst, n_src, 0.02, n_dst + 1, **hubs)
    blocks = [random_csr(n_dst, n_src, 0.03, 10 * n_dst + b, empty_rows=(b,), **hubs)
              for b in range(n_bid)]
    if n_bid == 1:
        b_ptr, b_idx, n_cols = blocks[0][0].numpy(), blocks[0][1].numpy(), n_src
    else:
        b_ptr, b_idx, n_cols = oracle.stitch_csr([(p_, i_, n_src) for p_, i_ in blocks])
    g = torch.Generator().manual_seed(h + f)
    vals = torch.randn(a_idx.numel(), h, generator=g)
    x = torch.randn(n_src, h, f, generator=g)
    q = torch.randn(n_bid, n_dst, h, generator=g)
    k = torch.randn(n_cols, h, generator=g)
    b_ptr_t, b_idx_t = torch.as_tensor(b_ptr), torch.as_tensor(b_idx)
    out, attn = graph_ext.hfused_forward(vals.to(dev), a_ptr.to(dev), a_idx.to(dev), x.to(dev),
                                         b_ptr_t.to(dev), b_idx_t.to(dev), q.to(dev), k.to(dev))
    want_out, want_attn = oracle.hfused_forward(vals, a_ptr, a_idx, x, b_ptr, b_idx, q.numpy(), k)
    abs_out = oracle.mh_spmm_forward(vals.abs(), a_ptr, a_idx, x.abs())
    assert_close(out, want_out, abs_sum=abs_out, what="spmm part")
    assert_close(attn, want_attn, what="sddmm part")


@pytest.mark.parametrize("n_dst,n_src,h,f,n_bid,long_rows", [
    (4096, 2048, 8, 4, 1, False), (300, 500, 1, 4, 1, False), (1000, 700, 3, 16, 2, False),
    (513, 129, 16, 64, 5, False), (64, 64, 4, 256, 1, False), (2000, 900, 4, 8, 1, True),
    (400, 300, 2, 6, 1, False), (400, 300, 20, 4, 1, False)])
def test_hfused_backward_against_the_oracle_ops(dev, n_dst, n_src, h, f, n_bid, long_rows):
    """The backward of both ops in two shared launches (per-row passes, then by-source
    gathers), and its fallback to the two ops, against the oracle's spmm / sddmm backward
    functions (spmm_cuda.cu:27-38, sddmm_cuda.cu:36-66); same bits on a second call."""
    hubs = dict(hub_rows=(3,), hub_degree=600) if long_rows else {}
    a_ptr, a_idx = random_csr(n_dst, n_src, 0.02, n_dst + 1, **hubs)
    blocks = [random_csr(n_dst, n_src, 0.03, 10 * n_dst + b, empty_rows=(b,), **hubs)
              for b in range(n_bid)]
    if n_bid == 1:
        b_ptr, b_idx, n_cols = blocks[0][0].numpy(), blocks[0][1].numpy(), n_src
    else:
        b_ptr, b_idx, n_cols = oracle.stitch_csr([(p_, i_, n_src) for p_, i_ in blocks])
    g = torch.Generator().manual_seed(h + f)
    vals = torch.randn(a_idx.numel(), h, generator=g)
    x = torch.randn(n_src, h, f, generator=g)
    gy = torch.randn(n_dst, h, f, generator=g)
    q = torch.randn(n_bid, n_dst, h, generator=g)
    k = torch.randn(n_cols, h, generator=g)
    b_ptr_t, b_idx_t = torch.as_tensor(b_ptr), torch.as_tensor(b_idx)
    attn = oracle.sddmm_forward(b_ptr, b_idx, q.numpy(), k.numpy())
    gattn = torch.randn(b_idx_t.numel(), h, generator=g)
    args = (vals.to(dev), a_ptr.to(dev), a_idx.to(dev), x.to(dev), gy.to(dev), b_ptr_t.to(dev),
            b_idx_t.to(dev), q.to(dev), k.to(dev), torch.as_tensor(attn).to(dev), gattn.to(dev))
    got = graph_ext.hfused_backward(*args)
    want_ga, want_gx = oracle.mh_spmm_backward(vals, a_ptr, a_idx, x.numpy(), gy.numpy())
    want_gq, want_gk = oracle.sddmm_backward(b_ptr, b_idx, q.numpy(), k.numpy(), attn, gattn.numpy())
    abs_ga = oracle.mh_spmm_backward(vals.abs(), a_ptr, a_idx, x.abs().numpy(), gy.abs().numpy())
    assert_close(got[0], want_ga, abs_sum=abs_ga[0], what="grad of the SpMM's edge values")
    assert_close(got[1], want_gx, abs_sum=abs_ga[1], what="grad of the SpMM's features")
    abs_gq, abs_gk = softmax_backward_abs_sums(b_ptr, b_idx, attn, gattn, n_cols)
    assert_close(got[2], want_gq, abs_sum=abs_gq, what="grad_query")
    assert_close(got[3], want_gk, abs_sum=abs_gk, what="grad_key")
    again = graph_ext.hfused_backward(*args)
    assert all(torch.equal(a, b) for a, b in zip(got, again))


def test_dtype_and_device_checks(dev):
    indptr, indices = random_csr(10, 10, 0.3, 0)
    v = torch.randn(indices.numel(), 2)
    x = torch.randn(10, 2, 4)
    with pytest.raises(RuntimeError):
        graph_ext.spmm_forward(v, indptr, indices, x)  # CPU tensors
    with pytest.raises(RuntimeError):
        graph_ext.spmm_forward(v.to(dev).double(), indptr.to(dev), indices.to(dev), x.to(dev))
    with pytest.raises(RuntimeError):
        graph_ext.sddmm_forward(indptr.to(dev), indices.to(dev), torch.randn(1, 9, 2, device=dev),
                                torch.randn(10, 2, device=dev))  # query rows != n_dst


@pytest.mark.parametrize("f", [16, 64])
def test_too_small_max_degree_hint_costs_speed_not_correctness(dev, monkeypatch, f):
    """The widest-row argument of the entry points is a hint: told (wrongly) that no row is
    long, the library builds no row plan and its row kernels walk the long rows themselves.
    Every op must still give the right answer."""
    from yitu_amd import _lib
    indptr, indices = powerlaw_graph(11, 40000, 77)
    n = indptr.numel() - 1
    assert int((indptr[1:] - indptr[:-1]).max()) > 500
    h = 4  # f = 64: rows of 256 floats, the fused forward's whole-wave layout
    g = torch.Generator().manual_seed(9)
    q, k = torch.randn(1, n, h, generator=g), torch.randn(n, h, generator=g)
    x, gy = torch.randn(n, h, f, generator=g), torch.randn(n, h, f, generator=g)
    ga = torch.randn(indices.numel(), h, generator=g)
    d = lambda t: t.to(dev)
    ip, ix = d(indptr), d(indices)

    def run():
        attn = graph_ext.sddmm_forward(ip, ix, d(q), d(k))
        gq, gk = graph_ext.sddmm_backward(ip, ix, d(q), d(k), attn, d(ga))
        out = graph_ext.spmm_forward(attn, ip, ix, d(x))
        gav, gx = graph_ext.spmm_backward(attn, ip, ix, d(x), d(gy))
        fo, fattn = graph_ext.gat_forward(ip, ix, d(q[0]), d(k), d(x))
        fb = graph_ext.gat_backward(ip, ix, d(q[0]), d(k), d(x), fattn, d(gy), out=fo)
        return [attn, gq, gk, out, gav, gx, fo] + list(fb)

    want = run()
    graph_ext.transposed(ip, ix, n)  # built with the true degrees; only the hints lie below
    monkeypatch.setattr(_lib, "max_degree", lambda t: 1)
    monkeypatch.setattr(_lib, "row_plan", lambda *a: None)
    tr = graph_ext.transposed(ip, ix, n)
    monkeypatch.setattr(tr, "max_degree_t", 1)
    monkeypatch.setattr(tr, "plan_t", None)
    got = run()
    for i, (a, b) in enumerate(zip(got, want)):
        assert_close(a, b, rtol=1e-4, atol=5e-4, what="result %d" % i)


def test_operands_that_are_not_vector_aligned(dev):
    """query / key / attn that start 4 bytes off a 16-byte boundary (views into a larger
    buffer): the one-lane-per-edge kernels read them as 16-byte vectors and must step aside
    for the scalar kernels; same results as with aligned operands."""
    indptr, indices = powerlaw_graph(10, 20000, 5)
    n, h, f = indptr.numel() - 1, 4, 64
    g = torch.Generator().manual_seed(4)
    q, k = torch.randn(n, h, generator=g).to(dev), torch.randn(n, h, generator=g).to(dev)
    x = torch.randn(n, h, f, generator=g).to(dev)
    ga = torch.randn(indices.numel(), h, generator=g).to(dev)
    ip, ix = indptr.to(dev), indices.to(dev)

    def shifted(t):
        buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=dev)
        v = buf[1:].view(t.shape)
        v.copy_(t)
        assert v.data_ptr() % 16 == 4 and v.is_contiguous()
        return v

    attn = graph_ext.sddmm_forward(ip, ix, q[None], k)
    gq, gk = graph_ext.sddmm_backward(ip, ix, q[None], k, attn, ga)
    out, _ = graph_ext.gat_forward(ip, ix, q, k, x)
    qs, ks = shifted(q), shifted(k)
    attn_s = graph_ext.sddmm_forward(ip, ix, qs[None], ks)
    gq_s, gk_s = graph_ext.sddmm_backward(ip, ix, qs[None], ks, shifted(attn), shifted(ga))
    out_s, _ = graph_ext.gat_forward(ip, ix, qs, ks, x)
    assert_close(attn_s, attn, rtol=1e-5, atol=1e-6, what="attn")
    assert_close(gq_s, gq, rtol=1e-4, atol=1e-5, what="grad_q")
    assert_close(gk_s, gk, rtol=1e-4, atol=2e-4, what="grad_k")
    assert_close(out_s, out, rtol=1e-5, atol=1e-4, what="out")


def test_max_degree_cache_does_not_outlive_its_tensor(dev):
    """Two graphs of the same size allocated one after the other land on the same device
    address; the widest-row cache must not hand the first one's answer to the second."""
    from yitu_amd import _lib
    a = torch.tensor([0, 1, 2, 3], dtype=torch.int32, device=dev)
    assert _lib.max_degree(a) == 1
    addr = a.data_ptr()
    del a
    b = torch.tensor([0, 0, 0, 300], dtype=torch.int32, device=dev)
    if b.data_ptr() == addr:  # the allocator reused the block (the case that matters)
        assert _lib.max_degree(b) == 300
    assert _lib.max_degree(b) == 300


# ---- degenerate graphs --------------------------------------------------------------

@pytest.mark.parametrize("n_dst,n_src", [(50, 40), (0, 40), (50, 0), (0, 0)])
def test_graph_without_edges(dev, n_dst, n_src):
    """No edges, and no rows on either side: every op returns zeros of the right
    shape (empty tensors have no address, so the library must not insist on one)."""
    h, f = 4, 16
    indptr = torch.zeros(n_dst + 1, dtype=torch.int32, device=dev)
    indices = torch.zeros(0, dtype=torch.int32, device=dev)
    g = torch.Generator().manual_seed(n_dst + n_src)
    x = torch.randn(n_src, h, f, generator=g).to(dev)
    q = torch.randn(n_dst, h, generator=g).to(dev)
    k = torch.randn(n_src, h, generator=g).to(dev)
    gy = torch.randn(n_dst, h, f, generator=g).to(dev)
    none = torch.zeros(0, h, device=dev)

    def zeros(t, *shape):
        return tuple(t.shape) == shape and not bool(t.any())

    assert zeros(graph_ext.spmm_forward(none, indptr, indices, x), n_dst, h, f)
    ga, gx = graph_ext.spmm_backward(none, indptr, indices, x, gy)
    assert zeros(ga, 0, h) and zeros(gx, n_src, h, f)
    assert zeros(graph_ext.sddmm_forward(indptr, indices, q[None], k), 0, h)
    gq, gk = graph_ext.sddmm_backward(indptr, indices, q[None], k, none, none)
    assert zeros(gq, 1, n_dst, h) and zeros(gk, n_src, h)
    out, attn = graph_ext.gat_forward(indptr, indices, q, k, x)
    assert zeros(out, n_dst, h, f) and zeros(attn, 0, h)
    gq, gk, gx = graph_ext.gat_backward(indptr, indices, q, k, x, attn, gy)
    assert zeros(gq, n_dst, h) and zeros(gk, n_src, h) and zeros(gx, n_src, h, f)
    # and through autograd
    blk = xblock.Block([n_dst, n_src], [indptr, indices])
    leaves = [t.clone().requires_grad_() for t in (q, k, x)]
    sparse.fused_gat(blk, *leaves).sum().backward()
    assert all(zeros(t.grad, *t.shape) for t in leaves)


@pytest.mark.parametrize("h,f", [(8, 32), (4, 64), (2, 128), (1, 256), (8, 64), (2, 256),
                                 (16, 64), (4, 256)])
def test_spmm_backward_one_gather_shapes(dev, h, f):
    """Rows of 256, 512 or 1024 floats: both gradients come from one pass over the by-source
    structure; against the oracle, with hub rows on both sides, and equal to the
    two-pass form (asked for one gradient at a time)."""
    indptr, indices = powerlaw_graph(12, 70000, 31 * h + f)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(h + f)
    values = torch.randn(indices.numel(), h, generator=g)
    x = torch.randn(n, h, f, generator=g)
    gy = torch.randn(n, h, f, generator=g)
    d = lambda t: t.to(dev)
    ga, gx = graph_ext.spmm_backward(d(values), d(indptr), d(indices), d(x), d(gy))
    want_ga, want_gx = oracle.mh_spmm_backward(values, indptr, indices, x, gy)
    _, abs_ga, abs_gx = spmm_abs_sums(values, indptr, indices, x, gy)
    assert_close(ga, want_ga, abs_sum=abs_ga)
    assert_close(gx, want_gx, abs_sum=abs_gx)
    ga2, _ = graph_ext.spmm_backward(d(values), d(indptr), d(indices), d(x), d(gy),
                                     need_grad_x=False)
    _, gx2 = graph_ext.spmm_backward(d(values), d(indptr), d(indices), d(x), d(gy),
                                     need_grad_a=False)
    assert_close(ga, ga2, abs_sum=abs_ga)
    assert_close(gx, gx2, abs_sum=abs_gx)
    again = graph_ext.spmm_backward(d(values), d(indptr), d(indices), d(x), d(gy))
    assert torch.equal(again[0], ga) and torch.equal(again[1], gx)


def test_spmm_backward_constant_weights_take_the_by_source_copy(dev):
    """grad_x alone with the same weight tensor passed again: from the second call on the
    weights are read from a copy in by-source order; same result, and an in-place change
    of the weights is noticed."""
    indptr, indices = powerlaw_graph(12, 50000, 17)
    n = indptr.numel() - 1
    g = torch.Generator().manual_seed(3)
    values = torch.rand(indices.numel(), 2, generator=g).to(dev)
    x = torch.randn(n, 2, 24, generator=g)
    gy = torch.randn(n, 2, 24, generator=g)
    ip, ix, xd, gyd = indptr.to(dev), indices.to(dev), x.to(dev), gy.to(dev)
    want = oracle.mh_spmm_backward(values.cpu(), indptr, indices, x, gy)[1]
    abs_gx = spmm_abs_sums(values.cpu(), indptr, indices, x, gy)[2]
    for _ in range(3):  # first call: through the permutation; then: the kept copy
        got = graph_ext.spmm_backward(values, ip, ix, xd, gyd, need_grad_a=False)[1]
        assert_close(got, want, abs_sum=abs_gx)
    values.mul_(2.0)
    for _ in range(3):
        got = graph_ext.spmm_backward(values, ip, ix, xd, gyd, need_grad_a=False)[1]
        assert_close(got, 2 * torch.as_tensor(want), abs_sum=2 * abs_gx)
