"""Pins the CPU oracle's graph_ext functions (multi-head SpMM, SDDMM + LeakyReLU
+ edge softmax, stitch_csr, b2gemm) against dense torch formulations with
autograd -- the method of the reference's own test_kernel.py -- and brute force."""
import numpy as np
import pytest
import torch
from torch import nn

import oracle
from helpers import assert_close, random_csr
from yitu_amd.xgnn_h import block as xblock
from yitu_amd.xgnn_h import convert


def _dense_mask(indptr, indices, n_dst, n_src):
    return convert.to_dense(n_dst, n_src, [indptr, indices], torch.ones(indices.numel()))


@pytest.mark.parametrize("n_dst,n_src,h,f,seed", [(1, 1, 1, 1, 0), (40, 55, 3, 7, 1), (130, 90, 8, 16, 2)])
def test_mh_spmm_forward_backward_equal_dense_bmm(n_dst, n_src, h, f, seed):
    """check_gspmm (test_kernel.py:25-94): y = bmm(dense_attn, x)."""
    indptr, indices = random_csr(n_dst, n_src, 0.15, seed, empty_rows=(0,) if n_dst > 1 else ())
    if indices.numel() == 0:
        indptr, indices = torch.tensor([0, 1], dtype=torch.int32), torch.tensor([0], dtype=torch.int32)
    g = torch.Generator().manual_seed(seed)
    values = torch.randn(indices.numel(), h, generator=g, dtype=torch.float64, requires_grad=True)
    x = torch.randn(n_src, h, f, generator=g, dtype=torch.float64, requires_grad=True)
    deg = (indptr[1:] - indptr[:-1]).long()
    rows = torch.repeat_interleave(torch.arange(n_dst), deg)
    dense = torch.zeros(h, n_dst, n_src, dtype=torch.float64)
    dense = dense.index_put((torch.arange(h)[:, None], rows[None, :], indices.long()[None, :]),
                            values.t())
    y = torch.bmm(dense, x.transpose(0, 1)).transpose(0, 1)
    gy = torch.randn(n_dst, h, f, generator=g, dtype=torch.float64)
    y.backward(gy)
    for f64 in (True, False):
        got = oracle.mh_spmm_forward(values.detach().numpy(), indptr, indices, x.detach().numpy(), f64)
        assert_close(got, y.detach().float())
    ga, gx = oracle.mh_spmm_backward(values.detach().numpy(), indptr, indices, x.detach().numpy(),
                                     gy.numpy())
    assert_close(ga, values.grad.float())
    assert_close(gx, x.grad.float())


def _dense_gat(q, k, mask):
    """test_kernel.py:133-151: LeakyReLU(0.2), -1e38 mask, softmax over sources, re-mask."""
    e = nn.functional.leaky_relu(q[:, None, :] + k[None, :, :], 0.2)  # [n_dst, n_src, H]
    e = torch.where(mask[:, :, None] > 0, e, torch.full_like(e, -1e38))
    a = torch.softmax(e.permute(2, 0, 1), dim=-1)  # [H, n_dst, n_src]
    return a * mask[None]


@pytest.mark.parametrize("n_dst,n_src,h,seed", [(30, 40, 1, 0), (64, 50, 4, 1), (90, 120, 16, 2)])
def test_sddmm_forward_backward_equal_dense_softmax(n_dst, n_src, h, seed):
    indptr, indices = random_csr(n_dst, n_src, 0.12, seed, empty_rows=(3,))
    mask = _dense_mask(indptr, indices, n_dst, n_src).double()
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n_dst, h, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(n_src, h, generator=g, dtype=torch.float64, requires_grad=True)
    a = _dense_gat(q, k, mask)
    deg = (indptr[1:] - indptr[:-1]).long()
    rows = torch.repeat_interleave(torch.arange(n_dst), deg)
    attn_edges = a[:, rows, indices.long()].t()  # [E, H]
    ge = torch.randn(indices.numel(), h, generator=g, dtype=torch.float64)
    attn_edges.backward(ge)
    got = oracle.sddmm_forward(indptr, indices, q.detach().numpy()[None], k.detach().numpy())
    assert_close(got, attn_edges.detach().float())
    # softmax rows sum to one wherever the row has edges
    sums = np.zeros((n_dst, h))
    np.add.at(sums, rows.numpy(), got)
    assert np.allclose(sums[deg.numpy() > 0], 1.0, atol=1e-5)
    gq, gk = oracle.sddmm_backward(indptr, indices, q.detach().numpy()[None], k.detach().numpy(),
                                   got, ge.numpy())
    assert_close(gq[0], q.grad.float())
    assert_close(gk, k.grad.float())


def _stitch_bruteforce(blocks):
    """The literal loops of block.py:46-55."""
    n_rows = len(blocks[0][0]) - 1
    new_indptr, new_indices = [], []
    for row in range(n_rows):
        cursor = 0
        new_indptr.append(len(new_indices))
        for bid, (indptr, indices, n_src) in enumerate(blocks):
            for i in range(indptr[row], indptr[row + 1]):
                new_indices.append((bid << 24) + cursor + indices[i])
            cursor += n_src
    new_indptr.append(len(new_indices))
    return new_indptr, new_indices


@pytest.mark.parametrize("n_blk,seed", [(2, 0), (5, 1), (16, 2)])
def test_stitch_csr_bit_exact(n_blk, seed):
    rng = np.random.default_rng(seed)
    n_dst = 23
    blocks = []
    for b in range(n_blk):
        n_src = int(rng.integers(1, 60))
        ip, ix = random_csr(n_dst, n_src, 0.1, seed * 100 + b, empty_rows=(b % n_dst,))
        blocks.append((ip, ix, n_src))
    want_ptr, want_idx = _stitch_bruteforce([(a.tolist(), b.tolist(), c) for a, b, c in blocks])
    got_ptr, got_idx, n_cols = oracle.stitch_csr(blocks)
    assert got_ptr.tolist() == want_ptr and got_idx.tolist() == want_idx
    assert n_cols == sum(b[2] for b in blocks)
    # the package's vectorised host implementation gives the same integers
    blk = xblock.stitch_csr([xblock.Block([n_dst, c], [a, b]) for a, b, c in blocks])
    assert blk.adj_sparse[0].dtype == torch.int32 and blk.adj_sparse[1].dtype == torch.int32
    assert blk.adj_sparse[0].tolist() == want_ptr and blk.adj_sparse[1].tolist() == want_idx
    assert blk.size == [n_dst, n_cols]


def test_stitch_rejects_more_than_16_blocks():
    ip, ix = random_csr(4, 4, 0.5, 0)
    with pytest.raises(AssertionError):
        oracle.stitch_csr([(ip, ix, 4)] * 17)
    with pytest.raises(AssertionError):
        xblock.stitch_csr([xblock.Block([4, 4], [ip, ix])] * 17)


def test_stitched_sddmm_spmm_equals_sum_over_relations():
    """check_stitch (test_kernel.py:236-359): softmax is per (row, block), so the
    stitched op equals the per-relation ops summed."""
    rng = np.random.default_rng(7)
    n_dst, h, f = 31, 3, 5
    blocks, srcs, dsts = [], [], []
    for b in range(4):
        n_src = int(rng.integers(5, 40))
        ip, ix = random_csr(n_dst, n_src, 0.15, 70 + b)
        blocks.append((ip, ix, n_src))
        srcs.append(rng.standard_normal((n_src, h, f)).astype(np.float32))
        dsts.append(rng.standard_normal((n_dst, h)).astype(np.float32))
    keys = [rng.standard_normal((b[2], h)).astype(np.float32) for b in blocks]
    want = np.zeros((n_dst, h, f), np.float32)
    for (ip, ix, _), x, q, k in zip(blocks, srcs, dsts, keys):
        a = oracle.sddmm_forward(ip, ix, q[None], k)
        want += oracle.mh_spmm_forward(a, ip, ix, x)
    sp, si, _ = oracle.stitch_csr(blocks)
    a = oracle.sddmm_forward(sp, si, np.stack(dsts), np.concatenate(keys))
    got = oracle.mh_spmm_forward(a, sp, si, np.concatenate(srcs))
    assert_close(got, want)


@pytest.mark.parametrize("n_bid,h,seed", [(2, 3, 0), (5, 1, 1), (16, 4, 2)])
def test_sddmm_multi_bid_forward_backward_equal_dense_per_block_softmax(n_bid, h, seed):
    """A stitched block tags every edge with a query block id (sddmm_cuda.cu:11-31,
    block.py:46-55); the softmax runs per (row, block id) (sddmm_cuda.cu:15-31) and the
    backward per the same groups (sddmm_cuda.cu:43-66). Independent statement: one dense
    masked softmax per block over that block's own columns, joined by autograd."""
    rng = np.random.default_rng(100 + seed)
    n_dst = 27
    blocks = []
    for b in range(n_bid):
        n_src = int(rng.integers(3, 30))
        ip, ix = random_csr(n_dst, n_src, 0.2, 1000 * seed + b, empty_rows=((b * 5) % n_dst,))
        blocks.append((ip, ix, n_src))
    sp, si, n_cols = oracle.stitch_csr(blocks)
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(n_bid, n_dst, h, generator=g, dtype=torch.float64, requires_grad=True)
    k = torch.randn(n_cols, h, generator=g, dtype=torch.float64, requires_grad=True)
    # dense attention of block b lives in columns [off_b, off_b + n_src_b) of a [H, n_dst, n_cols] tensor
    dense = torch.zeros(h, n_dst, n_cols, dtype=torch.float64)
    off = 0
    for b, (ip, ix, n_src) in enumerate(blocks):
        mask = _dense_mask(ip, ix, n_dst, n_src).double()
        dense = dense + nn.functional.pad(_dense_gat(q[b], k[off:off + n_src], mask),
                                          (off, n_cols - off - n_src))
        off += n_src
    deg = np.diff(sp).astype(np.int64)
    rows = torch.from_numpy(np.repeat(np.arange(n_dst), deg))
    cols = torch.from_numpy((si & 0xFFFFFF).astype(np.int64))
    attn_edges = dense[:, rows, cols].t()  # [E, H] in stitched CSR order
    ge = torch.randn(si.shape[0], h, generator=g, dtype=torch.float64)
    attn_edges.backward(ge)
    got = oracle.sddmm_forward(sp, si, q.detach().numpy(), k.detach().numpy())
    assert_close(got, attn_edges.detach().float())
    gq, gk = oracle.sddmm_backward(sp, si, q.detach().numpy(), k.detach().numpy(), got, ge.numpy())
    assert_close(gq, q.grad.float())
    assert_close(gk, k.grad.float())


def test_b2gemm_equals_two_linears():
    """check_bundle (test_kernel.py:187-233)."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(70, 24, generator=g, dtype=torch.float64, requires_grad=True)
    fc1 = nn.Linear(24, 9, bias=False).double()
    fc2 = nn.Linear(24, 9, bias=False).double()
    y1, y2 = fc1(x), fc2(x)
    g1 = torch.randn(70, 9, generator=g, dtype=torch.float64)
    g2 = torch.randn(70, 9, generator=g, dtype=torch.float64)
    (y1 * g1 + y2 * g2).sum().backward()
    ya, yb = oracle.b2gemm(x.detach().numpy(), fc1.weight.detach().numpy(), fc2.weight.detach().numpy())
    assert_close(ya, y1.detach().float())
    assert_close(yb, y2.detach().float())
    dx, dwa, dwb = oracle.b2gemm_backward(x.detach().numpy(), fc1.weight.detach().numpy(),
                                          fc2.weight.detach().numpy(), g1.numpy(), g2.numpy())
    assert_close(dx, x.grad.float())
    assert_close(dwa, fc1.weight.grad.float())
    assert_close(dwb, fc2.weight.grad.float())


def test_stack_blocks_places_every_block_in_the_union_matrix():
    """stack_blocks against a dense construction: block b lands at (row_offsets[b],
    col_offsets[b]) with its row scales as edge weights; inside a row the edges keep
    block order, then the block's own order."""
    rng = np.random.default_rng(5)
    shapes = [(7, 9), (7, 4), (5, 9), (3, 6)]       # (n_dst, n_src) per block
    row_off, col_off = [0, 0, 7, 12], [0, 9, 4, 13]  # overlapping row ranges (0 and 1), shared columns
    n_rows, n_cols = 15, 19
    blocks, scales, dense = [], [], np.zeros((n_rows, n_cols))
    for b, (nd, ns) in enumerate(shapes):
        ip, ix = random_csr(nd, ns, 0.4, 50 + b, empty_rows=(b,))
        sc = torch.tensor(rng.uniform(0.5, 2.0, nd), dtype=torch.float32)
        blocks.append(xblock.Block([nd, ns], [ip, ix]))
        scales.append(sc)
        for r in range(nd):
            for i in range(int(ip[r]), int(ip[r + 1])):
                dense[row_off[b] + r, col_off[b] + int(ix[i])] += float(sc[r])
    blk, values = xblock.stack_blocks(blocks, row_off, col_off, n_rows, n_cols, scales)
    indptr, indices = blk.adj_sparse
    assert indptr.dtype == torch.int32 and indices.dtype == torch.int32
    assert blk.size == [n_rows, n_cols] and values.shape == (indices.numel(), 1)
    assert indices.numel() == sum(b.adj_sparse[1].numel() for b in blocks)
    got = np.zeros((n_rows, n_cols))
    for r in range(n_rows):
        for i in range(int(indptr[r]), int(indptr[r + 1])):
            got[r, int(indices[i])] += float(values[i, 0])
    assert np.allclose(got, dense, atol=1e-6)
    # row 2 of the union: block 0's edges first, then block 1's, each in its own order
    want = [int(c) for c in blocks[0].adj_sparse[1][blocks[0].adj_sparse[0][2]:blocks[0].adj_sparse[0][3]]]
    want += [9 + int(c) for c in blocks[1].adj_sparse[1][blocks[1].adj_sparse[0][2]:blocks[1].adj_sparse[0][3]]]
    assert indices[indptr[2]:indptr[3]].tolist() == want
    # no scales: unit weights
    _, ones = xblock.stack_blocks(blocks, row_off, col_off, n_rows, n_cols)
    assert torch.equal(ones, torch.ones_like(values))


@pytest.mark.parametrize("n_dst,n_src,h,f,n_bid,seed", [(60, 45, 4, 8, 1, 0), (33, 70, 2, 5, 3, 1),
                                                        (90, 90, 1, 16, 16, 2)])
def test_all_core_float_builds_equal_the_serial_gradients(n_dst, n_src, h, f, n_bid, seed):
    """The *_omp functions exist to be timed on all cores; they are the same sums as the
    serial double-accumulate gradients they stand beside (by-source instead of scattered),
    and the by-source view they walk is the stable sort on the column."""
    indptr, indices = random_csr(n_dst, n_src, 0.15, seed, hub_rows=(3,), hub_degree=min(n_src, 40),
                                 empty_rows=(0,))
    rng = np.random.default_rng(seed)
    ip, ix = indptr.numpy(), indices.numpy().copy()
    ix |= (rng.integers(0, n_bid, ix.shape[0]).astype(np.int32) << 24)
    # a stitched row lists its blocks in ascending tag order
    for r in range(n_dst):
        seg = ix[ip[r]:ip[r + 1]]
        seg.sort()
    t_indptr, t_rows, t_perm = tr = oracle.csr_transpose(ip, ix, n_src)
    col = ix & 0xffffff
    rows = np.repeat(np.arange(n_dst), np.diff(ip))
    order = np.argsort(col, kind="stable")
    assert np.array_equal(t_perm, order) and np.array_equal(t_rows, rows[order])
    assert np.array_equal(np.diff(t_indptr), np.bincount(col, minlength=n_src))
    values = rng.standard_normal((ix.shape[0], h)).astype(np.float32)
    feat = rng.standard_normal((n_src, h, f)).astype(np.float32)
    gy = rng.standard_normal((n_dst, h, f)).astype(np.float32)
    ga, gx = oracle.mh_spmm_backward(values, ip, ix, feat, gy)
    ga2, gx2 = oracle.mh_spmm_backward_omp(values, ip, ix, feat, gy, tr)
    assert_close(ga2, ga)
    assert_close(gx2, gx)
    none_a, gx3 = oracle.mh_spmm_backward_omp(values, ip, ix, feat, gy, tr, need_grad_a=False)
    assert none_a is None and np.array_equal(gx3, gx2)
    q = rng.standard_normal((n_bid, n_dst, h)).astype(np.float32)
    k = rng.standard_normal((n_src, h)).astype(np.float32)
    attn = oracle.sddmm_forward(ip, ix, q, k)
    g_attn = rng.standard_normal(attn.shape).astype(np.float32)
    gq, gk = oracle.sddmm_backward(ip, ix, q, k, attn, g_attn)
    gq2, gk2 = oracle.sddmm_backward_omp(ip, ix, q, k, attn, g_attn, tr)
    # rows without an edge of a block keep grad_query 0 in both
    assert_close(gq2, gq)
    assert_close(gk2, gk)


@pytest.mark.parametrize("n,m,k", [(37, 20, 13), (8, 64, 64), (1, 5, 9)])
def test_all_core_float_gemm_equals_numpy(n, m, k):
    rng = np.random.default_rng(n + m + k)
    for ta in (False, True):
        for tb in (False, True):
            a = rng.standard_normal((k, n) if ta else (n, k)).astype(np.float32)
            b = rng.standard_normal((m, k) if tb else (k, m)).astype(np.float32)
            want = (a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64)
            assert_close(oracle.gemm_omp(a, b, ta, tb), want)
