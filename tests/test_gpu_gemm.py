"""GPU parity of the MFMA fp32 GEMM entry points (yitu_sgemm, yitu_b2gemm,
yitu_b2gemm_backward) against double-precision products."""
import numpy as np
import pytest
import torch
from torch import nn

import oracle
from helpers import assert_close
from yitu_amd import graph_ext
from yitu_amd.xgnn_h import bundle

pytestmark = pytest.mark.gpu


def _ref(a, b, ta, tb):
    a64, b64 = a.double(), b.double()
    return ((a64.t() if ta else a64) @ (b64.t() if tb else b64)).float()


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (7, 5, 3), (128, 128, 16), (130, 257, 33),
                                   (256, 128, 256), (1000, 40, 100), (64, 300, 1)])
def test_sgemm_all_layouts(dev, ta, tb, m, n, k):
    g = torch.Generator().manual_seed(m * 7 + n * 3 + k)
    a = torch.randn((k, m) if ta else (m, k), generator=g)
    b = torch.randn((n, k) if tb else (k, n), generator=g)
    got = graph_ext.sgemm(a.to(dev), b.to(dev), ta, tb)
    assert_close(got, _ref(a, b, ta, tb), atol=1e-4 * max(1.0, np.sqrt(k) / 4),
                 what="m=%d n=%d k=%d ta=%s tb=%s" % (m, n, k, ta, tb))


def test_sgemm_split_k_long_inner_dimension(dev):
    """dW = X^T G with K = number of nodes: few tiles, split along K, fixed-order reduce."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(70001, 96, generator=g)
    gy = torch.randn(70001, 130, generator=g)
    got = graph_ext.sgemm(x.to(dev), gy.to(dev), True, False)
    assert_close(got, _ref(x, gy, True, False), atol=1e-4 * np.sqrt(70001))
    again = graph_ext.sgemm(x.to(dev), gy.to(dev), True, False)
    assert torch.equal(got, again)


@pytest.mark.parametrize("ki,no", [(256, 256), (64, 256), (256, 64), (128, 256), (256, 128),
                                   (128, 128), (128, 64), (64, 128), (64, 64)])
@pytest.mark.parametrize("ks", [[70001], [49152], [30000, 10, 20001, 300], [7000] * 10])
def test_sgemm_weight_gradient_many_rows(dev, ks, ki, no):
    """dW = X^T G for operands of 64 / 128 / 256 columns and tens of thousands of rows: every
    chunk of rows keeps the whole product in registers (64 x 64 takes the tiled kernel); several node types in one launch
    (one with fewer rows than a stage, more than 8), a fixed order of additions, and the
    accumulating form."""
    g = torch.Generator().manual_seed(sum(ks))
    xs = [torch.randn(k, ki, generator=g) for k in ks]
    gs = [torch.randn(k, no, generator=g) for k in ks]
    dx, dg = [x.to(dev) for x in xs], [x.to(dev) for x in gs]
    run = lambda: graph_ext.sgemm_typed(dx, dg, True, False) if len(ks) > 1 \
        else [graph_ext.sgemm(dx[0], dg[0], True, False)]
    got = run()
    for x, y, c, k in zip(xs, gs, got, ks):
        assert_close(c, _ref(x, y, True, False), atol=1e-4 * np.sqrt(k), what="k=%d" % k)
    assert all(torch.equal(c, d) for c, d in zip(got, run()))


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("m,n,k", [(70001, 256, 256), (50000, 250, 128), (60000, 448, 64),
                                   (5000, 256, 256), (300, 40, 24), (1, 7, 3)])
def test_linear_forward_with_bias(dev, with_bias, m, n, k):
    """y = x w^T + bias: the bias is added inside the many-rows kernel (whole and ragged
    tiles and column blocks) or by a pass of its own after the tiled kernel."""
    g = torch.Generator().manual_seed(m + n + k)
    x, w = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g)
    b = torch.randn(n, generator=g) if with_bias else None
    got = graph_ext.linear_forward(x.to(dev), w.to(dev), None if b is None else b.to(dev))
    want = x.double() @ w.double().t()
    if b is not None:
        want = want + b.double()
    assert_close(got, want.float(), atol=1e-4 * max(1.0, np.sqrt(k) / 4))


@pytest.mark.parametrize("ms,n,k", [([30000, 0, 20001, 300], 256, 256), ([7000] * 10, 192, 128),
                                    ([900, 1, 77], 96, 40), ([40000, 30000], 250, 64)])
def test_linear_forward_typed(dev, ms, n, k):
    """Per-type Linear layers written as row slices of one buffer, some with and some without
    a bias: on the many-rows kernel (bias inside), on the tiled kernel (bias pass after it),
    with an empty type, with more than eight types, and against the layer-at-a-time call."""
    g = torch.Generator().manual_seed(sum(ms) + n + k)
    xs = [torch.randn(m, k, generator=g) for m in ms]
    ws = [torch.randn(n, k, generator=g) for _ in ms]
    bs = [torch.randn(n, generator=g) if i % 3 != 1 else None for i in range(len(ms))]
    y = torch.full((sum(ms), n), float("nan"), device=dev)
    parts, off = [], 0
    for m in ms:
        parts.append(y[off:off + m])
        off += m
    to = lambda t: None if t is None else t.to(dev)
    got = graph_ext.linear_forward_typed([to(x) for x in xs], [to(w) for w in ws],
                                         [to(b) for b in bs], out_list=parts)
    for x, w, b, c, part in zip(xs, ws, bs, got, parts):
        assert c.data_ptr() == part.data_ptr()
        want = x.double() @ w.double().t()
        if b is not None:
            want = want + b.double()
        assert_close(c, want.float(), atol=1e-4 * max(1.0, np.sqrt(k) / 4))
        if x.size(0):
            single = graph_ext.linear_forward(to(x), to(w), to(b))
            assert_close(c, single.cpu())


def test_sgemm_typed_gemm_shape(dev):
    """[n_t, 256] x [256, 256] of the heterogeneous configuration (fast path)."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1 << 15, 256, generator=g)
    w = torch.randn(256, 256, generator=g) * 0.02
    assert_close(graph_ext.sgemm(x.to(dev), w.to(dev)), _ref(x, w, False, False))


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("ms,n,k", [([50000], 256, 256), ([60000], 448, 64), ([70001], 256, 128),
                                    ([49157], 250, 128), ([20000], 520, 256), ([5000], 300, 64),
                                    ([30000, 0, 20001, 300], 256, 256), ([7000] * 10, 192, 128)])
def test_sgemm_many_rows_short_inner_dimension(dev, tb, ms, n, k):
    """Inner dimensions of 64 / 128 / 256 with tens of thousands of rows run with the weight
    held in registers and whole-row tiles: ragged last tiles, column counts that are not
    multiples of 4 / 32 / 256, several column blocks, several node types in one launch
    (an empty one among them, more than 8), both weight layouts; two shapes just outside
    (few rows, a narrow last column block) take the tiled kernel."""
    g = torch.Generator().manual_seed(sum(ms) + 3 * n + 5 * k + tb)
    a = [torch.randn(m, k, generator=g) for m in ms]
    b = [torch.randn((n, k) if tb else (k, n), generator=g) for _ in ms]
    da, db = [x.to(dev) for x in a], [w.to(dev) for w in b]
    got = graph_ext.sgemm_typed(da, db, False, tb) if len(ms) > 1 \
        else [graph_ext.sgemm(da[0], db[0], False, tb)]
    for x, w, c, m in zip(a, b, got, ms):
        assert tuple(c.shape) == (m, n)
        assert_close(c, _ref(x, w, False, tb), atol=1e-4 * max(1.0, np.sqrt(k) / 4),
                     what="m=%d n=%d k=%d tb=%s" % (m, n, k, tb))
    again = graph_ext.sgemm_typed(da, db, False, tb) if len(ms) > 1 \
        else [graph_ext.sgemm(da[0], db[0], False, tb)]
    assert all(torch.equal(c, d) for c, d in zip(got, again))


@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False)])
@pytest.mark.parametrize("sizes", [[(300, 64), (1, 64), (0, 64), (129, 64)],
                                   [(1024, 256), (512, 256), (256, 256)],
                                   [(50, 8)] * 11,                  # more than one group of 8
                                   [(40, 70001), (33, 5000), (64, 0)]])  # long, uneven, empty K
def test_sgemm_typed_equals_one_product_at_a_time(dev, ta, tb, sizes):
    """Problems of different height (and inner length) in one launch: each result is
    bit for bit what the single-problem entry point gives when the inner dimension is
    too short for a K split, and within the bar of a float64 product always."""
    n = 96
    g = torch.Generator().manual_seed(len(sizes) * 5 + ta * 2 + tb)
    if ta:  # the gradient form: a_i [k_i, m], b_i [k_i, n] with m shared
        sizes = [(64, k) for _, k in sizes]
    a_list = [torch.randn((k, m) if ta else (m, k), generator=g).to(dev) for m, k in sizes]
    b_list = [torch.randn((n, k) if tb else (k, n), generator=g).to(dev) for _, k in sizes]
    # (where the row strides differ between the problems the wrapper takes them one at a time)
    got = graph_ext.sgemm_typed(a_list, b_list, ta, tb)
    for (m, k), a, b, c in zip(sizes, a_list, b_list, got):
        assert tuple(c.shape) == (m, n)
        assert_close(c, _ref(a.cpu(), b.cpu(), ta, tb), atol=1e-4 * max(1.0, np.sqrt(k) / 4),
                     what="m=%d k=%d" % (m, k))
        if k < 256:  # no K split either way: the same sums in the same order
            assert torch.equal(c, graph_ext.sgemm(a, b, ta, tb))
    again = graph_ext.sgemm_typed(a_list, b_list, ta, tb)
    assert all(torch.equal(x, y) for x, y in zip(got, again))


def test_sgemm_typed_writes_row_slices_of_one_buffer(dev):
    g = torch.Generator().manual_seed(4)
    heights = [384, 128, 257, 5]
    xs = [torch.randn(m, 256, generator=g).to(dev) for m in heights]
    ws = [(torch.randn(256, 256, generator=g) * 0.02).to(dev) for _ in heights]
    buf = torch.full((sum(heights) + 3, 256), 7.0, device=dev)
    parts, off = [], 0
    for m in heights:
        parts.append(buf[off:off + m])
        off += m
    graph_ext.sgemm_typed(xs, ws, out_list=parts)
    for x, w, part in zip(xs, ws, parts):
        assert_close(part, _ref(x.cpu(), w.cpu(), False, False))
    assert torch.all(buf[off:] == 7.0)


@pytest.mark.parametrize("seed", range(6))
def test_check_bundle(dev, seed):
    """test_kernel.py:187-233 with seeded shapes: b2gemm vs two bias-free Linear layers,
    outputs and all three gradients, through GEMMBundleFunction."""
    rng = np.random.default_rng(seed)
    n, k, m = int(rng.integers(8, 1025)), int(rng.integers(8, 257)), int(rng.integers(1, 33))
    torch.manual_seed(seed)
    x = torch.randn(n, k, device=dev, requires_grad=True)
    fc1 = nn.Linear(k, m, bias=False).to(dev)
    fc2 = nn.Linear(k, m, bias=False).to(dev)
    y1, y2 = fc1(x), fc2(x)
    torch.sum(y1 + y2).backward()
    gx1, g1, g2 = x.grad.clone(), fc1.weight.grad.clone(), fc2.weight.grad.clone()
    x.grad.zero_()
    fc1.zero_grad()
    fc2.zero_grad()
    y3, y4 = bundle.GEMMBundleFunction.apply(x, fc1.weight, fc2.weight, fc1.bias, fc2.bias)
    torch.sum(y3 + y4).backward()
    assert torch.allclose(y1, y3, atol=1e-3) and torch.allclose(y2, y4, atol=1e-3)
    assert torch.allclose(g1, fc1.weight.grad, atol=1e-3)
    assert torch.allclose(g2, fc2.weight.grad, atol=1e-3)
    assert torch.allclose(gx1, x.grad, atol=1e-3)


def test_b2gemm_against_oracle(dev):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4096, 256, generator=g)
    wa = torch.randn(256, 256, generator=g) * 0.02
    wb = torch.randn(256, 256, generator=g) * 0.02
    ga = torch.randn(4096, 256, generator=g)
    gb = torch.randn(4096, 256, generator=g)
    ya, yb = graph_ext.b2gemm(x.to(dev), wa.to(dev), wb.to(dev))
    want_a, want_b = oracle.b2gemm(x.numpy(), wa.numpy(), wb.numpy())
    assert_close(ya, want_a)
    assert_close(yb, want_b)
    dx, dwa, dwb = graph_ext.b2gemm_backward(x.to(dev), wa.to(dev), wb.to(dev), ga.to(dev),
                                             gb.to(dev))
    want_dx, want_dwa, want_dwb = oracle.b2gemm_backward(x.numpy(), wa.numpy(), wb.numpy(),
                                                         ga.numpy(), gb.numpy())
    assert_close(dx, want_dx)
    assert_close(dwa, want_dwa, atol=1e-4 * 64)
    assert_close(dwb, want_dwb, atol=1e-4 * 64)


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1, 1, 8), (7, 5, 16), (128, 256, 32), (130, 257, 40),
                                   (1000, 100, 104), (4096, 256, 256), (300, 512, 0)])
def test_gemm_bf16_against_double(dev, tb, out_dtype, m, n, k):
    """bf16 operands are exact in fp32, so the product differs from the double one by the
    fp32 accumulation only (and by one bf16 rounding when the output is bf16)."""
    g = torch.Generator().manual_seed(m + 3 * n + 5 * k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    b = torch.randn((n, k) if tb else (k, n), generator=g).to(torch.bfloat16)
    got = graph_ext.gemm_bf16(a.to(dev), b.to(dev), trans_b=tb, out_dtype=out_dtype)
    want = a.double() @ (b.double().t() if tb else b.double())
    assert got.dtype == out_dtype and got.shape == (m, n)
    if out_dtype == torch.float32:
        assert_close(got, want.float(), atol=1e-4 * max(1.0, np.sqrt(k) / 4))
    else:
        # one bf16 rounding (relative 2^-9) on top of the fp32 accumulation error
        assert_close(got.float(), want.float(), rtol=2.0 ** -8,
                     atol=1e-4 * max(1.0, np.sqrt(k) / 4))


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(4100, 256, 256), (5000, 300, 64), (70001, 256, 48),
                                   (4096, 250, 128), (20000, 520, 256), (40000, 64, 16)])
def test_gemm_bf16_many_rows_short_inner_dimension(dev, out_dtype, m, n, k):
    """Inner dimensions of at most 256 with thousands of rows run with the weight held in
    registers and whole-row tiles: ragged last tile, column counts that are not multiples
    of 4 / 64 / 256, several column blocks, short inner dimensions."""
    g = torch.Generator().manual_seed(m + 3 * n + 5 * k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    b = torch.randn(n, k, generator=g).to(torch.bfloat16)
    got = graph_ext.gemm_bf16(a.to(dev), b.to(dev), trans_b=True, out_dtype=out_dtype)
    want = (a.double() @ b.double().t()).float()
    if out_dtype == torch.float32:
        assert_close(got, want, atol=1e-4 * max(1.0, np.sqrt(k) / 4))
    else:
        assert_close(got.float(), want, rtol=2.0 ** -8, atol=1e-4 * max(1.0, np.sqrt(k) / 4))
    assert torch.equal(got, graph_ext.gemm_bf16(a.to(dev), b.to(dev), trans_b=True,
                                                out_dtype=out_dtype))


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ms,n,k", [([5000, 0, 4097, 300], 256, 256),
                                    ([700] * 10, 192, 128),      # two launches of 8 and 2
                                    ([33, 64, 1], 256, 64),      # few rows: one product each
                                    ([3000, 2000], 72, 40)])     # not one of the grouped widths
def test_gemm_bf16_typed_against_double(dev, tb, out_dtype, ms, n, k):
    """Products of several node types in one call: row tiles of every type in one grid,
    a type's ragged last tile next to the first tile of the next, an empty type."""
    g = torch.Generator().manual_seed(sum(ms) + 3 * n + 5 * k)
    a = [torch.randn(m, k, generator=g).to(torch.bfloat16) for m in ms]
    b = [torch.randn((n, k) if tb else (k, n), generator=g).to(torch.bfloat16) for _ in ms]
    rows = torch.zeros(sum(ms), n, dtype=out_dtype, device=dev)
    outs = list(rows.split(ms))  # row slices of one buffer
    got = graph_ext.gemm_bf16_typed([x.to(dev) for x in a], [w.to(dev) for w in b], trans_b=tb,
                                    out_list=outs)
    for x, w, c, m in zip(a, b, got, ms):
        want = (x.double() @ (w.double().t() if tb else w.double())).float()
        assert c.dtype == out_dtype and c.shape == (m, n)
        if out_dtype == torch.float32:
            assert_close(c, want, atol=1e-4 * max(1.0, np.sqrt(k) / 4))
        else:
            assert_close(c.float(), want, rtol=2.0 ** -8, atol=1e-4 * max(1.0, np.sqrt(k) / 4))
    again = graph_ext.gemm_bf16_typed([x.to(dev) for x in a], [w.to(dev) for w in b], trans_b=tb,
                                      out_dtype=out_dtype)
    assert all(torch.equal(c, d) for c, d in zip(got, again))


@pytest.mark.parametrize("m,ki,no", [(1, 8, 8), (33, 8, 16), (100, 72, 40), (4096, 256, 256),
                                     (5000, 128, 264), (70000, 256, 256), (0, 16, 8)])
def test_gemm_bf16_tn_against_double(dev, m, ki, no):
    """The weight gradient X^T . dY with bf16 operands: exact products, fp32 sums over
    the m rows in a fixed order; the allowance follows sum |x| |g| (helpers.assert_close)."""
    g = torch.Generator().manual_seed(m + 3 * ki + 5 * no)
    a = torch.randn(m, ki, generator=g).to(torch.bfloat16)
    b = torch.randn(m, no, generator=g).to(torch.bfloat16)
    got = graph_ext.gemm_bf16_tn(a.to(dev), b.to(dev))
    want = (a.double().t() @ b.double()).float()
    abs_sum = (a.double().abs().t() @ b.double().abs()).float()
    assert got.dtype == torch.float32 and got.shape == (ki, no)
    assert_close(got, want, abs_sum=abs_sum, what="m=%d ki=%d no=%d" % (m, ki, no))
    assert torch.equal(got, graph_ext.gemm_bf16_tn(a.to(dev), b.to(dev)))  # reproducible
    # accumulate, and operands that are column slices of wider buffers
    if m > 0 and ki >= 16:
        wide_a = torch.randn(m, ki + 24, generator=g).to(torch.bfloat16).to(dev)
        wide_b = torch.randn(m, no + 8, generator=g).to(torch.bfloat16).to(dev)
        acc = torch.ones(ki, no, device=dev)
        graph_ext.gemm_bf16_tn(wide_a[:, 8:8 + ki], wide_b[:, :no], out=acc, accumulate=True)
        want2 = 1.0 + (wide_a[:, 8:8 + ki].double().t() @ wide_b[:, :no].double())
        abs2 = 1.0 + (wide_a[:, 8:8 + ki].double().abs().t() @ wide_b[:, :no].double().abs())
        assert_close(acc, want2.float(), abs_sum=abs2.float())


@pytest.mark.parametrize("ms,ki,no", [([70000, 0, 4097, 300], 256, 256), ([900] * 10, 72, 136),
                                      ([1, 31, 33], 8, 16)])
def test_gemm_bf16_tn_typed_against_double(dev, ms, ki, no):
    """Weight gradients of several node types in one call: the types' row chunks share a
    grid, a type without rows gives zeros; reproducible; `accumulate` adds."""
    g = torch.Generator().manual_seed(sum(ms) + ki + no)
    a = [torch.randn(m, ki, generator=g).to(torch.bfloat16) for m in ms]
    b = [torch.randn(m, no, generator=g).to(torch.bfloat16) for m in ms]
    da, db = [x.to(dev) for x in a], [x.to(dev) for x in b]
    got = graph_ext.gemm_bf16_tn_typed(da, db)
    for x, y, c, m in zip(a, b, got, ms):
        want = (x.double().t() @ y.double()).float()
        assert_close(c, want, atol=1e-4 * max(1.0, np.sqrt(max(m, 1))))
    again = graph_ext.gemm_bf16_tn_typed(da, db)
    assert all(torch.equal(c, d) for c, d in zip(got, again))
    acc = [torch.ones(ki, no, device=dev) for _ in ms]
    graph_ext.gemm_bf16_tn_typed(da, db, out_list=acc, accumulate=True)
    for c, d in zip(got, acc):
        assert_close(d, c + 1.0, atol=1e-4 * max(1.0, np.sqrt(max(max(ms), 1))))


def test_gemm_bf16_tn_rejects_unaligned_width(dev):
    a = torch.zeros(16, 12, dtype=torch.bfloat16, device=dev)
    b = torch.zeros(16, 8, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        graph_ext.gemm_bf16_tn(a, b)


def test_gemm_bf16_rejects_unaligned_k(dev):
    a = torch.zeros(4, 12, dtype=torch.bfloat16, device=dev)
    b = torch.zeros(12, 4, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        graph_ext.gemm_bf16(a, b)


@pytest.mark.parametrize("n,k,j,bias", [(1000, 256, 8, True), (33, 64, 1, False), (517, 512, 8, True),
                                        (260, 1024, 4, True), (129, 100, 16, True), (5, 768, 4, False),
                                        (2048, 256, 16, True)])
def test_skinny_linear_forward_backward(dev, n, k, j, bias):
    """Linear layers with a handful of outputs against float64 torch: y, grad_x written and
    accumulated in place, grad_w, grad_b."""
    g = torch.Generator().manual_seed(n + k + j)
    x, w = torch.randn(n, k, generator=g), torch.randn(j, k, generator=g)
    b = torch.randn(j, generator=g) if bias else None
    gy, base = torch.randn(n, j, generator=g), torch.randn(n, k, generator=g)
    d = lambda t: None if t is None else t.to(dev)
    y = graph_ext.skinny_linear(d(x), d(w), d(b))
    want = x.double() @ w.double().t() + (b.double() if bias else 0)
    assert_close(y, want.float(), atol=1e-4 * k ** 0.5)
    gx, gw, gb = graph_ext.skinny_linear_backward(d(x), d(w), d(gy), need_bias=bias)
    assert_close(gx, (gy.double() @ w.double()).float(), atol=1e-4 * j ** 0.5)
    assert_close(gw, (gy.double().t() @ x.double()).float(), atol=1e-4 * n ** 0.5)
    if bias:
        assert_close(gb, gy.double().sum(0).float(), atol=1e-4 * n ** 0.5)
    else:
        assert gb is None
    acc = d(base.clone())
    gx2, gw2, _ = graph_ext.skinny_linear_backward(d(x), d(w), d(gy), grad_x=acc, need_bias=bias)
    assert gx2 is acc
    assert_close(gx2, (gy.double() @ w.double() + base.double()).float(), atol=1e-4 * j ** 0.5)
    assert torch.equal(gw2, gw)


def test_skinny_linear_rejects_wide_outputs(dev):
    x, w = torch.zeros(4, 1024, device=dev), torch.zeros(8, 1024, device=dev)
    with pytest.raises(RuntimeError):
        graph_ext.skinny_linear(x, w)
    assert not graph_ext.skinny_linear_shape(1024, 8) and graph_ext.skinny_linear_shape(1024, 4)


@pytest.mark.parametrize("m,n", [(1, 1), (11132, 100), (64, 272), (65, 3), (5000, 1000), (70001, 256),
                                 (9000, 1024), (8193, 12), (300000, 64), (4097, 1028), (777, 4)])
def test_column_sum(dev, m, n):
    """Column counts that are multiples of 4 up to 1024 (16-byte reads, several rows side by
    side, also where 256 is not a multiple of n / 4) and others (one column per thread); row
    counts around the chunking's steps; the same bits on a second call."""
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, n, generator=g)
    got = graph_ext.column_sum(x.to(dev))
    assert_close(got, x.double().sum(0).float(), atol=1e-4 * m ** 0.5)
    assert torch.equal(got, graph_ext.column_sum(x.to(dev)))


@pytest.mark.parametrize("n,k,m,bias", [(1000, 256, 256, True), (77, 24, 64, True), (513, 100, 172, False),
                                        (300, 64, 4, True)])
def test_bundle_linear_matches_torch(dev, n, k, m, bias):
    """bundle.linear (MFMA GEMM or skinny product, fixed-order bias gradient) == F.linear,
    outputs and all three gradients."""
    torch.manual_seed(n + k + m)
    lin = nn.Linear(k, m, bias=bias).to(dev)
    x = torch.randn(n, k, device=dev, requires_grad=True)
    w = torch.randn(n, m, device=dev)
    y = bundle.linear(x, lin.weight, lin.bias)
    (y * w).sum().backward()
    got = [y.detach(), x.grad.clone(), lin.weight.grad.clone()] + ([lin.bias.grad.clone()] if bias else [])
    x.grad = None
    lin.zero_grad()
    y2 = lin(x)
    (y2 * w).sum().backward()
    want = [y2.detach(), x.grad, lin.weight.grad] + ([lin.bias.grad] if bias else [])
    for a, b in zip(got, want):
        assert_close(a, b, rtol=1e-4, atol=2e-4 * (n ** 0.5 if a.dim() < 2 or a.shape == lin.weight.shape else 1))


def test_typed_products_of_forty_small_layers(dev):
    """More layers than one launch takes (32), a few hundred rows each, outputs of 2 and of 32
    columns: the per-relation Linears and attention projections of a small heterogeneous
    graph. Forward with biases, both gradient products and the bias gradients in one
    grouped call each, against float64."""
    g = torch.Generator().manual_seed(77)
    for n_out, k in ((32, 32), (2, 64), (4, 24)):
        ms = [int(v) for v in torch.randint(0, 400, (40,), generator=g)]
        ms[5] = 0
        xs = [torch.randn(m, k, generator=g) for m in ms]
        ws = [torch.randn(n_out, k, generator=g) for _ in ms]
        bs = [torch.randn(n_out, generator=g) if i % 3 else None for i in range(len(ms))]
        to = lambda ts: [None if t is None else t.to(dev) for t in ts]
        got = graph_ext.linear_forward_typed(to(xs), to(ws), to(bs))
        for x, w, b, y in zip(xs, ws, bs, got):
            want = x.double() @ w.double().t() + (0 if b is None else b.double())
            assert_close(y, want, abs_sum=x.double().abs() @ w.double().abs().t())
        gys = [torch.randn(m, n_out, generator=g) for m in ms]
        gx = graph_ext.sgemm_typed(to(gys), to(ws))
        gw = graph_ext.sgemm_typed(to(gys), to(xs), trans_a=True)
        for gy, x, w, dx, dw in zip(gys, xs, ws, gx, gw):
            assert_close(dx, gy.double() @ w.double(), abs_sum=gy.double().abs() @ w.double().abs())
            assert_close(dw, gy.double().t() @ x.double(),
                         abs_sum=gy.double().abs().t() @ x.double().abs())
        # bias gradients: row slices of one buffer, one launch per 32 of them
        buf = torch.cat(gys).to(dev)
        parts, off = [], 0
        for m in ms:
            parts.append(buf[off:off + m])
            off += m
        sums = graph_ext.column_sum_typed(parts)
        for gy, s in zip(gys, sums):
            assert_close(s, gy.double().sum(0), abs_sum=gy.double().abs().sum(0))
        again = graph_ext.column_sum_typed(parts)
        assert all(torch.equal(a, b) for a, b in zip(sums, again))
    # long matrices take the two-stage sum of one matrix each
    long_parts = [torch.randn(9000, 8, generator=g).to(dev), torch.randn(10, 8, generator=g).to(dev)]
    for x, s in zip(long_parts, graph_ext.column_sum_typed(long_parts)):
        assert_close(s, x.double().sum(0), abs_sum=x.double().abs().sum(0))
