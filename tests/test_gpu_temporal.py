"""Temporal neighbour attention (fifth configuration) on the GPU: the layer built
on the HIP ops against a dense [B, k] masked-softmax formulation in plain torch
(time encoding cos(w dt + b), LeakyReLU(0.2), softmax over each root's sampled
neighbours, weighted sum, output projection, ReLU, LayerNorm), forward and
gradients. The reference holds no test for this layer and its attention core is
DGL code outside the tree, so the closed form is the pin."""
import numpy as np
import pytest
import torch

from yitu_amd import sampler_core
from yitu_amd.temporal import TemporalBlock, TimeEncode, TransfomerAttentionLayer
from helpers import assert_close, dense_temporal_attention

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("num_head", [1, 2])
def test_layer_matches_dense_masked_attention(dev, num_head):
    torch.manual_seed(0)
    rng = np.random.default_rng(0)
    n_nodes, n_events, k = 400, 6000, 20
    src = (rng.zipf(1.2, n_events) - 1) % n_nodes
    dst = (rng.zipf(1.2, n_events) - 1) % n_nodes
    ts = np.sort(rng.uniform(0, 1e6, n_events)).astype(np.float32)
    lists = [[] for _ in range(n_nodes)]
    for e, (s, d, t) in enumerate(zip(src, dst, ts)):
        lists[s].append((t, d, e))
        lists[d].append((t, s, e))
    indptr, indices, eid, tss = [0], [], [], []
    for l in lists:
        for t, d, e in sorted(l):
            indices.append(d), eid.append(e), tss.append(t)
        indptr.append(len(indices))
    smp = sampler_core.ParallelSampler(indptr, indices, eid, tss, 4, 1, 1, [k], True, False, 1, 0.0)
    ev = rng.integers(n_events * 9 // 10, n_events, 128)
    smp.sample(np.concatenate([src[ev], dst[ev]]), np.concatenate([ts[ev], ts[ev]]))
    tgb = smp.get_ret()[0]
    memory = torch.randn(n_nodes, 172, device=dev)
    blk = TemporalBlock.from_sampler(tgb, memory, device=dev)
    assert blk.num_edges() > 500
    layer = TransfomerAttentionLayer(172, 0, 100, num_head, 0.0, 0.0, 100).to(dev)
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
    ref_grads = [blk.h.grad] + [p.grad for p in layer.parameters()]
    for g, r, name in zip(grads, ref_grads, ["h"] + [n for n, _ in layer.named_parameters()]):
        # the frequency gradients sum products with time deltas of up to 10^6 that largely
        # cancel: both sides carry fp32 summation noise well above their other gradients'
        rtol = 1e-3 if name == "time_enc.w.weight" else 1e-4
        assert_close(g, r, rtol=rtol, atol=5e-4, what=name)


def test_time_encode_closed_form(dev):
    te = TimeEncode(100).to(dev)
    t = torch.tensor([0.0, 1.0, 1234.5, 1e6], device=dev)
    w = torch.from_numpy(1 / 10 ** np.linspace(0, 9, 100, dtype=np.float32)).to(dev)
    assert torch.allclose(te(t), torch.cos(t[:, None] * w[None, :]), atol=1e-6)
    assert te.w.weight.shape == (100, 1) and torch.all(te.w.bias == 0)


def test_empty_block_returns_zeros(dev):
    layer = TransfomerAttentionLayer(8, 0, 4, 1, 0.0, 0.0, 6).to(dev)
    blk = TemporalBlock(np.zeros(0, np.int64), 5, np.zeros(0, np.float32),
                        h=torch.randn(5, 8, device=dev), device=dev)
    out = layer(blk)
    assert out.shape == (5, 6) and torch.all(out == 0)


def _reference_layer(layer, blk, dtype=torch.float64):
    """The layer's arithmetic (layers.py:75-142) edge by edge in float64 torch ops, with
    autograd: per-root softmax through index_reduce / index_add."""
    import copy
    ref = copy.deepcopy(layer).to(dtype)
    n_dst, row = blk.n_dst, blk.row
    E = row.numel()
    h = blk.h.detach().to(dtype).requires_grad_() if layer.dim_node_feat > 0 else None
    f = blk.f.detach().to(dtype).requires_grad_() if layer.dim_edge_feat > 0 else None
    parts_q, parts_kv = [], []
    if h is not None:
        parts_q.append(h[:n_dst])
        parts_kv.append(h[n_dst:])
    if f is not None:
        parts_kv.append(f)
    if layer.dim_time > 0:
        # the argument of the cosine as float32 rounds it (product, then bias); the
        # reference rounds there as well (Linear(1, dim) in float32)
        w32, b32 = layer.time_enc.w.weight.detach()[:, 0], layer.time_enc.w.bias.detach()
        arg32 = (blk.dt[:, None] * w32[None, :] + b32).to(dtype)
        w, b = ref.time_enc.w.weight[:, 0], ref.time_enc.w.bias
        exact = blk.dt.to(dtype)[:, None] * w[None, :] + b
        parts_kv.append(torch.cos(exact + (arg32 - exact).detach()))
        parts_q.append(torch.cos(b)[None, :].expand(n_dst, -1))
    q = ref.w_q(torch.cat(parts_q, 1))[row]
    kv_in = torch.cat(parts_kv, 1)
    k, v = ref.w_k(kv_in), ref.w_v(kv_in)
    H, D = layer.num_head, layer.dim_out // layer.num_head
    logits = torch.nn.functional.leaky_relu((q * k).view(E, H, D).sum(-1), 0.2)
    top = torch.full((n_dst, H), -1e30, dtype=dtype, device=row.device)
    top = top.index_reduce(0, row, logits.detach(), "amax")
    p = torch.exp(logits - top[row])
    s = torch.zeros(n_dst, H, dtype=dtype, device=row.device).index_add(0, row, p)
    att = p / s[row]
    agg = torch.zeros(n_dst, H, D, dtype=dtype, device=row.device).index_add(
        0, row, v.view(E, H, D) * att[:, :, None]).reshape(n_dst, H * D)
    rst = torch.cat([agg, h[:n_dst]], 1) if h is not None else agg
    out = ref.layer_norm(torch.relu(ref.w_out(rst)))
    return ref, out, h, f


@pytest.mark.parametrize("dims", [
    # dim_node, dim_edge, dim_time, num_head, dim_out
    (172, 0, 100, 1, 100), (172, 0, 100, 4, 100), (16, 12, 8, 2, 32), (0, 5, 10, 1, 24),
    (20, 0, 0, 2, 64), (33, 7, 100, 8, 256), (9, 0, 3, 1, 6)])
def test_fused_layer_all_input_combinations(dev, dims):
    """The layer as one autograd node (input assembly, products, attention per root, ReLU +
    LayerNorm) for every combination of node / edge / time inputs the reference's branches
    cover, with roots that have no neighbour, one, 64, 65 and 150 (more than one chunk of
    the online softmax): output and every gradient against the float64 statement above,
    rtol 1e-5 / atol 1e-4 (looser for the frequency gradients, see above)."""
    dim_node, dim_edge, dim_time, num_head, dim_out = dims
    torch.manual_seed(sum(dims))
    counts = [0, 1, 64, 65, 150, 3, 0, 20, 20, 7] + [5] * 40
    n_dst = len(counts)
    row = np.repeat(np.arange(n_dst), counts)
    E = row.size
    dt = np.random.default_rng(0).uniform(0, 1e4, E).astype(np.float32)
    h = torch.randn(n_dst + E, dim_node, device=dev) if dim_node else None
    f = torch.randn(E, dim_edge, device=dev) if dim_edge else None
    blk = TemporalBlock(row, n_dst, dt, h=h, f=f, device=dev)
    layer = TransfomerAttentionLayer(dim_node, dim_edge, dim_time, num_head, 0.0, 0.0, dim_out).to(dev)
    with torch.no_grad():   # biases and phases away from their zero initial values
        for p in layer.parameters():
            if p.dim() == 1:
                p.add_(torch.randn_like(p) * 0.3)
    if h is not None:
        h.requires_grad_()
    if f is not None:
        f.requires_grad_()
    out = layer(blk)
    assert out.grad_fn.name().startswith("TemporalAttentionFunction")
    w = torch.randn_like(out)
    (out * w).sum().backward()
    ref, want, h_ref, f_ref = _reference_layer(layer, blk)
    (want * w.double()).sum().backward()
    assert_close(out, want.float(), atol=1e-4, what="out")
    pairs = [(n, p.grad, dict(ref.named_parameters())[n].grad) for n, p in layer.named_parameters()]
    if h is not None:
        pairs.append(("h", h.grad, h_ref.grad))
    if f is not None:
        pairs.append(("f", f.grad, f_ref.grad))
    for name, got, ref_grad in pairs:
        assert got is not None, name
        scale = 1e4 if name == "time_enc.w.weight" else 1.0   # sums of products with dt <= 10^4
        assert_close(got, ref_grad.float(), rtol=1e-4, atol=1e-4 * scale, what=name)
    # same bits on a second run
    layer.zero_grad()
    out2 = layer(blk)
    (out2 * w).sum().backward()
    assert torch.equal(out, out2)
    for name, got, _ in pairs[:len(list(layer.parameters()))]:
        assert torch.equal(got, dict(layer.named_parameters())[name].grad), name


def test_fused_layer_equals_the_composed_ops(dev, monkeypatch):
    """The same block through the fused node and through the composition of graph_ext ops
    that the layer used before (and still uses under dropout)."""
    from yitu_amd.temporal import fused
    torch.manual_seed(5)
    counts = np.random.default_rng(5).integers(0, 21, 300)
    row = np.repeat(np.arange(300), counts)
    dt = np.random.default_rng(6).uniform(0, 1e6, row.size).astype(np.float32)
    h = torch.randn(300 + row.size, 172, device=dev, requires_grad=True)
    blk = TemporalBlock(row, 300, dt, h=h, device=dev)
    layer = TransfomerAttentionLayer(172, 0, 100, 1, 0.0, 0.0, 100).to(dev)
    w = torch.randn(300, 100, device=dev)
    out = layer(blk)
    (out * w).sum().backward()
    got = [h.grad.clone()] + [p.grad.clone() for p in layer.parameters()]
    h.grad = None
    layer.zero_grad()
    monkeypatch.setattr(fused, "supported", lambda *a: False)
    out_c = layer(blk)
    assert not out_c.grad_fn.name().startswith("TemporalAttentionFunction")
    (out_c * w).sum().backward()
    assert_close(out, out_c, atol=1e-4)
    for g, r, name in zip(got, [h.grad] + [p.grad for p in layer.parameters()],
                          ["h"] + [n for n, _ in layer.named_parameters()]):
        rtol = 1e-3 if name == "time_enc.w.weight" else 1e-4
        assert_close(g, r, rtol=rtol, atol=5e-4, what=name)


def _reference_combined(layer, blk):
    """layers.py:81-103 in float64: one Linear per input part, results added."""
    import copy
    ref = copy.deepcopy(layer).double()
    n_dst, row = blk.n_dst, blk.row
    E = row.numel()
    dev = row.device
    O = layer.dim_out
    q = torch.zeros(E, O, dtype=torch.float64, device=dev)
    k = torch.zeros(E, O, dtype=torch.float64, device=dev)
    v = torch.zeros(E, O, dtype=torch.float64, device=dev)
    h = blk.h.detach().double().requires_grad_() if layer.dim_node_feat > 0 else None
    f = blk.f.detach().double().requires_grad_() if layer.dim_edge_feat > 0 else None
    if h is not None:
        q = q + ref.w_q_n(h[:n_dst])[row]
        k = k + ref.w_k_n(h[n_dst:])
        v = v + ref.w_v_n(h[n_dst:])
    if f is not None:
        k = k + ref.w_k_e(f)
        v = v + ref.w_v_e(f)
    if layer.dim_time > 0:
        w32, b32 = layer.time_enc.w.weight.detach()[:, 0], layer.time_enc.w.bias.detach()
        arg32 = (blk.dt[:, None] * w32[None, :] + b32).double()
        w, b = ref.time_enc.w.weight[:, 0], ref.time_enc.w.bias
        exact = blk.dt.double()[:, None] * w[None, :] + b
        te = torch.cos(exact + (arg32 - exact).detach())
        te0 = torch.cos(b)[None, :].expand(n_dst, -1)
        q = q + ref.w_q_t(te0)[row]
        k = k + ref.w_k_t(te)
        v = v + ref.w_v_t(te)
    H, D = layer.num_head, O // layer.num_head
    logits = torch.nn.functional.leaky_relu((q * k).view(E, H, D).sum(-1), 0.2)
    top = torch.full((n_dst, H), -1e300, dtype=torch.float64, device=dev)
    top = top.index_reduce(0, row, logits.detach(), "amax")
    p = torch.exp(logits - top[row])
    s = torch.zeros(n_dst, H, dtype=torch.float64, device=dev).index_add(0, row, p)
    att = p / s[row]
    agg = torch.zeros(n_dst, H, D, dtype=torch.float64, device=dev).index_add(
        0, row, v.view(E, H, D) * att[:, :, None]).reshape(n_dst, O)
    rst = torch.cat([agg, h[:n_dst]], 1) if h is not None else agg
    return ref, ref.layer_norm(torch.relu(ref.w_out(rst))), h, f


@pytest.mark.parametrize("dims", [(24, 6, 10, 2, 32), (24, 0, 10, 1, 16), (0, 6, 0, 1, 8),
                                  (12, 5, 0, 4, 32)])
def test_combined_branch(dev, dims):
    """combined=True (layers.py:53-66, 81-103): per-part Linears with the reference's
    parameter names, added up; computed as one product over concatenated weights. Against
    the part-by-part float64 statement, output and every gradient; (0, 6, 0): edge
    features only, where the query stays zero and the attention is uniform."""
    dim_node, dim_edge, dim_time, num_head, dim_out = dims
    torch.manual_seed(sum(dims))
    counts = [0, 1, 70, 3, 20] + [6] * 30
    n_dst = len(counts)
    row = np.repeat(np.arange(n_dst), counts)
    E = row.size
    dt = np.random.default_rng(1).uniform(0, 1e4, E).astype(np.float32)
    h = torch.randn(n_dst + E, dim_node, device=dev).requires_grad_() if dim_node else None
    f = torch.randn(E, dim_edge, device=dev).requires_grad_() if dim_edge else None
    blk = TemporalBlock(row, n_dst, dt, h=h, f=f, device=dev)
    layer = TransfomerAttentionLayer(dim_node, dim_edge, dim_time, num_head, 0.0, 0.0, dim_out,
                                     combined=True).to(dev)
    names = {n for n, _ in layer.named_parameters()}
    assert ("w_k_e.weight" in names) == (dim_edge > 0) and ("w_q_t.bias" in names) == (dim_time > 0)
    assert "w_q.weight" not in names and "w_k.weight" not in names
    out = layer(blk)
    w = torch.randn_like(out)
    (out * w).sum().backward()
    ref, want, h_ref, f_ref = _reference_combined(layer, blk)
    (want * w.double()).sum().backward()
    assert_close(out, want.float(), what="out")
    pairs = [(n, p.grad, dict(ref.named_parameters())[n].grad) for n, p in layer.named_parameters()]
    if h is not None:
        pairs.append(("h", h.grad, h_ref.grad))
    if f is not None:
        pairs.append(("f", f.grad, f_ref.grad))
    for name, got, ref_grad in pairs:
        assert got is not None, name
        scale = 1e4 if name == "time_enc.w.weight" else 1.0
        assert_close(got, ref_grad.float(), rtol=1e-4, atol=1e-4 * scale, what=name)
