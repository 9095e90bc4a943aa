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
from helpers import assert_close

pytestmark = pytest.mark.gpu


def _dense_reference(layer, h, row, dt, n_dst, k_max):
    """Dense masked attention with the layer's own parameters."""
    dev = h.device
    E = row.numel()
    slot = torch.zeros(E, dtype=torch.long, device=dev)
    counts = torch.bincount(row, minlength=n_dst)
    start = torch.cumsum(counts, 0) - counts
    slot = torch.arange(E, device=dev) - start[row]
    mask = torch.zeros(n_dst, k_max, dtype=torch.bool, device=dev)
    mask[row, slot] = True
    te = torch.cos(dt[:, None] * layer.time_enc.w.weight[:, 0][None, :] + layer.time_enc.w.bias)
    te0 = torch.cos(layer.time_enc.w.bias)[None, :].expand(n_dst, -1)
    q = layer.w_q(torch.cat([h[:n_dst], te0], 1))
    kv_in = torch.cat([h[n_dst:], te], 1)
    k, v = layer.w_k(kv_in), layer.w_v(kv_in)
    H, D = layer.num_head, layer.dim_out // layer.num_head
    Kd = torch.zeros(n_dst, k_max, H, D, device=dev)
    Vd = torch.zeros(n_dst, k_max, H, D, device=dev)
    Kd[row, slot] = k.reshape(E, H, D)
    Vd[row, slot] = v.reshape(E, H, D)
    logits = torch.einsum("bhd,bkhd->bkh", q.reshape(n_dst, H, D), Kd)
    logits = torch.nn.functional.leaky_relu(logits, 0.2)
    logits = logits.masked_fill(~mask[:, :, None], float("-inf"))
    att = torch.softmax(logits, dim=1)
    att = torch.nan_to_num(att, nan=0.0)  # roots without neighbours
    agg = torch.einsum("bkh,bkhd->bhd", att, Vd).reshape(n_dst, H * D)
    out = layer.w_out(torch.cat([agg, h[:n_dst]], 1))
    return layer.layer_norm(torch.relu(out))


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
    want = _dense_reference(layer, blk.h, blk.row, blk.dt, blk.n_dst, k)
    (want * w).sum().backward()
    assert_close(out, want, atol=2e-4)
    ref_grads = [blk.h.grad] + [p.grad for p in layer.parameters()]
    for g, r, name in zip(grads, ref_grads, ["h"] + [n for n, _ in layer.named_parameters()]):
        assert_close(g, r, rtol=1e-4, atol=5e-4, what=name)


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
