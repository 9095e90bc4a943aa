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
