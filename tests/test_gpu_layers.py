"""GCN / GAT / heterogeneous layers on the GPU against dense torch algebra, the
method of the reference's test_allclose.py (GCN layer == D_in^-1 A X W^T) and
test_kernel.py (GAT attention == masked dense softmax)."""
import numpy as np
import pytest
import torch
from torch import nn

from helpers import assert_close, random_csr
from yitu_amd.xgnn_h import block as xblock
from yitu_amd.xgnn_h import convert, layers

pytestmark = pytest.mark.gpu


def test_gcn_layer_equals_dense_right_norm(dev):
    """test_allclose.py:24-30,53-62: y = D_in^-1 A (X W^T + b)."""
    torch.manual_seed(0)
    n, fin, fout = 300, 40, 24
    indptr, indices = random_csr(n, n, 0.03, 1, empty_rows=(7,))
    blk = xblock.Block([n, n], [indptr, indices]).to(dev)
    norm = layers.right_norm(blk)
    layer = layers.GCNLayer(fin, fout).to(dev)
    x = torch.randn(n, fin, device=dev, requires_grad=True)
    y = layer(blk, norm, x)
    w = torch.randn_like(y)
    (y * w).sum().backward()
    got = [y.detach(), x.grad.clone(), layer.fc.weight.grad.clone()]
    x.grad = None
    layer.zero_grad()
    dense = convert.to_dense(n, n, [indptr, indices], torch.ones(indices.numel())).to(dev)
    deg = dense.sum(1, keepdim=True)
    yd = torch.where(deg > 0, 1.0 / deg.clamp(min=1), torch.zeros_like(deg)) * (dense @ layer.fc(x))
    (yd * w).sum().backward()
    assert torch.all(got[0][7] == 0)
    for a, b in zip(got, [yd.detach(), x.grad, layer.fc.weight.grad]):
        assert_close(a, b, atol=2e-4)


@pytest.mark.parametrize("fused", [True, False])
def test_gat_layer_equals_dense_attention(dev, fused):
    torch.manual_seed(1)
    n, fin, f, h = 257, 30, 16, 4
    indptr, indices = random_csr(n, n, 0.04, 2, hub_rows=(3,), hub_degree=200)
    blk = xblock.Block([n, n], [indptr, indices]).to(dev)
    layer = layers.GATLayer(fin, f, h, fused=fused).to(dev)
    x = torch.randn(n, fin, device=dev, requires_grad=True)
    y = layer(blk, x)
    w = torch.randn_like(y)
    (y * w).sum().backward()
    got = [y.detach(), x.grad.clone()] + [p.grad.clone() for p in layer.parameters()]
    x.grad = None
    layer.zero_grad()
    adj = convert.to_dense(n, n, [indptr, indices], torch.ones(indices.numel())).to(dev)
    hv = layer.linear_v(x)
    q, k = layer.linear_q(hv), layer.linear_k(hv)
    e = nn.functional.leaky_relu(q[:, None, :] + k[None, :, :], 0.2)
    e = torch.where(adj[:, :, None] > 0, e, torch.full_like(e, -1e38))
    a = torch.softmax(e.permute(2, 0, 1), dim=-1) * adj[None]
    yd = torch.bmm(a, hv.view(n, h, f).transpose(0, 1)).transpose(0, 1).mean(dim=1)
    (yd * w).sum().backward()
    want = [yd.detach(), x.grad] + [p.grad for p in layer.parameters()]
    for a_, b_ in zip(got, want):
        assert_close(a_, b_, rtol=1e-4, atol=5e-4)


def test_hetero_conv_mean_over_relations(dev):
    torch.manual_seed(2)
    sizes = {"a": 50, "b": 70}
    rels = [("a", "r0", "b"), ("b", "r1", "b"), ("b", "r2", "a")]
    hgraph, norms = {}, {}
    for i, (s, e, d) in enumerate(rels):
        ip, ix = random_csr(sizes[d], sizes[s], 0.1, 10 + i)
        blk = xblock.Block([sizes[d], sizes[s]], [ip, ix]).to(dev)
        hgraph[(s, e, d)] = blk
        norms[str((s, e, d))] = layers.right_norm(blk)
    conv = layers.HeteroGraphConv({e: layers.GCNLayer(12, 8) for _, e, _ in rels}).to(dev)
    xs = {t: torch.randn(n, 12, device=dev) for t, n in sizes.items()}
    out = conv(hgraph, xs, norms)
    b0 = conv.convs["r0"](hgraph[rels[0]], norms[str(rels[0])], (xs["a"], xs["b"]))
    b1 = conv.convs["r1"](hgraph[rels[1]], norms[str(rels[1])], (xs["b"], xs["b"]))
    assert_close(out["b"], (b0 + b1) / 2)
    assert out["a"].shape == (50, 8)


def test_two_layer_gcn_training_matches_dense_autograd(dev):
    """Twenty SGD steps of a 2-layer GCN built from the module-1 conv (forward and the
    reference-semantics backward through the C ABI) follow the same loss curve as a dense
    autograd model. The graph is symmetric, where aggregating dY with the forward CSR
    (the reference's backward, YiTu_GNN_kernel.cu:447-461) is the true gradient."""
    import types

    import torch.nn.functional as F_
    from yitu_amd import YiTu_GNN_kernel as K
    from yitu_amd.data import graphgen
    from yitu_amd.nn.GCNConv import GCNConv

    n, fin, hid, ncls = 600, 32, 16, 5
    g = torch.Generator().manual_seed(11)
    src = torch.randint(0, n, (4000,), generator=g)
    dst = torch.randint(0, n, (4000,), generator=g)
    loops = torch.arange(n)
    rows = torch.cat([src, dst, loops])  # both directions: symmetric
    cols = torch.cat([dst, src, loops])
    indptr, indices = graphgen.csr_from_edges(rows, cols, n)
    s = graphgen.gcn_norm(indptr)
    pp, p2n = K.build_part(32, indptr)
    info = types.SimpleNamespace(row_pointers=indptr.to(dev), column_index=indices.to(dev),
                                 degrees=s.to(dev), partPtr=pp.to(dev), part2Node=p2n.to(dev),
                                 partSize=32, dimWorker=32, warpPerBlock=8)
    dense = torch.zeros(n, n)
    r = torch.repeat_interleave(torch.arange(n), (indptr[1:] - indptr[:-1]).long())
    dense[r, indices.long()] = s[r] * s[indices.long()]
    dense = dense.to(dev)
    x = torch.randn(n, fin, generator=g).to(dev)
    teacher = torch.randn(fin, ncls, generator=g).to(dev)
    y = (dense @ (x @ teacher)).argmax(1)  # labels a GCN can fit

    torch.manual_seed(3)
    c1, c2 = GCNConv(fin, hid).to(dev), GCNConv(hid, ncls).to(dev)
    w1 = c1.weights.detach().clone().requires_grad_()
    w2 = c2.weights.detach().clone().requires_grad_()
    opt_a = torch.optim.SGD(list(c1.parameters()) + list(c2.parameters()), lr=0.5)
    opt_b = torch.optim.SGD([w1, w2], lr=0.5)
    losses_a, losses_b = [], []
    for _ in range(20):
        opt_a.zero_grad()
        la = F_.nll_loss(F_.log_softmax(c2(torch.relu(c1(x, info)), info), dim=1), y)
        la.backward()
        opt_a.step()
        opt_b.zero_grad()
        lb = F_.nll_loss(F_.log_softmax(dense @ (torch.relu(dense @ (x @ w1)) @ w2), dim=1), y)
        lb.backward()
        opt_b.step()
        losses_a.append(la.item())
        losses_b.append(lb.item())
    assert losses_a[-1] < losses_a[0] - 0.01          # it learns
    assert np.allclose(losses_a, losses_b, rtol=2e-4, atol=2e-5), (losses_a, losses_b)
    assert_close(c1.weights, w1, rtol=1e-3, atol=1e-4)
    assert_close(c2.weights, w2, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("per_relation", [True, False])
def test_stacked_hetero_gcn_equals_per_relation_convs(dev, per_relation):
    """One stacked edge-weighted SpMM == HeteroGraphConv over GCNLayers (model.py:137-171):
    outputs, input gradients and weight gradients, with weights per edge type or shared
    per source node type."""
    torch.manual_seed(4)
    sizes = {"a": 90, "b": 130, "c": 40}
    rels = [("a", "r0", "b"), ("b", "r1", "b"), ("b", "r2", "a"), ("c", "r3", "a"),
            ("a", "r4", "c")]
    fin, fout = 20, 12
    hgraph, norms = {}, {}
    for i, (s, e, d) in enumerate(rels):
        ip, ix = random_csr(sizes[d], sizes[s], 0.08, 30 + i, empty_rows=(i,))
        blk = xblock.Block([sizes[d], sizes[s]], [ip, ix]).to(dev)
        hgraph[(s, e, d)] = blk
        norms[str((s, e, d))] = layers.right_norm(blk)
    stacked = layers.StackedHeteroGCN(sizes, rels, fin, fout, per_relation=per_relation).to(dev)
    stacked.stack(hgraph, norms)
    conv = layers.HeteroGraphConv({e: layers.GCNLayer(fin, fout) for _, e, _ in rels}).to(dev)
    with torch.no_grad():
        for s, e, _ in rels:
            src = stacked.fcs[e if per_relation else s]
            conv.convs[e].fc.weight.copy_(src.weight)
            conv.convs[e].fc.bias.copy_(src.bias)
    xs = {t: torch.randn(n, fin, device=dev, requires_grad=True) for t, n in sizes.items()}
    ws = {t: torch.randn(n, fout, device=dev) for t, n in sizes.items()}

    out = stacked(xs)
    sum((out[t] * ws[t]).sum() for t in out).backward()
    got_x = {t: xs[t].grad.clone() for t in xs}
    got_w = {k: (fc.weight.grad.clone(), fc.bias.grad.clone()) for k, fc in stacked.fcs.items()}
    for t in xs:
        xs[t].grad = None

    want = conv(hgraph, xs, norms)
    sum((want[t] * ws[t]).sum() for t in want).backward()
    assert set(out) == set(want)
    for t in want:
        assert_close(out[t], want[t], rtol=1e-5, atol=1e-4)
    for t in xs:
        assert_close(got_x[t], xs[t].grad, rtol=1e-5, atol=1e-4)
    for k, (gw, gb) in got_w.items():
        if per_relation:
            ref_w, ref_b = conv.convs[k].fc.weight.grad, conv.convs[k].fc.bias.grad
        else:  # shared per source type: the sum over the relations that leave it
            ref_w = sum(conv.convs[e].fc.weight.grad for s, e, _ in rels if s == k)
            ref_b = sum(conv.convs[e].fc.bias.grad for s, e, _ in rels if s == k)
        assert_close(gw, ref_w, rtol=1e-5, atol=1e-4)
        assert_close(gb, ref_b, rtol=1e-5, atol=1e-4)
