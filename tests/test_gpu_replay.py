"""A training step recorded into a HIP graph (yitu_amd.utils.replay): replays must
reproduce the eager step bit for bit on this library's kernels, also with eager work in
between, and a step that cannot be replayed faithfully must be refused."""
import numpy as np
import pytest
import torch

from helpers import powerlaw_graph
from yitu_amd import YiTu_GNN_kernel as K
from yitu_amd.data import graphgen
from yitu_amd.utils.replay import ReplayedStep

pytestmark = pytest.mark.gpu


def test_gcn_layer_step_replays_like_eager(dev):
    """forward + backward of a GCN layer (dense product, aggregation with long rows through
    the row plan, both gradient products) replayed five times with new inputs written into
    the same buffers: same bits as the eager step on those inputs."""
    indptr, indices = powerlaw_graph(12, 60000, 3)
    n = indptr.numel() - 1
    rp, ci, deg = indptr.to(dev), indices.to(dev), graphgen.gcn_norm(indptr).to(dev)
    pp, p2n = K.build_part(32, rp)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(n, 48, generator=g).to(dev)
    w = (torch.randn(48, 32, generator=g) / 8).to(dev)
    dy = torch.randn(n, 32, generator=g).to(dev)

    def step():
        out = K.forward(x, w, rp, ci, deg, pp, p2n, 32, 32, 8)[0]
        dx, dw = K.backward(dy, x, w, rp, ci, deg, pp, p2n, 32, 32, 8)
        return [out, dx, dw]

    replayed = ReplayedStep(step, rtol=0, atol=0)
    for seed in range(5):
        x.copy_(torch.randn(n, 48, generator=g))
        dy.copy_(torch.randn(n, 32, generator=g))
        got = [t.clone() for t in replayed.replay()]
        want = step()
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_a_step_that_changes_between_runs_is_refused(dev):
    state = {"calls": 0}
    x = torch.ones(1000, device=dev)

    def step():
        state["calls"] += 1
        return [x * float(state["calls"])]  # the recording freezes one factor, eager moves on

    with pytest.raises(RuntimeError, match="differs from the eager step"):
        ReplayedStep(step)


@pytest.mark.parametrize("which", ["rgcn", "rgat"])
def test_stitched_hetero_model_step_replays_like_eager(dev, which):
    """The reference's heterogeneous models (test/common/model.py:174-229), captured, lowered
    and stitched, with their per-relation Linears grouped by the executor: forward + backward
    recorded into a HIP graph give the eager step's outputs and parameter gradients on every
    replay, also after new feature rows were written into the embedding tables."""
    import pipeline_cases as cases
    from yitu_amd import xgnn_h
    from yitu_amd.xgnn_h import models
    torch.manual_seed(5)
    hgraph = cases.hetero_graph(device=dev)
    kwargs = cases.hetero_kwargs(hgraph, device=dev, with_norms=which == "rgcn")
    model = (models.RGCNModel(hgraph, 16, 16, 4) if which == "rgcn"
             else models.RGATModel(hgraph, 16, 16, 4, n_heads=2)).to(dev)
    lowered = xgnn_h.Optimizer().lower(xgnn_h.Module2IR().transform(model, kwargs), kwargs)
    stitched = xgnn_h.Stitcher().transform(lowered, kwargs)
    executor = xgnn_h.Executor()
    executor.eval()  # no dropout: the replays can be compared with eager runs
    params = list(model.parameters())
    weights = {nty: torch.randn(num, 4, device=dev) for nty, num in hgraph.nty2num.items()}

    def step():
        for p in params:
            p.grad = None
        out = executor.run(stitched, kwargs)
        torch.autograd.backward([out[k] for k in out], [weights[k] for k in out])
        return [out[k] for k in out] + [p.grad for p in params if p.grad is not None]

    replayed = ReplayedStep(step, rtol=1e-5, atol=1e-6)
    tables = [p for p in params if p.dim() == 2 and p.size(0) in cases.NTYPES.values()]
    assert tables
    for _ in range(3):
        with torch.no_grad():
            for t in tables:
                t.copy_(torch.randn_like(t))
        got = [t.clone() for t in replayed.replay()]
        want = step()
        assert len(got) == len(want)
        for a, b in zip(got, want):
            assert torch.allclose(a, b, rtol=1e-5, atol=1e-6)
