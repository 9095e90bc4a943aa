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
