"""Lowered and stitched dataflows on the HIP ops against the same dataflow executed
as captured (message functions from their definitions): the equivalences the
reference checks in test_stitch.py:69-79 (stitched == lowered, atol 1e-3) and relies on
for its lowering, here at the fp32 parity tolerance and including every gradient."""
import pytest
import torch

import pipeline_cases as cases
from helpers import assert_close
from yitu_amd import xgnn_h
from yitu_amd.xgnn_h import ir, models

pytestmark = pytest.mark.gpu


def _run_with_grads(dataflow, kwargs, params, weights, leaf_inputs=()):
    for p in list(params) + list(leaf_inputs):
        p.grad = None
    executor = xgnn_h.Executor()
    executor.eval()
    out = executor.run(dataflow, kwargs)
    outs = out if isinstance(out, dict) else {"y": out}
    sum((outs[k] * weights[k]).sum() for k in outs).backward()
    grads = [p.grad.clone() if p.grad is not None else None for p in list(params) + list(leaf_inputs)]
    return {k: v.detach() for k, v in outs.items()}, grads


def _compare(a, b, rtol=1e-5, atol=1e-4):
    outs_a, grads_a = a
    outs_b, grads_b = b
    assert set(outs_a) == set(outs_b)
    for k in outs_a:
        assert_close(outs_a[k], outs_b[k], rtol=rtol, atol=atol, what="output " + k)
    for i, (ga, gb) in enumerate(zip(grads_a, grads_b)):
        assert (ga is None) == (gb is None)
        if ga is not None:
            assert_close(ga, gb, rtol=rtol, atol=atol, what="gradient %d" % i)


@pytest.mark.parametrize("fuse_gat,bundle_gemm", [(True, True), (True, False), (False, True),
                                                  (False, False)])
def test_gat_model_lowered_equals_captured(dev, fuse_gat, bundle_gemm):
    torch.manual_seed(5)
    g = cases.homo_graph(n=300, device=dev)
    model = models.GATModel(24, 16, 8, n_heads=4).to(dev)
    x = torch.randn(g.num_src_nodes(), 24, device=dev, requires_grad=True)
    kwargs = {"graph": g, "x": x}
    captured = xgnn_h.Module2IR().transform(model, kwargs)
    lowered = xgnn_h.Optimizer(fuse_gat=fuse_gat, bundle_gemm=bundle_gemm).lower(captured, kwargs)
    weights = {"y": torch.randn(g.num_dst_nodes(), 8, device=dev)}
    params = list(model.parameters())
    want = _run_with_grads(captured, kwargs, params, weights, [x])
    got = _run_with_grads(lowered, kwargs, params, weights, [x])
    _compare(got, want)
    # the model itself, run eagerly on real tensors, is the same function (torch's
    # index_add_ on the device adds in no fixed order, hence a tolerance)
    model.eval()
    assert_close(model(g, x), want[0]["y"])


def test_gcn_model_lowered_equals_captured(dev):
    torch.manual_seed(6)
    g = cases.homo_graph(n=300, device=dev)
    model = models.GCNModel(24, 16, 8).to(dev)
    x = torch.randn(g.num_src_nodes(), 24, device=dev, requires_grad=True)
    kwargs = {"graph": g, "x": x, "norm": g.right_norm()}
    captured = xgnn_h.Module2IR().transform(model, kwargs)
    lowered = xgnn_h.Optimizer().lower(captured, kwargs)
    weights = {"y": torch.randn(g.num_dst_nodes(), 8, device=dev)}
    params = list(model.parameters())
    _compare(_run_with_grads(lowered, kwargs, params, weights, [x]),
             _run_with_grads(captured, kwargs, params, weights, [x]))


@pytest.mark.parametrize("which", ["rgcn", "rgat"])
def test_hetero_model_lowered_and_stitched(dev, which):
    """captured == lowered == stitched for every destination type, outputs and the
    gradients of every embedding / layer parameter."""
    torch.manual_seed(7)
    hgraph = cases.hetero_graph(device=dev)
    if which == "rgcn":
        kwargs = cases.hetero_kwargs(hgraph, device=dev)
        model = models.RGCNModel(hgraph, 16, 16, 4).to(dev)
    else:
        kwargs = cases.hetero_kwargs(hgraph, device=dev, with_norms=False)
        model = models.RGATModel(hgraph, 16, 16, 4, n_heads=2).to(dev)
    captured = xgnn_h.Module2IR().transform(model, kwargs)
    lowered = xgnn_h.Optimizer().lower(captured, kwargs)
    stitched = xgnn_h.Stitcher().transform(lowered, kwargs)
    n_core = lambda d: sum(1 for n in ir.walk(d) if n.op in ("spmm", "gat"))  # noqa: E731
    assert n_core(stitched) < n_core(lowered)
    weights = {nty: torch.randn(num, 4, device=dev) for nty, num in hgraph.nty2num.items()}
    params = list(model.parameters())
    want = _run_with_grads(captured, kwargs, params, weights)
    _compare(_run_with_grads(lowered, kwargs, params, weights), want)
    _compare(_run_with_grads(stitched, kwargs, params, weights), want)


def test_single_root_stitch_like_the_reference_test(dev):
    """test_stitch.py:41-79: take the predicted category's root, lower, stitch, run both."""
    torch.manual_seed(8)
    hgraph = cases.hetero_graph(device=dev)
    kwargs = cases.hetero_kwargs(hgraph, device=dev)
    model = models.RGCNModel(hgraph, 16, 16, 4).to(dev)
    dataflow = xgnn_h.Module2IR().transform(model, kwargs)["paper"]
    dataflow_1 = xgnn_h.Optimizer().lower(dataflow, kwargs)
    dataflow_2 = xgnn_h.Stitcher().transform(dataflow_1, kwargs)
    executor = xgnn_h.Executor()
    executor.eval()
    y_1 = executor.run(dataflow_1, kwargs)
    y_2 = executor.run(dataflow_2, kwargs)
    assert_close(y_2, y_1)
    # training mode: dropout is live, two runs differ
    executor.train()
    assert not torch.equal(executor.run(dataflow_2, kwargs), executor.run(dataflow_2, kwargs))


def test_embedding_of_all_ids_in_order_is_the_table(dev, monkeypatch):
    """Node ids 0..n-1 in order: the executor hands on the table instead of gathering it, with
    the same outputs and parameter gradients, bit for bit, as the lookup; ids in another order,
    or changed in place after the first run, take the lookup."""
    torch.manual_seed(11)
    hgraph = cases.hetero_graph(device=dev)
    kwargs = cases.hetero_kwargs(hgraph, device=dev)
    model = models.RGCNModel(hgraph, 16, 16, 4).to(dev)
    lowered = xgnn_h.Optimizer().lower(xgnn_h.Module2IR().transform(model, kwargs), kwargs)
    weights = {nty: torch.randn(num, 4, device=dev) for nty, num in hgraph.nty2num.items()}
    params = list(model.parameters())
    taken = []
    whole_table = xgnn_h.Executor._whole_table

    def counting(self, node, v):
        res = whole_table(self, node, v)
        taken.append(res is not None)
        return res

    monkeypatch.setattr(xgnn_h.Executor, "_whole_table", counting)
    short = _run_with_grads(lowered, kwargs, params, weights)
    assert taken and all(taken)
    monkeypatch.setattr(xgnn_h.Executor, "_whole_table", lambda self, node, v: None)
    _compare(short, _run_with_grads(lowered, kwargs, params, weights), rtol=0, atol=0)

    # one executor, ids reversed in place between two runs: the second run looks them up
    monkeypatch.setattr(xgnn_h.Executor, "_whole_table", counting)
    executor = xgnn_h.Executor()
    executor.eval()
    first = executor.run(lowered, kwargs)
    for ids in kwargs["xs"].values():
        ids.copy_(ids.flip(0))
    del taken[:]
    second = executor.run(lowered, kwargs)
    assert taken and not any(taken)
    want = xgnn_h.Executor()
    want.eval()
    monkeypatch.setattr(xgnn_h.Executor, "_whole_table", lambda self, node, v: None)
    for nty, got in second.items():
        assert torch.equal(got, want.run(lowered, kwargs)[nty])
    assert any(not torch.equal(first[nty], second[nty]) for nty in first)
