"""Capture -> lower -> stitch of models written against the message-passing front
end (the reference's xgnn_h pipeline: ast.py, optimizer.py, stitcher.py, executor.py).
Everything here runs without a GPU: tracing is symbolic, and a dataflow that has not
been lowered executes from the definitions of the message functions, which this file
pins against dense algebra (the method of the reference's test_kernel.py:133-151 and
test_allclose.py:24-30)."""
import io

import pytest
import torch
from torch import nn

import pipeline_cases as cases
from helpers import assert_close
from yitu_amd import xgnn_h
from yitu_amd.xgnn_h import ir, models, mp


def test_message_functions_equal_dense_masked_attention():
    """u_add_v -> LeakyReLU -> edge_softmax -> u_mul_e -> aggregate_sum on real tensors
    == softmax over the neighbours of a dense masked score matrix, per head."""
    torch.manual_seed(0)
    g = cases.homo_graph()
    n, h, f = g.num_dst_nodes(), 3, 5
    q, k, x = torch.randn(n, h), torch.randn(n, h), torch.randn(n, h, f)
    g.src_node["q"], g.dst_node["k"], g.src_node["u"] = q, k, x
    g.message_func(mp.Fn.u_add_v("k", "q", "e"))
    g.edge["c"] = nn.functional.leaky_relu(g.edge["e"], 0.2)
    g.message_func(mp.Fn.edge_softmax("c", "a"))
    g.message_func(mp.Fn.u_mul_e("u", "a", "m"))
    g.reduce_func(mp.Fn.aggregate_sum("m", "v"))
    adj = cases.dense_adjacency(g.blk)
    score = nn.functional.leaky_relu(q[:, None, :] + k[None, :, :], 0.2)       # [dst, src, h]
    score = torch.where(adj[:, :, None] > 0, score, torch.full_like(score, -1e38))
    attn = torch.softmax(score, dim=1) * adj[:, :, None]
    want = torch.einsum("dsh,shf->dhf", attn, x)
    assert_close(g.dst_node["v"], want)
    # a row without edges aggregates to zero; attention rows sum to one elsewhere
    assert torch.all(g.dst_node["v"][5] == 0)
    rows, _, _ = mp.edge_endpoints(g.blk)
    sums = torch.zeros(n, h).index_add_(0, rows, g.edge["a"])
    assert_close(sums[adj.sum(1) > 0], torch.ones_like(sums[adj.sum(1) > 0]))


def test_gcn_model_eager_equals_dense_right_norm():
    """GCN layer on real tensors == D_in^-1 A (X W^T + b) (test_allclose.py:24-30)."""
    torch.manual_seed(1)
    g = cases.homo_graph()
    layer = models.GCNLayer(7, 4)
    x = torch.randn(g.num_src_nodes(), 7)
    got = layer(g, g.right_norm(), x)
    adj = cases.dense_adjacency(g.blk)
    want = g.right_norm() * (adj @ layer.fc(x))
    assert_close(got, want)


@pytest.mark.parametrize("which", ["gcn", "gat"])
def test_captured_dataflow_replays_the_model(which):
    torch.manual_seed(2)
    g = cases.homo_graph()
    x = torch.randn(g.num_src_nodes(), 9)
    if which == "gcn":
        model, kwargs = models.GCNModel(9, 6, 3), {"graph": g, "x": x, "norm": g.right_norm()}
    else:
        model, kwargs = models.GATModel(9, 6, 3, n_heads=2), {"graph": g, "x": x}
    model.eval()
    dataflow = xgnn_h.Module2IR().transform(model, kwargs)
    assert isinstance(dataflow, ir.Node) and dataflow.size == [g.num_dst_nodes(), 3]
    assert not g.src_node and not g.edge and not g.dst_node  # the trace leaves nothing behind
    executor = xgnn_h.Executor()
    with pytest.raises(RuntimeError):
        executor.run(dataflow, kwargs)  # dropout needs train() / eval()
    executor.eval()
    got = executor.run(dataflow, kwargs)
    assert_close(got, model(**kwargs), rtol=0, atol=0)
    # parameters are held by reference: an update is seen without tracing again
    with torch.no_grad():
        for p in model.parameters():
            p.mul_(1.5)
    assert_close(executor.run(dataflow, kwargs), model(**kwargs), rtol=0, atol=0)


def test_lowering_gat_patterns_and_options():
    g = cases.homo_graph()
    model = models.GATModel(9, 6, 3, n_heads=2)
    kwargs = {"graph": g, "x": torch.randn(g.num_src_nodes(), 9)}
    dataflow = xgnn_h.Module2IR().transform(model, kwargs)
    before = cases.ops_of(dataflow)
    assert before["edge.u_add_v"] == 2 and before["edge.edge_softmax"] == 2
    assert before["edge.u_mul_e"] == 2 and before["vert.aggregate_sum"] == 2
    assert before["linear"] == 6

    full = cases.ops_of(xgnn_h.Optimizer().lower(dataflow, kwargs))
    assert full["gat"] == 2 and full["bundle"] == 2 and full["select"] == 4
    assert full["linear"] == 2 and full["spmm"] == 0 and full["sddmm"] == 0
    assert not any(k.startswith(("edge", "vert")) for k in full)
    # the mean over heads that follows each attention is taken inside the fused op
    lowered = xgnn_h.Optimizer().lower(dataflow, kwargs)
    assert all(n.attrs.get("head_mean") for n in ir.walk(lowered) if n.op == "gat")
    assert not any(n.op == "call" and n.fn_name() == "mean" for n in ir.walk(lowered))
    assert lowered.op == "gat" and lowered.size == [g.num_dst_nodes(), 3]

    plain = cases.ops_of(xgnn_h.Optimizer(fuse_gat=False, bundle_gemm=False).lower(dataflow, kwargs))
    assert plain["sddmm"] == 2 and plain["spmm"] == 2 and plain["gat"] == 0
    assert plain["bundle"] == 0 and plain["linear"] == 6
    # lowering rebuilds the graph: the captured dataflow is unchanged, attributes included
    assert cases.ops_of(dataflow) == before
    assert all(set(n.attrs) <= {"fn", "args", "kwargs", "weight", "bias", "p", "width", "dtype"}
               for n in ir.walk(dataflow))


def test_lowering_leaves_other_slopes_and_shared_attention_alone():
    g = cases.homo_graph()

    class OtherSlope(models.GATLayer):
        def __init__(self):
            super().__init__(9, 4, 2)
            self.leaky_relu = nn.LeakyReLU(0.1)

    kwargs = {"graph": g, "x": torch.randn(g.num_src_nodes(), 9)}
    low = xgnn_h.Optimizer().lower(xgnn_h.Module2IR().transform(OtherSlope(), kwargs), kwargs)
    ops = cases.ops_of(low)
    # the kernels implement slope 0.2 only: the softmax stays a message function,
    # the aggregation still becomes an edge-weighted spmm
    assert ops["sddmm"] == 0 and ops["gat"] == 0 and ops["edge.edge_softmax"] == 1
    assert ops["spmm"] == 1 and "e" in [n for n in ir.walk(low) if n.op == "spmm"][0].inputs

    class ReturnsAttention(models.GATLayer):
        def forward(self, graph, x):
            out = super().forward(graph, x)
            return {"out": out, "attn": graph.edge["attn"]}

    low = xgnn_h.Optimizer().lower(
        xgnn_h.Module2IR().transform(ReturnsAttention(9, 4, 2), kwargs), kwargs)
    ops = cases.ops_of(low)
    assert ops["gat"] == 0 and ops["sddmm"] == 1 and ops["spmm"] == 1  # attention has two readers
    assert low["attn"].op == "sddmm"


def test_gcn_lowering():
    g = cases.homo_graph()
    kwargs = {"graph": g, "x": torch.randn(g.num_src_nodes(), 9), "norm": g.right_norm()}
    low = xgnn_h.Optimizer().lower(xgnn_h.Module2IR().transform(models.GCNModel(9, 6, 3), kwargs),
                                   kwargs)
    ops = cases.ops_of(low)
    assert ops["spmm"] == 2 and not any(k.startswith(("edge", "vert")) for k in ops)
    assert all("e" not in n.inputs for n in ir.walk(low) if n.op == "spmm")


def test_hetero_capture_names_relations_and_inputs():
    hgraph = cases.hetero_graph()
    kwargs = cases.hetero_kwargs(hgraph)
    model = models.RGCNModel(hgraph, 8, 8, 4)
    dataflow = xgnn_h.Module2IR().transform(model, kwargs)
    assert set(dataflow) == {"paper", "author", "venue"}
    names = {n.name for n in ir.walk(dataflow) if n.op in ("input", "graph")}
    assert "xs.paper" in names and "hgraph.0" in names
    assert "norms.%s" % str(cases.RELATIONS[2]) in names
    model.eval()
    executor = xgnn_h.Executor()
    executor.eval()
    got = executor.run(dataflow, kwargs)
    want = model(**kwargs)
    for nty in want:
        assert_close(got[nty], want[nty], rtol=0, atol=0)


@pytest.mark.parametrize("which", ["rgcn", "rgat"])
def test_stitching_replaces_sums_of_relations(which):
    hgraph = cases.hetero_graph()
    if which == "rgcn":
        kwargs = cases.hetero_kwargs(hgraph)
        model = models.RGCNModel(hgraph, 8, 8, 4)
    else:
        kwargs = cases.hetero_kwargs(hgraph, with_norms=False)
        model = models.RGATModel(hgraph, 8, 8, 4, n_heads=2)
    root = xgnn_h.Module2IR().transform(model, kwargs)["paper"]
    low = xgnn_h.Optimizer().lower(root, kwargs)
    n_rel = len(cases.RELATIONS)
    per_layer_core = "spmm" if which == "rgcn" else "gat"
    assert cases.ops_of(low)[per_layer_core] == n_rel + 4  # layer 1: all relations; layer 2: into paper
    stitched = xgnn_h.Stitcher().transform(low, kwargs)
    ops = cases.ops_of(stitched)
    # layer 2 reads all three types of layer 1: one stitched term per destination type
    # with several relations (paper: 4 -> 1, author: 2 -> 1), venue keeps its single one
    assert ops["spmm"] + ops["gat"] == 1 + 3
    if which == "rgat":
        # without the fused op the stitched terms keep the two-op form
        plain = xgnn_h.Optimizer(fuse_gat=False).lower(root, kwargs)
        two_op = cases.ops_of(xgnn_h.Stitcher().transform(plain, dict(kwargs)))
        assert two_op["gat"] == 0 and two_op["sddmm"] == two_op["spmm"] == 1 + 3
    if which == "rgcn":
        # the relations' Linears feed nothing else: one typed Linear per stitched term
        # writes the feature rows, nothing is concatenated
        assert ops["typed_linear"] == 3 and ops["concat"] == 0
        assert ops["edge_values"] == 3 and ops["sddmm"] == 0
    else:
        # the transformed features are also read by the projections: they stay as they are
        assert ops["concat"] >= 3 and ops["typed_linear"] == 0
        # the relations ran the fused attention op, so do the stitched terms (one query
        # block per relation)
        assert ops["sddmm"] == 0 and ops["stack"] == 3 and ops["gat"] == 1 + 3
    new = kwargs["stitch"]
    assert isinstance(new, mp.HeteroGraph) and len(new.hetero_graph) == 2
    (sty, ety, dty), g = next(iter(new))
    assert dty in ("paper", "author") and "-->" in sty and "-->" in ety
    # every stitched block is stitch_csr of its relations, in the order of its name
    for (sty, ety, dty), g in new:
        rels = list(zip(sty.split("-->"), ety.split("-->")))
        want = xgnn_h.block.stitch_csr([hgraph.hetero_graph[s, e, dty].blk for s, e in rels])
        assert torch.equal(g.blk.adj_sparse[0], want.adj_sparse[0])
        assert torch.equal(g.blk.adj_sparse[1], want.adj_sparse[1])
    # the lowered graph is left as it was
    assert cases.ops_of(low)[per_layer_core] == n_rel + 4


def test_stitcher_bin_limits():
    hgraph = cases.hetero_graph()
    kwargs = cases.hetero_kwargs(hgraph)
    low = xgnn_h.Optimizer().lower(
        xgnn_h.Module2IR().transform(models.RGCNModel(hgraph, 8, 8, 4), kwargs)["paper"], kwargs)
    two = xgnn_h.Stitcher(max_blocks=2).transform(low, dict(kwargs))
    # paper's four relations need two bins in each of the two layers; author's two
    # (layer 1 only: the root is the paper output) fit one
    sizes = sorted(len(n.inputs) - 1 for n in ir.walk(two) if n.op == "edge_values")
    assert sizes == [2, 2, 2, 2, 2]


def test_edge_values_follow_the_stitched_edge_order():
    hgraph = cases.hetero_graph()
    rels = [cases.RELATIONS[0], cases.RELATIONS[2], cases.RELATIONS[3]]
    blocks = [hgraph.hetero_graph[r].blk for r in rels]
    st = xgnn_h.block.stitch_csr(blocks)
    norms = [b.right_norm for b in blocks]
    node = ir.Node("edge_values", {"g": ir.Node("graph"), "0": ir.Node("input"),
                                   "1": ir.Node("input"), "2": ir.Node("input")})
    got = xgnn_h.Executor()._eval(node, {"g": st, "0": norms[0], "1": norms[1], "2": norms[2]}, {})
    indptr, indices = st.adj_sparse
    for r in range(st.size[0]):
        for i in range(int(indptr[r]), int(indptr[r + 1])):
            bid = int(indices[i]) >> 24
            assert float(got[i, 0]) == float(norms[bid][r, 0])


def test_printer_lists_nodes_in_evaluation_order():
    g = cases.homo_graph()
    kwargs = {"graph": g, "x": torch.randn(g.num_src_nodes(), 9), "norm": g.right_norm()}
    low = xgnn_h.Optimizer().lower(xgnn_h.Module2IR().transform(models.GCNLayer(9, 4), kwargs), kwargs)
    buf = io.StringIO()
    xgnn_h.Printer().dump(low, file=buf)
    n = g.num_dst_nodes()
    assert buf.getvalue().splitlines() == [
        "%%norm: [%d, 1] = input()" % n,
        "%%graph: [%d, %d] = graph()" % (n, n),
        "%%x: [%d, 9] = input()" % n,
        "%%0: [%d, 4] = linear(x: %%x)" % n,
        "%%1: [%d, 1, 4] = call.view(0: %%0)" % n,
        "%%2: [%d, 1, 4] = spmm(g: %%graph, x: %%1)" % n,
        "%%3: [%d, 4] = call.squeeze(0: %%2)" % n,
        "%%4: [%d, 4] = call.multiply(0: %%norm, 1: %%3)" % n,
    ]


def test_whole_embedding_table_is_aliased_only_under_autograd():
    """All ids in order make an embedding lookup the table itself. The alias is handed out
    only where an in-place write to it would raise (gradients on, a table that takes one);
    under no_grad and for a frozen table the lookup copies, so nothing downstream can write
    into the parameter."""
    import torch.nn.functional as F
    hgraph = cases.hetero_graph()
    kwargs = cases.hetero_kwargs(hgraph)
    model = models.RGCNModel(hgraph, 8, 8, 4)
    dataflow = xgnn_h.Module2IR().transform(model, kwargs)
    nodes = [n for n in ir.walk(dataflow) if n.op == "call" and n.attrs["fn"] is F.embedding]
    assert nodes
    node = nodes[0]
    executor = xgnn_h.Executor()
    table = torch.nn.Parameter(torch.randn(6, 3))
    ids = torch.arange(6)
    node_like = type("N", (), {"attrs": {"args": (ids, table), "kwargs": {}}})()
    executor.train()
    assert executor._whole_table(node_like, {}).data_ptr() == table.data_ptr()
    with torch.no_grad():
        assert executor._whole_table(node_like, {}) is None
    executor.eval()  # no dropout; gradients still flow, so autograd still guards the alias
    assert executor._whole_table(node_like, {}) is not None
    with pytest.raises(RuntimeError):
        executor._whole_table(node_like, {}).add_(1.0)
    table.requires_grad_(False)
    assert executor._whole_table(node_like, {}) is None
    table.requires_grad_(True)
    shuffled = type("N", (), {"attrs": {"args": (ids.flip(0), table), "kwargs": {}}})()
    assert executor._whole_table(shuffled, {}) is None
    executor.forget_tables()
    assert not executor._whole_tables


@pytest.mark.parametrize("which", ["rgcn", "rgat"])
def test_grouped_linears_equal_one_linear_at_a_time(which):
    """The executor runs the Linears of one depth and one shape as one grouped node
    (``Optimizer.group_linears``): same outputs and parameter gradients as one Linear at a
    time, and the per-relation Linears of a layer do end up in few groups."""
    hgraph = cases.hetero_graph()
    kwargs = cases.hetero_kwargs(hgraph, with_norms=which == "rgcn")
    torch.manual_seed(3)
    model = models.RGCNModel(hgraph, 8, 8, 4) if which == "rgcn" else \
        models.RGATModel(hgraph, 8, 8, 4, n_heads=2)
    model.eval()
    dataflow = xgnn_h.Module2IR().transform(model, kwargs)
    grouped = xgnn_h.Optimizer.group_linears(dataflow)
    n_linear = sum(1 for n in ir.walk(dataflow) if n.op == "linear")
    typed = [n for n in ir.walk(grouped) if n.op == "typed_linear"]
    left = sum(1 for n in ir.walk(grouped) if n.op == "linear")
    assert typed and sum(len(t.inputs) for t in typed) + left == n_linear
    assert len(typed) <= 8 and left <= 2  # a handful of launches for a dozen relations
    for t in typed:
        assert sorted(t.inputs) == sorted(str(i) for i in range(len(t.attrs["weights"])))
        assert sum(t.attrs["split"]) == t.size[0]
    params = list(model.parameters())
    results = []
    for flag in (False, True):
        for p in params:
            p.grad = None
        executor = xgnn_h.Executor(group_linears=flag)
        executor.eval()
        out = executor.run(dataflow, kwargs)
        sum((v * (i + 1.0)).sum() for i, v in enumerate(out.values())).backward()
        results.append(({k: v.detach().clone() for k, v in out.items()},
                        [None if p.grad is None else p.grad.clone() for p in params]))
    (out_a, grads_a), (out_b, grads_b) = results
    for k in out_a:
        assert_close(out_b[k], out_a[k], rtol=1e-6, atol=1e-6)
    for ga, gb in zip(grads_a, grads_b):
        assert (ga is None) == (gb is None)
        if ga is not None:
            assert_close(gb, ga, rtol=1e-5, atol=1e-6)
