"""Relation stitching for heterogeneous models (the role of
xgnn_h/stitcher.py). A heterogeneous layer sums, per destination type, one
term per relation:

    GCN  norm_r * squeeze(spmm(g_r, x_r))                    (model.py:7-30)
    GAT  mean_heads(spmm(g_r, sddmm(g_r, q_r, k_r), x_r))    (model.py:61-106)

Terms of the same shape are replaced by one term over the row-wise
concatenation of their blocks (``block.stitch_csr``): sources concatenated,
queries stacked per block (the softmax stays per relation through the block id
in the column word), and for GCN the per-relation row scale carried as a
per-edge weight, so the stitched term equals the sum of the terms it replaces.
The reference groups the relations of a destination type into two bins
(stitcher.py:7-38, 186-206) and drops the row scale when it rewrites GCN terms
(stitcher.py:281-283); here the bins are as few as the 16-block and 2^24-column
limits of a packed CSR allow, and the scale is kept.
"""
from typing import Dict, List, Optional

import torch

from . import block, ir, mp

_ADD = ("add", "__add__", "__radd__")
_MUL = ("multiply", "mul", "__mul__", "__rmul__")


def _call_operands(node: ir.Node, names) -> Optional[List[ir.Node]]:
    """Operand nodes of a ``call`` to one of ``names`` whose positional arguments
    are all traced tensors, else None."""
    if node.op != "call" or node.fn_name() not in names:
        return None
    args = node.attrs["args"]
    if not all(isinstance(a, ir.Slot) for a in args):
        return None
    return [node.inputs[a.key] for a in args]


def _is_add(node: ir.Node) -> bool:
    ops = _call_operands(node, _ADD)
    return ops is not None and len(ops) == 2 and not node.attrs["kwargs"]


def _unary_dim1(node: ir.Node, names) -> Optional[ir.Node]:
    """Input of ``squeeze`` / ``mean`` over dim 1, else None."""
    ops = _call_operands(node, names)
    if ops is None or len(ops) != 1:
        return None
    kwargs = node.attrs["kwargs"]
    if kwargs.get("dim") != 1 or any(k not in ("dim",) for k in kwargs):
        return None
    return ops[0]


class _Term:
    """One relation's contribution to a sum, taken apart."""

    def __init__(self, root, scale, post, core, rel_index, hgraph_key):
        self.root, self.scale, self.post, self.core = root, scale, post, core
        self.rel_index, self.hgraph_key = rel_index, hgraph_key
        self.attention = core.op == "gat" or "e" in core.inputs
        self.mean_inside = core.op == "gat" and bool(core.attrs.get("head_mean"))

    def qkx(self):
        c = self.core
        if c.op == "gat":
            return c.inputs["q"], c.inputs["k"], c.inputs["x"]
        if "e" in c.inputs:
            return c.inputs["e"].inputs["q"], c.inputs["e"].inputs["k"], c.inputs["x"]
        return None, None, c.inputs["x"]

    def signature(self):
        x = self.core.inputs["x"]
        post = "mean" if self.mean_inside else (self.post.fn_name() if self.post else None)
        return (self.attention, self.scale is not None, post, tuple(x.size[1:]), self.hgraph_key)


def _match_term(node: ir.Node, kwargs: dict) -> Optional[_Term]:
    cur, scale = node, None
    ops = _call_operands(cur, _MUL)
    if ops is not None and len(ops) == 2:
        for a, b in (ops, ops[::-1]):
            if a.op == "input" and len(a.size) == 2 and a.size[1] == 1:
                scale, cur = a, b
                break
        else:
            return None
    post = None
    inner = _unary_dim1(cur, ("squeeze", "mean"))
    if inner is not None:
        post, cur = cur, inner
    if cur.op not in ("spmm", "gat"):
        return None
    g = cur.inputs["g"]
    key, _, idx = g.name.partition(".")
    if g.op != "graph" or not idx.isdigit() or not isinstance(kwargs.get(key), mp.HeteroGraph):
        return None
    if cur.op == "spmm" and "e" in cur.inputs:
        attn = cur.inputs["e"]
        if attn.op != "sddmm" or attn.inputs["g"] is not g or len(attn.inputs["q"].size) != 2:
            return None
    if scale is not None and scale.size[0] != g.size[0]:
        return None
    return _Term(node, scale, post, cur, int(idx), key)


class Stitcher:
    def __init__(self, max_blocks: int = 16, max_columns: int = 1 << 24):
        assert 2 <= max_blocks <= 16
        self.max_blocks = max_blocks
        self.max_columns = max_columns
        self._readers: Dict[int, int] = {}

    def _pack(self, terms: List[_Term], hgraph: mp.HeteroGraph) -> List[List[_Term]]:
        """First-fit decreasing by edge count into bins of at most ``max_blocks``
        blocks and ``max_columns`` columns."""
        def blk(t):
            return hgraph.hetero_graph[tuple(hgraph.idx2rel[t.rel_index])].blk
        bins: List[List[_Term]] = []
        for t in sorted(terms, key=lambda t: -blk(t).num_edges()):
            for b in bins:
                if len(b) < self.max_blocks and \
                        sum(blk(o).size[1] for o in b) + blk(t).size[1] <= self.max_columns:
                    b.append(t)
                    break
            else:
                bins.append([t])
        return bins

    def _concat_features(self, xs, n_rows: int) -> ir.Node:
        """The feature rows of the stitched block: the relations' features one below the
        other. Where each of them is ``view(linear(x_i))`` read by nobody else, the
        Linears become one ``typed_linear`` node that writes its products straight into
        the row ranges of one buffer (a grouped GEMM launch, no concatenation pass)."""
        tail = xs[0].size[1:]
        inner = []
        for x in xs:
            ops = _call_operands(x, ("view", "reshape")) if len(x.size) == 3 else None
            lin = ops[0] if ops is not None and len(ops) == 1 else None
            if lin is None or lin.op != "linear" or len(lin.size) != 2 or \
                    lin.size[1] != tail[0] * tail[1] or self._readers.get(id(lin), 0) != 1 or \
                    self._readers.get(id(x), 0) != 1 or len(lin.inputs["x"].size) != 2:
                inner = None
                break
            inner.append(lin)
        if not inner:
            return ir.Node("concat", {str(i): n for i, n in enumerate(xs)}, size=[n_rows] + tail)
        flat = ir.Node("typed_linear", {str(i): lin.inputs["x"] for i, lin in enumerate(inner)},
                       {"weights": [lin.attrs["weight"] for lin in inner],
                        "biases": [lin.attrs["bias"] for lin in inner]},
                       size=[n_rows, tail[0] * tail[1]])
        return ir.Node("call", {"0": flat},
                       {"fn": torch.Tensor.view, "args": (ir.Slot("0"), [-1] + tail), "kwargs": {}},
                       size=[n_rows] + tail)

    def _stitch_bin(self, terms: List[_Term], hgraph: mp.HeteroGraph,
                    stitched: mp.HeteroGraph) -> ir.Node:
        rels = [tuple(hgraph.idx2rel[t.rel_index]) for t in terms]
        blocks = [hgraph.hetero_graph[r].blk for r in rels]
        new_blk = block.stitch_csr(blocks)
        dty = rels[0][2]
        assert all(r[2] == dty for r in rels)
        new_sty = "-->".join(r[0] for r in rels)
        new_ety = "-->".join(r[1] for r in rels)
        stitched.nty2num[new_sty] = new_blk.size[1]
        stitched.add_relation(new_sty, new_ety, dty, new_blk)
        idx = stitched.rel2idx[new_sty, new_ety, dty]
        g = ir.Node("graph", size=new_blk.size, name="stitch.%d" % idx)
        qs, ks, xs = zip(*(t.qkx() for t in terms))
        x = self._concat_features(xs, new_blk.size[1])
        inputs = {"g": g, "x": x}
        n_edges = new_blk.num_edges()
        if terms[0].attention:
            q = ir.Node("stack", {str(i): n for i, n in enumerate(qs)},
                        size=[len(qs)] + qs[0].size)
            k = ir.Node("concat", {str(i): n for i, n in enumerate(ks)},
                        size=[new_blk.size[1]] + ks[0].size[1:])
            if all(t.core.op == "gat" for t in terms):
                # the relations ran the fused attention op: so does the stitched term, with
                # one query block per relation (and the mean over heads inside, if they had it)
                mean = terms[0].mean_inside
                size = [new_blk.size[0]] + (xs[0].size[2:] if mean else xs[0].size[1:])
                out = ir.Node("gat", {"g": g, "q": q, "k": k, "x": x}, {"head_mean": mean}, size)
                if not mean and terms[0].post is not None:
                    (slot,) = terms[0].post.inputs
                    out = terms[0].post.with_inputs({slot: out})
                return out
            inputs["e"] = ir.Node("sddmm", {"g": g, "q": q, "k": k}, size=[n_edges, ks[0].size[1]])
        elif terms[0].scale is not None:
            scales = {str(i): t.scale for i, t in enumerate(terms)}
            inputs["e"] = ir.Node("edge_values", dict(g=g, **scales), size=[n_edges, 1])
        out = ir.Node("spmm", inputs, size=[new_blk.size[0]] + xs[0].size[1:])
        post = terms[0].post
        if terms[0].mean_inside:  # the terms carried their mean over heads inside the fused op
            out = ir.Node("call", {"0": out}, {"fn": torch.mean, "args": (ir.Slot("0"),),
                                               "kwargs": {"dim": 1}},
                          size=[out.size[0]] + out.size[2:])
        elif post is not None:
            (slot,) = post.inputs
            out = post.with_inputs({slot: out})
        return out

    def transform(self, dataflow: ir.Dataflow, kwargs: dict) -> ir.Dataflow:
        """Rewrites every sum of per-relation terms in ``dataflow`` (lowered by
        ``Optimizer.lower``). The stitched blocks are stored as a ``HeteroGraph``
        under ``kwargs['stitch']``, where the executor looks up ``stitch.<index>``."""
        consumers: Dict[int, List[ir.Node]] = {}
        for node in ir.walk(dataflow):
            for child in node.inputs.values():
                consumers.setdefault(id(child), []).append(node)
        self._readers = {key: len(nodes) for key, nodes in consumers.items()}

        def inner_add(node):  # an add whose only reader is another add
            readers = consumers.get(id(node), [])
            return _is_add(node) and len(readers) == 1 and _is_add(readers[0])

        stitched = mp.HeteroGraph()
        for v in kwargs.values():
            if isinstance(v, mp.HeteroGraph):
                stitched.device = v.device
                stitched.nty2num = dict(v.nty2num)
        memo: Dict[int, ir.Node] = {}

        def leaves_of(node, out):
            for child in _call_operands(node, _ADD):
                if inner_add(child):
                    leaves_of(child, out)
                else:
                    out.append(child)
            return out

        def rebuild(node: ir.Node) -> ir.Node:
            if id(node) in memo:
                return memo[id(node)]
            if _is_add(node) and not inner_add(node):
                new = self._rebuild_sum(node, [rebuild(l) for l in leaves_of(node, [])],
                                        kwargs, stitched)
            else:
                ins = {k: rebuild(c) for k, c in node.inputs.items()}
                changed = any(ins[k] is not node.inputs[k] for k in ins)
                new = node.with_inputs(ins) if changed else node
            memo[id(node)] = new
            # a rebuilt node has the readers of the node it stands for
            self._readers.setdefault(id(new), self._readers.get(id(node), 0))
            return new

        if isinstance(dataflow, ir.Node):
            result = rebuild(dataflow)
        else:
            result = {k: rebuild(v) for k, v in dataflow.items()}
        kwargs["stitch"] = stitched
        return result

    def _rebuild_sum(self, add_node: ir.Node, leaves: List[ir.Node], kwargs: dict,
                     stitched: mp.HeteroGraph) -> ir.Node:
        groups: Dict[tuple, List[_Term]] = {}
        summands: List[ir.Node] = []
        for leaf in leaves:
            term = _match_term(leaf, kwargs)
            if term is None:
                summands.append(leaf)
            else:
                groups.setdefault(term.signature(), []).append(term)
        for terms in groups.values():
            hgraph = kwargs[terms[0].hgraph_key]
            for bin_ in self._pack(terms, hgraph):
                if len(bin_) == 1:
                    summands.append(bin_[0].root)
                else:
                    summands.append(self._stitch_bin(bin_, hgraph, stitched))
        total = summands[0]
        a, b = (s.key for s in add_node.attrs["args"])
        for s in summands[1:]:
            total = ir.Node("call", {a: total, b: s}, add_node.attrs, add_node.size)
        return total
