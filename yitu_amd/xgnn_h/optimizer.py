"""Lowering of the message-passing operators to the sparse kernels (the role of
xgnn_h/optimizer.py):

* ``edge_softmax(leaky_relu(u_add_v(k, q)))``            -> ``sddmm(g, q, k)``
* ``aggregate_sum(copy_u(x))``                            -> ``spmm(g, x)``
* ``aggregate_sum(u_mul_e(x, e))``                        -> ``spmm(g, e, x)``
  (optimizer.py:10-87 matches the same three shapes)
* ``spmm(g, sddmm(g, q, k), x)`` with no other reader of the attention
  -> ``gat(g, q, k, x)``: the fused kernel, one pass per destination row
* the two ``linear`` nodes that produce q and k from one input
  -> one ``bundle`` GEMM launch (what ``_bundle_gemm``, optimizer.py:89-104,
  sets out to do and leaves empty)
"""
from torch.nn import functional as F

from . import ir

_SLOPE = 0.2  # the LeakyReLU slope the attention kernels implement (ops.cuh:1-3)


def _leaky_input(node: ir.Node):
    """The input of a ``leaky_relu`` call with the kernels' slope, else None."""
    if node.op != "call" or node.attrs["fn"] is not F.leaky_relu:
        return None
    args, kwargs = node.attrs["args"], node.attrs["kwargs"]
    slope = kwargs.get("negative_slope", args[1] if len(args) > 1 else 0.01)
    if abs(slope - _SLOPE) > 1e-12 or not isinstance(args[0], ir.Slot):
        return None
    return node.inputs[args[0].key]


class Optimizer:
    def __init__(self, fuse_gat: bool = True, bundle_gemm: bool = True):
        self.fuse_gat = fuse_gat
        self.bundle_gemm = bundle_gemm

    # -- message passing -> sddmm / spmm ------------------------------------
    @staticmethod
    def _lower_node(node: ir.Node, _original: ir.Node = None) -> ir.Node:
        if node.op == "edge" and node.attrs["fn"] == "edge_softmax":
            logits = _leaky_input(node.inputs["e"])
            if logits is not None and logits.op == "edge" and logits.attrs["fn"] == "u_add_v" \
                    and logits.inputs["g"] is node.inputs["g"]:
                return ir.Node("sddmm", {"g": node.inputs["g"], "q": logits.inputs["v"],
                                         "k": logits.inputs["u"]}, size=node.size)
        if node.op == "vert" and node.attrs["fn"] == "aggregate_sum":
            msg = node.inputs["e"]
            if msg.op == "edge" and msg.inputs["g"] is node.inputs["g"]:
                if msg.attrs["fn"] == "copy_u":
                    return ir.Node("spmm", {"g": node.inputs["g"], "x": msg.inputs["u"]},
                                   size=node.size)
                if msg.attrs["fn"] == "u_mul_e":
                    return ir.Node("spmm", {"g": node.inputs["g"], "e": msg.inputs["e"],
                                            "x": msg.inputs["u"]}, size=node.size)
        return node

    # -- spmm(sddmm) -> gat --------------------------------------------------
    @staticmethod
    def _fuse_gat(dataflow: ir.Dataflow) -> ir.Dataflow:
        uses = ir.use_counts(dataflow)
        attention_of = {}  # id(rewritten sddmm) -> readers of the sddmm it stands for

        def rule(node: ir.Node, original: ir.Node) -> ir.Node:
            if node.op == "sddmm":
                attention_of[id(node)] = uses.get(id(original), 0)
            attn = node.inputs.get("e") if node.op == "spmm" else None
            if attn is None or attn.op != "sddmm" or attn.inputs["g"] is not node.inputs["g"]:
                return node
            # the attention must have no other reader and one query block
            if attention_of.get(id(attn)) != 1 or len(attn.inputs["q"].size) != 2:
                return node
            return ir.Node("gat", {"g": node.inputs["g"], "q": attn.inputs["q"],
                                   "k": attn.inputs["k"], "x": node.inputs["x"]}, size=node.size)

        return Optimizer._fuse_head_mean(ir.rewrite(dataflow, rule))

    # -- mean(gat, dim=1) -> gat with the mean inside ------------------------
    @staticmethod
    def _fuse_head_mean(dataflow: ir.Dataflow) -> ir.Dataflow:
        uses = ir.use_counts(dataflow)
        sole_reader = set()  # ids of rewritten gat nodes whose original has one reader

        def rule(node: ir.Node, original: ir.Node) -> ir.Node:
            if node.op == "gat" and uses.get(id(original)) == 1:
                sole_reader.add(id(node))
            if node.op != "call" or node.fn_name() != "mean" or len(node.inputs) != 1:
                return node
            (inner,) = node.inputs.values()
            kwargs = node.attrs["kwargs"]
            if inner.op != "gat" or id(inner) not in sole_reader or kwargs.get("dim") != 1 or \
                    set(kwargs) != {"dim"} or len(node.attrs["args"]) != 1:
                return node
            return ir.Node("gat", inner.inputs, {"head_mean": True}, node.size)

        return ir.rewrite(dataflow, rule)

    # -- linear_q(h), linear_k(h) -> one launch ------------------------------
    @staticmethod
    def _bundle(dataflow: ir.Dataflow) -> ir.Dataflow:
        bundles = {}

        def rule(node: ir.Node, _original: ir.Node) -> ir.Node:
            if node.op not in ("sddmm", "gat"):
                return node
            q, k = node.inputs["q"], node.inputs["k"]
            if q.op != "linear" or k.op != "linear" or q is k or q.inputs["x"] is not k.inputs["x"]:
                return node
            wq, wk = q.attrs["weight"], k.attrs["weight"]
            if wq.shape != wk.shape or wq.stride() != wk.stride() or len(q.inputs["x"].size) != 2:
                return node
            key = (id(q), id(k))
            if key not in bundles:
                both = ir.Node("bundle", {"x": q.inputs["x"]},
                               {"weights": (wq, wk), "biases": (q.attrs["bias"], k.attrs["bias"])})
                bundles[key] = (ir.Node("select", {"x": both}, {"index": 0}, q.size),
                                ir.Node("select", {"x": both}, {"index": 1}, k.size))
            inputs = dict(node.inputs)
            inputs["q"], inputs["k"] = bundles[key]
            return node.with_inputs(inputs)

        return ir.rewrite(dataflow, rule)

    # -- the Linears of one depth and one shape -> one grouped launch ---------
    @staticmethod
    def group_linears(dataflow: ir.Dataflow, min_group: int = 2,
                      max_rows: int = 16384) -> ir.Dataflow:
        """A heterogeneous model applies one Linear per relation (model.py:137-171 over
        :25-29, :70-71): at the scale of the reference's own benchmark that is a hundred
        products of a few hundred rows, each a launch of its own forward and three more
        backward. Linears (and the two halves of a ``bundle``) that sit at the same depth of
        the dataflow cannot depend on each other; those of one weight shape become one
        ``typed_linear`` node, a grouped GEMM launch that writes all their outputs into one
        buffer, and every former Linear reads its rows back through one ``split`` (whose
        backward is one concatenation of the incoming gradients). The executor applies this
        to whatever dataflow it is given (lowered or stitched), once per dataflow. Only
        Linears over at most ``max_rows`` rows are joined: that is where launches dominate; on
        inputs of 10^5 rows a product fills the chip by itself and the concatenation of the
        gradients is a pass over memory that separate Linears do not make (the attention model
        at the fourth configuration's scale: 22.7 ms per step ungrouped, 26.1 ms grouped)."""
        depth = {}
        for node in ir.walk(dataflow):
            depth[id(node)] = 1 + max([depth[id(c)] for c in node.inputs.values()], default=0)
        # units: (key, original node, which weight of it)
        groups = {}
        for node in ir.walk(dataflow):
            if node.op == "linear":
                ws = [(node.attrs["weight"], node.attrs["bias"])]
            elif node.op == "bundle":
                ws = list(zip(node.attrs["weights"], node.attrs["biases"]))
            else:
                continue
            x = node.inputs["x"]
            if x.size is None or len(x.size) != 2 or any(w.dim() != 2 for w, _ in ws) or \
                    int(x.size[0]) > max_rows:
                continue
            for which, (w, _) in enumerate(ws):
                key = (depth[id(node)], node.op, which, tuple(w.shape))
                groups.setdefault(key, []).append(node)
        place = {}  # (id(original node), which) -> (typed node, position in it)
        for key, members in groups.items():
            if len(members) < min_group:
                continue
            which = key[2]
            sizes = [int(m.inputs["x"].size[0]) for m in members]
            pick = (lambda m: (m.attrs["weight"], m.attrs["bias"])) if key[1] == "linear" else \
                (lambda m: (m.attrs["weights"][which], m.attrs["biases"][which]))
            typed = ir.Node("typed_linear", {},
                            {"weights": [pick(m)[0] for m in members],
                             "biases": [pick(m)[1] for m in members], "split": sizes},
                            size=[sum(sizes), int(key[3][0])])
            for i, m in enumerate(members):
                place[(id(m), which)] = (typed, i)
        if not place:
            return dataflow

        def piece(typed, i, size):
            return ir.Node("select", {"x": typed}, {"index": i}, size)

        def rule(node: ir.Node, original: ir.Node) -> ir.Node:
            if original.op == "linear" and (id(original), 0) in place:
                typed, i = place[(id(original), 0)]
                typed.inputs[str(i)] = node.inputs["x"]
                return piece(typed, i, node.size)
            if original.op == "bundle":
                # register the (rewritten) input with both typed nodes; readers follow below
                for which in (0, 1):
                    if (id(original), which) in place:
                        typed, i = place[(id(original), which)]
                        typed.inputs[str(i)] = node.inputs["x"]
                return node
            if original.op == "select" and original.inputs["x"].op == "bundle":
                hit = place.get((id(original.inputs["x"]), original.attrs["index"]))
                if hit is not None:
                    return piece(hit[0], hit[1], node.size)
            return node

        return ir.rewrite(dataflow, rule)

    def lower(self, dataflow: ir.Dataflow, kwargs: dict = None) -> ir.Dataflow:
        dataflow = ir.rewrite(dataflow, self._lower_node)
        if self.fuse_gat:
            dataflow = self._fuse_gat(dataflow)
        if self.bundle_gemm:
            dataflow = self._bundle(dataflow)
        return dataflow
