"""Dataflow graph of a traced model (the role of xgnn_h/ir.py).

The reference keeps one Python class per operator (ir.py:7-310). Here a node
is generic: an operator name, named inputs, attributes and the result size.
Any torch function the model calls becomes a ``call`` node that the executor
replays as-is, so the set of supported layers is not limited to a fixed list;
only the message-passing operators and what they are lowered to have names of
their own:

==============  ===========================================================
op              meaning (inputs)
==============  ===========================================================
``input``       tensor argument of the model, looked up by ``name``
``graph``       a ``Block`` argument (``name`` = ``kwarg`` or ``kwarg.idx``)
``call``        ``attrs['fn'](*args, **kwargs)`` with ``Slot`` markers
``linear``      ``F.linear(x, weight, bias)`` (x)
``dropout``     ``F.dropout(x, p, training)`` (x)
``edge``        message function ``attrs['fn']`` (g + operands) -> [E, H]
``vert``        reduce function ``attrs['fn']`` (g, e) -> [n_dst, H, F]
``sddmm``       LeakyReLU(q[row] + k[col]) softmax per row (g, q, k)
``spmm``        sum_e w[e,h] x[col_e,h,:] (g, x, optional e)
``gat``         spmm(g, sddmm(g, q, k), x) as one op (g, q, k, x)
``bundle``      two linears of one input as one GEMM launch (x) -> pair
``select``      item ``attrs['index']`` of a pair (x)
``concat``      ``torch.cat`` along dim 0 (inputs '0', '1', ...)
``stack``       ``torch.stack`` along dim 0
``edge_values`` per-edge weights of a stitched block from per-relation row
                scales (g, '0', '1', ...)
==============  ===========================================================
"""
from typing import Callable, Dict, Iterable, List, Union


class Slot:
    """Marks, inside the argument template of a ``call`` node, the position of
    the traced tensor held in ``inputs[key]``."""
    __slots__ = ("key",)

    def __init__(self, key: str):
        self.key = key

    def __repr__(self):
        return "Slot(%s)" % self.key


class Node:
    __slots__ = ("op", "inputs", "attrs", "size", "name")

    def __init__(self, op: str, inputs: Dict[str, "Node"] = None, attrs: dict = None,
                 size: Iterable[int] = None, name: str = ""):
        self.op = op
        self.inputs = dict(inputs or {})
        self.attrs = dict(attrs or {})
        self.size = list(size) if size is not None else None
        self.name = name

    def with_inputs(self, inputs: Dict[str, "Node"]) -> "Node":
        return Node(self.op, inputs, self.attrs, self.size, self.name)

    def fn_name(self) -> str:
        fn = self.attrs.get("fn")
        return fn if isinstance(fn, str) else getattr(fn, "__name__", str(fn))

    def __repr__(self):
        label = self.name or (self.fn_name() if "fn" in self.attrs else "")
        return "<%s %s %s>" % (self.op, label, self.size)


Dataflow = Union[Node, Dict[str, Node]]


def roots_of(dataflow: Dataflow) -> List[Node]:
    if isinstance(dataflow, Node):
        return [dataflow]
    if isinstance(dataflow, dict):
        return list(dataflow.values())
    raise NotImplementedError("a dataflow is a Node or a dict of Nodes")


def walk(dataflow: Dataflow) -> List[Node]:
    """Every node once, inputs before their consumers."""
    order, seen = [], set()
    stack = [(r, False) for r in reversed(roots_of(dataflow))]
    while stack:
        node, expanded = stack.pop()
        if expanded:
            order.append(node)
            continue
        if id(node) in seen:
            continue
        seen.add(id(node))
        stack.append((node, True))
        for child in reversed(list(node.inputs.values())):
            if id(child) not in seen:
                stack.append((child, False))
    return order


def use_counts(dataflow: Dataflow) -> Dict[int, int]:
    """id(node) -> number of (consumer, slot) pairs that read it; roots count once more."""
    uses: Dict[int, int] = {}
    for node in walk(dataflow):
        for child in node.inputs.values():
            uses[id(child)] = uses.get(id(child), 0) + 1
    for root in roots_of(dataflow):
        uses[id(root)] = uses.get(id(root), 0) + 1
    return uses


def rewrite(dataflow: Dataflow, rule: Callable[[Node, Node], Node]) -> Dataflow:
    """Rebuilds the graph bottom-up. ``rule(node, original)`` receives each node with
    its inputs already rewritten, and the node of the input graph it stands for (for
    facts gathered beforehand, such as use counts); it returns the node to use in its
    place (possibly the same one). Shared sub-graphs stay shared; the input graph is
    not modified."""
    done: Dict[int, Node] = {}
    for node in walk(dataflow):
        new_inputs = {k: done[id(v)] for k, v in node.inputs.items()}
        if any(new_inputs[k] is not node.inputs[k] for k in new_inputs):
            node_in = node.with_inputs(new_inputs)
        else:
            node_in = node
        done[id(node)] = rule(node_in, node)
    if isinstance(dataflow, Node):
        return done[id(dataflow)]
    return {k: done[id(v)] for k, v in dataflow.items()}
