"""Symbolic tensors for capturing a model's dataflow (the role of
xgnn_h/trace.py). The reference's ``Tracer`` is a real tensor that remembers
the last function applied to it and is walked backwards afterwards
(trace.py:4-39, ast.py:11-180). This one carries no data: it wraps a ``meta``
tensor for shape inference, and every torch function applied to it appends a
node to the dataflow graph right away, so capture costs no device work and is
not limited to a fixed list of functions.
"""
import torch
from torch.nn import functional as F

from . import ir


class Tracer(torch.Tensor):
    """A meta tensor with the dataflow node that produces it in ``.node``."""

    @staticmethod
    def wrap(meta: torch.Tensor, node: ir.Node) -> "Tracer":
        assert meta.device.type == "meta"
        t = torch.Tensor._make_subclass(Tracer, meta, False)
        t.node = node
        return t

    @staticmethod
    def placeholder(like: torch.Tensor, name: str) -> "Tracer":
        meta = torch.empty(like.shape, dtype=like.dtype, device="meta")
        return Tracer.wrap(meta, ir.Node("input", size=like.shape, name=name,
                                         attrs={"dtype": like.dtype}))

    def __repr__(self):
        return "Tracer(%r)" % (self.node,)

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        inputs = {}

        def template(v):
            # traced tensors become slots, real tensors (parameters) stay by reference
            if isinstance(v, Tracer):
                key = str(len(inputs))
                inputs[key] = v.node
                return ir.Slot(key)
            if isinstance(v, (list, tuple)):
                return type(v)(template(i) for i in v)
            if isinstance(v, dict):
                return {k: template(i) for k, i in v.items()}
            return v

        def to_meta(v):
            if isinstance(v, Tracer):
                return v.as_subclass(torch.Tensor)
            if isinstance(v, torch.Tensor):
                return torch.empty(v.shape, dtype=v.dtype, device="meta")
            if isinstance(v, (list, tuple)):
                return type(v)(to_meta(i) for i in v)
            if isinstance(v, dict):
                return {k: to_meta(i) for k, i in v.items()}
            return v

        with torch._C.DisableTorchFunctionSubclass():
            out = func(*to_meta(args), **to_meta(kwargs))
        if not isinstance(out, (torch.Tensor, tuple, list)):
            return out  # sizes, dtypes, booleans: plain Python values
        if isinstance(out, (tuple, list)) and not all(isinstance(o, torch.Tensor) for o in out):
            return out
        t_args, t_kwargs = template(args), template(kwargs)
        node = cls._structured(func, args, kwargs, inputs)
        if node is None:
            node = ir.Node("call", inputs, {"fn": func, "args": t_args, "kwargs": t_kwargs})
        if isinstance(out, torch.Tensor):
            node.size = list(out.shape)
            return Tracer.wrap(out, node)
        items = []
        for i, o in enumerate(out):
            items.append(Tracer.wrap(o, ir.Node("select", {"x": node}, {"index": i}, o.shape)))
        return type(out)(items)

    @staticmethod
    def _structured(func, args, kwargs, inputs):
        """Nodes the optimizer matches on get a fixed shape instead of an argument template."""
        def bind(names):
            bound = dict(zip(names, args))
            bound.update(kwargs)
            return bound

        if func is F.linear:
            b = bind(("input", "weight", "bias"))
            if isinstance(b["input"], Tracer) and not isinstance(b["weight"], Tracer) \
                    and not isinstance(b.get("bias"), Tracer):
                return ir.Node("linear", {"x": b["input"].node},
                               {"weight": b["weight"], "bias": b.get("bias")})
        if func is F.dropout:
            b = bind(("input", "p", "training", "inplace"))
            if isinstance(b["input"], Tracer):
                return ir.Node("dropout", {"x": b["input"].node}, {"p": b.get("p", 0.5)})
        return None
