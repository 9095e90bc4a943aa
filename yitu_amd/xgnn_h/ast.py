"""Model -> dataflow graph (the role of xgnn_h/ast.py). The model is called
once on symbolic tensors; the graph is complete when the call returns, so there
is no backward walk over recorded calls (ast.py:11-180)."""
import torch
from torch import nn

from . import ir, mp
from .trace import Tracer


class Module2IR:
    def transform(self, model: nn.Module, kwargs: dict) -> ir.Dataflow:
        """Runs ``model(**kwargs)`` with every tensor replaced by a placeholder.
        Tensor arguments are named after their keyword (``xs.paper`` for the entry
        ``paper`` of a dict argument ``xs``), graphs ``graph`` or ``hgraph.<index of
        the relation>``; ``Executor.run`` resolves the same names against the
        arguments it is given. Returns the root node, or a dict of roots when the
        model returns a dict."""
        graphs = []

        def symbolic(value, name):
            if isinstance(value, torch.Tensor):
                return Tracer.placeholder(value, name)
            if isinstance(value, dict):
                return {k: symbolic(v, "%s.%s" % (name, k)) for k, v in value.items()}
            if isinstance(value, (list, tuple)):
                return [symbolic(v, "%s.%d" % (name, i)) for i, v in enumerate(value)]
            if isinstance(value, mp.Graph):
                value._placeholder = ir.Node("graph", size=value.blk.size, name=name)
                graphs.append(value)
                return value
            if isinstance(value, mp.HeteroGraph):
                for rel, g in value.hetero_graph.items():
                    symbolic(g, "%s.%d" % (name, value.rel2idx[rel]))
                return value
            raise NotImplementedError("argument %r of type %s" % (name, type(value).__name__))

        traced = {k: symbolic(v, k) for k, v in kwargs.items()}
        try:
            output = model(**traced)
        finally:
            for g in graphs:  # the stores hold symbolic tensors: drop them
                g._placeholder = None
                g.clear()
        if isinstance(output, dict):
            return {k: self._root(v) for k, v in output.items()}
        return self._root(output)

    @staticmethod
    def _root(value):
        if not isinstance(value, Tracer):
            raise NotImplementedError("the model must return traced tensors")
        return value.node
