"""Conv modules over the module-1 ops (YiTu_GNN/nn/__init__.py). Only the
single-GPU classes exist here: the reference swaps in a DGL message-passing
GraphConv when DGL_DIST_MODE is set (nn/__init__.py:3-6), which is outside the
sparse kernel path."""
from .GCNConv import GCNConv, GNNAFunction
from .GINConv import GINConv, GNNAFunction_GIN

__all__ = ["GCNConv", "GINConv", "GNNAFunction", "GNNAFunction_GIN"]
