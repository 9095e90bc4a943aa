"""What the two conv layers share: how the graph arguments of the module-1 ops
are read off the ``inputInfo`` carrier, and the weight initialisation."""
import math

import torch

# attribute names of the carrier, in the positional order the ops take them
# (YiTu_GNN.cpp:247-258); ``degrees`` is used by the GCN ops only
GRAPH_FIELDS = ("row_pointers", "column_index")
PARTITION_FIELDS = ("partPtr", "part2Node", "partSize", "dimWorker", "warpPerBlock")


def graph_arguments(info, *middle):
    """(row_pointers, column_index, *middle, partPtr, part2Node, partSize, dimWorker,
    warpPerBlock): the tail of every op's argument list. ``middle`` is the one
    argument that differs between the ops (the degree scale, or epsilon)."""
    return (tuple(getattr(info, f) for f in GRAPH_FIELDS) + tuple(middle) +
            tuple(getattr(info, f) for f in PARTITION_FIELDS))


class DenseWeight(torch.nn.Module):
    """A [input_dim, output_dim] parameter named ``weights`` drawn from
    U(-1/sqrt(output_dim), 1/sqrt(output_dim)) (GCNConv.py:58-66, GINConv.py:58-67)."""

    def __init__(self, input_dim, output_dim):
        super().__init__()
        # drawn, then redrawn by reset_parameters, like the reference: a seeded run
        # consumes the generator the same way
        self.weights = torch.nn.Parameter(torch.randn(input_dim, output_dim))
        self.reset_parameters()

    def reset_parameters(self):
        bound = 1.0 / math.sqrt(self.weights.size(1))
        with torch.no_grad():
            self.weights.uniform_(-bound, bound)
