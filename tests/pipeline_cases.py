"""Small seeded graphs and models shared by the capture / lower / stitch tests."""
import torch

from helpers import random_csr
from yitu_amd import xgnn_h
from yitu_amd.xgnn_h import layers, models, mp

NTYPES = {"paper": 60, "author": 45, "venue": 12}
# four relations reach "paper" (three of them with norms of their own), two reach "author"
RELATIONS = [("author", "writes", "paper"), ("paper", "cites", "paper"),
             ("venue", "publishes", "paper"), ("author", "reviews", "paper"),
             ("paper", "written_by", "author"), ("venue", "invites", "author"),
             ("paper", "appears_in", "venue")]


def homo_graph(n=48, seed=3, device=None):
    ip, ix = random_csr(n, n, 0.12, seed, empty_rows=(5,), hub_rows=(2,), hub_degree=n - 3)
    blk = xgnn_h.Block([n, n], [ip, ix])
    if device is not None:
        blk = blk.to(device)
    blk.right_norm = layers.right_norm(blk)
    return mp.Graph(blk)


def hetero_graph(seed=11, device=None):
    blocks = {}
    for i, (s, e, d) in enumerate(RELATIONS):
        ip, ix = random_csr(NTYPES[d], NTYPES[s], 0.15, seed + i, empty_rows=(i,))
        blk = xgnn_h.Block([NTYPES[d], NTYPES[s]], [ip, ix])
        if device is not None:
            blk = blk.to(device)
        blk.right_norm = layers.right_norm(blk)
        blocks[(s, e, d)] = blk
    return mp.HeteroGraph.from_blocks(NTYPES, blocks, device=device)


def hetero_kwargs(hgraph, device=None, with_norms=True):
    kwargs = {"hgraph": hgraph,
              "xs": {nty: torch.arange(num, dtype=torch.int64, device=device)
                     for nty, num in hgraph.nty2num.items()}}
    if with_norms:
        kwargs["norms"] = {str(rel): g.right_norm() for rel, g in hgraph.hetero_graph.items()}
    return kwargs


def dense_adjacency(blk):
    indptr, indices = blk.adj_sparse
    rows = torch.repeat_interleave(torch.arange(blk.size[0], device=indptr.device),
                                   (indptr[1:] - indptr[:-1]).long())
    a = torch.zeros(blk.size[0], blk.size[1], device=indptr.device)
    a[rows, (indices.long() & 0xFFFFFF)] = 1.0
    return a


def ops_of(dataflow):
    from collections import Counter
    return Counter(n.op + ("." + n.fn_name() if n.op in ("edge", "vert") else "")
                   for n in xgnn_h.ir.walk(dataflow))
