"""Message-passing front end that model code is written against (the role of
xgnn_h/mp.py): ``Graph`` with ``src_node`` / ``dst_node`` / ``edge`` stores,
``message_func`` / ``reduce_func`` taking the ``Fn`` descriptors, and
``HeteroGraph`` as a dictionary of relations.

With traced tensors the functions append ``edge`` / ``vert`` nodes to the
dataflow graph (the reference returns zero-filled dummies of the right shape,
mp.py:7-31). With real tensors they compute the result directly from the
definitions below, which is also what the executor does for a dataflow that
has not been lowered; the reference cannot run either case.
"""
from typing import Dict, Tuple

import torch

from . import block, ir
from .trace import Tracer

COL_MASK = 0xFFFFFF  # low 24 bits of a packed column id (block.py:53)


class Fn:
    """Descriptors of the message / reduce functions (mp.py:34-75)."""

    @staticmethod
    def copy_u(u, e):
        return {"func": "copy_u", "u": u, "out": e}

    @staticmethod
    def u_add_v(u, v, e):
        return {"func": "u_add_v", "u": u, "v": v, "out": e}

    @staticmethod
    def u_mul_e(u, e, v):
        return {"func": "u_mul_e", "u": u, "e": e, "out": v}

    @staticmethod
    def edge_softmax(e1, e2):
        return {"func": "edge_softmax", "e": e1, "out": e2}

    @staticmethod
    def aggregate_sum(e, v):
        return {"func": "aggregate_sum", "e": e, "out": v}


# --------------------------------------------------------------------------- #
# definitions of the functions on real tensors
# --------------------------------------------------------------------------- #
def edge_endpoints(blk: block.Block) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(destination row, source column, block id) of every edge of a packed CSR."""
    indptr, indices = blk.adj_sparse
    deg = (indptr[1:] - indptr[:-1]).to(torch.int64)
    rows = torch.repeat_interleave(torch.arange(deg.numel(), device=indptr.device), deg)
    idx = indices.to(torch.int64)
    return rows, idx & COL_MASK, idx >> 24


def apply_edge(fn: str, blk: block.Block, **t) -> torch.Tensor:
    rows, cols, bids = edge_endpoints(blk)
    if fn == "u_add_v":  # u: per source [n_src, H]; v: per destination [n_dst, H] or [n_bid, n_dst, H]
        v = t["v"][rows] if t["v"].dim() == 2 else t["v"][bids, rows]
        return t["u"][cols] + v
    if fn == "copy_u":   # [n_src, H, F] -> [E, H, F]
        return t["u"][cols]
    if fn == "u_mul_e":  # [n_src, H, F] x [E, H] -> [E, H, F]
        return t["u"][cols] * t["e"].unsqueeze(-1)
    if fn == "edge_softmax":  # over the edges of a destination row (and block id), per head
        e = t["e"]
        n_dst = blk.size[0]
        seg = rows + bids * n_dst
        n_seg = n_dst * (int(bids.max()) + 1 if bids.numel() else 1)
        top = torch.full((n_seg, e.size(1)), float("-inf"), dtype=e.dtype, device=e.device)
        top = top.scatter_reduce(0, seg[:, None].expand_as(e), e, "amax", include_self=True)
        p = torch.exp(e - top[seg])
        total = torch.zeros_like(top).index_add_(0, seg, p)
        return p / total[seg]
    raise NotImplementedError("message function %r" % fn)


def apply_vert(fn: str, blk: block.Block, **t) -> torch.Tensor:
    if fn != "aggregate_sum":
        raise NotImplementedError("reduce function %r" % fn)
    rows, _, _ = edge_endpoints(blk)
    e = t["e"]
    out = torch.zeros((blk.size[0],) + tuple(e.shape[1:]), dtype=e.dtype, device=e.device)
    return out.index_add_(0, rows, e)


# --------------------------------------------------------------------------- #
class Graph:
    """One relation: a ``Block`` plus named tensors on its sources, destinations
    and edges (mp.py:78-170)."""

    def __init__(self, blk: block.Block):
        self.blk = blk
        self.edge = dict()
        self.src_node = dict()
        self.dst_node = dict()
        self._placeholder = None  # the ``graph`` node while a trace is running

    def device(self):
        for v in self.src_node.values():
            return v.device
        raise RuntimeError("no source tensor set yet")

    def num_edges(self):
        return self.blk.num_edges()

    def num_src_nodes(self):
        return self.blk.num_src_nodes()

    def num_dst_nodes(self):
        return self.blk.num_dst_nodes()

    def num_features(self):
        width = None
        for v in self.src_node.values():
            if v.dim() == 3:
                assert width in (None, v.size(-1))
                width = v.size(-1)
        assert width
        return width

    def right_norm(self):
        return self.blk.right_norm

    def clear(self):
        self.edge.clear()
        self.src_node.clear()
        self.dst_node.clear()

    def _operands(self, desc: dict) -> Dict[str, torch.Tensor]:
        # a name is looked up in all three stores (the reference's models keep the
        # query under src_node and the key under dst_node, model.py:91-92)
        found = {}
        for role, name in desc.items():
            if role in ("func", "out"):
                continue
            for store in (self.edge, self.src_node, self.dst_node):
                if name in store:
                    found[role] = store[name]
            if role not in found:
                raise KeyError("no tensor named %r on this graph" % name)
        return found

    def _apply(self, kind: str, desc: dict):
        ops = self._operands(desc)
        fn = desc["func"]
        if not any(isinstance(v, Tracer) for v in ops.values()):
            apply = apply_edge if kind == "edge" else apply_vert
            return apply(fn, self.blk, **ops)
        if self._placeholder is None:
            raise RuntimeError("traced tensors on a graph that is not an argument of the trace")
        inputs = {"g": self._placeholder}
        for role, v in ops.items():
            if not isinstance(v, Tracer):
                raise NotImplementedError("mixing traced and real tensors in %s" % fn)
            inputs[role] = v.node
        heads = {v.size(1) for v in ops.values()}
        assert len(heads) == 1, "operands disagree on the number of heads"
        n_heads = heads.pop()
        if kind == "edge":
            # the per-edge feature rows of copy_u / u_mul_e are never materialised: like
            # the reference, the message is sized [E, H] and remembers the row width
            width = ops["u"].size(2) if fn in ("copy_u", "u_mul_e") else None
            size = [self.num_edges(), n_heads]
            attrs = {"fn": fn, "width": width}
            dtype = next(iter(ops.values())).dtype
        else:
            width = inputs["e"].attrs.get("width") or self.num_features()
            size = [self.num_dst_nodes(), n_heads, width]
            attrs = {"fn": fn}
            dtype = ops["e"].dtype
        node = ir.Node(kind, inputs, attrs, size)
        return Tracer.wrap(torch.empty(size, dtype=dtype, device="meta"), node)

    def message_func(self, desc: dict):
        self.edge[desc["out"]] = self._apply("edge", desc)

    def reduce_func(self, desc: dict):
        self.dst_node[desc["out"]] = self._apply("vert", desc)

    @staticmethod
    def from_dglgraph(graph):
        """mp.py:132-170: CSR by destination of a homogeneous DGL graph."""
        adj = graph.adj(transpose=True, scipy_fmt="csr")
        n = graph.num_nodes()
        blk = block.Block(size=[n, n],
                          adj=[torch.IntTensor(adj.indptr).to(graph.device),
                               torch.IntTensor(adj.indices).to(graph.device)],
                          right_norm=torch.div(1.0, graph.in_degrees()).unsqueeze(-1))
        return Graph(blk)


class HeteroGraph:
    """Relations keyed by (source type, edge type, destination type), with the
    bookkeeping the models and the stitcher read (mp.py:173-241)."""

    def __init__(self):
        self.device = None
        self.etypes = []
        self.nty2num = {}
        self.idx2rel = {}
        self.rel2idx = {}
        self.hetero_graph = {}

    def __iter__(self):
        return iter(self.hetero_graph.items())

    def add_relation(self, sty, ety, dty, blk: block.Block):
        assert blk.size == [self.nty2num[dty], self.nty2num[sty]]
        idx = len(self.idx2rel)
        self.idx2rel[idx] = [sty, ety, dty]
        self.rel2idx[sty, ety, dty] = idx
        self.hetero_graph[sty, ety, dty] = Graph(blk)
        if ety not in self.etypes:
            self.etypes.append(ety)

    @staticmethod
    def from_blocks(nty2num: dict, blocks: dict, device=None):
        """``blocks``: {(source type, edge type, destination type): Block}."""
        hgraph = HeteroGraph()
        hgraph.device = device
        hgraph.nty2num = dict(nty2num)
        for (sty, ety, dty), blk in blocks.items():
            hgraph.add_relation(sty, ety, dty, blk)
        return hgraph

    @staticmethod
    def from_dglgraph(graph):
        """mp.py:186-241: one Block per canonical edge type of a DGL heterograph."""
        hgraph = HeteroGraph()
        hgraph.device = graph.device
        hgraph.nty2num = {nty: graph.num_nodes(nty) for nty in graph.ntypes}
        for sty, ety, dty in graph.canonical_etypes:
            adj = graph.adj(transpose=True, scipy_fmt="csr", etype=(sty, ety, dty))
            blk = block.Block(
                size=[graph.num_nodes(dty), graph.num_nodes(sty)],
                adj=[torch.IntTensor(adj.indptr).to(graph.device),
                     torch.IntTensor(adj.indices).to(graph.device)],
                right_norm=torch.div(1.0, graph.in_degrees(etype=(sty, ety, dty))).unsqueeze(-1))
            hgraph.add_relation(sty, ety, dty, blk)
        hgraph.etypes = list(graph.etypes)
        return hgraph


def from_dglgraph(graph):
    """mp.py:244-250. DGL is imported only by the caller that holds a DGL graph."""
    if graph.is_homogeneous:
        return Graph.from_dglgraph(graph)
    return HeteroGraph.from_dglgraph(graph)
