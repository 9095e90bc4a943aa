"""T-CSR of an event stream: per node, its events in time order
(YiTu_GNN/YiTu_T/gen_graph.py:40-95). Built with stable device sorts, so it runs
where the events live (GPU or CPU tensors).

Entry order inside a node is ascending timestamp; events of equal timestamp keep
their order in the stream (the reference uses numpy's default, unstable argsort
there, gen_graph.py:82, so for equal timestamps its order is unspecified; for
distinct timestamps the result is identical)."""
import torch


def build_tcsr(src, dst, ts, num_nodes, add_reverse=True):
    """``src``, ``dst`` integer tensors [E], ``ts`` float tensor [E] (any order).
    Returns (indptr int32 [num_nodes + 1], indices int32, eid int32, ts float32):
    node ``src[e]`` gets the entry (dst[e], e, ts[e]); with ``add_reverse`` node
    ``dst[e]`` also gets (src[e], e, ts[e]) (gen_graph.py --add_reverse)."""
    src = src.to(torch.int64)
    dst = dst.to(torch.int64)
    ts = ts.to(torch.float32)
    n_events = src.numel()
    eid = torch.arange(n_events, device=src.device)
    if add_reverse:
        # stream order: event e contributes entry 2e (to src) then 2e + 1 (to dst)
        node = torch.stack([src, dst], 1).reshape(-1)
        other = torch.stack([dst, src], 1).reshape(-1)
        eid = torch.stack([eid, eid], 1).reshape(-1)
        t = torch.stack([ts, ts], 1).reshape(-1)
    else:
        node, other, t = src, dst, ts
    by_time = torch.sort(t, stable=True).indices
    by_node = torch.sort(node[by_time], stable=True).indices
    order = by_time[by_node]
    counts = torch.bincount(node, minlength=num_nodes)
    indptr = torch.zeros(num_nodes + 1, dtype=torch.int64, device=src.device)
    indptr[1:] = torch.cumsum(counts, 0)
    return (indptr.to(torch.int32), other[order].to(torch.int32), eid[order].to(torch.int32),
            t[order])
