"""Drop-in for the reference's ``YiTu_GNN.rabbit`` extension module
(ccsrc/reorder/reorder.cpp:293-295): ``reorder(edge_index) -> edge_index``.

``reorder_with_perm`` additionally returns the permutation (new id of every old
vertex), which the reference computes and throws away, and ``permute_rows``
applies it to a feature matrix on the GPU.
"""
import ctypes

import numpy as np
import torch

from . import _host


def _run(edge_index, want_edges=True, threads=1):
    if not isinstance(edge_index, torch.Tensor):
        edge_index = torch.as_tensor(np.asarray(edge_index))
    if edge_index.is_cuda:
        raise RuntimeError("rabbit.reorder expects a CPU tensor")
    if edge_index.dim() != 2 or edge_index.size(0) != 2:
        raise RuntimeError("edge_index must be [2, n_edges]")
    if edge_index.dtype != torch.int32:
        raise RuntimeError("edge_index must be int32 (torch.IntTensor)")
    if not edge_index.is_contiguous():
        raise RuntimeError("in_edge_index must be contiguous")  # CHECK_INPUT, reorder.cpp:232-233
    m = edge_index.size(1)
    n = int(edge_index.max()) + 1 if m else 0
    out = torch.zeros_like(edge_index) if want_edges else None
    perm = torch.empty(n, dtype=torch.int32)
    n_out = ctypes.c_int64(0)
    rc = _host.lib().yitu_rabbit_reorder_threads(
        ctypes.c_void_p(out.data_ptr() if out is not None else 0), ctypes.c_void_p(perm.data_ptr()),
        ctypes.c_int64(n), ctypes.byref(n_out), ctypes.c_void_p(edge_index.data_ptr()),
        ctypes.c_int64(m), ctypes.c_int(int(threads)))
    if rc != 0:
        raise RuntimeError("rabbit reorder failed: %s" % _host.lib().yitu_host_last_error().decode())
    return out, perm


def reorder(in_edge_index, threads=1):
    """int32 CPU [2, E] -> int32 [2, E]: the same edges, in the same order, with
    both end points renamed by the Rabbit-Order permutation (reorder.cpp:282-289).
    ``threads``: 1 (default) aggregates on one thread and gives the same permutation
    every time; more threads (0 = all) follow the reference's lock-free protocol
    (rabbit_order.hpp:554-621) and, like it, give a valid but timing-dependent one."""
    return _run(in_edge_index, threads=threads)[0]


def reorder_with_perm(in_edge_index, threads=1):
    """Returns (relabelled edge_index, perm) with perm[old id] = new id."""
    return _run(in_edge_index, threads=threads)


def permute_rows(x, perm):
    """Rows of ``x`` moved to their new ids: out[perm[v]] = x[v]."""
    out = torch.empty_like(x)
    out[perm.to(x.device).long()] = x
    return out
