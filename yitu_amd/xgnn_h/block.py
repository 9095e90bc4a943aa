"""CSR holder and multi-relation CSR packing (xgnn_h/block.py)."""
from typing import List

import torch


class Block:
    """``size = [n_dst, n_src]``, ``adj_sparse = [indptr, indices]`` (block.py:5-33)."""

    def __init__(self, size: list, adj: list, right_norm=None):
        self.size = size
        self.adj_sparse = adj
        self.right_norm = right_norm

    def to(self, device):
        self.adj_sparse = [self.adj_sparse[0].to(device), self.adj_sparse[1].to(device)]
        if self.right_norm is not None:
            self.right_norm = self.right_norm.to(device)
        return self

    def by_query_block(self, n_blocks: int):
        """A stitched block seen as ``n_dst * n_blocks`` rows: row ``r * n_blocks + b`` holds
        the edges of destination ``r`` that carry block tag ``b`` (they are contiguous: a
        stitched row is sorted by tag, then column). Same ``indices`` tensor, so per-graph
        state derived from it is shared. A softmax per (destination, block), which is what a
        stitched attention term asks for, is a plain per-row softmax over this view. Built
        once per block and kept."""
        kept = getattr(self, "_by_query_block", None)
        if kept is None or kept[0] != n_blocks or kept[2] is not self.adj_sparse[1]:
            indptr, indices = self.adj_sparse
            n_dst = indptr.numel() - 1
            deg = (indptr[1:] - indptr[:-1]).to(torch.int64)
            rows = torch.repeat_interleave(torch.arange(n_dst, device=indptr.device), deg)
            key = rows * n_blocks + (indices.to(torch.int64) >> 24)
            if key.numel() > 1:
                assert bool((key[1:] >= key[:-1]).all()), "rows must be sorted by block tag"
            counts = torch.bincount(key, minlength=n_dst * n_blocks)
            v_indptr = torch.zeros(n_dst * n_blocks + 1, dtype=torch.int32, device=indptr.device)
            v_indptr[1:] = torch.cumsum(counts, 0)
            view = Block([n_dst * n_blocks, self.size[1]], [v_indptr, indices])
            kept = (n_blocks, view, indices)
            self._by_query_block = kept
        return kept[1]

    def num_edges(self):
        indices = self.adj_sparse[1]
        assert indices.dim() == 1
        return indices.numel()

    def num_src_nodes(self):
        return self.size[1]

    def num_dst_nodes(self):
        indptr = self.adj_sparse[0]
        assert indptr.dim() == 1
        assert self.size[0] == indptr.size(0) - 1
        return self.size[0]


def stitch_csr(block_list: List[Block]):
    """Row-wise concatenation of up to 16 blocks with equal row counts
    (block.py:36-67): block b's columns are shifted by the source counts of
    blocks 0..b-1 and tagged ``(b << 24) + col``. The reference walks every edge
    in a Python loop; this is the same integer result from vectorised tensor ops
    on whichever device the blocks live on."""
    lens = [blk.size[0] for blk in block_list]
    n_rows = min(lens)
    assert len(lens) <= 16
    assert min(lens) == max(lens)
    dev = block_list[0].adj_sparse[0].device
    rows, keys, blk_of = [], [], []
    cursor = 0
    for bid, blk in enumerate(block_list):
        indptr, indices = blk.adj_sparse
        assert indptr.numel() == n_rows + 1
        deg = (indptr[1:] - indptr[:-1]).to(torch.int64)
        col = indices.to(torch.int64) + cursor
        if col.numel():
            assert int(col.max()) <= 2 ** 24
        rows.append(torch.repeat_interleave(torch.arange(n_rows, device=dev), deg))
        keys.append((bid << 24) + col)
        blk_of.append(torch.full((col.numel(),), bid, dtype=torch.int64, device=dev))
        cursor += blk.size[1]
    rows = torch.cat(rows)
    keys = torch.cat(keys)
    blk_of = torch.cat(blk_of)
    # order: by row, then by block, keeping each block's own edge order (stable)
    order = torch.argsort(rows * 16 + blk_of, stable=True)
    new_indices = keys[order].to(torch.int32)
    counts = torch.bincount(rows, minlength=n_rows)
    new_indptr = torch.zeros(n_rows + 1, dtype=torch.int64, device=dev)
    new_indptr[1:] = torch.cumsum(counts, 0)
    n_cols = sum(blk.size[1] for blk in block_list)
    return Block(size=[n_rows, n_cols], adj=[new_indptr.to(torch.int32), new_indices])


def stack_blocks(block_list: List[Block], row_offsets: List[int], col_offsets: List[int],
                 n_rows: int, n_cols: int, row_scales: List[torch.Tensor] = None):
    """Places blocks in one [n_rows, n_cols] CSR over a union node space: block
    ``b`` occupies rows ``row_offsets[b] + r`` and columns ``col_offsets[b] + c``.
    Where ``stitch_csr`` (block.py:36-67) joins blocks of one destination set side
    by side for one launch, this also stacks different destination sets, so that
    a whole heterogeneous layer (per-relation aggregate, sum over the relations
    of a destination type) is a single edge-weighted SpMM.

    Returns ``(Block, values [E, 1])``; ``values[e] = row_scales[b][r]`` of the
    block and row the edge came from (1 when no scales are given). Inside a row,
    edges are ordered by block, then in the block's own order; columns are plain
    ids (no block tag), so ``n_cols`` is limited to 2^24 like any packed CSR.
    """
    assert len(block_list) == len(row_offsets) == len(col_offsets) and len(block_list) > 0
    assert n_cols <= 2 ** 24
    dev = block_list[0].adj_sparse[0].device
    rows, cols, vals, blk_of = [], [], [], []
    for bid, blk in enumerate(block_list):
        indptr, indices = blk.adj_sparse
        assert row_offsets[bid] + blk.size[0] <= n_rows and col_offsets[bid] + blk.size[1] <= n_cols
        deg = (indptr[1:] - indptr[:-1]).to(torch.int64)
        r = torch.repeat_interleave(torch.arange(blk.size[0], device=dev), deg)
        rows.append(r + row_offsets[bid])
        cols.append((indices.to(torch.int64) & 0xFFFFFF) + col_offsets[bid])
        if row_scales is not None:
            vals.append(row_scales[bid].reshape(-1).to(torch.float32)[r])
        else:
            vals.append(torch.ones(r.numel(), dtype=torch.float32, device=dev))
        blk_of.append(torch.full((r.numel(),), bid, dtype=torch.int64, device=dev))
    rows, cols, vals, blk_of = torch.cat(rows), torch.cat(cols), torch.cat(vals), torch.cat(blk_of)
    order = torch.argsort(rows * len(block_list) + blk_of, stable=True)
    new_indptr = torch.zeros(n_rows + 1, dtype=torch.int64, device=dev)
    new_indptr[1:] = torch.cumsum(torch.bincount(rows, minlength=n_rows), 0)
    return (Block(size=[n_rows, n_cols],
                  adj=[new_indptr.to(torch.int32), cols[order].to(torch.int32)]),
            vals[order].unsqueeze(-1).contiguous())
