"""Structure of the row plan written by yitu_plan_build (integer work: exact).

The plan's layout is read back from the device buffer: a 512-byte header
(counters; band width and count), the long-row table and the item records. The checks
are invariants that any correct plan must satisfy, stated independently of how
the builder derives it: the items of a long row tile the row's edge range
without gap or overlap in item-id order, no item exceeds 64 edges, every item
appears exactly once in the record list, the list is in ascending order of the
items' middle source ids, the bands cover the source ids, and the number of items
stays inside the bound that sizes the callers' workspaces.
"""
import numpy as np
import pytest
import torch

from helpers import powerlaw_graph, random_csr
from yitu_amd import _lib

pytestmark = pytest.mark.gpu

CHUNK = 64
BAND_SHIFT, MAX_BANDS, MIN_SEGMENT = 17, 64, 16


def read_plan(plan, nnz):
    raw = plan.cpu().numpy().view(np.int32)
    max_rows = nnz // CHUNK + 1
    max_items = nnz // CHUNK + nnz // 16 + max_rows + 1
    n_items, n_rows, overflow = raw[0], raw[1], raw[2]
    band_shift, n_bands = int(raw[64]), int(raw[65])
    local_rows, sampled_rows = int(raw[66]), int(raw[67])
    rows_off = 128
    rows = raw[rows_off:rows_off + 4 * max_rows].reshape(-1, 4)[:n_rows]
    rec_off = rows_off + ((16 * max_rows + 255) // 256 * 256) // 4
    records = raw[rec_off:rec_off + 4 * max_items].reshape(-1, 4)
    return dict(n_items=int(n_items), n_rows=int(n_rows), overflow=int(overflow),
                band_shift=band_shift, n_bands=n_bands, rows=rows, local=local_rows,
                sampled=sampled_rows,
                records=records[:n_items], tail=records[n_items:], max_items=max_items)


def check_plan(indptr, indices, n_src, col_mask, dev):
    nnz = indices.numel()
    plan = _lib.row_plan(indptr.to(dev), indices.to(dev), n_src, col_mask)
    ip = indptr.numpy().astype(np.int64)
    deg = np.diff(ip)
    long_rows = np.nonzero(deg >= CHUNK)[0]
    if plan is None:
        assert long_rows.size == 0
        return None
    torch.cuda.synchronize()
    p = read_plan(plan, nnz)
    assert p["overflow"] == 0
    assert p["n_items"] <= p["max_items"]
    # the long-row table lists exactly the rows with >= 64 edges
    assert sorted(p["rows"][:, 0].tolist()) == long_rows.tolist()
    rec = p["records"]
    beg, end, item, tag = rec[:, 0].astype(np.int64), rec[:, 1].astype(np.int64), rec[:, 2], rec[:, 3]
    row = tag & 0x7fffffff
    single = tag < 0
    assert np.array_equal(np.sort(item), np.arange(p["n_items"]))          # every item once
    assert np.all(end > beg) and np.all(end - beg <= CHUNK)
    assert not p["tail"].any()                                               # unused slots cleared
    by_item = np.argsort(item)
    b, e, r, s = beg[by_item], end[by_item], row[by_item], single[by_item]
    for rr, first, count, _ in p["rows"]:
        assert count >= 1
        assert count <= deg[rr] // CHUNK + min(p["n_bands"], deg[rr] // MIN_SEGMENT)  # workspace bound
        sl = slice(first, first + count)
        assert np.all(r[sl] == rr)
        assert b[sl][0] == ip[rr] and e[sl][-1] == ip[rr + 1]                # tiles the row ...
        assert np.array_equal(b[sl][1:], e[sl][:-1])                         # ... in item order
        assert np.all(s[sl] == (count == 1))
    # locality: up to 4 evenly spaced edges of every row below 64 edges are sampled; local
    # = source within 1/64 of the id space (at least 1,024 ids) of the row's own position
    n_dst = deg.size
    cols_all = (indices.numpy() & col_mask).astype(np.int64)
    own = np.arange(n_dst, dtype=np.int64) * n_src // max(n_dst, 1)
    n_sampled = n_local = 0
    for k in range(4):
        take = (deg < CHUNK) & (deg > k)
        ns = np.minimum(deg[take], 4)
        c = cols_all[ip[:-1][take] + deg[take] * k // ns]
        n_sampled += int(take.sum())
        n_local += int((np.abs(c - own[take]) <= max(n_src >> 6, 1024)).sum())
    assert p["sampled"] == n_sampled and p["local"] == n_local
    # bands of 2^17 ids, wider only when that would give more than 64 of them
    assert p["band_shift"] >= BAND_SHIFT and 1 <= p["n_bands"] <= MAX_BANDS
    assert ((max(n_src, 1) - 1) >> p["band_shift"]) + 1 == p["n_bands"]
    assert p["band_shift"] == BAND_SHIFT or ((max(n_src, 1) - 1) >> (p["band_shift"] - 1)) + 1 > MAX_BANDS
    # the records are in ascending band (middle source id, 16 bits) order
    cols = (indices.numpy() & col_mask).astype(np.int64)
    mid = cols[(beg + end) // 2]
    shift = 0
    while ((max(n_src, 1) - 1) >> shift) >= (1 << 16):
        shift += 1
    assert np.all(np.diff(mid >> shift) >= 0)
    # an item is pure when it gathers from one group of bands of its row: a row of deg
    # edges may be cut into the largest power of two <= deg / 16 pieces (at most the
    # number of bands), i.e. at the boundaries of groups of ceil(bands / pieces) bands
    d = deg[row]
    allowed = np.minimum(2 ** np.floor(np.log2(np.maximum(d // MIN_SEGMENT, 1))).astype(np.int64),
                         p["n_bands"])
    allowed = np.where(2 * allowed * MIN_SEGMENT <= d, p["n_bands"], allowed)
    per_group = -(-p["n_bands"] // allowed)
    p["pure"] = ((cols[beg] >> p["band_shift"]) // per_group ==
                 (cols[end - 1] >> p["band_shift"]) // per_group)
    return p


def test_power_law_graph(dev):
    indptr, indices = powerlaw_graph(19, 6000000, 5)
    p = check_plan(indptr, indices, 1 << 19, 0x7fffffff, dev)
    # 4 bands of 2^17 sources: the cuts happen for real, and most items gather from
    # one band group only (segments shorter than 16 edges are merged into a neighbour)
    assert p["n_bands"] == 4
    assert p["pure"].mean() > 0.6


@pytest.mark.parametrize("hub_degree", [64, 65, 127, 128, 200, 1000, 4096])
def test_hub_rows(dev, hub_degree):
    n = 4096
    indptr, indices = random_csr(n, n, 0.003, hub_degree, hub_rows=(0, 77, n - 1),
                                 hub_degree=hub_degree, empty_rows=(3,))
    check_plan(indptr, indices, n, 0x7fffffff, dev)


def test_columns_not_sorted_inside_rows(dev):
    """Module-2 indices carry a block id above bit 24, so the masked columns of a
    row are sorted per block only: the cuts must still tile every row."""
    n = 2048
    indptr, indices = random_csr(n, n, 0.05, 9, hub_rows=(5, 6), hub_degree=1500)
    rng = np.random.default_rng(0)
    bid = torch.from_numpy(rng.integers(0, 3, indices.numel()).astype(np.int32))
    ip = indptr.numpy()
    tagged = indices | (bid << 24)
    # canonical module-2 order: sorted by (bid, col) inside every row
    rows = torch.repeat_interleave(torch.arange(n), torch.from_numpy(np.diff(ip)).long())
    order = np.lexsort((tagged.numpy(), rows.numpy()))
    tagged = tagged[torch.from_numpy(order)].contiguous()
    check_plan(indptr, tagged, n, 0xffffff, dev)


def test_more_sources_than_edges(dev):
    """A huge, mostly unused source range (32 bands of 2^17 ids) must still give a
    valid plan."""
    n_dst, n_src = 64, 1 << 22
    rng = np.random.default_rng(1)
    rows = np.repeat(np.arange(n_dst), 200)
    cols = rng.integers(0, n_src, rows.size)
    from yitu_amd.data import graphgen
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(rows), torch.from_numpy(cols),
                                              n_dst, n_src)
    check_plan(indptr, indices, n_src, 0x7fffffff, dev)


def test_no_long_rows(dev):
    indptr, indices = random_csr(500, 500, 0.01, 2)
    assert check_plan(indptr, indices, 500, 0x7fffffff, dev) is None


def test_locality_of_a_planted_graph_and_of_its_shuffle(dev):
    """Most rows of a graph with planted communities (contiguous ids) are local, few of the
    same graph with shuffled ids are: the flag the row kernels deal their rows by."""
    from yitu_amd.data import graphgen
    n_comm, size = 256, 512
    n = n_comm * size
    rng = np.random.default_rng(3)
    dst = np.repeat(np.arange(n), 40)
    src = dst // size * size + rng.integers(0, size, dst.size)
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(dst), torch.from_numpy(src), n, n)
    p = check_plan(indptr, indices, n, 0x7fffffff, dev)
    assert p["local"] == p["sampled"] == 4 * n
    shuffle = rng.permutation(n)
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(shuffle[dst]),
                                              torch.from_numpy(shuffle[src]), n, n)
    p = check_plan(indptr, indices, n, 0x7fffffff, dev)
    assert p["local"] * 8 < p["sampled"]
