"""Device-side edge list -> canonical CSR (yitu_coo_to_csr) against scipy's
coo_matrix(...).tocsr(), the routine the reference's dataset loader uses
(YiTu_GNN/data/dataset.py:116-129). Integer work: bit-exact."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from yitu_amd.data import csr, graphgen

pytestmark = pytest.mark.gpu


def _scipy_csr(rows, cols, n_rows, n_cols):
    m = sp.coo_matrix((np.ones(rows.size, np.float32), (rows, cols)), shape=(n_rows, n_cols)).tocsr()
    m.sum_duplicates()
    m.sort_indices()
    return m.indptr.astype(np.int32), m.indices.astype(np.int32)


@pytest.mark.parametrize("n_rows,n_cols,n_edges,seed", [
    (1, 1, 1, 0), (10, 10, 0, 1), (100, 100, 1000, 2), (257, 33, 5000, 3), (33, 4000, 5000, 4),
    (5000, 5000, 200000, 5), (3, 3, 10000, 6)])
def test_matches_scipy(dev, n_rows, n_cols, n_edges, seed):
    rng = np.random.default_rng(seed)
    rows = rng.integers(0, n_rows, n_edges)
    cols = rng.integers(0, n_cols, n_edges)
    indptr, indices = csr.coo_to_csr(torch.from_numpy(rows).to(dev), torch.from_numpy(cols).to(dev),
                                     n_rows, n_cols)
    want_ptr, want_idx = _scipy_csr(rows, cols, n_rows, n_cols)
    assert indptr.dtype == torch.int32 and indices.dtype == torch.int32
    assert np.array_equal(indptr.cpu().numpy(), want_ptr)
    assert np.array_equal(indices.cpu().numpy(), want_idx)


def test_power_law_graph_matches_the_host_build(dev):
    """2^18 nodes, 4 M draws with many duplicates: same bits as the torch build."""
    src, dst = graphgen.rmat(18, 4_000_000, 9, self_loops=True, device=dev)
    want_ptr, want_idx = graphgen.csr_by_destination(src, dst, 1 << 18)
    indptr, indices = csr.coo_to_csr(dst, src, 1 << 18)
    assert torch.equal(indptr, want_ptr) and torch.equal(indices, want_idx)


def test_out_of_range_id_is_an_error(dev):
    rows = torch.tensor([0, 1, 5], device=dev)
    cols = torch.tensor([0, 1, 2], device=dev)
    with pytest.raises(RuntimeError, match="outside"):
        csr.coo_to_csr(rows, cols, 4, 4)
    with pytest.raises(RuntimeError, match="outside"):
        csr.coo_to_csr(cols, torch.tensor([0, -1, 2], device=dev), 4, 4)


def test_common_dataset_builds_its_csr_on_the_device(dev):
    from yitu_amd.data.dataset import CommonDataset
    rng = np.random.default_rng(0)
    ei = rng.integers(0, 500, (2, 6000))
    ds = CommonDataset(None, 8, 3, edge_index=ei, num_nodes=500, device=dev)
    want_ptr, want_idx = _scipy_csr(ei[0], ei[1], 500, 500)
    assert not ds.row_pointers.is_cuda and ds.row_pointers.dtype == torch.int32
    assert np.array_equal(ds.row_pointers.numpy(), want_ptr)
    assert np.array_equal(ds.column_index.numpy(), want_idx)
    assert torch.allclose(ds.degrees.cpu(), torch.sqrt(torch.clamp(
        torch.from_numpy(np.diff(want_ptr)).float(), min=1.0)))


def test_forget_after_a_raw_pointer_refill(dev):
    """The plan / by-source caches key on torch's version counter, which a kernel that
    writes through the raw pointer does not move: after such a refill ``forget`` must be
    called, and then the next op sees the new graph. A second stream that uses a plan built
    on another stream waits for the build."""
    import oracle
    from helpers import assert_close, powerlaw_graph
    from yitu_amd import graph_ext
    n = 1 << 12
    ip_a, ix_a = powerlaw_graph(12, 60000, 1)
    ip_b, ix_b = powerlaw_graph(12, 60000, 2)
    m = min(ix_a.numel(), ix_b.numel())
    # same-sized buffers: truncate both graphs to m edges
    def clip(ip, ix):
        ip = torch.clamp(ip, max=m)
        return ip.contiguous(), ix[:m].contiguous()
    ip_a, ix_a = clip(ip_a, ix_a)
    ip_b, ix_b = clip(ip_b, ix_b)
    indptr, indices = ip_a.to(dev), ix_a.to(dev)
    g = torch.Generator().manual_seed(0)
    values = torch.rand(m, 2, generator=g)
    x = torch.randn(n, 2, 16, generator=g)
    got_a = graph_ext.spmm_forward(values.to(dev), indptr, indices, x.to(dev))
    assert_close(got_a, oracle.mh_spmm_forward(values, ip_a, ix_a, x))
    # refill in place through raw pointers (what a device-side CSR builder does)
    version = indices._version
    torch.cuda.synchronize()
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    for dst, src in ((indptr, ip_b), (indices, ix_b)):
        assert hip.hipMemcpy(ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()),
                             ctypes.c_size_t(src.numel() * 4), 1) == 0
    assert indices._version == version  # torch did not notice
    graph_ext.forget(indptr, indices)
    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):
        got_b = graph_ext.spmm_forward(values.to(dev), indptr, indices, x.to(dev))
    side.synchronize()
    assert_close(got_b, oracle.mh_spmm_forward(values, ip_b, ix_b, x))
    # the plan built on the side stream, used from the default stream
    got_b2 = graph_ext.spmm_forward(values.to(dev), indptr, indices, x.to(dev))
    assert torch.equal(got_b2, got_b)


@pytest.mark.parametrize("ps", [1, 7, 32, 64, 1000])
@pytest.mark.parametrize("last_empty", [False, True])
def test_build_part_on_the_device(dev, ps, last_empty):
    """build_part (YiTu_GNN.cpp:203-245) built on the GPU from a device indptr: the same
    integers as the oracle's restatement of the reference loop, including the sentinel that
    stays 0 behind an empty last row; hub rows of several waves' worth of groups, empty rows."""
    import oracle
    from helpers import random_csr
    from yitu_amd import YiTu_GNN_kernel as K
    indptr, _ = random_csr(3000, 3000, 0.004, ps, hub_rows=(5, 2998), hub_degree=2500,
                           empty_rows=(0, 17) + ((2999,) if last_empty else ()))
    if not last_empty:
        assert indptr[-1] > indptr[-2]
    pp, p2n = K.build_part(ps, indptr.to(dev))
    want_pp, want_p2n = oracle.build_part(ps, indptr.numpy())
    assert pp.is_cuda and pp.dtype == torch.int32 and p2n.dtype == torch.int32
    assert np.array_equal(pp.cpu().numpy(), want_pp) and np.array_equal(p2n.cpu().numpy(), want_p2n)


def test_build_part_on_the_device_empty_graph(dev):
    from yitu_amd import YiTu_GNN_kernel as K
    pp, p2n = K.build_part(8, torch.zeros(5, dtype=torch.int32, device=dev))
    assert pp.tolist() == [0] and p2n.numel() == 0
    pp, p2n = K.build_part(8, torch.zeros(1, dtype=torch.int32, device=dev))
    assert pp.tolist() == [0] and p2n.numel() == 0
