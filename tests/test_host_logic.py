"""CPU tests of the host-side mirror: build_part, InputInfo, CommonDataset, the
C-ABI library's exported symbols."""
import ctypes
import os
import re

import numpy as np
import pytest
import scipy.sparse as sp
import torch

import oracle
from helpers import random_csr
from yitu_amd import YiTu_GNN_kernel as K
from yitu_amd.data.dataset import CommonDataset
from yitu_amd.utils.input_info import InputInfo

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "yitu_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(yitu_[a-z0-9_]+)\s*\(", header))
    assert len(names) >= 8
    lib = ctypes.CDLL(os.path.join(ROOT, "yitu_amd", "libyitu_hip.so"))
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, "declared but not exported: %s" % missing
    lib.yitu_abi_version.restype = ctypes.c_int
    from yitu_amd import _lib as binding
    assert lib.yitu_abi_version() == binding.ABI_VERSION == 4


def test_host_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "yitu_host.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(yitu_[a-z0-9_]+)\s*\(", header))
    assert len(names) >= 10
    lib = ctypes.CDLL(os.path.join(ROOT, "yitu_amd", "libyitu_host.so"))
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, "declared but not exported: %s" % missing


@pytest.mark.parametrize("ps", [1, 4, 32])
@pytest.mark.parametrize("last_empty", [False, True])
def test_build_part_matches_oracle(ps, last_empty):
    indptr, _ = random_csr(60, 60, 0.15, ps, hub_rows=(2,), hub_degree=55,
                           empty_rows=(0, 59) if last_empty else (0,))
    pp, p2n = K.build_part(ps, indptr)
    want_pp, want_p2n = oracle.build_part(ps, indptr.numpy())
    assert pp.dtype == torch.int32 and p2n.dtype == torch.int32 and not pp.is_cuda
    assert np.array_equal(pp.numpy(), want_pp) and np.array_equal(p2n.numpy(), want_p2n)
    # what the reference's caller does with its float tensors is a no-op here
    assert torch.equal(pp.int(), pp)


def test_build_part_empty_graph():
    pp, p2n = K.build_part(8, torch.zeros(5, dtype=torch.int32))
    assert pp.tolist() == [0] and p2n.tolist() == []


def test_common_dataset_csr_and_degrees(tmp_path):
    rng = np.random.default_rng(0)
    n, m = 100, 700
    src, dst = rng.integers(0, n, m), rng.integers(0, n, m)
    src[0], dst[0] = n - 1, n - 1
    path = tmp_path / "g.npz"
    np.savez(path, src_li=src, dst_li=dst, num_nodes=n)
    ds = CommonDataset(str(path), dim=8, num_class=3, load_from_txt=False, device="cpu")
    ref = sp.coo_matrix((np.ones(m), (src, dst)), shape=(n, n)).tocsr()
    assert np.array_equal(ds.row_pointers.numpy(), ref.indptr)
    assert np.array_equal(ds.column_index.numpy(), ref.indices)
    deg = np.maximum(np.diff(ref.indptr), 1)
    assert np.allclose(ds.degrees.numpy(), np.sqrt(deg.astype(np.float32)))
    assert ds.avg_degree == m / n
    assert ds.avg_edgeSpan == np.mean(np.abs(src - dst))
    assert ds.x.shape == (n, 8) and ds.y.shape == (n,)
    txt = tmp_path / "g.txt"
    np.savetxt(txt, np.stack([src, dst], 1), fmt="%d")
    ds2 = CommonDataset(str(txt), dim=8, num_class=3, load_from_txt=True, device="cpu")
    assert torch.equal(ds2.row_pointers, ds.row_pointers)
    assert torch.equal(ds2.column_index, ds.column_index)


def test_input_info_auto_decider():
    class DS:
        num_nodes, avg_degree, avg_edgeSpan, num_features = 10000, 11.3, 3000.0, 64
        reorder_flag = False

        def rabbit_reorder(self):
            self.called = True

    ds = DS()
    info = InputInfo(partSize=32, dimWorker=32, warpPerBlock=8, sharedMem=100, hiddenDim=16,
                     dataset_obj=ds, enable_rabbit=True, manual_mode=False)
    info.decider()
    assert info.partSize == 11
    assert info.dimWorker_input == 32 and info.dimWorker_hidden == 16
    assert 1 <= info.warpPerBlock_input <= 8 and 1 <= info.warpPerBlock_hidden <= 8
    # sqrt(3000) = 54.8 > sqrt(10000) / 100 = 1 -> reorder
    assert info.reorder_status is True and ds.reorder_flag is True and ds.called
    assert info.set_input().dimWorker == 32 and info.set_hidden().dimWorker == 16
    with pytest.raises(ValueError):
        InputInfo(sharedMem=100)


def test_auto_knobs_hand_computed():
    """input_info.py:79-127 worked by hand. Average degree 50, 1000 input and 300 hidden
    features, 8 KB budget: input estimate 8 * (200 + 4000 + 400) B = 36.8 KB -> capped at
    8 KB -> int(8000 / 4200) = 1 row per workgroup; hidden estimate 8 * (200 + 300 + 400) B
    = 7.2 KB (the hidden width enters unscaled) -> int(7200 / 1400) = 5."""
    from yitu_amd.utils.input_info import auto_knobs, worth_reordering
    k = auto_knobs(50.9, 1000, 300, 8.0)
    assert tuple(k) == (50, 1, 5, 32, 32)
    assert tuple(auto_knobs(11.3, 64, 16, 40.0)) == (11, 8, 8, 32, 16)
    assert worth_reordering(3000.0, 10000) and not worth_reordering(0.5, 10000)
