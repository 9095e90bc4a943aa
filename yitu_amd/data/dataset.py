"""Edge list -> CSR + per-node scale, as the module-1 callers expect it
(YiTu_GNN/data/dataset.py). The CSR is the canonical form scipy's
coo_matrix(...).tocsr() gives the reference (rows = first edge column, sorted,
duplicates merged, int32); ``degrees = sqrt(max(row length, 1))``
(dataset.py:131-133)."""
import time

import numpy as np
import torch

from . import graphgen


class CommonDataset(torch.nn.Module):
    """``path`` is a text file of ``src dst`` lines (load_from_txt) or an .npz
    with ``src_li``, ``dst_li``, ``num_nodes`` (dataset.py:64-109). ``edge_index``
    may be given directly instead of a path as an int array [2, E]."""

    def __init__(self, path, dim, num_class, load_from_txt=True, verbose=False, device="cuda",
                 edge_index=None, num_nodes=None):
        super().__init__()
        self.load_from_txt = load_from_txt
        self.num_nodes = 0
        self.num_features = dim
        self.num_classes = num_class
        self.edge_index = None
        self.reorder_flag = False
        self.verbose_flag = verbose
        self.device = torch.device(device)
        self.avg_degree = -1
        self.avg_edgeSpan = -1
        self.init_edges(path, edge_index, num_nodes)
        self.init_embedding(dim)
        self.init_labels(num_class)
        n = self.num_nodes
        mask = lambda frac: torch.arange(n, device=self.device) < int(n * frac)
        self.train_mask, self.val_mask, self.test_mask = mask(1), mask(0.3), mask(0.1)

    def init_edges(self, path, edge_index=None, num_nodes=None):
        start = time.perf_counter()
        if edge_index is not None:
            src_li, dst_li = np.asarray(edge_index[0]), np.asarray(edge_index[1])
            self.num_nodes = int(num_nodes) if num_nodes is not None else int(
                max(src_li.max(), dst_li.max())) + 1
        elif self.load_from_txt:
            arr = np.loadtxt(path, dtype=np.int64, ndmin=2)
            src_li, dst_li = arr[:, 0], arr[:, 1]
            self.num_nodes = int(max(src_li.max(), dst_li.max())) + 1
        else:
            if not path.endswith(".npz"):
                raise ValueError("graph file must be a .npz file")
            graph_obj = np.load(path)
            src_li, dst_li = graph_obj["src_li"], graph_obj["dst_li"]
            self.num_nodes = int(graph_obj["num_nodes"])
        self.num_edges = len(src_li)
        self.edge_index = np.stack([src_li, dst_li])
        if self.verbose_flag:
            print("# Loading (s): {:.3f}".format(time.perf_counter() - start))
        self.avg_degree = self.num_edges / self.num_nodes
        self.avg_edgeSpan = np.mean(np.abs(np.subtract(src_li, dst_li)))
        self._build_csr()

    def _build_csr(self):
        src = torch.as_tensor(self.edge_index[0], dtype=torch.int64)
        dst = torch.as_tensor(self.edge_index[1], dtype=torch.int64)
        if self.device.type == "cuda":
            # sort + merge on the device, then back to the host tensors the callers expect
            from . import csr
            indptr, indices = csr.coo_to_csr(src.to(self.device), dst.to(self.device),
                                             self.num_nodes)
            indptr, indices = indptr.cpu(), indices.cpu()
        else:
            indptr, indices = graphgen.csr_from_edges(src, dst, self.num_nodes)
        self.row_pointers = indptr  # CPU int32, as torch.IntTensor in the reference
        self.column_index = indices
        deg = (indptr[1:] - indptr[:-1]).to(torch.float32).clamp_(min=1.0)
        self.degrees = torch.sqrt(deg).to(self.device)

    def init_embedding(self, dim):
        self.x = torch.randn(self.num_nodes, dim).to(self.device)

    def init_labels(self, num_class):
        self.y = torch.ones(self.num_nodes).long().to(self.device)

    def rabbit_reorder(self):
        """Relabels the vertices by community order and rebuilds the CSR
        (dataset.py:149-190); a no-op unless ``reorder_flag`` is set."""
        if not self.reorder_flag:
            return
        from .. import rabbit
        self.edge_index = rabbit.reorder(torch.IntTensor(self.edge_index)).numpy()
        self._build_csr()
