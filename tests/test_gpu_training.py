"""Module-1 training end to end, the way the reference's single-GPU examples run it
(examples/YiTu_GNN/single/gin/main.py:17-119, gin.py, gcn.py): Planetoid-format .npz
(single/data_process.py:78-91) -> CommonDataset -> InputInfo.decider (with the vertex
reorder) -> build_part -> 5-layer GIN / 2-layer GCN under Adam, against the same model
in dense autograd from the same initial weights. The graph is symmetric, where the
reference's backward (aggregating dY over the forward CSR) is the true gradient."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from yitu_amd import YiTu_GNN_kernel
from yitu_amd.data.dataset import CommonDataset
from yitu_amd.nn import GCNConv, GINConv
from yitu_amd.utils.input_info import InputInfo

pytestmark = pytest.mark.gpu


class GIN(torch.nn.Module):  # single/gin/gin.py
    def __init__(self, in_features, num_hidden, num_classes):
        super().__init__()
        dims = [in_features] + [num_hidden] * 4 + [num_classes]
        for i in range(5):
            setattr(self, "conv%d" % (i + 1), GINConv(dims[i], dims[i + 1]))

    def forward(self, x, input_info):
        x = F.relu(self.conv1(x, input_info.set_input()))
        for conv in (self.conv2, self.conv3, self.conv4):
            x = F.relu(conv(x, input_info.set_hidden()))
        return F.log_softmax(self.conv5(x, input_info.set_hidden()), dim=1)


class GCN(torch.nn.Module):  # single/gcn/gcn.py
    def __init__(self, in_features, num_hidden, num_classes):
        super().__init__()
        self.conv1 = GCNConv(in_features, num_hidden)
        self.conv2 = GCNConv(num_hidden, num_classes)

    def forward(self, x, input_info):
        x = F.relu(self.conv1(x, input_info.set_input()))
        return F.log_softmax(self.conv2(x, input_info.set_hidden()), dim=1)


def _write_npz(path, n, m, seed):
    """A symmetric graph with self loops in the on-disk layout of data_process.py:78-91."""
    rng = np.random.default_rng(seed)
    a, b = rng.integers(0, n, m), rng.integers(0, n, m)
    loops = np.arange(n)
    src = np.concatenate([a, b, loops])
    dst = np.concatenate([b, a, loops])
    np.savez(path, feat=rng.normal(size=(n, 4)).astype(np.float32), label=np.zeros(n, np.int64),
             test_mask=np.zeros(n, bool), train_mask=np.ones(n, bool), val_mask=np.zeros(n, bool),
             src_li=src, dst_li=dst, num_edges=len(src), num_nodes=n, n_classes=4)


def _prepare(tmp_path, dev, manual_mode):
    path = str(tmp_path / "toy.npz")
    n, dim, hidden, classes = 700, 24, 16, 4
    _write_npz(path, n, 3000, seed=21)
    torch.manual_seed(13)
    dataset = CommonDataset(path, dim, classes, load_from_txt=False, device=dev)
    assert dataset.num_nodes == n and dataset.x.shape == (n, dim)
    info = InputInfo(dataset.row_pointers, dataset.column_index, dataset.degrees, 32, 32, 8, 100,
                     hiddenDim=hidden, dataset_obj=dataset, enable_rabbit=True,
                     manual_mode=manual_mode)
    before = dataset.column_index.clone()
    info.decider()
    # ids are spread uniformly: sqrt(mean |src - dst|) is far above sqrt(n) / 100
    assert info.reorder_status is True and dataset.reorder_flag is True
    assert not torch.equal(dataset.column_index, before)  # the dataset was relabelled
    if manual_mode:   # manual mode hands the new CSR to the carrier (input_info.py:65-72)
        assert info.row_pointers is dataset.row_pointers
        assert info.partSize == 32
    else:             # automatic mode derives the knobs and keeps the CSR it was given
        assert info.partSize == int(dataset.avg_degree)
        assert info.dimWorker_input == 24 and info.dimWorker_hidden == 16
    part_ptr, part2node = YiTu_GNN_kernel.build_part(info.partSize, info.row_pointers)
    info.row_pointers = info.row_pointers.to(dev)
    info.column_index = info.column_index.to(dev)
    info.partPtr = part_ptr.int().to(dev)
    info.part2Node = part2node.int().to(dev)
    if manual_mode:  # one of the two modes also trains with the per-edge column scales
        info.prepare_edge_scale()
        assert info.edge_scale.shape == info.column_index.shape
    # dense form of the CSR the model will run on
    rp, ci = info.row_pointers.cpu(), info.column_index.cpu().long()
    rows = torch.repeat_interleave(torch.arange(n), (rp[1:] - rp[:-1]).long())
    adj = torch.zeros(n, n)
    adj[rows, ci] = 1.0
    assert torch.equal(adj, adj.t())
    return dataset, info, adj.to(dev), (dim, hidden, classes)


@pytest.mark.parametrize("manual_mode", [True, False])
def test_gin_five_layers_follows_dense_autograd(dev, tmp_path, manual_mode):
    dataset, info, adj, (dim, hidden, classes) = _prepare(tmp_path, dev, manual_mode)
    x = dataset.x
    teacher = torch.randn(dim, classes, device=dev)
    y = (adj @ (x @ teacher)).argmax(1)
    torch.manual_seed(17)
    model = GIN(dim, hidden, classes).to(dev)
    convs = [getattr(model, "conv%d" % i) for i in range(1, 6)]
    ws = [c.weights.detach().clone().requires_grad_() for c in convs]
    eps = convs[0].eplison
    opt_a = torch.optim.Adam(model.parameters(), lr=0.01)
    opt_b = torch.optim.Adam(ws, lr=0.01)
    curve_a, curve_b = [], []
    for _ in range(25):
        model.train()
        opt_a.zero_grad()
        la = F.nll_loss(model(x, info), y)
        la.backward()
        opt_a.step()
        opt_b.zero_grad()
        h = x
        for i, w in enumerate(ws):
            h = (eps * (adj @ h)) @ w
            if i < 4:
                h = torch.relu(h)
        lb = F.nll_loss(F.log_softmax(h, dim=1), y)
        lb.backward()
        opt_b.step()
        curve_a.append(la.item())
        curve_b.append(lb.item())
    assert curve_a[-1] < curve_a[0]
    assert np.allclose(curve_a, curve_b, rtol=2e-3, atol=1e-4), (curve_a, curve_b)


def test_gcn_two_layers_from_npz_follows_dense_autograd(dev, tmp_path):
    dataset, info, adj, (dim, hidden, classes) = _prepare(tmp_path, dev, manual_mode=True)
    x = dataset.x
    # the carrier's degrees are those of the CSR before the reorder; take the relabelled ones
    info.degrees = dataset.degrees
    s = 1.0 / info.degrees            # the example passes sqrt(deg); the op multiplies by it, so
    info.degrees = s                  # the symmetric normalisation needs the reciprocal
    assert info.edge_scale is None    # replacing the scale vector dropped the per-edge scales
    info.prepare_edge_scale()
    norm_adj = s[:, None] * adj * s[None, :]
    y = (norm_adj @ (x @ torch.randn(dim, classes, device=dev))).argmax(1)
    torch.manual_seed(19)
    model = GCN(dim, hidden, classes).to(dev)
    w1 = model.conv1.weights.detach().clone().requires_grad_()
    w2 = model.conv2.weights.detach().clone().requires_grad_()
    opt_a = torch.optim.Adam(model.parameters(), lr=0.01)
    opt_b = torch.optim.Adam([w1, w2], lr=0.01)
    curve_a, curve_b = [], []
    for _ in range(25):
        opt_a.zero_grad()
        la = F.nll_loss(model(x, info), y)
        la.backward()
        opt_a.step()
        opt_b.zero_grad()
        lb = F.nll_loss(F.log_softmax(norm_adj @ (torch.relu(norm_adj @ (x @ w1)) @ w2), dim=1), y)
        lb.backward()
        opt_b.step()
        curve_a.append(la.item())
        curve_b.append(lb.item())
    assert curve_a[-1] < curve_a[0]
    assert np.allclose(curve_a, curve_b, rtol=2e-3, atol=1e-4), (curve_a, curve_b)
