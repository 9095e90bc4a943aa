"""Shared test helpers: small seeded graphs and the tolerances of the parity bar."""
import numpy as np
import torch

from yitu_amd.data import graphgen

# fp32 outputs and gradients: rtol 1e-5 / atol 1e-4; bf16-in / fp32-accumulate: rtol 1e-2
RTOL_F32, ATOL_F32 = 1e-5, 1e-4
RTOL_BF16, ATOL_BF16 = 1e-2, 1e-4


def assert_close(got, want, rtol=RTOL_F32, atol=ATOL_F32, what=""):
    got = got.detach().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got)
    want = want.detach().cpu().numpy() if isinstance(want, torch.Tensor) else np.asarray(want)
    assert got.shape == want.shape, "%s shape %s vs %s" % (what, got.shape, want.shape)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    bound = atol + rtol * np.abs(want.astype(np.float64))
    bad = err > bound
    if bad.any():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError("%s: %d / %d elements off; worst at %s got %r want %r" %
                             (what, bad.sum(), bad.size, i, got[i], want[i]))


def random_csr(n_dst, n_src, density, seed, hub_rows=(), hub_degree=0, empty_rows=()):
    """Canonical CSR with a given density plus optional hub / empty rows."""
    rng = np.random.default_rng(seed)
    rows, cols = np.nonzero(rng.random((n_dst, n_src)) < density)
    keep = ~np.isin(rows, np.asarray(list(empty_rows), dtype=np.int64))
    rows, cols = rows[keep], cols[keep]
    for r in hub_rows:
        c = rng.choice(n_src, size=min(hub_degree, n_src), replace=False)
        rows = np.concatenate([rows, np.full(c.shape, r)])
        cols = np.concatenate([cols, c])
    indptr, indices = graphgen.csr_from_edges(torch.from_numpy(rows), torch.from_numpy(cols),
                                              n_dst, n_src)
    return indptr, indices


def powerlaw_graph(scale, m, seed):
    src, dst = graphgen.rmat(scale, m, seed, self_loops=True)
    return graphgen.csr_by_destination(src, dst, 1 << scale)


def dense_temporal_attention(layer, h, row, dt, n_dst, k_max):
    """Dense masked attention with the layer's own parameters."""
    dev = h.device
    E = row.numel()
    slot = torch.zeros(E, dtype=torch.long, device=dev)
    counts = torch.bincount(row, minlength=n_dst)
    start = torch.cumsum(counts, 0) - counts
    slot = torch.arange(E, device=dev) - start[row]
    mask = torch.zeros(n_dst, k_max, dtype=torch.bool, device=dev)
    mask[row, slot] = True
    te = torch.cos(dt[:, None] * layer.time_enc.w.weight[:, 0][None, :] + layer.time_enc.w.bias)
    te0 = torch.cos(layer.time_enc.w.bias)[None, :].expand(n_dst, -1)
    q = layer.w_q(torch.cat([h[:n_dst], te0], 1))
    kv_in = torch.cat([h[n_dst:], te], 1)
    k, v = layer.w_k(kv_in), layer.w_v(kv_in)
    H, D = layer.num_head, layer.dim_out // layer.num_head
    Kd = torch.zeros(n_dst, k_max, H, D, device=dev)
    Vd = torch.zeros(n_dst, k_max, H, D, device=dev)
    Kd[row, slot] = k.reshape(E, H, D)
    Vd[row, slot] = v.reshape(E, H, D)
    logits = torch.einsum("bhd,bkhd->bkh", q.reshape(n_dst, H, D), Kd)
    logits = torch.nn.functional.leaky_relu(logits, 0.2)
    logits = logits.masked_fill(~mask[:, :, None], float("-inf"))
    att = torch.softmax(logits, dim=1)
    att = torch.nan_to_num(att, nan=0.0)  # roots without neighbours
    agg = torch.einsum("bkh,bkhd->bhd", att, Vd).reshape(n_dst, H * D)
    out = layer.w_out(torch.cat([agg, h[:n_dst]], 1))
    return layer.layer_norm(torch.relu(out))
