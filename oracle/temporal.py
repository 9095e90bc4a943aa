"""Dense restatement of the temporal neighbour attention layer (TEST INFRASTRUCTURE ONLY).

``TransfomerAttentionLayer.forward`` (YiTu_GNN/YiTu_T/layers.py:75-142, the branch with
node features and time encodings, :104-125) gathers, per root, the sampled neighbours'
``[h | cos(w dt + b)]`` rows, projects them to keys and values, scores them against the
root's query with LeakyReLU(0.2), normalises over the root's neighbours (DGL's
``edge_softmax``) and sums the values, then applies ``w_out`` on ``[agg | h_root]``, ReLU
and LayerNorm. Here the same arithmetic runs on a dense ``[roots, k_max]`` neighbour grid
with a mask, in plain torch on whatever device the inputs live on: the checker of the GPU
layer and, on CPU tensors, the timed CPU baseline of the benchmark. ``TimeEncode``
(layers.py:6-17) is ``cos(t w + b)``.

The reference's layer is DGL code outside the tree and holds no test; this statement is
what the GPU layer is pinned to (forward and all gradients through autograd).
"""
import torch


def dense_temporal_attention(layer, h, row, dt, n_dst, k_max):
    """``layer``: any object with the reference's parameter names (``time_enc.w``,
    ``w_q``, ``w_k``, ``w_v``, ``w_out``, ``layer_norm``, ``num_head``, ``dim_out``).
    ``h`` [n_dst + E, dim]: root rows then neighbour rows; ``row`` [E]: root of each
    neighbour, sorted; ``dt`` [E]."""
    dev = h.device
    E = row.numel()
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
