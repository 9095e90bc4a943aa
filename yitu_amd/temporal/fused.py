"""The temporal attention layer (YiTu_GNN/YiTu_T/layers.py:75-142) as one autograd node
of twelve launches: input assembly, Q | K | V as one grouped product, attention per root,
output product, ReLU + LayerNorm; the backward mirrors it. Biases ride as one more column
of every weight matrix against a column of ones, so no launch adds a bias or sums a bias
gradient. Everything goes through the C ABI (``yitu_tattn_*``, ``yitu_sgemm*``); torch
only provides the memory."""
import ctypes

import torch

from .. import _lib
from .._lib import c_i64, c_int, c_size, check, ptr, stream_ptr

c_f32 = ctypes.c_float

MAX_OUT, MAX_HEADS = 256, 8


def supported(dim_node, dim_edge, dim_time, dim_out, num_head):
    """Shapes the fused kernels take: a query made of node or time features, rows of at
    most 256 floats, at most 8 heads."""
    return (dim_node + dim_time > 0 and 1 <= dim_out <= MAX_OUT and dim_time <= MAX_OUT
            and 1 <= num_head <= MAX_HEADS and dim_out % num_head == 0)


def _gemm(L, dev, c, a, b, m, n, k, trans_a, trans_b, lda, ldb, ldc, ws):
    rc = L.yitu_sgemm(ptr(c), ptr(a), ptr(b), c_i64(m), c_i64(n), c_i64(k), c_int(trans_a),
                      c_int(trans_b), c_i64(lda), c_i64(ldb), c_i64(ldc), c_int(0), ptr(ws),
                      c_size(ws.numel() if ws is not None else 0), stream_ptr(dev))
    check(rc, "yitu_sgemm")


def _gemm_typed(L, dev, cs, as_, bs, ms, ks, n, trans_a, trans_b, lda, ldb, ldc, ws):
    count = len(cs)
    pointers = lambda ts: (ctypes.c_void_p * count)(*[t.data_ptr() for t in ts])
    sizes = lambda v: (ctypes.c_int64 * count)(*v)
    rc = L.yitu_sgemm_typed(pointers(cs), pointers(as_), pointers(bs), sizes(ms), sizes(ks),
                            c_i64(count), c_i64(n), c_int(trans_a), c_int(trans_b), c_i64(lda),
                            c_i64(ldb), c_i64(ldc), c_int(0), ptr(ws),
                            c_size(ws.numel() if ws is not None else 0), stream_ptr(dev))
    check(rc, "yitu_sgemm_typed")


def _carve(buf, *shapes):
    """Views of one fp32 buffer, each starting on a 64-float boundary."""
    out, pos = [], 0
    for shape in shapes:
        n = 1
        for s in shape:
            n *= s
        out.append(buf[pos:pos + n].view(*shape))
        pos += (n + 63) // 64 * 64
    return out


def _room(*shapes):
    total = 0
    for shape in shapes:
        n = 1
        for s in shape:
            n *= s
        total += (n + 63) // 64 * 64
    return max(total, 64)


class TemporalAttentionFunction(torch.autograd.Function):
    """apply(indptr, n_dst, num_head, eps, h, f, dt, time_w, time_b, w_q, b_q, w_k, b_k, w_v,
    b_v, w_out, b_out, ln_w, ln_b) -> [n_dst, dim_out]. ``h`` [n_dst + E, dim_node] or None,
    ``f`` [E, dim_edge] or None, ``time_w`` [dim_time, 1] / ``time_b`` or None."""

    @staticmethod
    def forward(ctx, indptr, n_dst, num_head, eps, h, f, dt, time_w, time_b, w_q, b_q, w_k, b_k,
                w_v, b_v, w_out, b_out, ln_w, ln_b):
        dev = w_k.device
        L = _lib.lib()
        E = int(dt.numel())
        B = int(n_dst)
        Dn = 0 if h is None else h.size(1)
        De = 0 if f is None else f.size(1)
        Dt = 0 if time_w is None else time_w.size(0)
        O = w_k.size(0)
        L.yitu_tattn_row_length.restype = ctypes.c_int64
        LD = int(L.yitu_tattn_row_length(c_i64(Dn), c_i64(De), c_i64(Dt), c_i64(O)))
        shapes = ((E, LD), (B, LD), (B, LD), (2 * O, LD), (2 * O, LD), (O, LD), (E, 2 * O),
                  (B, 2 * O), (E, num_head), (B, O))
        buf = torch.empty(_room(*shapes), dtype=torch.float32, device=dev)
        x_kv, x_q, x_r, w_kv, w_q2, w_r, kv, q2, attn, pre = _carve(buf, *shapes)
        out = torch.empty((B, O), dtype=torch.float32, device=dev)
        cont = lambda t: None if t is None else t.contiguous()
        h, f, dt, time_w, time_b = cont(h), cont(f), cont(dt), cont(time_w), cont(time_b)
        params = [cont(t) for t in (w_q, b_q, w_k, b_k, w_v, b_v, w_out, b_out)]
        ln_w, ln_b = cont(ln_w), cont(ln_b)
        stream = stream_ptr(dev)
        with torch.cuda.device(dev):
            check(L.yitu_tattn_prepare(
                ptr(x_kv), ptr(x_q), ptr(x_r), ptr(w_kv), ptr(w_q2), ptr(w_r), ptr(h), ptr(f),
                ptr(dt), ptr(time_w), ptr(time_b), *[ptr(t) for t in params], c_i64(B), c_i64(E),
                c_i64(Dn), c_i64(De), c_i64(Dt), c_i64(O), c_i64(LD), stream), "yitu_tattn_prepare")
            if E > 0:
                _gemm_typed(L, dev, [kv, q2], [x_kv, x_q], [w_kv, w_q2], [E, B], [LD, LD], 2 * O,
                            0, 1, LD, LD, 2 * O, None)
            else:
                _gemm(L, dev, q2, x_q, w_q2, B, 2 * O, LD, 0, 1, LD, LD, 2 * O, None)
            check(L.yitu_tattn_forward(ptr(x_r), ptr(attn), ptr(q2), ptr(kv), ptr(indptr), c_i64(B),
                                       c_i64(E), c_i64(O), c_i64(num_head), c_i64(LD), stream),
                  "yitu_tattn_forward")
            _gemm(L, dev, pre, x_r, w_r, B, O, LD, 0, 1, LD, LD, O, None)
            check(L.yitu_relu_layernorm_forward(ptr(out), ptr(pre), ptr(ln_w), ptr(ln_b), c_i64(B),
                                                c_i64(O), c_f32(eps), stream),
                  "yitu_relu_layernorm_forward")
        ctx.dims = (B, E, Dn, De, Dt, O, int(num_head), LD, float(eps))
        ctx.views = (x_kv, x_q, x_r, w_kv, w_q2, w_r, kv, q2, attn, pre)  # views of one buffer
        ctx.save_for_backward(indptr, dt, time_w, time_b, ln_w)
        return out

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_out):
        B, E, Dn, De, Dt, O, H, LD, eps = ctx.dims
        x_kv, x_q, x_r, w_kv, w_q2, w_r, kv, q2, attn, pre = ctx.views
        indptr, dt, time_w, time_b, ln_w = ctx.saved_tensors
        dev = grad_out.device
        L = _lib.lib()
        L.yitu_tattn_partial_rows.restype = ctypes.c_int64
        rows_ln = int(L.yitu_tattn_partial_rows(c_i64(B)))
        rows_t = int(L.yitu_tattn_partial_rows(c_i64(B + E)))
        grad_out = grad_out.contiguous()
        shapes = ((B, 2 * O), (B, LD), (B, 2 * O), (E, 2 * O), (E, H, 2), (E, LD), (B, LD),
                  (rows_ln, 2 * O), (rows_t, 2 * max(Dt, 1)), (2 * O, LD), (O, LD), (O, LD))
        buf = torch.empty(_room(*shapes), dtype=torch.float32, device=dev)
        (d_pre2, dx_r, dq2, dkv, scratch, dx_kv, dx_q, part_ln, part_t, dw_kv, dw_q,
         dw_r) = _carve(buf, *shapes)
        # weight gradients with the bias gradient as their last column: [w_k | b_k ; w_v | b_v],
        # [w_q | b_q], [w_out | b_out]; the last launch unpacks them into one tensor per parameter
        Dkv, Dq, Dr = Dn + De + Dt, Dn + Dt, O + Dn
        gshapes = ((O, Dq), (O,), (O, Dkv), (O,), (O, Dkv), (O,), (O, Dr), (O,), (2, O),
                   (2, max(Dt, 1)))
        gbuf = torch.empty(_room(*gshapes), dtype=torch.float32, device=dev)
        g_wq, g_bq, g_wk, g_bk, g_wv, g_bv, g_wo, g_bo, d_ln, d_time = _carve(gbuf, *gshapes)
        need_h = Dn > 0 and ctx.needs_input_grad[4]
        need_f = De > 0 and ctx.needs_input_grad[5]
        grad_h = torch.empty((B + E, Dn), dtype=torch.float32, device=dev) if need_h else None
        grad_f = torch.empty((E, De), dtype=torch.float32, device=dev) if need_f else None
        ws_bytes = _lib.size_fn("yitu_sgemm_workspace_bytes")(c_i64(2 * O), c_i64(LD),
                                                              c_i64(max(E, B)), c_i64(3))
        ws = _lib.workspace(ws_bytes, dev)
        stream = stream_ptr(dev)
        with torch.cuda.device(dev):
            check(L.yitu_relu_layernorm_backward(ptr(d_pre2), ptr(part_ln), ptr(grad_out), ptr(pre),
                                                 ptr(ln_w), c_i64(B), c_i64(O), c_i64(2 * O),
                                                 c_f32(eps), stream), "yitu_relu_layernorm_backward")
            _gemm(L, dev, dx_r, d_pre2, w_r, B, LD, O, 0, 0, 2 * O, LD, LD, None)
            check(L.yitu_tattn_backward(ptr(dq2), ptr(dkv), ptr(scratch), ptr(dx_r), ptr(q2), ptr(kv),
                                        ptr(attn), ptr(indptr), c_i64(B), c_i64(E), c_i64(O),
                                        c_i64(H), c_i64(LD), stream), "yitu_tattn_backward")
            if E > 0:
                _gemm_typed(L, dev, [dx_kv, dx_q], [dkv, dq2], [w_kv, w_q2], [E, B], [2 * O, O], LD,
                            0, 0, 2 * O, LD, LD, None)
                _gemm_typed(L, dev, [dw_kv, dw_q, dw_r], [dkv, dq2, d_pre2], [x_kv, x_q, x_r],
                            [2 * O, O, O], [E, B, B], LD, 1, 0, 2 * O, LD, LD, ws)
            else:
                dw_kv.zero_()
                _gemm(L, dev, dx_q, dq2, w_q2, B, LD, O, 0, 0, 2 * O, LD, LD, None)
                _gemm_typed(L, dev, [dw_q, dw_r], [dq2, d_pre2], [x_q, x_r], [O, O], [B, B], LD, 1, 0,
                            2 * O, LD, LD, ws)
            check(L.yitu_tattn_finalize(ptr(grad_h), ptr(grad_f), ptr(part_t), ptr(dx_kv), ptr(dx_q),
                                        ptr(dx_r), ptr(dt), ptr(time_w), ptr(time_b), c_i64(B),
                                        c_i64(E), c_i64(Dn), c_i64(De), c_i64(Dt), c_i64(O),
                                        c_i64(LD), stream), "yitu_tattn_finalize")
            check(L.yitu_tattn_collect(
                ptr(d_ln), ptr(d_time), ptr(g_wq), ptr(g_bq), ptr(g_wk), ptr(g_bk), ptr(g_wv),
                ptr(g_bv), ptr(g_wo), ptr(g_bo), ptr(part_ln), c_i64(rows_ln), ptr(part_t),
                c_i64(rows_t), ptr(dw_kv), ptr(dw_q), ptr(dw_r), c_i64(Dn), c_i64(De), c_i64(Dt),
                c_i64(O), c_i64(LD), stream), "yitu_tattn_collect")
        g_time_w = d_time[0, :Dt].reshape(Dt, 1) if Dt > 0 else None
        g_time_b = d_time[1, :Dt] if Dt > 0 else None
        return (None, None, None, None, grad_h, grad_f, None, g_time_w, g_time_b,
                g_wq, g_bq, g_wk, g_bk, g_wv, g_bv, g_wo, g_bo, d_ln[0], d_ln[1])
