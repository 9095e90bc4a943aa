// Backward of the multi-head edge-weighted SpMM:
//   grad_a[i,h]   = <grad_out[row_i,h,:], feat[col_i,h,:]>      (per-edge dot, this file)
//   grad_x[c,h,:] = sum_{i: col_i = c} values[i,h] grad_out[row_i,h,:]
// The second sum is a row gather over the transposed structure and reuses the
// forward kernels (launch_spmm with the edge permutation), so neither needs
// atomics.
#include "../../include/yitu_hip.h"
#include "spmm_rows.hpp"

namespace yitu {

struct DotParams {
    SpmmParams sp;          // indptr, indices, feat, n_rows, L, F, H, col_mask, plan
    const float *grad_out;  // [n_dst, L]
    float *grad_a;          // [nnz, H]
    int lph;  // lanes per head (F / VEC) when that is a power of two <= G, else 0
    int long_rows_only;  // the rows below the plan threshold were handled by another kernel
};

// Dot products of the row's grad_out tile `gt` with the n edges in window lanes
// [first, first + n); edge k of them is CSR edge e0 + k.
template <int VEC, int G, int KT, int UNROLL = (KT >= 4 ? 2 : 4)>
__device__ __forceinline__ void dot_window(const DotParams &p, const float (&gt)[KT][VEC],
                                           const TileLanes<VEC, G, KT, W_EDGEHEAD> &tl,
                                           const EdgeWindow &win, int first, int n, int e0,
                                           int c0) {
    constexpr int SLOTS = kWave / G;
    const int lane = lane_id();
    const int slot = lane / G, sub = lane % G;
    const float *__restrict__ feat = static_cast<const float *>(p.sp.feat);
    const int L = p.sp.L, F = p.sp.F, H = p.sp.H;
    // heads present in this column tile, for the generic reduction
    const int h_lo = c0 / F;
    const int h_hi = min(H - 1, (min(L, c0 + G * VEC * KT) - 1) / F);

    for (int s0 = 0; s0 < n; s0 += SLOTS * UNROLL) {
        float v[UNROLL][KT][VEC];
        // all gathers of the group first
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int k = min(s0 + u * SLOTS + slot, n - 1);
            const int c = __shfl(win.col, first + k, kWave);
            if (s0 + u * SLOTS < n) {  // wave-uniform
#pragma unroll
                for (int t = 0; t < KT; t++)
                    RowLoad<VEC, float>::ld(feat + (size_t)c * L + tl.off[t], v[u][t]);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            if (s0 + u * SLOTS >= n) break;  // wave-uniform
            const int k = s0 + u * SLOTS + slot;
            const bool valid = k < n;
            const size_t e = (size_t)(e0 + min(k, n - 1));
            float part[KT];
#pragma unroll
            for (int t = 0; t < KT; t++) {
                float d = 0.0f;
#pragma unroll
                for (int i = 0; i < VEC; i++) d += gt[t][i] * v[u][t][i];
                part[t] = d;
            }
            if (p.lph > 0) {
                // a head is lph consecutive lanes of one tile
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    float d = part[t];
                    for (int o = p.lph >> 1; o >= 1; o >>= 1) d += __shfl_xor(d, o, kWave);
                    if (valid && tl.live[t] && (sub & (p.lph - 1)) == 0)
                        p.grad_a[e * H + tl.head[t]] = d;
                }
            } else {
                // generic shapes: one masked reduction per head present in the tile
                for (int h = h_lo; h <= h_hi; h++) {
                    float d = 0.0f;
#pragma unroll
                    for (int t = 0; t < KT; t++)
                        if (tl.live[t] && tl.head[t] == h) d += part[t];
                    d = group_sum<G>(d);
                    if (valid && sub == 0) {
                        float *dst = p.grad_a + e * H + h;
                        // a head that started in an earlier column pass keeps its partial
                        if (h * F < c0)
                            *dst += d;
                        else
                            *dst = d;
                    }
                }
            }
        }
    }
}

template <int VEC, int G, int KT>
__device__ __forceinline__ void load_grad_tile(float (&gt)[KT][VEC], const DotParams &p,
                                               const TileLanes<VEC, G, KT, W_EDGEHEAD> &tl,
                                               int row) {
#pragma unroll
    for (int t = 0; t < KT; t++) {
        RowLoad<VEC, float>::ld(p.grad_out + (size_t)row * p.sp.L + tl.off[t], gt[t]);
        if (!tl.live[t])
#pragma unroll
            for (int i = 0; i < VEC; i++) gt[t][i] = 0.0f;
    }
}

// Short rows: a wave walks rows_per_wave consecutive rows through a sliding edge window.
template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void dot_rows_kernel(DotParams p) {
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.sp.n_rows);
    const int r0 = (blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * rpw;
    if (r0 >= p.sp.n_rows) return;
    const int n_here = min(rpw, p.sp.n_rows - r0);
    const int my_ptr = p.sp.indptr[r0 + min(lane, n_here)];
    const int limit = __shfl(my_ptr, n_here, kWave);
    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;
    for (int i = 0; i < n_here; i++) {
        const int beg = __shfl(my_ptr, i, kWave), end = __shfl(my_ptr, i + 1, kWave);
        if (end == beg || end - beg >= p.sp.plan.threshold) continue;
        for (int c0 = 0; c0 < p.sp.L; c0 += G * VEC * KT) {
            const TileLanes<VEC, G, KT, W_EDGEHEAD> tl(p.sp, c0);
            float gt[KT][VEC];
            load_grad_tile<VEC, G, KT>(gt, p, tl, r0 + i);
            for (int b = beg; b < end; b += kWave) {
                const int n = min(kWave, end - b);
                if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                    load_window<W_NONE>(win, p.sp, b, limit);
                dot_window<VEC, G, KT>(p, gt, tl, win, b - win.base, n, b, c0);
            }
        }
    }
}

// Long rows: the plan's band-ordered items, kItemsPerWave per wave.
template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void dot_items_kernel(DotParams p) {
    const int lane = lane_id();
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int e_beg[kItemsPerWave], n_edges[kItemsPerWave], row[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            e_beg[j] = __shfl(my_rec.x, j, kWave);
            const int end = __shfl(my_rec.y, j, kWave);
            row[j] = __shfl(my_rec.w, j, kWave) & 0x7fffffff;
            n_edges[j] = j < n_here ? end - e_beg[j] : 0;
            if (n_edges[j] > 0) load_window<W_NONE>(win[j], p.sp, e_beg[j], end);
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            if (n_edges[j] <= 0) continue;
            for (int c0 = 0; c0 < p.sp.L; c0 += G * VEC * KT) {
                const TileLanes<VEC, G, KT, W_EDGEHEAD> tl(p.sp, c0);
                float gt[KT][VEC];
                load_grad_tile<VEC, G, KT>(gt, p, tl, row[j]);
                dot_window<VEC, G, KT>(p, gt, tl, win[j], 0, n_edges[j], e_beg[j], c0);
            }
        }
    }
}

template <int VEC, int G, int KT>
static int dot_launch(const DotParams &p, bool has_items, hipStream_t stream) {
    if (!p.long_rows_only) {
        dot_rows_kernel<VEC, G, KT>
            <<<(int)ceil_div(p.sp.n_rows, kWavesPerBlock * rows_per_wave(p.sp.n_rows)), kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    if (has_items) {
        const int grid = (int)std::min<int64_t>(
            ceil_div(p.sp.plan.max_items, kWavesPerBlock * kItemsPerWave), 1 << 16);
        dot_items_kernel<VEC, G, KT><<<grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int VEC>
static int dot_dispatch(DotParams &p, bool has_items, hipStream_t stream) {
    const int lanes = (p.sp.L + VEC - 1) / VEC;
    const int lph = p.sp.F % VEC == 0 ? p.sp.F / VEC : 0;
    p.lph = (lph > 0 && lph <= 64 && (lph & (lph - 1)) == 0) ? lph : 0;
    if constexpr (VEC == 4) {
        if (lanes <= 16) return dot_launch<4, 16, 1>(p, has_items, stream);
        if (lanes <= 32) return dot_launch<4, 32, 1>(p, has_items, stream);
        if (lanes <= 64) return dot_launch<4, 64, 1>(p, has_items, stream);
        if (lanes <= 128) return dot_launch<4, 64, 2>(p, has_items, stream);
        return dot_launch<4, 64, 4>(p, has_items, stream);
    } else {
        if (lanes <= 64) return dot_launch<VEC, 64, 1>(p, has_items, stream);
        return dot_launch<VEC, 64, 4>(p, has_items, stream);
    }
}


// The body of yitu_spmm_backward. With long_rows_only the per-edge dot skips
// the rows below the plan threshold (the fused GAT backward has done them).
int spmm_backward_run(float *grad_a, float *grad_x, const float *values, const int32_t *indptr,
                      const int32_t *indices, const float *features, const float *grad_out,
                      const int32_t *t_indptr, const int32_t *t_rows, const int32_t *t_perm,
                      int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads,
                      int64_t n_features, int64_t max_degree, int64_t max_degree_t,
                      const void *plan, const void *plan_t, void *workspace,
                      size_t workspace_bytes, bool long_rows_only, hipStream_t stream) {
    YITU_REQUIRE(n_dst >= 0 && n_src >= 0 && nnz >= 0 && n_heads >= 0 && n_features >= 0,
                 "negative size");
    const int64_t L = n_heads * n_features;
    if (L == 0) return 0;
    YITU_REQUIRE(n_dst < INT32_MAX && n_src <= (1 << 24) && L < (1 << 20) && nnz < INT32_MAX,
                 "size out of range (columns are 24-bit)");
    YITU_REQUIRE(indptr && (nnz == 0 || (indices && features && grad_out)), "null input");
    if (nnz == 0 && n_src == 0) return 0;  // both gradients are empty
    YITU_REQUIRE(grad_a || grad_x, "no output requested");
    YITU_REQUIRE(!grad_x || nnz == 0 || values, "grad_x needs the edge values");
    YITU_REQUIRE(!grad_x || (t_indptr && (nnz == 0 || (t_rows && t_perm))),
                 "grad_x needs the transposed structure (yitu_csr_transpose)");

    if (grad_a && grad_x && nnz > 0 && n_dst > 0 && n_src > 0 && !long_rows_only &&
        spmm_backward_one_gather_shape(n_heads, n_features, features, grad_out, grad_x))
        return spmm_backward_one_gather(grad_a, grad_x, values, features, grad_out, t_indptr,
                                        t_rows, t_perm, n_dst, n_src, nnz, n_heads, n_features,
                                        max_degree_t, plan_t, workspace, workspace_bytes, stream);
    if (grad_a && nnz > 0 && n_dst > 0) {
        DotParams p{};
        p.sp.indptr = indptr;
        p.sp.indices = indices;
        p.sp.feat = features;
        p.sp.n_rows = (int)n_dst;
        p.sp.n_src = (int)n_src;
        p.sp.L = (int)L;
        p.sp.F = (int)n_features;
        p.sp.H = (int)n_heads;
        p.sp.col_mask = 0xffffff;
        p.grad_out = grad_out;
        p.grad_a = grad_a;
        p.long_rows_only = long_rows_only ? 1 : 0;
        bool has_items = false;
        void *rest = nullptr;
        size_t rest_bytes = 0;
        int rc = plan_resolve(p.sp.plan, has_items, plan, indptr, indices, n_dst, n_src, nnz,
                              0xffffff, max_degree, workspace, workspace_bytes, &rest, &rest_bytes,
                              stream);
        if (rc) return rc;
        const bool al = aligned16(features) && aligned16(grad_out);
        if (n_features % 4 == 0 && al)
            rc = dot_dispatch<4>(p, has_items, stream);
        else if (n_features % 2 == 0 && al)
            rc = dot_dispatch<2>(p, has_items, stream);
        else
            rc = dot_dispatch<1>(p, has_items, stream);
        if (rc) return rc;
    }
    if (grad_x && n_src > 0) {
        // grad_x = A^T-weighted gather: rows = sources, "columns" = destination rows
        SpmmParams sp{};
        sp.indptr = t_indptr;
        sp.indices = t_rows;
        sp.feat = grad_out;
        sp.out = grad_x;
        sp.values = values;
        sp.eperm = t_perm;
        sp.n_rows = (int)n_src;
        sp.n_src = (int)n_dst;
        sp.L = (int)L;
        sp.F = (int)n_features;
        sp.H = (int)n_heads;
        sp.col_mask = 0x7fffffff;
        sp.alpha = 1.0f;
        return launch_spmm(sp, W_EDGEHEAD, false, nnz, max_degree_t, plan_t, workspace,
                           workspace_bytes, stream);
    }
    return 0;
}

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API int yitu_spmm_backward(float *grad_a, float *grad_x, const float *values,
                                const int32_t *indptr, const int32_t *indices,
                                const float *features, const float *grad_out,
                                const int32_t *t_indptr, const int32_t *t_rows,
                                const int32_t *t_perm, int64_t n_dst, int64_t n_src, int64_t nnz,
                                int64_t n_heads, int64_t n_features, int64_t max_degree,
                                int64_t max_degree_t, const void *plan, const void *plan_t,
                                void *workspace, size_t workspace_bytes, void *stream_) {
    return spmm_backward_run(grad_a, grad_x, values, indptr, indices, features, grad_out, t_indptr,
                             t_rows, t_perm, n_dst, n_src, nnz, n_heads, n_features, max_degree,
                             max_degree_t, plan, plan_t, workspace, workspace_bytes, false,
                             static_cast<hipStream_t>(stream_));
}
