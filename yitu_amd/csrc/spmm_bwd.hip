// Backward of the multi-head edge-weighted SpMM:
//   grad_a[i,h]   = <grad_out[row_i,h,:], feat[col_i,h,:]>      (per-edge dot, this file)
//   grad_x[c,h,:] = sum_{i: col_i = c} values[i,h] grad_out[row_i,h,:]
// The second sum is a row gather over the transposed structure and reuses the
// forward kernels (launch_spmm with the edge permutation), so neither needs
// atomics.
#include "../../include/yitu_hip.h"
#include "dot_rows.hpp"

namespace yitu {

// Long rows: the plan's band-ordered items, kItemsPerWave per wave.
template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void dot_items_kernel(DotParams p) {
    const int lane = lane_id();
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int e_beg[kItemsPerWave], n_edges[kItemsPerWave], row[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            e_beg[j] = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            row[j] = __builtin_amdgcn_readlane(my_rec.w, j) & 0x7fffffff;
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
