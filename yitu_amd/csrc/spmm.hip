// Instantiation table and host-side launch logic of the row-split SpMM.
#include "packed_rows.hpp"

#include <cstdarg>

namespace yitu {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
const char *last_error() { return g_error; }

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(float *p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (; i < n; i += stride) p[i] = 0.0f;
}

int fill_zero(float *p, int64_t n, hipStream_t stream) {
    if (n <= 0) return 0;
    const int grid = (int)std::min<int64_t>(ceil_div(n, kBlock), 8192);
    fill_zero_kernel<<<grid, kBlock, 0, stream>>>(p, n);
    YITU_LAUNCH_CHECK();
    return 0;
}

// w[e] = scale[col[e]]: the per-edge column scale of the GCN norm, computed once
// per graph so that the aggregation kernels read it in edge order.
__global__ __launch_bounds__(kBlock) void edge_scale_kernel(float *__restrict__ w,
                                                            const int32_t *__restrict__ indices,
                                                            const float *__restrict__ scale,
                                                            int64_t nnz, int col_mask) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (; i < nnz; i += stride) w[i] = scale[indices[i] & col_mask];
}

int edge_scale_fill(float *w, const int32_t *indices, const float *scale, int64_t nnz, int col_mask,
                    hipStream_t stream) {
    if (nnz <= 0) return 0;
    edge_scale_kernel<<<(int)std::min<int64_t>(ceil_div(nnz, kBlock), 16384), kBlock, 0, stream>>>(
        w, indices, scale, nnz, col_mask);
    YITU_LAUNCH_CHECK();
    return 0;
}

size_t spmm_workspace_bytes(int64_t nnz, int64_t L, bool with_plan) {
    size_t b = align_up(sizeof(float) * (size_t)plan_max_items(nnz) * (size_t)L, 256);
    if (!with_plan) b += plan_temp_bytes(nnz);
    return b + 256;
}

template <int VEC, int G, int KT, int WMODE, typename TIN>
static int launch_variant(const SpmmParams &p, bool has_items, hipStream_t stream) {
    int grid = (int)ceil_div(p.n_rows, kWavesPerBlock * rows_per_wave(p.n_rows));
    if (grid >= 64) grid = (grid + 7) / 8 * 8;  // whole eighths for row_block
    spmm_rows_kernel<VEC, G, KT, WMODE, TIN><<<grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (has_items) {
        // whole-wave rows (1 KB and more per gather): one item per wave and a grid that walks
        // the list once; narrower rows: four items per wave, the grid capped
        constexpr int IPW = (G == kWave && KT == 1) ? 1 : kItemsPerWave;
        const int item_grid = (int)std::min<int64_t>(
            ceil_div(p.plan.max_items, kWavesPerBlock * IPW), IPW == 1 ? 1 << 20 : 1 << 16);
        spmm_items_kernel<VEC, G, KT, WMODE, TIN, IPW><<<item_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        const int red_grid = (int)std::min<int64_t>(p.plan.max_rows, 1 << 16);
        constexpr int RV = VEC >= 4 ? 4 : VEC;  // VEC | L whenever this variant is chosen
        if (p.L % RV == 0)
            spmm_reduce_kernel<WMODE, RV><<<red_grid, kBlock, 0, stream>>>(p);
        else
            spmm_reduce_kernel<WMODE, 1><<<red_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int WMODE, typename TIN, int VEC>
static int dispatch_shape(const SpmmParams &p, bool with_hub, hipStream_t stream) {
    const int lanes = (p.L + VEC - 1) / VEC;
    if constexpr (VEC >= 4) {
        if (lanes <= 16) return launch_variant<VEC, 16, 1, WMODE, TIN>(p, with_hub, stream);
        if (lanes <= 32) return launch_variant<VEC, 32, 1, WMODE, TIN>(p, with_hub, stream);
        if (lanes <= 64) return launch_variant<VEC, 64, 1, WMODE, TIN>(p, with_hub, stream);
        if (lanes <= 128) return launch_variant<VEC, 64, 2, WMODE, TIN>(p, with_hub, stream);
        if constexpr (VEC == 4) return launch_variant<VEC, 64, 4, WMODE, TIN>(p, with_hub, stream);
        return launch_variant<VEC, 64, 2, WMODE, TIN>(p, with_hub, stream);
    } else {
        if (lanes <= 64) return launch_variant<VEC, 64, 1, WMODE, TIN>(p, with_hub, stream);
        return launch_variant<VEC, 64, 4, WMODE, TIN>(p, with_hub, stream);
    }
}

// Unweighted fp32 rows of 1, 2 or 4 floats: one lane per edge.
template <int VEC>
static int launch_tiny(const SpmmParams &p, bool has_items, hipStream_t stream) {
    const int R = packed_rows_per_wave(p.n_rows);
    tiny_rows_packed_kernel<VEC>
        <<<(int)ceil_div(p.n_rows, (int64_t)kWavesPerBlock * R), kBlock, 0, stream>>>(p, R);
    YITU_LAUNCH_CHECK();
    if (has_items && p.cols_are_edges) {
        // a row's edges are contiguous: sum them in place, no items
        edge_sum_long_kernel<VEC>
            <<<(int)std::min<int64_t>(std::max<int64_t>(p.plan.max_rows, 2), 1 << 14), kBlock, 0,
               stream>>>(p);
        YITU_LAUNCH_CHECK();
        return 0;
    }
    if (has_items) {
        const int item_grid = (int)std::min<int64_t>(
            ceil_div(p.plan.max_items, kWavesPerBlock * kItemsPerWave), 1 << 16);
        tiny_items_kernel<VEC><<<item_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        spmm_reduce_kernel<W_NONE, VEC>
            <<<(int)std::min<int64_t>(p.plan.max_rows, 1 << 16), kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int WMODE>
static int dispatch_type(const SpmmParams &p, bool bf16_in, bool with_hub, hipStream_t stream) {
    if constexpr (WMODE == W_NONE) {
        if (!bf16_in && aligned16(p.feat) && aligned16(p.out)) {
            if (p.L == 4) return launch_tiny<4>(p, with_hub, stream);
            if (p.L == 2) return launch_tiny<2>(p, with_hub, stream);
            if (p.L == 1) return launch_tiny<1>(p, with_hub, stream);
        }
    }
    // a lane's VEC elements must stay inside one head and one aligned vector
    const int unit = WMODE == W_EDGEHEAD ? p.F : p.L;
    if (bf16_in) {
        if (unit % 8 == 0 && aligned16(p.feat) && aligned16(p.out))
            return dispatch_shape<WMODE, bf16_t, 8>(p, with_hub, stream);
        return dispatch_shape<WMODE, bf16_t, 1>(p, with_hub, stream);
    }
    if (unit % 4 == 0 && aligned16(p.feat) && aligned16(p.out))
        return dispatch_shape<WMODE, float, 4>(p, with_hub, stream);
    if (unit % 2 == 0 && aligned16(p.feat) && aligned16(p.out))
        return dispatch_shape<WMODE, float, 2>(p, with_hub, stream);
    return dispatch_shape<WMODE, float, 1>(p, with_hub, stream);
}

int launch_spmm(SpmmParams &p, int wmode, bool bf16_in, int64_t nnz, int64_t max_degree_hint,
                const void *plan, void *workspace, size_t workspace_bytes, hipStream_t stream) {
    if (p.n_rows == 0 || p.L == 0) return 0;
    YITU_REQUIRE(nnz < (int64_t)1 << 31 && (int64_t)p.n_rows * p.L < ((int64_t)1 << 40),
                 "problem exceeds the int32 edge-index range");
    bool with_hub = false;
    void *rest = nullptr;
    size_t rest_bytes = 0;
    int rc = plan_resolve(p.plan, with_hub, plan, p.indptr, p.indices, p.n_rows, p.n_src, nnz,
                          p.col_mask, max_degree_hint, workspace, workspace_bytes, &rest,
                          &rest_bytes, stream);
    if (rc) return rc;
    p.partial = nullptr;
    if (with_hub) {
        const size_t need = sizeof(float) * (size_t)p.plan.max_items * (size_t)p.L;
        YITU_REQUIRE(rest && rest_bytes >= need,
                     "workspace too small for the partial rows: need %zu more bytes, got %zu", need,
                     rest_bytes);
        p.partial = static_cast<float *>(rest);
    }
    switch (wmode) {
        case W_NONE: return dispatch_type<W_NONE>(p, bf16_in, with_hub, stream);
        case W_DEGPROD: return dispatch_type<W_DEGPROD>(p, bf16_in, with_hub, stream);
        case W_EDGEHEAD: return dispatch_type<W_EDGEHEAD>(p, bf16_in, with_hub, stream);
    }
    set_error("unknown weight mode %d", wmode);
    return -1;
}

}  // namespace yitu
