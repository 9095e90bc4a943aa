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
    const int32_t *indptr;
    const int32_t *indices;
    const float *feat;      // [n_src, L]
    const float *grad_out;  // [n_dst, L]
    float *grad_a;          // [nnz, H]
    int n_rows, L, F, H;
    int lph;       // lanes per head (F / VEC) when that is a power of two <= G, else 0
    int hub_threshold;
    HubQueue hub;  // only the row/item lists are used
};

// Dot products for edges [e_beg, e_end) of `row`; gt holds the row's grad_out tile.
template <int VEC, int G, int KT>
__device__ __forceinline__ void dot_edges(const DotParams &p, int row, int e_beg, int e_end) {
    constexpr int SLOTS = kWave / G;
    const int lane = lane_id();
    const int slot = lane / G, sub = lane % G;
    const float *__restrict__ feat = p.feat;

    for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
        int off[KT], head[KT];
        bool live[KT];
        float gt[KT][VEC];
#pragma unroll
        for (int t = 0; t < KT; t++) {
            off[t] = c0 + (t * G + sub) * VEC;
            live[t] = off[t] < p.L;
            if (!live[t]) off[t] = 0;
            head[t] = off[t] / p.F;
            RowLoad<VEC, float>::ld(p.grad_out + (size_t)row * p.L + off[t], gt[t]);
            if (!live[t])
#pragma unroll
                for (int i = 0; i < VEC; i++) gt[t][i] = 0.0f;
        }
        // first head of this column tile, used by the generic reduction
        const int h_lo = c0 / p.F;
        const int h_hi = min(p.H - 1, (min(p.L, c0 + G * VEC * KT) - 1) / p.F);

        for (int base = e_beg; base < e_end; base += kWave) {
            const int n = min(kWave, e_end - base);
            const int my_col = p.indices[base + min(lane, n - 1)] & 0xffffff;
            for (int s = 0; s < n; s += SLOTS) {
                const int src = s + slot;
                const bool valid = src < n;
                const int c = __shfl(my_col, src, kWave);
                float part[KT];
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    float v[VEC];
                    RowLoad<VEC, float>::ld(feat + (size_t)c * p.L + off[t], v);
                    float d = 0.0f;
#pragma unroll
                    for (int i = 0; i < VEC; i++) d += gt[t][i] * v[i];
                    part[t] = d;
                }
                const size_t e = (size_t)(base + src);
                if (p.lph > 0 && p.lph <= G) {
                    // a head is lph consecutive lanes of one tile
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        float d = part[t];
                        for (int o = p.lph >> 1; o >= 1; o >>= 1) d += __shfl_xor(d, o, kWave);
                        if (valid && live[t] && (sub & (p.lph - 1)) == 0)
                            p.grad_a[e * p.H + head[t]] = d;
                    }
                } else {
                    // generic shapes: one masked reduction per head present in the tile
                    for (int h = h_lo; h <= h_hi; h++) {
                        float d = 0.0f;
#pragma unroll
                        for (int t = 0; t < KT; t++)
                            if (live[t] && head[t] == h) d += part[t];
                        d = group_sum<G>(d);
                        if (valid && sub == 0) {
                            float *dst = p.grad_a + e * p.H + h;
                            // a head that started in an earlier column pass keeps its partial
                            if (h * p.F < c0)
                                *dst += d;
                            else
                                *dst = d;
                        }
                    }
                }
            }
        }
    }
}

template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void spmm_bwd_dot_rows_kernel(DotParams p) {
    const int row = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (row >= p.n_rows) return;
    const int beg = p.indptr[row], end = p.indptr[row + 1];
    if (end == beg) return;
    if (end - beg >= p.hub_threshold) {
        queue_hub_row(p.hub, row, end - beg);
        return;
    }
    dot_edges<VEC, G, KT>(p, row, beg, end);
}

template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void spmm_bwd_dot_hub_kernel(DotParams p) {
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);
    const int wave = threadIdx.x / kWave;
    constexpr int kPerWave = kHubChunk / kWavesPerBlock;
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int4 it = p.hub.items[item];
        const int beg = p.indptr[it.x] + it.y * kHubChunk;
        const int end = min(p.indptr[it.x + 1], beg + kHubChunk);
        const int wbeg = min(end, beg + wave * kPerWave), wend = min(end, wbeg + kPerWave);
        if (wend > wbeg) dot_edges<VEC, G, KT>(p, it.x, wbeg, wend);
    }
}

template <int VEC, int G, int KT>
static int dot_launch(const DotParams &p, bool with_hub, hipStream_t stream) {
    if (with_hub) {
        zero_hub_counters_kernel<<<1, kWave, 0, stream>>>(p.hub.counters);
        YITU_LAUNCH_CHECK();
    }
    spmm_bwd_dot_rows_kernel<VEC, G, KT>
        <<<(int)ceil_div(p.n_rows, kWavesPerBlock), kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (with_hub) {
        spmm_bwd_dot_hub_kernel<VEC, G, KT>
            <<<(int)std::min<int64_t>(p.hub.max_items, 4096), kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int VEC>
static int dot_dispatch(DotParams &p, bool with_hub, hipStream_t stream) {
    const int lanes = (p.L + VEC - 1) / VEC;
    const int lph = p.F % VEC == 0 ? p.F / VEC : 0;
    p.lph = (lph > 0 && lph <= 64 && (lph & (lph - 1)) == 0) ? lph : 0;
    if constexpr (VEC == 4) {
        if (lanes <= 16) return dot_launch<4, 16, 1>(p, with_hub, stream);
        if (lanes <= 32) return dot_launch<4, 32, 1>(p, with_hub, stream);
        if (lanes <= 64) return dot_launch<4, 64, 1>(p, with_hub, stream);
        if (lanes <= 128) return dot_launch<4, 64, 2>(p, with_hub, stream);
        return dot_launch<4, 64, 4>(p, with_hub, stream);
    } else {
        if (lanes <= 64) return dot_launch<VEC, 64, 1>(p, with_hub, stream);
        return dot_launch<VEC, 64, 4>(p, with_hub, stream);
    }
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
                                int64_t max_degree_t, void *workspace, size_t workspace_bytes,
                                void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_dst >= 0 && n_src >= 0 && nnz >= 0 && n_heads >= 0 && n_features >= 0,
                 "negative size");
    const int64_t L = n_heads * n_features;
    if (L == 0) return 0;
    YITU_REQUIRE(n_dst < INT32_MAX && n_src <= (1 << 24) && L < (1 << 20) && nnz < INT32_MAX,
                 "size out of range (columns are 24-bit)");
    YITU_REQUIRE(indptr && (nnz == 0 || (indices && features && grad_out)), "null input");
    YITU_REQUIRE(grad_a || grad_x, "no output requested");
    YITU_REQUIRE(!grad_x || nnz == 0 || values, "grad_x needs the edge values");
    YITU_REQUIRE(!grad_x || (t_indptr && (nnz == 0 || (t_rows && t_perm))),
                 "grad_x needs the transposed structure (yitu_csr_transpose)");

    if (grad_a && nnz > 0 && n_dst > 0) {
        DotParams p{};
        p.indptr = indptr;
        p.indices = indices;
        p.feat = features;
        p.grad_out = grad_out;
        p.grad_a = grad_a;
        p.n_rows = (int)n_dst;
        p.L = (int)L;
        p.F = (int)n_features;
        p.H = (int)n_heads;
        const bool with_hub =
            nnz >= kHubThreshold && !(max_degree >= 0 && max_degree < kHubThreshold);
        p.hub_threshold = with_hub ? kHubThreshold : 0x7fffffff;
        if (with_hub) {
            int rc = hub512_queue_init(p.hub, workspace, workspace_bytes, nnz);
            if (rc) return rc;
        }
        int rc;
        const bool al = aligned16(features) && aligned16(grad_out);
        if (n_features % 4 == 0 && al)
            rc = dot_dispatch<4>(p, with_hub, stream);
        else if (n_features % 2 == 0 && al)
            rc = dot_dispatch<2>(p, with_hub, stream);
        else
            rc = dot_dispatch<1>(p, with_hub, stream);
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
        return launch_spmm(sp, W_EDGEHEAD, false, nnz, max_degree_t, workspace, workspace_bytes,
                           stream);
    }
    return 0;
}
