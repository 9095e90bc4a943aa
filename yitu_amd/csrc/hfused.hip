// Horizontally fused SpMM || SDDMM: one launch that runs the edge-weighted SpMM of
// graph A and the SDDMM + LeakyReLU + edge softmax of graph B side by side
// (hfused_forward, YiTu_GNN/YiTu_H/src/entry.cpp:136-155; hfused_cuda.cu:5-45,96-137,
// where one thread walks row r of both graphs in turn). The two ops share nothing
// but the launch: here the first workgroups of the grid run the SpMM row kernel's
// body on A and the rest the SDDMM row kernel's body on B, so the chip is filled by
// both at once, which is the point for the small per-relation graphs of a
// heterogeneous layer where each op alone leaves most CUs idle. The single launch
// applies when neither graph has a row that needs the long-row machinery (A: 64
// edges, B: 512 edges) and the shapes are the vectorised ones; otherwise the two
// ops run one after the other.
#include "../../include/yitu_hip.h"
#include "sddmm_kernels.hpp"
#include "spmm_rows.hpp"

namespace yitu {

namespace {

template <int G, int KT, int HP>
__global__ __launch_bounds__(kBlock) void hfused_rows_kernel(SpmmParams a, int a_blocks,
                                                             SddmmParams b) {
    if ((int)blockIdx.x < a_blocks)
        spmm_rows_body<4, G, KT, W_EDGEHEAD, float>(a, blockIdx.x, a_blocks);
    else
        sddmm_fwd_rows_body<HP>(b, blockIdx.x - a_blocks);
}

template <int G, int KT>
int launch_heads(const SpmmParams &a, const SddmmParams &b, hipStream_t stream) {
    int ga = (int)ceil_div(a.n_rows, kWavesPerBlock * rows_per_wave(a.n_rows));
    if (ga >= 64) ga = (ga + 7) / 8 * 8;  // as the SpMM launches its row kernel (row_block)
    const int gb = (int)ceil_div(b.n_dst, kWavesPerBlock);
#define YITU_HF(HP)                                                              \
    hfused_rows_kernel<G, KT, HP><<<ga + gb, kBlock, 0, stream>>>(a, ga, b);     \
    break
    switch (b.H <= 1 ? 1 : b.H <= 2 ? 2 : b.H <= 4 ? 4 : b.H <= 8 ? 8 : 16) {
        case 1: YITU_HF(1);
        case 2: YITU_HF(2);
        case 4: YITU_HF(4);
        case 8: YITU_HF(8);
        default: YITU_HF(16);
    }
#undef YITU_HF
    YITU_LAUNCH_CHECK();
    return 0;
}

}  // namespace

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API size_t yitu_hfused_forward_workspace_bytes(int64_t n_rows, int64_t nnz_a, int64_t row_len,
                                                    int64_t nnz_b, int64_t n_heads, int64_t n_bid) {
    return std::max(yitu_spmm_workspace_bytes(nnz_a, row_len, 0),
                    yitu_sddmm_workspace_bytes(n_rows, nnz_b, n_heads, n_bid, 0));
}

YITU_API int yitu_hfused_forward(float *spmm_out, float *attn, const float *spmm_values,
                                 const int32_t *spmm_indptr, const int32_t *spmm_indices,
                                 const float *spmm_features, const int32_t *sddmm_indptr,
                                 const int32_t *sddmm_indices, const float *sddmm_query,
                                 const float *sddmm_key, int64_t n_rows, int64_t n_src_a,
                                 int64_t nnz_a, int64_t n_heads, int64_t n_features,
                                 int64_t n_src_b, int64_t nnz_b, int64_t n_bid,
                                 int64_t max_degree_a, int64_t max_degree_b, void *workspace,
                                 size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_rows >= 0 && n_src_a >= 0 && nnz_a >= 0 && n_heads >= 0 && n_features >= 0 &&
                     n_src_b >= 0 && nnz_b >= 0,
                 "negative size");
    const int64_t L = n_heads * n_features;
    const bool one_launch =
        n_rows > 0 && nnz_a > 0 && nnz_b > 0 && L > 0 && n_features % 4 == 0 && L <= 1024 &&
        n_heads <= 16 && n_bid >= 1 && n_bid <= 16 && n_rows < INT32_MAX &&
        n_src_a <= (1 << 24) && n_src_b <= (1 << 24) && nnz_a < INT32_MAX && nnz_b < INT32_MAX &&
        max_degree_a >= 0 && max_degree_a < kPlanThreshold && max_degree_b >= 0 &&
        max_degree_b < kHubThreshold && spmm_out && attn && spmm_values && spmm_indptr &&
        spmm_indices && spmm_features && sddmm_indptr && sddmm_indices && sddmm_query &&
        sddmm_key && aligned16(spmm_features) && aligned16(spmm_out);
    if (!one_launch) {
        // long rows or an unvectorised shape: the two ops, each with its own kernels
        int rc = yitu_spmm_forward(spmm_out, spmm_values, spmm_indptr, spmm_indices, spmm_features,
                                   n_rows, n_src_a, nnz_a, n_heads, n_features, max_degree_a,
                                   nullptr, workspace, workspace_bytes, stream_);
        if (rc) return rc;
        return yitu_sddmm_forward(attn, sddmm_indptr, sddmm_indices, sddmm_query, sddmm_key, n_rows,
                                  n_src_b, nnz_b, n_heads, n_bid, max_degree_b, nullptr, workspace,
                                  workspace_bytes, stream_);
    }
    SpmmParams a{};
    a.indptr = spmm_indptr;
    a.indices = spmm_indices;
    a.feat = spmm_features;
    a.out = spmm_out;
    a.values = spmm_values;
    a.n_rows = (int)n_rows;
    a.n_src = (int)n_src_a;
    a.L = (int)L;
    a.F = (int)n_features;
    a.H = (int)n_heads;
    a.col_mask = 0xffffff;
    a.alpha = 1.0f;
    a.plan = plan_none();
    SddmmParams b{};
    b.indptr = sddmm_indptr;
    b.indices = sddmm_indices;
    b.query = sddmm_query;
    b.key = sddmm_key;
    b.attn = attn;
    b.n_dst = (int)n_rows;
    b.H = (int)n_heads;
    b.n_bid = (int)n_bid;
    b.hub_threshold = 0x7fffffff;
    b.hub = HubQueue{};
    const int lanes = (int)(L / 4);
    if (lanes <= 16) return launch_heads<16, 1>(a, b, stream);
    if (lanes <= 32) return launch_heads<32, 1>(a, b, stream);
    if (lanes <= 64) return launch_heads<64, 1>(a, b, stream);
    if (lanes <= 128) return launch_heads<64, 2>(a, b, stream);
    return launch_heads<64, 4>(a, b, stream);
}
