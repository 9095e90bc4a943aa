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
#include "dot_rows.hpp"
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

// ---- backward ---------------------------------------------------------------------
// Two launches, each shared by the two graphs. The first runs the per-row passes: the
// per-edge dot products of A (grad of the SpMM's edge values) beside the softmax
// backward of B (grad_query and the per-edge logit gradient). The second runs the two
// by-source gathers that depend on them: grad_x of A over A^T beside grad_key of B
// as the sum of B^T's per-edge logit gradients. The reference's fused backward
// (hfused_cuda.cu:47-94) scatters both with atomics from one thread per row.
template <int G, int KT, int HP>
__global__ __launch_bounds__(kBlock) void hfused_bwd_rows_kernel(DotParams a, int a_blocks,
                                                                 SddmmParams b) {
    if ((int)blockIdx.x < a_blocks)
        dot_rows_body<4, G, KT>(a, blockIdx.x);
    else
        sddmm_bwd_rows_body<HP>(b, blockIdx.x - a_blocks);
}

// TINY = heads of B when they are 1, 2 or 4 (one lane per edge), else 0 (one lane per head)
template <int G, int KT, int TINY>
__global__ __launch_bounds__(kBlock) void hfused_bwd_sources_kernel(SpmmParams a, int a_blocks,
                                                                    SpmmParams b) {
    if ((int)blockIdx.x < a_blocks) {
        spmm_rows_body<4, G, KT, W_EDGEHEAD, float>(a, blockIdx.x, a_blocks);
    } else {
        if constexpr (TINY > 0)
            tiny_rows_body<TINY>(b, blockIdx.x - a_blocks);
        else
            spmm_rows_body<1, 64, 1, W_NONE, float>(b, blockIdx.x - a_blocks, 0);
    }
}

template <int G, int KT>
int launch_backward(const DotParams &a, const SddmmParams &b, const SpmmParams &at,
                    const SpmmParams &bt, hipStream_t stream) {
    {
        const int ga = (int)ceil_div(a.sp.n_rows, kWavesPerBlock * rows_per_wave(a.sp.n_rows));
        const int gb = (int)ceil_div(b.n_dst, kWavesPerBlock);
#define YITU_HF(HP)                                                                  \
    hfused_bwd_rows_kernel<G, KT, HP><<<ga + gb, kBlock, 0, stream>>>(a, ga, b);    \
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
    }
    int ga = (int)ceil_div(at.n_rows, kWavesPerBlock * rows_per_wave(at.n_rows));
    if (ga >= 64) ga = (ga + 7) / 8 * 8;
    const int gb = (int)ceil_div(bt.n_rows, kWavesPerBlock * rows_per_wave(bt.n_rows));
    const bool tiny = aligned16(bt.feat) && aligned16(bt.out);
    if (tiny && bt.L == 1)
        hfused_bwd_sources_kernel<G, KT, 1><<<ga + gb, kBlock, 0, stream>>>(at, ga, bt);
    else if (tiny && bt.L == 2)
        hfused_bwd_sources_kernel<G, KT, 2><<<ga + gb, kBlock, 0, stream>>>(at, ga, bt);
    else if (tiny && bt.L == 4)
        hfused_bwd_sources_kernel<G, KT, 4><<<ga + gb, kBlock, 0, stream>>>(at, ga, bt);
    else
        hfused_bwd_sources_kernel<G, KT, 0><<<ga + gb, kBlock, 0, stream>>>(at, ga, bt);
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

YITU_API size_t yitu_hfused_backward_workspace_bytes(int64_t n_rows, int64_t n_src_a,
                                                     int64_t nnz_a, int64_t row_len,
                                                     int64_t n_src_b, int64_t nnz_b,
                                                     int64_t n_heads, int64_t n_bid) {
    (void)n_src_a;
    (void)n_src_b;
    return std::max(yitu_spmm_workspace_bytes(nnz_a, row_len, 0),
                    std::max(yitu_sddmm_workspace_bytes(n_rows, nnz_b, n_heads, n_bid, 0),
                             yitu_spmm_workspace_bytes(nnz_b, n_heads, 0)));
}

YITU_API int yitu_hfused_backward(
    float *grad_values, float *grad_features, float *grad_query, float *grad_key, float *grad_edge,
    const float *spmm_values, const int32_t *spmm_indptr, const int32_t *spmm_indices,
    const float *spmm_features, const float *spmm_grad, const int32_t *spmm_t_indptr,
    const int32_t *spmm_t_rows, const int32_t *spmm_t_perm, const int32_t *sddmm_indptr,
    const int32_t *sddmm_indices, const float *sddmm_query, const float *sddmm_key,
    const float *sddmm_attn, const float *sddmm_grad, const int32_t *sddmm_t_indptr,
    const int32_t *sddmm_t_perm, int64_t n_rows, int64_t n_src_a, int64_t nnz_a, int64_t n_heads,
    int64_t n_features, int64_t n_src_b, int64_t nnz_b, int64_t n_bid, int64_t max_degree_a,
    int64_t max_degree_a_t, int64_t max_degree_b, int64_t max_degree_b_t, void *workspace,
    size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_rows >= 0 && n_src_a >= 0 && nnz_a >= 0 && n_heads >= 0 && n_features >= 0 &&
                     n_src_b >= 0 && nnz_b >= 0,
                 "negative size");
    YITU_REQUIRE(spmm_t_indptr && sddmm_t_indptr && (nnz_a == 0 || (spmm_t_rows && spmm_t_perm)) &&
                     (nnz_b == 0 || (sddmm_t_perm && grad_edge)),
                 "both by-source structures (yitu_csr_transpose) and a grad_edge buffer are needed");
    const int64_t L = n_heads * n_features;
    const auto known_below = [](int64_t d, int limit) { return d >= 0 && d < limit; };
    const bool two_launches =
        n_rows > 0 && nnz_a > 0 && nnz_b > 0 && n_src_a > 0 && n_src_b > 0 && L > 0 &&
        n_features % 4 == 0 && L <= 1024 && n_heads <= 16 && n_bid >= 1 && n_bid <= 16 &&
        n_rows < INT32_MAX && n_src_a <= (1 << 24) && n_src_b <= (1 << 24) && nnz_a < INT32_MAX &&
        nnz_b < INT32_MAX && known_below(max_degree_a, kPlanThreshold) &&
        known_below(max_degree_a_t, kPlanThreshold) && known_below(max_degree_b, kHubThreshold) &&
        known_below(max_degree_b_t, kPlanThreshold) && grad_values && grad_features &&
        grad_query && grad_key && spmm_values && spmm_indptr && spmm_indices && spmm_features &&
        spmm_grad && sddmm_indptr && sddmm_indices && sddmm_query && sddmm_key && sddmm_attn &&
        sddmm_grad && aligned16(spmm_features) && aligned16(spmm_grad) && aligned16(grad_features);
    // big graphs with rows of 256 / 512 / 1,024 floats: the SpMM backward's single by-source
    // gather for both of its gradients saves more than the shared launches do
    const bool one_gather_pays =
        nnz_a * L > ((int64_t)1 << 24) &&
        spmm_backward_one_gather_shape(n_heads, n_features, spmm_features, spmm_grad, grad_features);
    if (!two_launches || one_gather_pays) {
        int rc = spmm_backward_run(grad_values, grad_features, spmm_values, spmm_indptr,
                                   spmm_indices, spmm_features, spmm_grad, spmm_t_indptr,
                                   spmm_t_rows, spmm_t_perm, n_rows, n_src_a, nnz_a, n_heads,
                                   n_features, max_degree_a, max_degree_a_t, nullptr, nullptr,
                                   workspace, workspace_bytes, false, stream);
        if (rc) return rc;
        return sddmm_backward_run(grad_query, grad_key, grad_edge, sddmm_indptr, sddmm_indices,
                                  sddmm_query, sddmm_key, sddmm_attn, sddmm_grad, sddmm_t_indptr,
                                  sddmm_t_perm, n_rows, n_src_b, nnz_b, n_heads, n_bid,
                                  max_degree_b, max_degree_b_t, nullptr, nullptr, workspace,
                                  workspace_bytes, 0, stream);
    }
    DotParams a{};
    a.sp.indptr = spmm_indptr;
    a.sp.indices = spmm_indices;
    a.sp.feat = spmm_features;
    a.sp.n_rows = (int)n_rows;
    a.sp.n_src = (int)n_src_a;
    a.sp.L = (int)L;
    a.sp.F = (int)n_features;
    a.sp.H = (int)n_heads;
    a.sp.col_mask = 0xffffff;
    a.sp.plan = plan_none();
    a.grad_out = spmm_grad;
    a.grad_a = grad_values;
    const int lph = (int)(n_features / 4);
    a.lph = (lph <= 64 && (lph & (lph - 1)) == 0) ? lph : 0;
    SddmmParams b{};
    b.indptr = sddmm_indptr;
    b.indices = sddmm_indices;
    b.query = sddmm_query;
    b.key = sddmm_key;
    b.attn = const_cast<float *>(sddmm_attn);
    b.grad_out = sddmm_grad;
    b.grad_q = grad_query;
    b.grad_k = nullptr;
    b.grad_e = grad_edge;
    b.n_dst = (int)n_rows;
    b.H = (int)n_heads;
    b.n_bid = (int)n_bid;
    b.hub_threshold = 0x7fffffff;
    b.hub = HubQueue{};
    SpmmParams at{};
    at.indptr = spmm_t_indptr;
    at.indices = spmm_t_rows;
    at.feat = spmm_grad;
    at.out = grad_features;
    at.values = spmm_values;
    at.eperm = spmm_t_perm;
    at.n_rows = (int)n_src_a;
    at.n_src = (int)n_rows;
    at.L = (int)L;
    at.F = (int)n_features;
    at.H = (int)n_heads;
    at.col_mask = 0x7fffffff;
    at.alpha = 1.0f;
    at.plan = plan_none();
    SpmmParams bt{};
    bt.indptr = sddmm_t_indptr;
    bt.indices = sddmm_t_perm;
    bt.feat = grad_edge;
    bt.out = grad_key;
    bt.n_rows = (int)n_src_b;
    bt.n_src = (int)nnz_b;
    bt.L = bt.F = (int)n_heads;
    bt.H = 1;
    bt.col_mask = 0x7fffffff;
    bt.alpha = 1.0f;
    bt.plan = plan_none();
    const int lanes = (int)(L / 4);
    if (lanes <= 16) return launch_backward<16, 1>(a, b, at, bt, stream);
    if (lanes <= 32) return launch_backward<32, 1>(a, b, at, bt, stream);
    if (lanes <= 64) return launch_backward<64, 1>(a, b, at, bt, stream);
    if (lanes <= 128) return launch_backward<64, 2>(a, b, at, bt, stream);
    return launch_backward<64, 4>(a, b, at, bt, stream);
}
