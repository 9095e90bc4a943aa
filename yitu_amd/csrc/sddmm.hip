// Host side and C ABI of the SDDMM + LeakyReLU + edge-softmax op.
#include "../../include/yitu_hip.h"
#include "sddmm_kernels.hpp"

namespace yitu {

// ---- host side -------------------------------------------------------------
static inline int64_t sd_max_rows(int64_t nnz) { return nnz / kHubThreshold + 1; }
static inline int64_t sd_max_items(int64_t nnz) { return nnz / kHubChunk + sd_max_rows(nnz) + 1; }

static size_t sddmm_ws_bytes(int64_t nnz, int64_t H, int64_t n_bid) {
    size_t b = 256;
    b += align_up(sizeof(int4) * (size_t)sd_max_rows(nnz), 256);
    b += align_up(sizeof(int4) * (size_t)sd_max_items(nnz), 256);
    b += align_up(sizeof(float) * 3 * (size_t)(sd_max_items(nnz) * n_bid * H), 256);
    b += align_up(sizeof(float) * 3 * (size_t)(sd_max_rows(nnz) * n_bid * H), 256);
    return b;
}

static int sddmm_setup(SddmmParams &p, int64_t nnz, int64_t max_degree, void *workspace,
                       size_t workspace_bytes, bool &with_hub) {
    with_hub = nnz >= kHubThreshold && !(max_degree >= 0 && max_degree < kHubThreshold);
    p.hub_threshold = with_hub ? kHubThreshold : 0x7fffffff;
    p.hub = HubQueue{};
    if (!with_hub) return 0;
    const size_t need = sddmm_ws_bytes(nnz, p.H, p.n_bid);
    YITU_REQUIRE(workspace && workspace_bytes >= need, "workspace too small: need %zu bytes", need);
    YITU_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "workspace must be 256-byte aligned");
    char *w = static_cast<char *>(workspace);
    p.hub.counters = reinterpret_cast<HubCounters *>(w);
    w += 256;
    p.hub.max_rows = (int)sd_max_rows(nnz);
    p.hub.max_items = (int)sd_max_items(nnz);
    p.hub.chunk = kHubChunk;
    p.hub.rows = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)p.hub.max_rows, 256);
    p.hub.items = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)p.hub.max_items, 256);
    p.hub.partial = reinterpret_cast<float *>(w);
    w += align_up(sizeof(float) * 3 * (size_t)p.hub.max_items * p.n_bid * p.H, 256);
    p.rowstat = reinterpret_cast<float *>(w);
    return 0;
}

template <int HP>
static int sddmm_fwd_launch(const SddmmParams &p, bool with_hub, hipStream_t stream) {
    const int grid = (int)ceil_div(p.n_dst, kWavesPerBlock);
    if (with_hub) {
        zero_hub_counters_kernel<<<1, kWave, 0, stream>>>(p.hub.counters);
        YITU_LAUNCH_CHECK();
    }
    sddmm_fwd_rows_kernel<HP><<<grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (with_hub) {
        const int ig = (int)std::min<int64_t>(p.hub.max_items, 4096);
        sddmm_fwd_hub_stats_kernel<HP><<<ig, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        sddmm_fwd_hub_combine_kernel<<<(int)std::min<int64_t>(p.hub.max_rows, 512), kBlock, 0,
                                       stream>>>(p);
        YITU_LAUNCH_CHECK();
        sddmm_fwd_hub_norm_kernel<HP><<<ig, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int HP>
static int sddmm_bwd_launch(const SddmmParams &p, bool with_hub, hipStream_t stream) {
    const int grid = (int)ceil_div(p.n_dst, kWavesPerBlock);
    if (with_hub) {
        zero_hub_counters_kernel<<<1, kWave, 0, stream>>>(p.hub.counters);
        YITU_LAUNCH_CHECK();
    }
    sddmm_bwd_rows_kernel<HP><<<grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (with_hub) {
        const int ig = (int)std::min<int64_t>(p.hub.max_items, 4096);
        sddmm_bwd_hub_sums_kernel<HP><<<ig, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        sddmm_bwd_hub_combine_kernel<<<(int)std::min<int64_t>(p.hub.max_rows, 512), kBlock, 0,
                                       stream>>>(p);
        YITU_LAUNCH_CHECK();
        sddmm_bwd_hub_apply_kernel<HP><<<ig, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

#define YITU_DISPATCH_HP(H, CALL)                 \
    do {                                          \
        if ((H) <= 1) return CALL(1);             \
        if ((H) <= 2) return CALL(2);             \
        if ((H) <= 4) return CALL(4);             \
        if ((H) <= 8) return CALL(8);             \
        if ((H) <= 16) return CALL(16);           \
        if ((H) <= 32) return CALL(32);           \
        return CALL(64);                          \
    } while (0)

static int sddmm_fwd_dispatch(const SddmmParams &p, bool with_hub, hipStream_t s) {
#define CALL_FWD(N) sddmm_fwd_launch<N>(p, with_hub, s)
    YITU_DISPATCH_HP(p.H, CALL_FWD);
#undef CALL_FWD
}
static int sddmm_bwd_dispatch(const SddmmParams &p, bool with_hub, hipStream_t s) {
#define CALL_BWD(N) sddmm_bwd_launch<N>(p, with_hub, s)
    YITU_DISPATCH_HP(p.H, CALL_BWD);
#undef CALL_BWD
}

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API size_t yitu_sddmm_workspace_bytes(int64_t n_dst, int64_t nnz, int64_t n_heads,
                                           int64_t n_bid, int with_plan) {
    // the backward's gather pass reuses the buffer as SpMM workspace
    size_t b = std::max(sddmm_ws_bytes(nnz, n_heads, n_bid),
                        spmm_workspace_bytes(nnz, n_heads, with_plan != 0));
    if (n_bid == 1)
        b = std::max(b, attn_workspace_bytes(n_dst, nnz, n_heads) +
                            (with_plan ? 0 : plan_temp_bytes(nnz)));
    return b;
}

static int sddmm_check(const int32_t *indptr, const int32_t *indices, const float *query,
                       const float *key, int64_t n_dst, int64_t n_src, int64_t nnz, int64_t H,
                       int64_t n_bid) {
    YITU_REQUIRE(n_dst >= 0 && n_src >= 0 && nnz >= 0 && H >= 0, "negative size");
    YITU_REQUIRE(n_bid >= 1 && n_bid <= 16, "n_bid must be in [1, 16] (4-bit block tag)");
    YITU_REQUIRE(n_src <= (1 << 24), "column ids are 24-bit");
    YITU_REQUIRE(n_dst < INT32_MAX && nnz < INT32_MAX && nnz * H < ((int64_t)1 << 40),
                 "size out of range");
    YITU_REQUIRE(indptr, "null indptr");
    YITU_REQUIRE(nnz == 0 || (indices && query && key), "null input with nnz > 0");
    return 0;
}

YITU_API int yitu_sddmm_forward(float *attn, const int32_t *indptr, const int32_t *indices,
                                const float *query, const float *key, int64_t n_dst,
                                int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_bid,
                                int64_t max_degree, const void *plan, void *workspace,
                                size_t workspace_bytes, void *stream) {
    int rc = sddmm_check(indptr, indices, query, key, n_dst, n_src, nnz, n_heads, n_bid);
    if (rc) return rc;
    if (n_dst == 0 || nnz == 0 || n_heads == 0) return 0;
    YITU_REQUIRE(attn, "null output");
    if (n_bid == 1 && n_heads <= 64)
        return attn_forward_run(attn, indptr, indices, query, key, n_dst, n_src, nnz, n_heads,
                                max_degree, plan, workspace, workspace_bytes,
                                static_cast<hipStream_t>(stream));
    SddmmParams p{};
    p.indptr = indptr;
    p.indices = indices;
    p.query = query;
    p.key = key;
    p.attn = attn;
    p.n_dst = (int)n_dst;
    p.H = (int)n_heads;
    p.n_bid = (int)n_bid;
    bool with_hub;
    rc = sddmm_setup(p, nnz, max_degree, workspace, workspace_bytes, with_hub);
    if (rc) return rc;
    return sddmm_fwd_dispatch(p, with_hub, static_cast<hipStream_t>(stream));
}

namespace yitu {
int sddmm_backward_run(float *grad_query, float *grad_key, float *grad_edge, const int32_t *indptr,
                       const int32_t *indices, const float *query, const float *key,
                       const float *attn, const float *grad_out, const int32_t *t_indptr,
                       const int32_t *t_perm, int64_t n_dst, int64_t n_src, int64_t nnz,
                       int64_t n_heads, int64_t n_bid, int64_t max_degree, int64_t max_degree_t,
                       const void *plan, const void *plan_t, void *workspace,
                       size_t workspace_bytes, int skip_below, hipStream_t stream) {
    int rc = sddmm_check(indptr, indices, query, key, n_dst, n_src, nnz, n_heads, n_bid);
    if (rc) return rc;
    if (n_heads == 0) return 0;
    YITU_REQUIRE((grad_query || n_dst == 0) && (grad_key || n_src == 0), "null output");
    const bool gather = t_indptr != nullptr;
    YITU_REQUIRE(!gather || (t_perm && grad_edge) || nnz == 0,
                 "the gather form needs t_perm and a grad_edge buffer");
    if (!gather) {
        // scatter form: float atomics into a zeroed grad_key
        rc = fill_zero(grad_key, n_src * n_heads, stream);
        if (rc) return rc;
    }
    if (n_dst > 0 && nnz > 0 && skip_below == 0 && gather && n_bid == 1 && n_heads <= 64) {
        // one query block: windowed row kernel + row-plan items
        rc = attn_backward_run(grad_query, grad_edge, indptr, indices, query, key, attn, grad_out,
                               n_dst, n_src, nnz, n_heads, max_degree, plan, workspace,
                               workspace_bytes, stream);
        if (rc) return rc;
    } else if (n_dst > 0 && skip_below != INT32_MAX) {  // INT32_MAX: only the grad_key gather
        SddmmParams p{};
        p.indptr = indptr;
        p.indices = indices;
        p.query = query;
        p.key = key;
        p.attn = const_cast<float *>(attn);
        p.grad_out = grad_out;
        p.grad_q = grad_query;
        p.grad_k = gather ? nullptr : grad_key;
        p.grad_e = gather ? grad_edge : nullptr;
        p.n_dst = (int)n_dst;
        p.H = (int)n_heads;
        p.n_bid = (int)n_bid;
        p.skip_below = skip_below;
        bool with_hub;
        rc = sddmm_setup(p, nnz, max_degree, workspace, workspace_bytes, with_hub);
        if (rc) return rc;
        rc = sddmm_bwd_dispatch(p, with_hub, stream);
        if (rc) return rc;
    }
    if (gather && n_src > 0) {
        // grad_key[c, :] = sum over the transposed row c of grad_edge[t_perm[j], :]:
        // the scatter-add as a deterministic row gather with the edge id as "column"
        SpmmParams sp{};
        sp.indptr = t_indptr;
        sp.indices = t_perm;
        sp.feat = grad_edge;
        sp.out = grad_key;
        sp.n_rows = (int)n_src;
        sp.n_src = (int)nnz;
        sp.L = sp.F = (int)n_heads;
        sp.H = 1;
        sp.col_mask = 0x7fffffff;
        sp.alpha = 1.0f;
        // the plan of the transposed structure fits: same row bounds, other columns
        return launch_spmm(sp, W_NONE, false, nnz, max_degree_t, plan_t, workspace,
                           workspace_bytes, stream);
    }
    return 0;
}
}  // namespace yitu

YITU_API int yitu_sddmm_backward(float *grad_query, float *grad_key, float *grad_edge,
                                 const int32_t *indptr, const int32_t *indices, const float *query,
                                 const float *key, const float *attn, const float *grad_out,
                                 const int32_t *t_indptr, const int32_t *t_perm, int64_t n_dst,
                                 int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_bid,
                                 int64_t max_degree, int64_t max_degree_t, const void *plan,
                                 const void *plan_t, void *workspace, size_t workspace_bytes,
                                 void *stream_) {
    return sddmm_backward_run(grad_query, grad_key, grad_edge, indptr, indices, query, key, attn,
                              grad_out, t_indptr, t_perm, n_dst, n_src, nnz, n_heads, n_bid,
                              max_degree, max_degree_t, plan, plan_t, workspace, workspace_bytes,
                              0, static_cast<hipStream_t>(stream_));
}
