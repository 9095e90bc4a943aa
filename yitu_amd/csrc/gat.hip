// Fused GAT attention: SDDMM(u_add_v) -> LeakyReLU(0.2) -> edge softmax ->
// attention-weighted aggregate in one pass over each destination row, and the
// matching backward assembled from the dot / softmax-backward / transposed
// gather kernels. The reference runs these as separate launches
// (sddmm_cuda.cu:5-33 then spmm_cuda.cu:4-21); the contract of the fused op is
// their composition gspmm(blk, fused_gsddmm(blk, q, k), x).
//
// Forward mapping (wave64, one wave per destination row):
//   phase A  softmax statistics (max, sum) per head with HP lanes per edge;
//   phase B  per sub-batch of 64/HP edges: every (edge, head) probability is
//            computed exactly once in the (edge, head) lane layout, stored to
//            attn (one contiguous run), then broadcast lane-to-lane to the
//            (slot, column) layout that gathers x[col] tiles and accumulates.
// Hub rows: chunk statistics and their per-row combine reuse the SDDMM kernels,
// a chunk-apply kernel writes attn and per-chunk partial rows, the SpMM reduce
// kernel adds those in chunk order.
#include "../../include/yitu_hip.h"
#include "sddmm_kernels.hpp"

namespace yitu {

struct GatParams {
    const int32_t *indptr;
    const int32_t *indices;
    const float *query;  // [n_dst, H]
    const float *key;    // [n_src, H]
    const float *feat;   // [n_src, L]
    float *out;          // [n_dst, L]
    float *attn;         // [nnz, H] or null
    int n_dst, L, F, H;
    int HP;              // heads rounded up to a power of two (<= 64)
    int hub_threshold;
    HubQueue hub;          // hub.partial: per-item partial rows [item][L]
    const float *rowstat;  // [hub row][H][3]: max, 1/sum
};

// (max, sum) over the lanes that share lane % hp, hp a runtime power of two
__device__ __forceinline__ MaxSum ms_wave_rt(MaxSum a, int hp) {
    for (int o = 32; o >= hp; o >>= 1) {
        MaxSum b{__shfl_xor(a.m, o, kWave), __shfl_xor(a.s, o, kWave)};
        a = ms_merge(a, b);
    }
    return a;
}

__device__ __forceinline__ MaxSum gat_stats(const GatParams &p, int e_beg, int e_end, float qv) {
    const int lane = lane_id();
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    MaxSum a = ms_init();
    if (hl < p.H) {
        for (int e = e_beg + esub; e < e_end; e += eps) {
            const int col = p.indices[e] & kColMask;
            a = ms_push(a, leaky(qv + p.key[(size_t)col * p.H + hl]));
        }
    }
    return a;
}

// Phase B over edges [e_beg, e_end): writes attn and accumulates the weighted
// feature tiles of column block c0. m / inv are this lane's head statistics in
// the (edge, head) layout (lane % HP = head).
template <int VEC, int G, int KT>
__device__ __forceinline__ void gat_accumulate(float (&acc)[KT][VEC], const GatParams &p,
                                               int e_beg, int e_end, int c0, float qv, float m,
                                               float inv, bool write_attn) {
    constexpr int SLOTS = kWave / G;
    constexpr int UNROLL = KT >= 4 ? 2 : 4;
    const int lane = lane_id();
    const int slot = lane / G, sub = lane % G;
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    const float *__restrict__ feat = p.feat;

    int off[KT], head[KT];
    bool live[KT];
#pragma unroll
    for (int t = 0; t < KT; t++) {
        off[t] = c0 + (t * G + sub) * VEC;
        live[t] = off[t] < p.L;
        if (!live[t]) off[t] = 0;
        head[t] = off[t] / p.F;
    }

    for (int e0 = e_beg; e0 < e_end; e0 += eps) {
        const int nb = min(eps, e_end - e0);
        const int e = e0 + esub;
        const int col = p.indices[min(e, e_end - 1)] & kColMask;
        float pv = 0.0f;
        if (e < e_end && hl < p.H) {
            pv = expf(leaky(qv + p.key[(size_t)col * p.H + hl]) - m) * inv;
            if (write_attn) p.attn[(size_t)e * p.H + hl] = pv;
        }
        for (int j0 = 0; j0 < nb; j0 += SLOTS * UNROLL) {
            float v[UNROLL][KT][VEC];
            float w[UNROLL][KT];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int ej = j0 + u * SLOTS + slot;
                const bool valid = ej < nb;
                const int src = valid ? ej * p.HP : 0;  // lane holding edge ej (head 0)
                const int c = __shfl(col, src, kWave);
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    const float wt = __shfl(pv, src + head[t], kWave);
                    w[u][t] = (valid && live[t]) ? wt : 0.0f;
                }
                // steps wholly past the sub-batch load nothing (wave-uniform test)
                if (j0 + u * SLOTS < nb) {
#pragma unroll
                    for (int t = 0; t < KT; t++)
                        RowLoad<VEC, float>::ld(feat + (size_t)c * p.L + off[t], v[u][t]);
                } else {
#pragma unroll
                    for (int t = 0; t < KT; t++)
#pragma unroll
                        for (int i = 0; i < VEC; i++) v[u][t][i] = 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < VEC; i++) acc[t][i] += w[u][t] * v[u][t][i];
        }
    }
}

template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void gat_fwd_rows_kernel(GatParams p) {
    const int lane = lane_id();
    const int row = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (row >= p.n_dst) return;
    const int beg = p.indptr[row], end = p.indptr[row + 1];
    const int deg = end - beg;
    if (deg >= p.hub_threshold) {
        queue_hub_row(p.hub, row, deg);
        return;
    }
    const int sub = lane % G, slot = lane / G;
    const int hl = lane & (p.HP - 1);
    float qv = 0.0f, m = 0.0f, inv = 0.0f;
    if (deg > 0) {
        qv = hl < p.H ? p.query[(size_t)row * p.H + hl] : 0.0f;
        MaxSum a = ms_wave_rt(gat_stats(p, beg, end, qv), p.HP);
        m = a.m;
        inv = 1.0f / a.s;
    }
    for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
        float acc[KT][VEC];
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int i = 0; i < VEC; i++) acc[t][i] = 0.0f;
        if (deg > 0) {
            gat_accumulate<VEC, G, KT>(acc, p, beg, end, c0, qv, m, inv, p.attn && c0 == 0);
            fold_slots<VEC, G, KT>(acc);
        }
        if (slot == 0) {
#pragma unroll
            for (int t = 0; t < KT; t++) {
                const int o = c0 + (t * G + sub) * VEC;
                if (o < p.L) store_row<VEC>(p.out + (size_t)row * p.L + o, acc[t]);
            }
        }
    }
}

template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void gat_fwd_hub_apply_kernel(GatParams p) {
    __shared__ float red[kWavesPerBlock][G * VEC * KT];
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);
    const int lane = lane_id(), wave = threadIdx.x / kWave;
    const int sub = lane % G, slot = lane / G;
    const int hl = lane & (p.HP - 1);
    constexpr int kPerWave = kHubChunk / kWavesPerBlock;
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int4 it = p.hub.items[item];
        const int row = it.x;
        const int beg = p.indptr[row] + it.y * kHubChunk;
        const int end = min(p.indptr[row + 1], beg + kHubChunk);
        const int wbeg = min(end, beg + wave * kPerWave), wend = min(end, wbeg + kPerWave);
        float qv = 0.0f, m = 0.0f, inv = 0.0f;
        if (hl < p.H) {
            qv = p.query[(size_t)row * p.H + hl];
            const float *rs = p.rowstat + ((size_t)it.z * p.H + hl) * 3;
            m = rs[0];
            inv = rs[1];
        }
        for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
            float acc[KT][VEC];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < VEC; i++) acc[t][i] = 0.0f;
            if (wend > wbeg) {
                gat_accumulate<VEC, G, KT>(acc, p, wbeg, wend, c0, qv, m, inv, p.attn && c0 == 0);
                fold_slots<VEC, G, KT>(acc);
            }
            __syncthreads();
            if (slot == 0) {
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < VEC; i++) red[wave][(t * G + sub) * VEC + i] = acc[t][i];
            }
            __syncthreads();
            for (int e = threadIdx.x; e < G * VEC * KT; e += kBlock) {
                const int o = c0 + e;
                if (o < p.L) {
                    float s = red[0][e];
#pragma unroll
                    for (int w = 1; w < kWavesPerBlock; w++) s += red[w][e];
                    p.hub.partial[(size_t)item * p.L + o] = s;
                }
            }
        }
    }
}

// ---- host side ----------------------------------------------------------------
static inline int64_t gat_max_rows(int64_t nnz) { return nnz / kHubThreshold + 1; }
static inline int64_t gat_max_items(int64_t nnz) { return nnz / kHubChunk + gat_max_rows(nnz) + 1; }

struct GatWorkspace {
    HubCounters *counters;
    int4 *rows, *items;
    float *stats;    // [item][H][3]
    float *rowstat;  // [hub row][H][3]
    float *partial;  // [item][L]
    int max_rows, max_items;
};

static size_t gat_ws_bytes(int64_t nnz, int64_t H, int64_t L) {
    size_t b = 256;
    b += 2 * align_up(sizeof(int4) * (size_t)gat_max_items(nnz), 256);
    b += align_up(sizeof(float) * 3 * (size_t)(gat_max_items(nnz) * H), 256);
    b += align_up(sizeof(float) * 3 * (size_t)(gat_max_rows(nnz) * H), 256);
    b += align_up(sizeof(float) * (size_t)(gat_max_items(nnz) * L), 256);
    return b;
}

static void gat_ws_carve(GatWorkspace &g, void *workspace, int64_t nnz, int64_t H, int64_t L) {
    char *w = static_cast<char *>(workspace);
    g.max_rows = (int)gat_max_rows(nnz);
    g.max_items = (int)gat_max_items(nnz);
    g.counters = reinterpret_cast<HubCounters *>(w);
    w += 256;
    g.rows = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)g.max_items, 256);
    g.items = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)g.max_items, 256);
    g.stats = reinterpret_cast<float *>(w);
    w += align_up(sizeof(float) * 3 * (size_t)g.max_items * H, 256);
    g.rowstat = reinterpret_cast<float *>(w);
    w += align_up(sizeof(float) * 3 * (size_t)g.max_rows * H, 256);
    g.partial = reinterpret_cast<float *>(w);
}

template <int HP>
static int gat_hub_stats_launch(const SddmmParams &sp, hipStream_t stream) {
    sddmm_fwd_hub_stats_kernel<HP>
        <<<(int)std::min<int64_t>(sp.hub.max_items, 4096), kBlock, 0, stream>>>(sp);
    YITU_LAUNCH_CHECK();
    sddmm_fwd_hub_combine_kernel<<<(int)std::min<int64_t>(sp.hub.max_rows, 512), kBlock, 0,
                                   stream>>>(sp);
    YITU_LAUNCH_CHECK();
    return 0;
}

template <int VEC, int G, int KT>
static int gat_fwd_launch(GatParams &p, const GatWorkspace &g, bool with_hub, hipStream_t stream) {
    if (with_hub) {
        zero_hub_counters_kernel<<<1, kWave, 0, stream>>>(g.counters);
        YITU_LAUNCH_CHECK();
    }
    gat_fwd_rows_kernel<VEC, G, KT>
        <<<(int)ceil_div(p.n_dst, kWavesPerBlock), kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (!with_hub) return 0;
    // chunk statistics + per-row combine: the SDDMM hub kernels on the same queue
    SddmmParams sp{};
    sp.indptr = p.indptr;
    sp.indices = p.indices;
    sp.query = p.query;
    sp.key = p.key;
    sp.n_dst = p.n_dst;
    sp.H = p.H;
    sp.n_bid = 1;
    sp.hub = p.hub;
    sp.hub.partial = g.stats;
    sp.rowstat = g.rowstat;
    int rc;
    switch (p.HP) {
        case 1: rc = gat_hub_stats_launch<1>(sp, stream); break;
        case 2: rc = gat_hub_stats_launch<2>(sp, stream); break;
        case 4: rc = gat_hub_stats_launch<4>(sp, stream); break;
        case 8: rc = gat_hub_stats_launch<8>(sp, stream); break;
        case 16: rc = gat_hub_stats_launch<16>(sp, stream); break;
        case 32: rc = gat_hub_stats_launch<32>(sp, stream); break;
        default: rc = gat_hub_stats_launch<64>(sp, stream); break;
    }
    if (rc) return rc;
    gat_fwd_hub_apply_kernel<VEC, G, KT>
        <<<(int)std::min<int64_t>(p.hub.max_items, 4096), kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    SpmmParams rp{};
    rp.out = p.out;
    rp.L = p.L;
    rp.alpha = 1.0f;
    rp.hub = p.hub;
    spmm_hub_reduce_kernel<W_NONE, 4>
        <<<(int)std::min<int64_t>(p.hub.max_rows, 1024), kBlock, 0, stream>>>(rp);
    YITU_LAUNCH_CHECK();
    return 0;
}

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API size_t yitu_gat_workspace_bytes(int64_t nnz, int64_t n_heads, int64_t n_features) {
    const int64_t L = n_heads * n_features;
    size_t b = gat_ws_bytes(nnz, n_heads, L);
    b = std::max(b, (size_t)yitu_spmm_workspace_bytes(nnz, L));
    b = std::max(b, (size_t)yitu_sddmm_workspace_bytes(nnz, n_heads, 1));
    return b;
}

YITU_API int yitu_gat_forward(float *out, float *attn, const int32_t *indptr,
                              const int32_t *indices, const float *query, const float *key,
                              const float *features, int64_t n_dst, int64_t n_src, int64_t nnz,
                              int64_t n_heads, int64_t n_features, int64_t max_degree,
                              void *workspace, size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_dst >= 0 && n_src >= 0 && nnz >= 0 && n_heads >= 0 && n_features >= 0,
                 "negative size");
    const int64_t L = n_heads * n_features;
    if (n_dst == 0 || L == 0) return 0;
    YITU_REQUIRE(out && indptr, "null output or indptr");
    YITU_REQUIRE(nnz == 0 || (indices && query && key && features), "null input with nnz > 0");
    YITU_REQUIRE(n_dst < INT32_MAX && n_src <= (1 << 24) && L < (1 << 20) && nnz < INT32_MAX,
                 "size out of range (columns are 24-bit)");
    const bool fused_ok = n_features % 4 == 0 && n_heads <= 64 && aligned16(features) &&
                          aligned16(out);
    if (!fused_ok) {
        // shapes outside the fused kernel's vector layout: the two-op composition
        YITU_REQUIRE(attn, "this shape needs the attn buffer (unfused path)");
        int rc = yitu_sddmm_forward(attn, indptr, indices, query, key, n_dst, n_src, nnz, n_heads,
                                    1, max_degree, workspace, workspace_bytes, stream_);
        if (rc) return rc;
        return yitu_spmm_forward(out, attn, indptr, indices, features, n_dst, n_src, nnz, n_heads,
                                 n_features, max_degree, workspace, workspace_bytes, stream_);
    }
    GatParams p{};
    p.indptr = indptr;
    p.indices = indices;
    p.query = query;
    p.key = key;
    p.feat = features;
    p.out = out;
    p.attn = attn;
    p.n_dst = (int)n_dst;
    p.L = (int)L;
    p.F = (int)n_features;
    p.H = (int)n_heads;
    p.HP = 1;
    while (p.HP < p.H) p.HP <<= 1;
    const bool with_hub = nnz >= kHubThreshold && !(max_degree >= 0 && max_degree < kHubThreshold);
    p.hub_threshold = with_hub ? kHubThreshold : 0x7fffffff;
    GatWorkspace g{};
    if (with_hub) {
        const size_t need = gat_ws_bytes(nnz, n_heads, L);
        YITU_REQUIRE(workspace && workspace_bytes >= need, "workspace too small: need %zu bytes",
                     need);
        YITU_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                     "workspace must be 256-byte aligned");
        gat_ws_carve(g, workspace, nnz, n_heads, L);
        p.hub.counters = g.counters;
        p.hub.rows = g.rows;
        p.hub.items = g.items;
        p.hub.partial = g.partial;
        p.hub.max_rows = g.max_rows;
        p.hub.max_items = g.max_items;
        p.hub.chunk = kHubChunk;
        p.rowstat = g.rowstat;
    }
    const int lanes = (int)(L / 4);
    if (lanes <= 16) return gat_fwd_launch<4, 16, 1>(p, g, with_hub, stream);
    if (lanes <= 32) return gat_fwd_launch<4, 32, 1>(p, g, with_hub, stream);
    if (lanes <= 64) return gat_fwd_launch<4, 64, 1>(p, g, with_hub, stream);
    if (lanes <= 128) return gat_fwd_launch<4, 64, 2>(p, g, with_hub, stream);
    return gat_fwd_launch<4, 64, 4>(p, g, with_hub, stream);
}

YITU_API int yitu_gat_backward(float *grad_query, float *grad_key, float *grad_features,
                               float *grad_attn_scratch, float *grad_edge_scratch,
                               const int32_t *indptr, const int32_t *indices, const float *query,
                               const float *key, const float *features, const float *attn,
                               const float *grad_out, const int32_t *t_indptr,
                               const int32_t *t_rows, const int32_t *t_perm, int64_t n_dst,
                               int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_features,
                               int64_t max_degree, int64_t max_degree_t, void *workspace,
                               size_t workspace_bytes, void *stream) {
    YITU_REQUIRE(grad_query && grad_key && grad_features, "null output");
    YITU_REQUIRE(nnz == 0 || (grad_attn_scratch && grad_edge_scratch),
                 "gat_backward needs two [nnz, H] scratch buffers");
    YITU_REQUIRE(t_indptr && (nnz == 0 || (t_rows && t_perm)),
                 "gat_backward needs the transposed structure (yitu_csr_transpose)");
    // d attn = <grad_out[row], x[col]> per edge and head; grad_x = attn-weighted
    // gather of grad_out over the transposed structure
    int rc = yitu_spmm_backward(grad_attn_scratch, grad_features, attn, indptr, indices, features,
                                grad_out, t_indptr, t_rows, t_perm, n_dst, n_src, nnz, n_heads,
                                n_features, max_degree, max_degree_t, workspace, workspace_bytes,
                                stream);
    if (rc) return rc;
    // softmax + LeakyReLU backward; grad_key gathered over the transposed structure
    return yitu_sddmm_backward(grad_query, grad_key, grad_edge_scratch, indptr, indices, query,
                               key, attn, grad_attn_scratch, t_indptr, t_perm, n_dst, n_src, nnz,
                               n_heads, 1, max_degree, max_degree_t, workspace, workspace_bytes,
                               stream);
}
