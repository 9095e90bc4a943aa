// Kernels of the SDDMM(u_add_v) + LeakyReLU(0.2) + per-destination edge softmax,
// forward and backward, for packed indices (bid << 24 | col) and up to 16 query
// blocks. With one query block the op runs on the windowed / row-plan kernels of
// gat.hip instead; these kernels serve stitched multi-block graphs and the
// atomic form of the backward.
//
// Mapping (wave64): one wave per destination row; a step covers 64 / HP edges
// with HP lanes (the head count rounded up to a power of two) per edge, so the
// attn / grad_out accesses of a step are one contiguous run and the per-head
// reductions are butterflies over the lanes that share (lane % HP).
// The softmax is evaluated with a running (max, sum) pair, so inputs are read
// once for the statistics and once more for the normalised write.
// Rows with >= kHubThreshold edges are queued and handled by three chunk-level
// kernels (chunk statistics, per-row combine, chunk apply) so that a 10^5-edge
// row is spread over hundreds of workgroups instead of one wave.
#pragma once
#include <cfloat>

#include "spmm_rows.hpp"

namespace yitu {

// ---- queue of long rows for the multi-block kernels (rows of 512+ edges are
// spread over workgroups of 512-edge chunks) -----------------------------------
constexpr int kHubChunk = 512;      // edges per hub work item
constexpr int kHubThreshold = 512;  // rows with >= this many edges go to the chunk kernels

struct HubCounters {
    int n_items;
    int n_rows;
    int overflow;  // set when the queue capacity was exceeded; the hub kernels then do nothing
    int pad;
};

struct HubQueue {
    HubCounters *counters;  // zeroed before the row kernel
    int4 *rows;             // {row, first_item, n_chunks, 0}
    int4 *items;            // {row, chunk, index into rows[], 0}
    float *partial;         // [n_items, L]
    int max_rows;
    int max_items;
    int chunk;              // edges per item
};

// Appends a hub row and its ceil(deg / kHubChunk) chunk items to the queue.
// Called by all lanes of the wave that owns the row.
__device__ __forceinline__ void queue_hub_row(const HubQueue &q, int row, int deg) {
    const int lane = lane_id();
    const int n_chunks = (deg + q.chunk - 1) / q.chunk;
    int first = 0, slot_r = 0;
    if (lane == 0) {
        first = atomicAdd(&q.counters->n_items, n_chunks);
        slot_r = atomicAdd(&q.counters->n_rows, 1);
    }
    first = __shfl(first, 0, kWave);
    slot_r = __shfl(slot_r, 0, kWave);
    if (slot_r < q.max_rows && first + n_chunks <= q.max_items) {
        if (lane == 0) q.rows[slot_r] = make_int4(row, first, n_chunks, 0);
        for (int c = lane; c < n_chunks; c += kWave)
            q.items[first + c] = make_int4(row, c, slot_r, 0);
    } else if (lane == 0) {
        atomicExch(&q.counters->overflow, 1);
    }
}

static __global__ void zero_hub_counters_kernel(HubCounters *c) {
    if (threadIdx.x == 0) {
        c->n_items = 0;
        c->n_rows = 0;
        c->overflow = 0;
        c->pad = 0;
    }
}

constexpr float kSlope = 0.2f;  // LeakyReLU slope fixed by the reference (sddmm_cuda.cu:22)
constexpr int kColMask = 0xffffff;

__device__ __forceinline__ float leaky(float x) { return fmaxf(0.0f, x) + kSlope * fminf(0.0f, x); }

struct SddmmParams {
    const int32_t *indptr;
    const int32_t *indices;
    const float *query;  // [n_bid, n_dst, H]
    const float *key;    // [n_src, H]
    float *attn;         // fwd: out [nnz, H]; bwd: in
    const float *grad_out;  // bwd: [nnz, H]
    float *grad_q;          // bwd: [n_bid, n_dst, H]
    float *grad_k;          // bwd, atomic mode: [n_src, H] (pre-zeroed)
    float *grad_e;          // bwd, gather mode: [nnz, H] per-edge logit gradient
    int n_dst;
    int H;
    int n_bid;
    int hub_threshold;
    int skip_below;  // bwd: rows with fewer edges were handled by another kernel
    HubQueue hub;   // hub.partial = per-item statistics [item][n_bid][H][3]
    float *rowstat; // [hub row][n_bid][H][3]
};

// (max, sum) of a softmax prefix; merging two prefixes is associative.
struct MaxSum {
    float m, s;
};
__device__ __forceinline__ MaxSum ms_init() { return {-FLT_MAX, 0.0f}; }
__device__ __forceinline__ MaxSum ms_push(MaxSum a, float l) {
    const float m = fmaxf(a.m, l);
    return {m, a.s * expf(a.m - m) + expf(l - m)};
}
__device__ __forceinline__ MaxSum ms_merge(MaxSum a, MaxSum b) {
    const float m = fmaxf(a.m, b.m);
    return {m, a.s * expf(a.m - m) + b.s * expf(b.m - m)};
}
template <int HP>
__device__ __forceinline__ MaxSum ms_wave(MaxSum a) {
#pragma unroll
    for (int o = 32; o >= HP; o >>= 1) {
        MaxSum b{__shfl_xor(a.m, o, kWave), __shfl_xor(a.s, o, kWave)};
        a = ms_merge(a, b);
    }
    return a;
}

// =============================== forward =====================================

// Statistics of edges [e_beg, e_end) of `row` for block b and this lane's head.
template <int HP>
__device__ __forceinline__ MaxSum fwd_stats(const SddmmParams &p, int row, int e_beg, int e_end,
                                            int b, int h, bool act_h, float qv) {
    constexpr int EPS = kWave / HP;
    const int esub = lane_id() / HP;
    MaxSum a = ms_init();
    for (int e0 = e_beg; e0 < e_end; e0 += EPS) {
        const int e = e0 + esub;
        if (e < e_end && act_h) {
            const int idx = p.indices[e];
            if (p.n_bid == 1 || ((unsigned)idx >> 24) == (unsigned)b) {
                const float l = leaky(qv + p.key[(size_t)(idx & kColMask) * p.H + h]);
                a = ms_push(a, l);
            }
        }
    }
    return a;
}

template <int HP>
__device__ __forceinline__ void fwd_write(const SddmmParams &p, int e_beg, int e_end, int b, int h,
                                          bool act_h, float qv, float m, float inv) {
    constexpr int EPS = kWave / HP;
    const int esub = lane_id() / HP;
    for (int e0 = e_beg; e0 < e_end; e0 += EPS) {
        const int e = e0 + esub;
        if (e < e_end && act_h) {
            const int idx = p.indices[e];
            if (p.n_bid == 1 || ((unsigned)idx >> 24) == (unsigned)b) {
                const float l = leaky(qv + p.key[(size_t)(idx & kColMask) * p.H + h]);
                p.attn[(size_t)e * p.H + h] = expf(l - m) * inv;
            }
        }
    }
}

template <int HP>
__device__ __forceinline__ void sddmm_fwd_rows_body(const SddmmParams &p, int block) {
    const int row = block * kWavesPerBlock + threadIdx.x / kWave;
    if (row >= p.n_dst) return;
    const int beg = p.indptr[row], end = p.indptr[row + 1];
    if (end == beg) return;
    if (end - beg >= p.hub_threshold) {
        queue_hub_row(p.hub, row, end - beg);
        return;
    }
    const int hl = lane_id() % HP;
    for (int h0 = 0; h0 < p.H; h0 += HP) {
        const int h = h0 + hl;
        const bool act_h = h < p.H;
        for (int b = 0; b < p.n_bid; b++) {
            const float qv = act_h ? p.query[((size_t)b * p.n_dst + row) * p.H + h] : 0.0f;
            MaxSum a = ms_wave<HP>(fwd_stats<HP>(p, row, beg, end, b, h, act_h, qv));
            fwd_write<HP>(p, beg, end, b, h, act_h, qv, a.m, 1.0f / a.s);
        }
    }
}

template <int HP>
__global__ __launch_bounds__(kBlock) void sddmm_fwd_rows_kernel(SddmmParams p) {
    sddmm_fwd_rows_body<HP>(p, blockIdx.x);
}

// stats layout: [(item or hub row) * n_bid + b] * H + h, three floats each
__device__ __forceinline__ size_t stat_index(const SddmmParams &p, int slot, int b, int h) {
    return (((size_t)slot * p.n_bid + b) * p.H + h) * 3;
}

template <int HP>
__global__ __launch_bounds__(kBlock) void sddmm_fwd_hub_stats_kernel(SddmmParams p) {
    __shared__ float sm[kWavesPerBlock][HP][2];
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);
    const int wave = threadIdx.x / kWave, lane = lane_id(), hl = lane % HP;
    constexpr int kPerWave = kHubChunk / kWavesPerBlock;
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int4 it = p.hub.items[item];
        const int row = it.x, chunk = it.y;
        const int beg = p.indptr[row] + chunk * kHubChunk;
        const int end = min(p.indptr[row + 1], beg + kHubChunk);
        const int wbeg = min(end, beg + wave * kPerWave), wend = min(end, wbeg + kPerWave);
        for (int h0 = 0; h0 < p.H; h0 += HP) {
            const int h = h0 + hl;
            const bool act_h = h < p.H;
            for (int b = 0; b < p.n_bid; b++) {
                const float qv = act_h ? p.query[((size_t)b * p.n_dst + row) * p.H + h] : 0.0f;
                MaxSum a = ms_wave<HP>(fwd_stats<HP>(p, row, wbeg, wend, b, h, act_h, qv));
                __syncthreads();
                if (lane < HP) {
                    sm[wave][lane][0] = a.m;
                    sm[wave][lane][1] = a.s;
                }
                __syncthreads();
                if (wave == 0 && lane < HP && act_h) {
                    MaxSum t{sm[0][lane][0], sm[0][lane][1]};
#pragma unroll
                    for (int w = 1; w < kWavesPerBlock; w++)
                        t = ms_merge(t, MaxSum{sm[w][lane][0], sm[w][lane][1]});
                    float *st = p.hub.partial + stat_index(p, item, b, h);
                    st[0] = t.m;
                    st[1] = t.s;
                }
            }
        }
    }
}

// one thread per (hub row, b, h): merges the chunk statistics in chunk order
static __global__ __launch_bounds__(kBlock) void sddmm_fwd_hub_combine_kernel(SddmmParams p) {
    if (p.hub.counters->overflow) return;
    const int n_hub = min(p.hub.counters->n_rows, p.hub.max_rows);
    const int per_row = p.n_bid * p.H;
    const int64_t total = (int64_t)n_hub * per_row;
    for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < total;
         t += (int64_t)gridDim.x * kBlock) {
        const int hub = (int)(t / per_row), bh = (int)(t % per_row);
        const int4 r = p.hub.rows[hub];
        MaxSum a = ms_init();
        for (int c = 0; c < r.z; c++) {
            const float *st = p.hub.partial + ((size_t)(r.y + c) * per_row + bh) * 3;
            a = ms_merge(a, MaxSum{st[0], st[1]});
        }
        float *rs = p.rowstat + ((size_t)hub * per_row + bh) * 3;
        rs[0] = a.m;
        rs[1] = 1.0f / a.s;
    }
}

template <int HP>
__global__ __launch_bounds__(kBlock) void sddmm_fwd_hub_norm_kernel(SddmmParams p) {
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);
    const int wave = threadIdx.x / kWave, hl = lane_id() % HP;
    constexpr int kPerWave = kHubChunk / kWavesPerBlock;
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int4 it = p.hub.items[item];
        const int row = it.x, chunk = it.y, hub = it.z;
        const int beg = p.indptr[row] + chunk * kHubChunk;
        const int end = min(p.indptr[row + 1], beg + kHubChunk);
        const int wbeg = min(end, beg + wave * kPerWave), wend = min(end, wbeg + kPerWave);
        for (int h0 = 0; h0 < p.H; h0 += HP) {
            const int h = h0 + hl;
            const bool act_h = h < p.H;
            for (int b = 0; b < p.n_bid; b++) {
                const float qv = act_h ? p.query[((size_t)b * p.n_dst + row) * p.H + h] : 0.0f;
                float m = 0.0f, inv = 0.0f;
                if (act_h) {
                    const float *rs = p.rowstat + stat_index(p, hub, b, h);
                    m = rs[0];
                    inv = rs[1];
                }
                fwd_write<HP>(p, wbeg, wend, b, h, act_h, qv, m, inv);
            }
        }
    }
}

// =============================== backward ====================================
// Per (row, b, h), with x_i = q + k_i the pre-activation and d_i its slope:
//   S  = sum_i attn_i g_i
//   gv_i = attn_i (g_i - S) d_i        -> grad_k[col_i] (scatter) / grad_e[i]
//   grad_q = sum_i gv_i = A1 - S A2,   A1 = sum attn g d,  A2 = sum attn d
struct Sums3 {
    float s, a1, a2;
};

template <int HP>
__device__ __forceinline__ Sums3 bwd_sums(const SddmmParams &p, int e_beg, int e_end, int b, int h,
                                          bool act_h, float qv) {
    constexpr int EPS = kWave / HP;
    const int esub = lane_id() / HP;
    Sums3 r{0.0f, 0.0f, 0.0f};
    for (int e0 = e_beg; e0 < e_end; e0 += EPS) {
        const int e = e0 + esub;
        if (e < e_end && act_h) {
            const int idx = p.indices[e];
            if (p.n_bid == 1 || ((unsigned)idx >> 24) == (unsigned)b) {
                const float x = qv + p.key[(size_t)(idx & kColMask) * p.H + h];
                const float d = x < 0.0f ? kSlope : 1.0f;
                const float a = p.attn[(size_t)e * p.H + h];
                const float g = p.grad_out[(size_t)e * p.H + h];
                r.s += a * g;
                r.a1 += a * g * d;
                r.a2 += a * d;
            }
        }
    }
    return r;
}
template <int HP>
__device__ __forceinline__ Sums3 sums_wave(Sums3 r) {
    r.s = wave_sum_strided<HP>(r.s);
    r.a1 = wave_sum_strided<HP>(r.a1);
    r.a2 = wave_sum_strided<HP>(r.a2);
    return r;
}

template <int HP>
__device__ __forceinline__ void bwd_apply(const SddmmParams &p, int e_beg, int e_end, int b, int h,
                                          bool act_h, float qv, float S) {
    constexpr int EPS = kWave / HP;
    const int esub = lane_id() / HP;
    for (int e0 = e_beg; e0 < e_end; e0 += EPS) {
        const int e = e0 + esub;
        if (e < e_end && act_h) {
            const int idx = p.indices[e];
            if (p.n_bid == 1 || ((unsigned)idx >> 24) == (unsigned)b) {
                const int col = idx & kColMask;
                const float x = qv + p.key[(size_t)col * p.H + h];
                const float d = x < 0.0f ? kSlope : 1.0f;
                const float a = p.attn[(size_t)e * p.H + h];
                const float g = p.grad_out[(size_t)e * p.H + h];
                const float gv = a * (g - S) * d;
                if (p.grad_e) p.grad_e[(size_t)e * p.H + h] = gv;
                if (p.grad_k) atomicAdd(&p.grad_k[(size_t)col * p.H + h], gv);
            }
        }
    }
}

template <int HP>
__device__ __forceinline__ void sddmm_bwd_rows_body(const SddmmParams &p, int block) {
    const int row = block * kWavesPerBlock + threadIdx.x / kWave;
    if (row >= p.n_dst) return;
    const int beg = p.indptr[row], end = p.indptr[row + 1];
    if (end - beg < p.skip_below) return;
    const int lane = lane_id(), hl = lane % HP;
    const bool hub = end - beg >= p.hub_threshold;
    if (hub) queue_hub_row(p.hub, row, end - beg);
    for (int h0 = 0; h0 < p.H; h0 += HP) {
        const int h = h0 + hl;
        const bool act_h = h < p.H;
        for (int b = 0; b < p.n_bid; b++) {
            const size_t qi = ((size_t)b * p.n_dst + row) * p.H + h;
            if (hub) continue;  // grad_q of hub rows is written by the combine kernel
            if (end == beg) {
                if (lane < HP && act_h) p.grad_q[qi] = 0.0f;
                continue;
            }
            const float qv = act_h ? p.query[qi] : 0.0f;
            Sums3 r = sums_wave<HP>(bwd_sums<HP>(p, beg, end, b, h, act_h, qv));
            if (lane < HP && act_h) p.grad_q[qi] = r.a1 - r.s * r.a2;
            bwd_apply<HP>(p, beg, end, b, h, act_h, qv, r.s);
        }
    }
}

template <int HP>
__global__ __launch_bounds__(kBlock) void sddmm_bwd_rows_kernel(SddmmParams p) {
    sddmm_bwd_rows_body<HP>(p, blockIdx.x);
}

template <int HP>
__global__ __launch_bounds__(kBlock) void sddmm_bwd_hub_sums_kernel(SddmmParams p) {
    __shared__ float sm[kWavesPerBlock][HP][3];
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);
    const int wave = threadIdx.x / kWave, lane = lane_id(), hl = lane % HP;
    constexpr int kPerWave = kHubChunk / kWavesPerBlock;
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int4 it = p.hub.items[item];
        const int row = it.x, chunk = it.y;
        const int beg = p.indptr[row] + chunk * kHubChunk;
        const int end = min(p.indptr[row + 1], beg + kHubChunk);
        const int wbeg = min(end, beg + wave * kPerWave), wend = min(end, wbeg + kPerWave);
        for (int h0 = 0; h0 < p.H; h0 += HP) {
            const int h = h0 + hl;
            const bool act_h = h < p.H;
            for (int b = 0; b < p.n_bid; b++) {
                const float qv = act_h ? p.query[((size_t)b * p.n_dst + row) * p.H + h] : 0.0f;
                Sums3 r = sums_wave<HP>(bwd_sums<HP>(p, wbeg, wend, b, h, act_h, qv));
                __syncthreads();
                if (lane < HP) {
                    sm[wave][lane][0] = r.s;
                    sm[wave][lane][1] = r.a1;
                    sm[wave][lane][2] = r.a2;
                }
                __syncthreads();
                if (wave == 0 && lane < HP && act_h) {
                    float *st = p.hub.partial + stat_index(p, item, b, h);
#pragma unroll
                    for (int k = 0; k < 3; k++) {
                        float t = sm[0][lane][k];
#pragma unroll
                        for (int w = 1; w < kWavesPerBlock; w++) t += sm[w][lane][k];
                        st[k] = t;
                    }
                }
            }
        }
    }
}

static __global__ __launch_bounds__(kBlock) void sddmm_bwd_hub_combine_kernel(SddmmParams p) {
    if (p.hub.counters->overflow) return;
    const int n_hub = min(p.hub.counters->n_rows, p.hub.max_rows);
    const int per_row = p.n_bid * p.H;
    const int64_t total = (int64_t)n_hub * per_row;
    for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < total;
         t += (int64_t)gridDim.x * kBlock) {
        const int hub = (int)(t / per_row), bh = (int)(t % per_row);
        const int4 r = p.hub.rows[hub];
        float s = 0.0f, a1 = 0.0f, a2 = 0.0f;
        for (int c = 0; c < r.z; c++) {
            const float *st = p.hub.partial + ((size_t)(r.y + c) * per_row + bh) * 3;
            s += st[0];
            a1 += st[1];
            a2 += st[2];
        }
        p.rowstat[((size_t)hub * per_row + bh) * 3] = s;
        const int b = bh / p.H, h = bh % p.H;
        p.grad_q[((size_t)b * p.n_dst + r.x) * p.H + h] = a1 - s * a2;
    }
}

template <int HP>
__global__ __launch_bounds__(kBlock) void sddmm_bwd_hub_apply_kernel(SddmmParams p) {
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);
    const int wave = threadIdx.x / kWave, hl = lane_id() % HP;
    constexpr int kPerWave = kHubChunk / kWavesPerBlock;
    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int4 it = p.hub.items[item];
        const int row = it.x, chunk = it.y, hub = it.z;
        const int beg = p.indptr[row] + chunk * kHubChunk;
        const int end = min(p.indptr[row + 1], beg + kHubChunk);
        const int wbeg = min(end, beg + wave * kPerWave), wend = min(end, wbeg + kPerWave);
        for (int h0 = 0; h0 < p.H; h0 += HP) {
            const int h = h0 + hl;
            const bool act_h = h < p.H;
            for (int b = 0; b < p.n_bid; b++) {
                const float qv = act_h ? p.query[((size_t)b * p.n_dst + row) * p.H + h] : 0.0f;
                const float S = act_h ? p.rowstat[stat_index(p, hub, b, h)] : 0.0f;
                bwd_apply<HP>(p, wbeg, wend, b, h, act_h, qv, S);
            }
        }
    }
}

// One query block (n_bid = 1): windowed row kernels + row-plan items (gat.hip).
size_t attn_workspace_bytes(int64_t n_dst, int64_t nnz, int64_t H);
int attn_forward_run(float *attn, const int32_t *indptr, const int32_t *indices,
                     const float *query, const float *key, int64_t n_dst, int64_t n_src,
                     int64_t nnz, int64_t n_heads, int64_t max_degree, const void *plan,
                     void *workspace, size_t workspace_bytes, hipStream_t stream);
int attn_backward_run(float *grad_query, float *grad_edge, const int32_t *indptr,
                      const int32_t *indices, const float *query, const float *key,
                      const float *attn, const float *grad_attn, int64_t n_dst, int64_t n_src,
                      int64_t nnz, int64_t n_heads, int64_t max_degree, const void *plan,
                      void *workspace, size_t workspace_bytes, hipStream_t stream);

// The body of yitu_sddmm_backward; rows with fewer than skip_below edges are
// left alone (the fused GAT backward has already written their results).
int sddmm_backward_run(float *grad_query, float *grad_key, float *grad_edge, const int32_t *indptr,
                       const int32_t *indices, const float *query, const float *key,
                       const float *attn, const float *grad_out, const int32_t *t_indptr,
                       const int32_t *t_perm, int64_t n_dst, int64_t n_src, int64_t nnz,
                       int64_t n_heads, int64_t n_bid, int64_t max_degree, int64_t max_degree_t,
                       const void *plan, const void *plan_t, void *workspace,
                       size_t workspace_bytes, int skip_below, hipStream_t stream);

}  // namespace yitu
