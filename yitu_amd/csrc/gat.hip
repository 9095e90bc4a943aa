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
// Rows of 64 or more edges take the row plan's band-ordered 64-edge items:
// item statistics, per-row merge, item apply (attn + partial rows), and the SpMM
// reduce kernel, which adds a row's partials in a fixed order.
//
// Backward: one pass over the by-source structure gathers grad_out[row] once per
// edge and produces both d_attn (dot with the source's own row) and grad_x
// (attn-weighted sum); the softmax + LeakyReLU backward and the grad_key sum
// then work on [nnz, H] edge arrays only.
#include "../../include/yitu_hip.h"
#include "sddmm_kernels.hpp"

namespace yitu {

struct GatParams {
    SpmmParams sp;       // indptr, indices, feat = x [n_src, L], out, n_rows, L, F, H, plan, partial
    const float *query;  // [n_dst, H]
    const float *key;    // [n_src, H]
    float *attn;         // [nnz, H] or null
    int HP;              // heads rounded up to a power of two (<= 64)
    float *item_stats;   // [plan item id][H][2]: (max, sum) of the item's logits
    float *row_stats;    // [n_dst][H][2]: (max, 1/sum) of the planned rows
    float *stats_out;    // optional output, same layout, for every row (then row_stats == stats_out)
};

// (max, sum) over the lanes that share lane % hp, hp a runtime power of two
__device__ __forceinline__ MaxSum ms_wave_rt(MaxSum a, int hp) {
    for (int o = 32; o >= hp; o >>= 1) {
        MaxSum b{__shfl_xor(a.m, o, kWave), __shfl_xor(a.s, o, kWave)};
        a = ms_merge(a, b);
    }
    return a;
}

// Softmax statistics of the n edges in window lanes [first, first + n) for this
// lane's head (lane % HP), in the (edge, head) lane layout.
__device__ __forceinline__ MaxSum gat_stats_window(const GatParams &p, const EdgeWindow &win,
                                                   int first, int n, float qv) {
    const int lane = lane_id();
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    const int H = p.sp.H;
    MaxSum a = ms_init();
    // four steps of key gathers in flight before the first is used
    for (int k0 = 0; k0 < n; k0 += 4 * eps) {
        float kv[4];
        bool ok[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int k = k0 + u * eps + esub;
            const int col = __shfl(win.col, first + min(k, n - 1), kWave);
            ok[u] = k < n && hl < H;
            kv[u] = ok[u] ? p.key[(size_t)col * H + hl] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (ok[u]) a = ms_push(a, leaky(qv + kv[u]));
    }
    return a;
}

// Phase B for the n edges in window lanes [first, first + n) (CSR edges e0 ...):
// every (edge, head) probability is computed once in the (edge, head) layout,
// stored to attn, then broadcast to the (slot, column) layout that gathers the
// x[col] tiles. m / inv are this lane's head statistics (lane % HP = head).
template <int VEC, int G, int KT>
__device__ __forceinline__ void gat_apply_window(float (&acc)[KT][VEC], const GatParams &p,
                                                 const TileLanes<VEC, G, KT, W_EDGEHEAD> &tl,
                                                 const EdgeWindow &win, int first, int n, int e0,
                                                 float qv, float m, float inv, bool write_attn) {
    constexpr int SLOTS = kWave / G;
    constexpr int UNROLL = KT >= 4 ? 2 : 4;
    const int lane = lane_id();
    const int slot = lane / G;
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    const int H = p.sp.H, L = p.sp.L;
    const float *__restrict__ feat = static_cast<const float *>(p.sp.feat);

    for (int k0 = 0; k0 < n; k0 += eps) {
        const int nb = min(eps, n - k0);
        const int k = k0 + esub;
        const int col = __shfl(win.col, first + min(k, n - 1), kWave);
        float pv = 0.0f;
        if (k < n && hl < H) {
            pv = expf(leaky(qv + p.key[(size_t)col * H + hl]) - m) * inv;
            if (write_attn) p.attn[(size_t)(e0 + k) * H + hl] = pv;
        }
        for (int j0 = 0; j0 < nb; j0 += SLOTS * UNROLL) {
            float v[UNROLL][KT][VEC];
            float w[UNROLL][KT];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                const int ej = j0 + u * SLOTS + slot;
                const bool valid = ej < nb;
                const int src = valid ? ej * p.HP : 0;  // lane holding edge ej, head 0
                const int c = __shfl(col, src, kWave);
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    const float wt = __shfl(pv, src + tl.head[t], kWave);
                    w[u][t] = (valid && tl.live[t]) ? wt : 0.0f;
                }
                if (j0 + u * SLOTS < nb) {  // wave-uniform: steps past the sub-batch load nothing
#pragma unroll
                    for (int t = 0; t < KT; t++)
                        RowLoad<VEC, float>::ld(feat + (size_t)c * L + tl.off[t], v[u][t]);
                } else {
#pragma unroll
                    for (int t = 0; t < KT; t++)
#pragma unroll
                        for (int i = 0; i < VEC; i++) v[u][t][i] = 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                // a slot without an edge has loaded edge 0's row: 0 x value is not 0 for
                // every value, so the row is dropped (here, after the loads are out)
                const bool valid = SLOTS == 1 || j0 + u * SLOTS + slot < nb;
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < VEC; i++)
                        acc[t][i] += w[u][t] * (valid ? v[u][t][i] : 0.0f);
            }
        }
    }
}

// Short rows, fully fused: a wave walks rows_per_wave rows; per row statistics,
// then probabilities + aggregate, all from the sliding edge window.
template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void gat_rows_kernel(GatParams p) {
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.sp.n_rows);
    const int r0 = (blockIdx.x * kWavesPerBlock + wave_id()) * rpw;
    if (r0 >= p.sp.n_rows) return;
    const int n_here = min(rpw, p.sp.n_rows - r0);
    const int my_ptr = p.sp.indptr[r0 + min(lane, n_here)];
    const int limit = __builtin_amdgcn_readlane(my_ptr, n_here);
    const int sub = lane % G, slot = lane / G;
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H, L = p.sp.L;
    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;
    for (int i = 0; i < n_here; i++) {
        const int row = r0 + i;
        const int beg = __builtin_amdgcn_readlane(my_ptr, i), end = __builtin_amdgcn_readlane(my_ptr, i + 1);
        const int deg = end - beg;
        if (deg >= p.sp.plan.threshold) continue;
        float qv = 0.0f, m = 0.0f, inv = 0.0f;
        if (deg > 0) {
            qv = hl < H ? p.query[(size_t)row * H + hl] : 0.0f;
            MaxSum a = ms_init();
            for (int b = beg; b < end; b += kWave) {
                const int n = min(kWave, end - b);
                if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                    load_window<W_NONE>(win, p.sp, b, limit);
                a = ms_merge(a, gat_stats_window(p, win, b - win.base, n, qv));
            }
            a = ms_wave_rt(a, p.HP);
            m = a.m;
            inv = 1.0f / a.s;
        }
        if (p.stats_out && lane < p.HP && hl < H) {
            p.stats_out[((size_t)row * H + hl) * 2] = m;
            p.stats_out[((size_t)row * H + hl) * 2 + 1] = inv;
        }
        for (int c0 = 0; c0 < L; c0 += G * VEC * KT) {
            const TileLanes<VEC, G, KT, W_EDGEHEAD> tl(p.sp, c0);
            float acc[KT][VEC];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int k = 0; k < VEC; k++) acc[t][k] = 0.0f;
            for (int b = beg; b < end; b += kWave) {
                const int n = min(kWave, end - b);
                if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                    load_window<W_NONE>(win, p.sp, b, limit);
                gat_apply_window<VEC, G, KT>(acc, p, tl, win, b - win.base, n, b, qv, m, inv,
                                             p.attn && c0 == 0);
            }
            if (deg > 0) fold_slots<VEC, G, KT>(acc);
            if (slot == 0) {
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    const int o = c0 + (t * G + sub) * VEC;
                    if (o < L) store_row<VEC>(p.sp.out + (size_t)row * L + o, acc[t]);
                }
            }
        }
    }
}

// Long rows, step 1: (max, sum) of every plan item.
__global__ __launch_bounds__(kBlock) void gat_item_stats_kernel(GatParams p) {
    const int lane = lane_id();
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        // all windows and query values first, so the items' key gathers do not
        // each wait behind their own index load
        EdgeWindow win[kItemsPerWave];
        int n[kItemsPerWave], item[kItemsPerWave];
        float qv[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            const int beg = __builtin_amdgcn_readlane(my_rec.x, j), end = __builtin_amdgcn_readlane(my_rec.y, j);
            item[j] = __builtin_amdgcn_readlane(my_rec.z, j);
            const int row = __builtin_amdgcn_readlane(my_rec.w, j) & 0x7fffffff;
            n[j] = j < n_here ? end - beg : 0;
            qv[j] = 0.0f;
            if (n[j] > 0) {
                load_window<W_NONE>(win[j], p.sp, beg, end);
                if (hl < H) qv[j] = p.query[(size_t)row * H + hl];
            }
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            if (n[j] <= 0) continue;
            MaxSum a = ms_wave_rt(gat_stats_window(p, win[j], 0, n[j], qv[j]), p.HP);
            if (lane < p.HP && lane < H) {
                p.item_stats[((size_t)item[j] * H + lane) * 2] = a.m;
                p.item_stats[((size_t)item[j] * H + lane) * 2 + 1] = a.s;
            }
        }
    }
}

// Step 2: merge the item statistics of every planned row in item order.
__global__ __launch_bounds__(kBlock) void gat_row_combine_kernel(GatParams p) {
    if (p.sp.plan.counters->overflow) return;
    const int n_rows = min(p.sp.plan.counters->n_rows, p.sp.plan.max_rows);
    const int H = p.sp.H;
    const int lane = lane_id();
    // one wave per planned row: lane = (item slot, head), merged by a fixed butterfly
    const int hl = lane & (p.HP - 1), c0 = lane / p.HP, step = kWave / p.HP;
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int slot = blockIdx.x * kWavesPerBlock + wave_id(); slot < n_rows;
         slot += n_waves) {
        const int4 r = p.sp.plan.rows[slot];
        MaxSum a = ms_init();
        if (hl < H) {
            for (int c = c0; c < r.z; c += step) {
                const float *st = p.item_stats + ((size_t)(r.y + c) * H + hl) * 2;
                a = ms_merge(a, MaxSum{st[0], st[1]});
            }
        }
        a = ms_wave_rt(a, p.HP);
        if (lane < p.HP && lane < H) {
            p.row_stats[((size_t)r.x * H + lane) * 2] = a.m;
            p.row_stats[((size_t)r.x * H + lane) * 2 + 1] = 1.0f / a.s;
        }
    }
}

// Step 3: probabilities and weighted aggregate of every item, in band order.
template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void gat_item_apply_kernel(GatParams p) {
    const int lane = lane_id();
    const int sub = lane % G, slot = lane / G;
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H, L = p.sp.L;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int e_beg[kItemsPerWave], n_edges[kItemsPerWave], item_id[kItemsPerWave],
            row_tag[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            e_beg[j] = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            item_id[j] = __builtin_amdgcn_readlane(my_rec.z, j);
            row_tag[j] = __builtin_amdgcn_readlane(my_rec.w, j);
            n_edges[j] = j < n_here ? end - e_beg[j] : 0;
            if (n_edges[j] > 0) load_window<W_NONE>(win[j], p.sp, e_beg[j], end);
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            if (n_edges[j] <= 0) continue;
            const bool single = row_tag[j] < 0;
            const int row = row_tag[j] & 0x7fffffff;
            float qv = 0.0f, m = 0.0f, inv = 0.0f;
            if (hl < H) {
                qv = p.query[(size_t)row * H + hl];
                m = p.row_stats[((size_t)row * H + hl) * 2];
                inv = p.row_stats[((size_t)row * H + hl) * 2 + 1];
            }
            float *dst = single ? p.sp.out + (size_t)row * L
                                : p.sp.partial + (size_t)item_id[j] * L;
            for (int c0 = 0; c0 < L; c0 += G * VEC * KT) {
                const TileLanes<VEC, G, KT, W_EDGEHEAD> tl(p.sp, c0);
                float acc[KT][VEC];
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int k = 0; k < VEC; k++) acc[t][k] = 0.0f;
                gat_apply_window<VEC, G, KT>(acc, p, tl, win[j], 0, n_edges[j], e_beg[j], qv, m,
                                             inv, p.attn && c0 == 0);
                fold_slots<VEC, G, KT>(acc);
                if (slot == 0) {
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        const int o = c0 + (t * G + sub) * VEC;
                        if (o < L) store_row<VEC>(dst + o, acc[t]);
                    }
                }
            }
        }
    }
}

// ---- planned rows without the probabilities as an output ------------------------
// When no [nnz, H] probabilities are asked for, an item does not wait for its
// row's statistics: it weighs its edges by exp(logit - the item's own max) and
// leaves the sum unnormalised, next to its (max, sum). The reduction then scales
// item c of a row by exp(max_c - max_row) / sum_row. That drops the separate pass
// over the items' keys. Rows of one item are normalised and written at once.
template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void gat_item_local_kernel(GatParams p) {
    const int lane = lane_id();
    const int sub = lane % G, slot = lane / G;
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H, L = p.sp.L;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int e_beg[kItemsPerWave], n_edges[kItemsPerWave], item_id[kItemsPerWave],
            row_tag[kItemsPerWave];
        float qv[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            e_beg[j] = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            item_id[j] = __builtin_amdgcn_readlane(my_rec.z, j);
            row_tag[j] = __builtin_amdgcn_readlane(my_rec.w, j);
            n_edges[j] = j < n_here ? end - e_beg[j] : 0;
            qv[j] = 0.0f;
            if (n_edges[j] > 0) {
                load_window<W_NONE>(win[j], p.sp, e_beg[j], end);
                if (hl < H) qv[j] = p.query[(size_t)(row_tag[j] & 0x7fffffff) * H + hl];
            }
        }
        MaxSum st[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            st[j] = ms_init();
            if (n_edges[j] > 0)
                st[j] = ms_wave_rt(gat_stats_window(p, win[j], 0, n_edges[j], qv[j]), p.HP);
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            if (n_edges[j] <= 0) continue;
            const bool single = row_tag[j] < 0;
            const int row = row_tag[j] & 0x7fffffff;
            if (lane < p.HP && lane < H) {
                p.item_stats[((size_t)item_id[j] * H + lane) * 2] = st[j].m;
                p.item_stats[((size_t)item_id[j] * H + lane) * 2 + 1] = st[j].s;
            }
            const float inv = single ? 1.0f / st[j].s : 1.0f;
            float *dst = single ? p.sp.out + (size_t)row * L
                                : p.sp.partial + (size_t)item_id[j] * L;
            for (int c0 = 0; c0 < L; c0 += G * VEC * KT) {
                const TileLanes<VEC, G, KT, W_EDGEHEAD> tl(p.sp, c0);
                float acc[KT][VEC];
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int k = 0; k < VEC; k++) acc[t][k] = 0.0f;
                gat_apply_window<VEC, G, KT>(acc, p, tl, win[j], 0, n_edges[j], e_beg[j], qv[j],
                                             st[j].m, inv, false);
                fold_slots<VEC, G, KT>(acc);
                if (slot == 0) {
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        const int o = c0 + (t * G + sub) * VEC;
                        if (o < L) store_row<VEC>(dst + o, acc[t]);
                    }
                }
            }
        }
    }
}

// The same with the head count (rounded up to a power of two) known at compile time:
// the HP sub-batches of 64 / HP edges that an item can hold stay in registers, so every
// (edge, head) logit is made once. The statistics are a maximum, then one exponential per
// logit, then a sum (the running (max, sum) pair costs two exponentials per element and
// per butterfly step), each reduced over the lanes that share a head in log2(64 / HP)
// steps, and the exponentials are the weights of the aggregate: no second key gather.
// Per item about 700 vector instructions against 1,250; the kernel above was bound by
// instruction issue wherever most of its gathers hit L2.
template <int VEC, int G, int KT, int HP>
__global__ __launch_bounds__(kBlock) void gat_item_local_hp_kernel(GatParams p) {
    constexpr int EPS = kWave / HP;  // edges per sub-batch
    constexpr int kLocalItems = 1;   // items of a group
    constexpr int SLOTS = kWave / G;
    constexpr int UNROLL = KT >= 4 ? 2 : (KT == 2 ? 4 : 8);  // row gathers in flight (KT = 1: 4 / 8 / 16 measured 811 / 767 / 822 us)
    const int lane = lane_id();
    const int sub = lane % G, slot = lane / G;
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int hl = lane & (HP - 1), esub = lane / HP;
    const int H = p.sp.H, L = p.sp.L;
    const float *__restrict__ feat = static_cast<const float *>(p.sp.feat);
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kLocalItems;
         pos0 < n_items; pos0 += n_waves * kLocalItems) {
        const int n_here = min(kLocalItems, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        int col[kLocalItems], n_edges[kLocalItems], item_id[kLocalItems],
            row_tag[kLocalItems];
        float qv[kLocalItems];
#pragma unroll
        for (int j = 0; j < kLocalItems; j++) {
            const int beg = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            item_id[j] = __builtin_amdgcn_readlane(my_rec.z, j);
            row_tag[j] = __builtin_amdgcn_readlane(my_rec.w, j);
            n_edges[j] = j < n_here ? end - beg : 0;
            // lane e holds the source of the item's edge e (the last one again past the end)
            col[j] = p.sp.indices[beg + min(lane, max(n_edges[j], 1) - 1)] & kColMask;
            qv[j] = hl < H ? p.query[(size_t)(row_tag[j] & 0x7fffffff) * H + hl] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < kLocalItems; j++) {
            if (n_edges[j] <= 0) continue;  // wave-uniform
            const int n = n_edges[j];
            // (edge, head) layout: sub-batch r, lane (esub, hl) = edge r EPS + esub, head hl
            float pv[HP];
            int cr[HP];
#pragma unroll
            for (int r = 0; r < HP; r++) {
                const int k = r * EPS + esub;
                cr[r] = __shfl(col[j], min(k, n - 1), kWave);
                const float kv = hl < H ? p.key[(size_t)cr[r] * H + hl] : 0.0f;
                pv[r] = (k < n && hl < H) ? leaky(qv[j] + kv) : -FLT_MAX;
            }
            float m = pv[0];
#pragma unroll
            for (int r = 1; r < HP; r++) m = fmaxf(m, pv[r]);
            m = wave_max_strided<HP>(m);
            float ssum = 0.0f;
#pragma unroll
            for (int r = 0; r < HP; r++) {
                pv[r] = (r * EPS + esub < n && hl < H) ? expf(pv[r] - m) : 0.0f;
                ssum += pv[r];
            }
            ssum = wave_sum_strided<HP>(ssum);
            const bool single = row_tag[j] < 0;
            const int row = row_tag[j] & 0x7fffffff;
            if (lane < HP && lane < H) {
                p.item_stats[((size_t)item_id[j] * H + lane) * 2] = m;
                p.item_stats[((size_t)item_id[j] * H + lane) * 2 + 1] = ssum;
            }
            if (single) {
                const float inv = 1.0f / ssum;
#pragma unroll
                for (int r = 0; r < HP; r++) pv[r] *= inv;
            }
            float *dst = single ? p.sp.out + (size_t)row * L
                                : p.sp.partial + (size_t)item_id[j] * L;
            for (int c0 = 0; c0 < L; c0 += G * VEC * KT) {
                const TileLanes<VEC, G, KT, W_EDGEHEAD> tl(p.sp, c0);
                float acc[KT][VEC];
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int k = 0; k < VEC; k++) acc[t][k] = 0.0f;
#pragma unroll
                for (int r = 0; r < HP; r++) {
                    if (r * EPS >= n) break;  // wave-uniform
                    const int nb = min(EPS, n - r * EPS);
                    for (int j0 = 0; j0 < nb; j0 += SLOTS * UNROLL) {
                        float v[UNROLL][KT][VEC], w[UNROLL][KT];
#pragma unroll
                        for (int u = 0; u < UNROLL; u++) {
                            const int ej = j0 + u * SLOTS + slot;
                            const bool valid = ej < nb;
                            const int src = valid ? ej * HP : 0;  // lane of (edge ej, head 0)
                            int c;
                            if constexpr (SLOTS == 1)  // one edge for the whole wave: a scalar
                                c = __builtin_amdgcn_readlane(cr[r], src);
                            else
                                c = __shfl(cr[r], src, kWave);
#pragma unroll
                            for (int t = 0; t < KT; t++) {
                                const float wt = __shfl(pv[r], src + tl.head[t], kWave);
                                w[u][t] = (valid && tl.live[t]) ? wt : 0.0f;
                            }
                            if (j0 + u * SLOTS < nb) {  // wave-uniform
#pragma unroll
                                for (int t = 0; t < KT; t++)
                                    RowLoad<VEC, float>::ld(feat + (size_t)c * L + tl.off[t], v[u][t]);
                            } else {
#pragma unroll
                                for (int t = 0; t < KT; t++)
#pragma unroll
                                    for (int i = 0; i < VEC; i++) v[u][t][i] = 0.0f;
                            }
                        }
#pragma unroll
                        for (int u = 0; u < UNROLL; u++) {
                            const bool valid = SLOTS == 1 || j0 + u * SLOTS + slot < nb;  // as above
#pragma unroll
                            for (int t = 0; t < KT; t++)
#pragma unroll
                                for (int i = 0; i < VEC; i++)
                                    acc[t][i] += w[u][t] * (valid ? v[u][t][i] : 0.0f);
                        }
                    }
                }
                fold_slots<VEC, G, KT>(acc);
                if (slot == 0) {
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        const int o = c0 + (t * G + sub) * VEC;
                        if (o < L) store_row_streaming<VEC>(dst + o, acc[t]);
                    }
                }
            }
        }
    }
}

// s += exp(max_c - m_row) * src[c * L] for c = first, first + step, ... < n, in
// that order; st points at the first item's (max, sum) of this lane's head.
__device__ __forceinline__ void sum_scaled_partials(float (&s)[4], const float *src,
                                                    const float *st, int H, float m_row, int L,
                                                    int first, int n, int step) {
    int c = first;
    for (; c + 3 * step < n; c += 4 * step) {
        float v[4][4], w[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            RowLoad<4, float>::ld(src + (size_t)(c + u * step) * L, v[u]);
            w[u] = st[(size_t)(c + u * step) * H * 2];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const float f = expf(w[u] - m_row);
#pragma unroll
            for (int i = 0; i < 4; i++) s[i] += f * v[u][i];
        }
    }
    for (; c < n; c += step) {
        float v[4];
        RowLoad<4, float>::ld(src + (size_t)c * L, v);
        const float f = expf(st[(size_t)c * H * 2] - m_row);
#pragma unroll
        for (int i = 0; i < 4; i++) s[i] += f * v[i];
    }
}

// Adds the unnormalised item sums of every planned row with more than one item
// (after gat_row_combine_kernel), four columns per lane; the head width is a
// multiple of four, so a lane's columns share a head. Work split and summation
// order as in spmm_reduce_kernel.
__global__ __launch_bounds__(kBlock) void gat_scaled_reduce_kernel(GatParams p) {
    __shared__ float red[kBlock * 4];
    if (p.sp.plan.counters->overflow) return;
    const int n_hub = min(p.sp.plan.counters->n_rows, p.sp.plan.max_rows);
    const int L = p.sp.L, H = p.sp.H, F = p.sp.F;
    const int lanes_total = L / 4;
    const int half = gridDim.x / 2;
    if ((int)blockIdx.x < half) {
        const int lane = lane_id();
        int lanes = 1;
        while (lanes < lanes_total && lanes < kWave) lanes <<= 1;
        const int slots = kWave / lanes;
        const int slot = lane / lanes, sub = lane % lanes;
        const int stride = half * kWavesPerBlock;
        for (int h = blockIdx.x * kWavesPerBlock + wave_id(); h < n_hub; h += stride) {
            const int4 r = p.sp.plan.rows[h];
            if (r.z <= 1 || r.z > kReduceWaveItems) continue;
            for (int l0 = 0; l0 < lanes_total; l0 += lanes) {
                const bool live = l0 + sub < lanes_total;
                float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                float inv = 0.0f;
                if (live) {
                    const int head = (l0 + sub) * 4 / F;
                    const float *rs = p.row_stats + ((size_t)r.x * H + head) * 2;
                    inv = rs[1];
                    sum_scaled_partials(s, p.sp.partial + (size_t)r.y * L + (size_t)(l0 + sub) * 4,
                                        p.item_stats + ((size_t)r.y * H + head) * 2, H, rs[0], L,
                                        slot, r.z, slots);
                }
                for (int o = kWave / 2; o >= lanes; o >>= 1)
#pragma unroll
                    for (int i = 0; i < 4; i++) s[i] += __shfl_xor(s[i], o, kWave);
                if (live && slot == 0) {
#pragma unroll
                    for (int i = 0; i < 4; i++) s[i] *= inv;
                    store_row_streaming<4>(p.sp.out + (size_t)r.x * L + (size_t)(l0 + sub) * 4, s);
                }
            }
        }
        return;
    }
    for (int h = blockIdx.x - half; h < n_hub; h += gridDim.x - half) {
        const int4 r = p.sp.plan.rows[h];
        if (r.z <= kReduceWaveItems) continue;
        for (int l0 = 0; l0 < lanes_total; l0 += kBlock) {
            const int lanes = min(kBlock, lanes_total - l0);
            const int groups = kBlock / lanes;
            const int g = threadIdx.x / lanes, l = threadIdx.x % lanes;
            float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            float inv = 0.0f;
            if (g < groups) {
                const int head = (l0 + l) * 4 / F;
                const float *rs = p.row_stats + ((size_t)r.x * H + head) * 2;
                inv = rs[1];
                sum_scaled_partials(s, p.sp.partial + (size_t)r.y * L + (size_t)(l0 + l) * 4,
                                    p.item_stats + ((size_t)r.y * H + head) * 2, H, rs[0], L, g,
                                    r.z, groups);
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < 4; i++) red[threadIdx.x * 4 + i] = s[i];
            __syncthreads();
            if (g == 0) {
                for (int gg = 1; gg < groups; gg++)
#pragma unroll
                    for (int i = 0; i < 4; i++) s[i] += red[(gg * lanes + l) * 4 + i];
#pragma unroll
                for (int i = 0; i < 4; i++) s[i] *= inv;
                store_row_streaming<4>(p.sp.out + (size_t)r.x * L + (size_t)(l0 + l) * 4, s);
            }
        }
    }
}

// ---- backward of the softmax + LeakyReLU ----------------------------------------
// Given d_attn per edge and head, the three row sums
//   S = sum a d_attn,  A1 = sum a d_attn s,  A2 = sum a s   (s = LeakyReLU slope)
// give the per-edge logit gradient a (d_attn - S) s and grad_q = A1 - S A2.
struct GatBwdParams {
    SpmmParams sp;  // indptr, indices, n_rows, H, col_mask, plan
    const float *grad_out;  // unused by the attention-only kernels
    const float *query, *key, *attn;
    float *grad_q;  // [n_dst, H]
    float *grad_e;  // [nnz, H] per-edge logit gradient
    // planned rows (three kernels: item sums, row combine, item apply)
    float *grad_a;      // [nnz, H] d_attn (input)
    float *item_sums;   // [plan item id][H][3]: (S, A1, A2) over the item's edges
    float *row_sum;     // [n_dst][H]: S of every planned row
    int HP;             // heads rounded up to a power of two (item sums / combine lane layout)
};

constexpr int kDotUnroll = 4;  // gathers in flight per wave in the backward dots
constexpr int kSrcItems = 2;   // plan items a wave of the by-source item kernels takes per turn (1 / 2 / 4:
                               // 974 / 953 / 1004 us on a 2^18-node graph, 5.57 / 5.47 / 5.37 ms on a 2^21-node one)

// One wave per planned row adds its items' sums (lane = (item slot, head),
// fixed butterfly), writes S of the row and grad_q = A1 - S A2.
__global__ __launch_bounds__(kBlock) void gat_bwd_combine_kernel(GatBwdParams p) {
    if (p.sp.plan.counters->overflow) return;
    const int n_rows = min(p.sp.plan.counters->n_rows, p.sp.plan.max_rows);
    const int lane = lane_id();
    const int H = p.sp.H;
    const int h = lane & (p.HP - 1), c0 = lane / p.HP, step = kWave / p.HP;
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int slot = blockIdx.x * kWavesPerBlock + wave_id(); slot < n_rows;
         slot += n_waves) {
        const int4 r = p.sp.plan.rows[slot];
        float s = 0.0f, a1 = 0.0f, a2 = 0.0f;
        if (h < H) {
            for (int c = c0; c < r.z; c += step) {
                const float *st = p.item_sums + ((size_t)(r.y + c) * H + h) * 3;
                s += st[0];
                a1 += st[1];
                a2 += st[2];
            }
        }
        for (int o = kWave / 2; o >= p.HP; o >>= 1) {
            s += __shfl_xor(s, o, kWave);
            a1 += __shfl_xor(a1, o, kWave);
            a2 += __shfl_xor(a2, o, kWave);
        }
        if (lane < p.HP && h < H) {
            p.row_sum[(size_t)r.x * H + h] = s;
            p.grad_q[(size_t)r.x * H + h] = a1 - s * a2;
        }
    }
}

// Per-edge logit gradient of the planned rows' edges, (edge, head) per lane.
__global__ __launch_bounds__(kBlock) void gat_bwd_apply_kernel(GatBwdParams p) {
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int lane = lane_id();
    const int H = p.sp.H;
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int beg[kItemsPerWave], n[kItemsPerWave];
        float qv[kItemsPerWave], S[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            beg[j] = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            const int row = __builtin_amdgcn_readlane(my_rec.w, j) & 0x7fffffff;
            n[j] = j < n_here ? end - beg[j] : 0;
            qv[j] = S[j] = 0.0f;
            if (n[j] > 0) {
                load_window<W_NONE>(win[j], p.sp, beg[j], end);
                if (hl < H) {
                    qv[j] = p.query[(size_t)row * H + hl];
                    S[j] = p.row_sum[(size_t)row * H + hl];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            for (int k0 = 0; k0 < n[j]; k0 += 4 * eps) {
                float a[4], g[4], kv[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int k = k0 + u * eps + esub;
                    const int col = __shfl(win[j].col, min(k, n[j] - 1), kWave);
                    a[u] = g[u] = kv[u] = 0.0f;
                    if (k < n[j] && hl < H) {
                        const size_t e = (size_t)(beg[j] + k) * H + hl;
                        a[u] = p.attn[e];
                        g[u] = p.grad_a[e];
                        kv[u] = p.key[(size_t)col * H + hl];
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int k = k0 + u * eps + esub;
                    if (k < n[j] && hl < H)
                        p.grad_e[(size_t)(beg[j] + k) * H + hl] =
                            a[u] * (g[u] - S[j]) * (qv[j] + kv[u] < 0.0f ? kSlope : 1.0f);
                }
            }
        }
    }
}

// ---- attention only (the stand-alone SDDMM + LeakyReLU + edge softmax, one
// query block): the statistics / write halves of the fused kernels above, and
// the softmax backward over (edge, head) lanes. --------------------------------

// Probabilities of the n edges in window lanes [first, first + n) (CSR edges e0 ...).
__device__ __forceinline__ void attn_write_window(const GatParams &p, const EdgeWindow &win,
                                                  int first, int n, int e0, float qv, float m,
                                                  float inv) {
    const int lane = lane_id();
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    const int H = p.sp.H;
    for (int k0 = 0; k0 < n; k0 += 4 * eps) {
        float kv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int k = k0 + u * eps + esub;
            const int col = __shfl(win.col, first + min(k, n - 1), kWave);
            kv[u] = (k < n && hl < H) ? p.key[(size_t)col * H + hl] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int k = k0 + u * eps + esub;
            if (k < n && hl < H)
                p.attn[(size_t)(e0 + k) * H + hl] = expf(leaky(qv + kv[u]) - m) * inv;
        }
    }
}

// Short rows: rows_per_wave rows per wave through the sliding edge window.
__global__ __launch_bounds__(kBlock) void attn_rows_kernel(GatParams p) {
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.sp.n_rows);
    const int r0 = (blockIdx.x * kWavesPerBlock + wave_id()) * rpw;
    if (r0 >= p.sp.n_rows) return;
    const int n_here = min(rpw, p.sp.n_rows - r0);
    const int my_ptr = p.sp.indptr[r0 + min(lane, n_here)];
    const int limit = __builtin_amdgcn_readlane(my_ptr, n_here);
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H;
    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;
    for (int i = 0; i < n_here; i++) {
        const int beg = __builtin_amdgcn_readlane(my_ptr, i), end = __builtin_amdgcn_readlane(my_ptr, i + 1);
        const int n = end - beg;
        if (n == 0 || n >= p.sp.plan.threshold) continue;
        const float qv = hl < H ? p.query[(size_t)(r0 + i) * H + hl] : 0.0f;
        if (n > kWave) {
            // no plan although the row is long (a caller's max-degree hint was too small):
            // two walks over the row's windows, slow but right
            MaxSum a = ms_init();
            for (int b = beg; b < end; b += kWave) {
                load_window<W_NONE>(win, p.sp, b, limit);
                a = ms_merge(a, gat_stats_window(p, win, 0, min(kWave, end - b), qv));
            }
            a = ms_wave_rt(a, p.HP);
            for (int b = beg; b < end; b += kWave) {
                load_window<W_NONE>(win, p.sp, b, limit);
                attn_write_window(p, win, 0, min(kWave, end - b), b, qv, a.m, 1.0f / a.s);
            }
            continue;
        }
        if (win.base < 0 || beg < win.base || end > win.base + kWave)
            load_window<W_NONE>(win, p.sp, beg, limit);
        const MaxSum a = ms_wave_rt(gat_stats_window(p, win, beg - win.base, n, qv), p.HP);
        attn_write_window(p, win, beg - win.base, n, beg, qv, a.m, 1.0f / a.s);
    }
}

// Planned rows, step 3 (after gat_item_stats_kernel and gat_row_combine_kernel).
__global__ __launch_bounds__(kBlock) void attn_item_write_kernel(GatParams p) {
    const int lane = lane_id();
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int beg[kItemsPerWave], n[kItemsPerWave];
        float qv[kItemsPerWave], m[kItemsPerWave], inv[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            beg[j] = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            const int row = __builtin_amdgcn_readlane(my_rec.w, j) & 0x7fffffff;
            n[j] = j < n_here ? end - beg[j] : 0;
            qv[j] = m[j] = inv[j] = 0.0f;
            if (n[j] > 0) {
                load_window<W_NONE>(win[j], p.sp, beg[j], end);
                if (hl < H) {
                    qv[j] = p.query[(size_t)row * H + hl];
                    m[j] = p.row_stats[((size_t)row * H + hl) * 2];
                    inv[j] = p.row_stats[((size_t)row * H + hl) * 2 + 1];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++)
            if (n[j] > 0) attn_write_window(p, win[j], 0, n[j], beg[j], qv[j], m[j], inv[j]);
    }
}

// Softmax + LeakyReLU backward sums of the n edges in window lanes [first, ...):
// S = sum a g, A1 = sum a g s, A2 = sum a s for this lane's head (lane % HP),
// g = grad_a (the gradient that arrives at attn). Not yet reduced over lanes.
__device__ __forceinline__ void attn_bwd_sums_window(const GatBwdParams &p, const EdgeWindow &win,
                                                     int first, int n, int e0, float qv, float &S,
                                                     float &A1, float &A2) {
    const int lane = lane_id();
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    const int H = p.sp.H;
    for (int k0 = 0; k0 < n; k0 += 4 * eps) {
        float a[4], g[4], kv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int k = k0 + u * eps + esub;
            const int col = __shfl(win.col, first + min(k, n - 1), kWave);
            a[u] = g[u] = kv[u] = 0.0f;  // a = 0 makes a lane past the range add nothing
            if (k < n && hl < H) {
                const size_t e = (size_t)(e0 + k) * H + hl;
                a[u] = p.attn[e];
                g[u] = p.grad_a[e];
                kv[u] = p.key[(size_t)col * H + hl];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const float sl = qv + kv[u] < 0.0f ? kSlope : 1.0f;
            S += a[u] * g[u];
            A1 += a[u] * g[u] * sl;
            A2 += a[u] * sl;
        }
    }
}

// Per-edge logit gradient a (g - S) slope of the n edges in window lanes [first, first + n)
// (CSR edges e0 ...), (edge, head) per lane.
__device__ __forceinline__ void attn_bwd_write_window(const GatBwdParams &p, const EdgeWindow &win,
                                                      int first, int n, int e0, float qv, float S) {
    const int lane = lane_id();
    const int hl = lane & (p.HP - 1), esub = lane / p.HP, eps = kWave / p.HP;
    const int H = p.sp.H;
    for (int k0 = 0; k0 < n; k0 += 4 * eps) {
        float a[4], g[4], kv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int k = k0 + u * eps + esub;
            const int col = __shfl(win.col, first + min(k, n - 1), kWave);
            a[u] = g[u] = kv[u] = 0.0f;
            if (k < n && hl < H) {
                const size_t e = (size_t)(e0 + k) * H + hl;
                a[u] = p.attn[e];
                g[u] = p.grad_a[e];
                kv[u] = p.key[(size_t)col * H + hl];
            }
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int k = k0 + u * eps + esub;
            if (k < n && hl < H)
                p.grad_e[(size_t)(e0 + k) * H + hl] =
                    a[u] * (g[u] - S) * (qv + kv[u] < 0.0f ? kSlope : 1.0f);
        }
    }
}

__device__ __forceinline__ void attn_bwd_reduce(float &S, float &A1, float &A2, int hp) {
    for (int o = kWave / 2; o >= hp; o >>= 1) {
        S += __shfl_xor(S, o, kWave);
        A1 += __shfl_xor(A1, o, kWave);
        A2 += __shfl_xor(A2, o, kWave);
    }
}

__global__ __launch_bounds__(kBlock) void attn_bwd_rows_kernel(GatBwdParams p) {
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.sp.n_rows);
    const int r0 = (blockIdx.x * kWavesPerBlock + wave_id()) * rpw;
    if (r0 >= p.sp.n_rows) return;
    const int n_here = min(rpw, p.sp.n_rows - r0);
    const int my_ptr = p.sp.indptr[r0 + min(lane, n_here)];
    const int limit = __builtin_amdgcn_readlane(my_ptr, n_here);
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H;
    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;
    for (int i = 0; i < n_here; i++) {
        const int row = r0 + i;
        const int beg = __builtin_amdgcn_readlane(my_ptr, i), end = __builtin_amdgcn_readlane(my_ptr, i + 1);
        const int n = end - beg;
        if (n >= p.sp.plan.threshold) continue;
        if (n == 0) {
            if (lane < p.HP && hl < H) p.grad_q[(size_t)row * H + hl] = 0.0f;
            continue;
        }
        const float qv = hl < H ? p.query[(size_t)row * H + hl] : 0.0f;
        float S = 0.0f, A1 = 0.0f, A2 = 0.0f;
        if (n > kWave) {
            // no plan although the row is long (a max-degree hint that was too small):
            // sums over all windows first, then the per-edge gradients
            for (int b = beg; b < end; b += kWave) {
                load_window<W_NONE>(win, p.sp, b, limit);
                attn_bwd_sums_window(p, win, 0, min(kWave, end - b), b, qv, S, A1, A2);
            }
            attn_bwd_reduce(S, A1, A2, p.HP);
            if (lane < p.HP && hl < H) p.grad_q[(size_t)row * H + hl] = A1 - S * A2;
            for (int b = beg; b < end; b += kWave) {
                load_window<W_NONE>(win, p.sp, b, limit);
                attn_bwd_write_window(p, win, 0, min(kWave, end - b), b, qv, S);
            }
            continue;
        }
        if (win.base < 0 || beg < win.base || end > win.base + kWave)
            load_window<W_NONE>(win, p.sp, beg, limit);
        const int first = beg - win.base;
        attn_bwd_sums_window(p, win, first, n, beg, qv, S, A1, A2);
        attn_bwd_reduce(S, A1, A2, p.HP);
        if (lane < p.HP && hl < H) p.grad_q[(size_t)row * H + hl] = A1 - S * A2;
        attn_bwd_write_window(p, win, first, n, beg, qv, S);
    }
}

__global__ __launch_bounds__(kBlock) void attn_bwd_item_sums_kernel(GatBwdParams p) {
    const int lane = lane_id();
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int hl = lane & (p.HP - 1);
    const int H = p.sp.H;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int beg[kItemsPerWave], n[kItemsPerWave], item[kItemsPerWave];
        float qv[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            beg[j] = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            item[j] = __builtin_amdgcn_readlane(my_rec.z, j);
            const int row = __builtin_amdgcn_readlane(my_rec.w, j) & 0x7fffffff;
            n[j] = j < n_here ? end - beg[j] : 0;
            qv[j] = 0.0f;
            if (n[j] > 0) {
                load_window<W_NONE>(win[j], p.sp, beg[j], end);
                if (hl < H) qv[j] = p.query[(size_t)row * H + hl];
            }
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            if (n[j] <= 0) continue;
            float S = 0.0f, A1 = 0.0f, A2 = 0.0f;
            attn_bwd_sums_window(p, win[j], 0, n[j], beg[j], qv[j], S, A1, A2);
            attn_bwd_reduce(S, A1, A2, p.HP);
            if (lane < p.HP && hl < H) {
                float *st = p.item_sums + ((size_t)item[j] * H + hl) * 3;
                st[0] = S;
                st[1] = A1;
                st[2] = A2;
            }
        }
    }
}

}  // namespace yitu

#include "attn_packed.hpp"

namespace yitu {

// ---- backward over the transposed structure: one gather for every gradient -------
// Walking the edges by source c, the source's own row x[c] is local and the
// gathered row is grad_out[row_e]. That single gather gives both
//   d_attn[e,h]   = <grad_out[row_e,h,:], x[c,h,:]>
//   grad_x[c,h,:] = sum_e attn[e,h] grad_out[row_e,h,:]
// so the backward needs one pass over the feature rows instead of two. Rows of
// L = 256 KT floats (KT = 1, 2, 4): lane l holds floats [256 t + 4 l, +4) of every
// tile t, a head owns LPH = F / 4 consecutive lanes of one tile (HPT = 64 / LPH heads
// per tile), the dot of edge k is kept by lane (k % LPH) of each head and stored
// through the edge permutation.
struct GatSrcParams {
    SpmmParams sp;   // indptr / indices / eperm = by-source structure, values = attn,
                     // feat = grad_out, out = grad_x, plan = its row plan, partial
    const float *x;  // [n_src, L]
    float *grad_a;   // [nnz, H], CSR order: d_attn (FULL = false) or the logit gradient (FULL)
    int grad_a_vec;  // grad_a is 16-byte aligned and H a multiple of 4: vector stores
    // FULL: the forward output is at hand, so the softmax row sum S[r,h] = sum_e a d_attn
    // = <grad_out[r,h,:], out[r,h,:]> is known before the pass and the whole
    // softmax + LeakyReLU backward happens per edge, here
    // [n_dst, H]: (S, query, softmax max, 1 / softmax sum) side by side: everything an edge
    // needs from its destination, in one line (max and 1 / sum only with `recompute`)
    const float4 *row_sq;
    const float *stats;  // forward's row statistics [n_dst, H, 2] = (max, 1 / sum), or null
    int recompute;       // attn is not read: a = exp(LeakyReLU(query + key) - max) / sum
    const float *key;      // [n_src, H]
    float *grad_k;         // [n_src, H]
    float *partial_k;      // [plan item id, H] partial grad_k of multi-item sources
    // The gathered rows. Normally grad_out [n_dst, L]. When the caller's output was the
    // mean over heads, its gradient g [n_dst, F] stands for grad_out[r,h,:] = g[r,:] / H:
    // the gather shrinks to F floats per edge, every head's lanes reading the same ones.
    int g_ld;        // floats between gathered rows: L, or F
    int head_mean;   // nonzero: the second form
    float g_scale;   // 1, or 1 / H
};

// (S[r,h], query[r,h]) with S[r,h] = <grad_out[r,h,:], out[r,h,:]>, kRowsPerWave rows
// per wave. The pair is what an edge needs from its destination.
template <int LPH, int KT>
__global__ __launch_bounds__(kBlock) void gat_row_dot_kernel(float4 *__restrict__ row_sq,
                                                             const float *__restrict__ grad_out,
                                                             const float *__restrict__ out,
                                                             const float *__restrict__ query,
                                                             const float *__restrict__ stats,
                                                             int n_rows, int g_ld, int head_mean,
                                                             float g_scale) {
    constexpr int HPT = kWave / LPH, H = HPT * KT, L = 256 * KT, U = KT == 1 ? 4 : 2;
    const int lane = lane_id();
    const int g_lane = (head_mean ? lane % LPH : lane) * 4, g_tile = head_mean ? 0 : 256;
    const int r0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kRowsPerWave;
    for (int i0 = 0; i0 < kRowsPerWave && r0 + i0 < n_rows; i0 += U) {
        float d[U][KT];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int r = min(r0 + i0 + u, n_rows - 1);
#pragma unroll
            for (int t = 0; t < KT; t++) {
                // both arrays are read once, front to back: streaming loads
                typedef float f4 __attribute__((ext_vector_type(4)));
                const f4 a = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(
                    grad_out + (size_t)r * g_ld + t * g_tile + g_lane));
                const f4 b = __builtin_nontemporal_load(
                    reinterpret_cast<const f4 *>(out + (size_t)r * L + t * 256 + lane * 4));
                d[u][t] = (a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3]) * g_scale;
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int r = r0 + i0 + u;
#pragma unroll
            for (int t = 0; t < KT; t++) {
                float s = d[u][t];
                s = group_sum<LPH>(s);
                const int head = t * HPT + lane / LPH;
                if (lane % LPH == 0 && r < n_rows) {
                    const size_t at = (size_t)r * H + head;
                    row_sq[at] = make_float4(s, query[at], stats ? stats[at * 2] : 0.0f,
                                             stats ? stats[at * 2 + 1] : 0.0f);
                }
            }
        }
    }
}

// FULL: kc[t] = key[c, head] of the source; gk[t] accumulates this lane's share of
// grad_key[c, head], head = t HPT + lane / LPH.
template <int LPH, int KT, bool FULL>
__device__ __forceinline__ void gat_src_window(const GatSrcParams &p, const EdgeWindow &win,
                                               int first, int n, const float (&xt)[KT][4],
                                               float (&acc)[KT][4], const float (&kc)[KT],
                                               float (&gk)[KT]) {
    constexpr int NS = kWave / LPH;  // edge groups of LPH edges in a window; also heads per tile
    constexpr int U = KT == 1 ? kDotUnroll : 2;  // row gathers in flight
    const int lane = lane_id();
    const int h = lane / LPH, sub = lane % LPH;
    const int H = p.sp.H;
    const float *__restrict__ g = static_cast<const float *>(p.sp.feat);
    const int g_lane = (p.head_mean ? sub : lane) * 4, g_tile = p.head_mean ? 0 : 256;
    const float g_scale = p.g_scale;
    // What is needed per (edge, head) is fetched once, before the row gathers, in the
    // layout of the epilogue: lane (h, sub) owns edge j * LPH + sub. The attention
    // weight reaches the accumulate loop by a lane shuffle.
    // The first rows are asked for before anything else: they depend on the window only,
    // while the per-edge values below wait for a gather of their own.
    float v0[U][KT][4];
#pragma unroll
    for (int u = 0; u < U; u++) {
        if (u < n) {  // wave-uniform
            const int r = __builtin_amdgcn_readlane(win.col, first + u);
#pragma unroll
            for (int t = 0; t < KT; t++)
                RowLoad<4, float>::ld(g + (size_t)r * p.g_ld + t * g_tile + g_lane, v0[u][t]);
        }
    }
    float ea[NS][KT], eS[NS][KT], eq[NS][KT];
#pragma unroll
    for (int j = 0; j < NS; j++) {
#pragma unroll
        for (int t = 0; t < KT; t++) ea[j][t] = eS[j][t] = eq[j][t] = 0.0f;
        if (j * LPH >= n) continue;  // wave-uniform: most short rows fill one group only
        const int k = min(j * LPH + sub, n - 1);
        const int vr = __shfl(win.vrow, first + k, kWave);
        const int r = __shfl(win.col, first + k, kWave);
#pragma unroll
        for (int t = 0; t < KT; t++) {
            const int head = t * NS + h;
            if constexpr (FULL) {
                const float4 sq = p.row_sq[(size_t)r * H + head];
                eS[j][t] = sq.x;
                eq[j][t] = sq.y;
                ea[j][t] = p.recompute ? expf(leaky(sq.y + kc[t]) - sq.z) * sq.w
                                       : p.sp.values[(size_t)vr * H + head];
            } else {
                ea[j][t] = p.sp.values[(size_t)vr * H + head];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < NS; j++) {
        if (j * LPH >= n) break;  // wave-uniform
        float keep[KT];
#pragma unroll
        for (int t = 0; t < KT; t++) keep[t] = 0.0f;
        for (int kk = 0; kk < LPH && j * LPH + kk < n; kk += U) {
            float v[U][KT][4], a[U][KT];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int k = j * LPH + kk + u;
                if (k < n) {  // wave-uniform
                    const int r = __builtin_amdgcn_readlane(win.col, first + k);
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        if (j == 0 && kk == 0) {
#pragma unroll
                            for (int i = 0; i < 4; i++) v[u][t][i] = v0[u][t][i];
                        } else {
                            RowLoad<4, float>::ld(g + (size_t)r * p.g_ld + t * g_tile + g_lane,
                                                  v[u][t]);
                        }
                        a[u][t] = __shfl(ea[j][t], (lane - sub) + kk + u, kWave) * g_scale;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int k = j * LPH + kk + u;
                if (k < n) {
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        float d = xt[t][0] * v[u][t][0] + xt[t][1] * v[u][t][1] +
                                  xt[t][2] * v[u][t][2] + xt[t][3] * v[u][t][3];
                        d = group_sum<LPH>(d);
                        if (sub == kk + u) keep[t] = d * g_scale;
#pragma unroll
                        for (int i = 0; i < 4; i++) acc[t][i] += a[u][t] * v[u][t][i];
                    }
                }
            }
        }
        const int k = j * LPH + sub;
        const int vr = __shfl(win.vrow, first + min(k, n - 1), kWave);
        // The per-(edge, head) results go to grad_a through the edge permutation: scattered
        // stores. The W heads of an edge that sit in lanes LPH apart are collected by the
        // first of them and leave as one 8- or 16-byte store: a store of 4 bytes costs the
        // L2 a request of its own, four per edge.
        constexpr int W = NS >= 4 ? 4 : NS;
#pragma unroll
        for (int t = 0; t < KT; t++) {
            float val = keep[t];
            if constexpr (FULL) {
                val = ea[j][t] * (keep[t] - eS[j][t]) * (eq[j][t] + kc[t] < 0.0f ? kSlope : 1.0f);
                if (k < n) gk[t] += val;
            }
            if constexpr (W == 1) {
                if (k < n) p.grad_a[(size_t)vr * H + t * NS + h] = val;
            } else {
                float w[W];
                w[0] = val;
#pragma unroll
                for (int i = 1; i < W; i++) w[i] = __shfl(val, lane + i * LPH, kWave);
                if (k < n && h % W == 0) {
                    float *dst = p.grad_a + (size_t)vr * H + t * NS + h;
                    if (p.grad_a_vec) {
                        typedef float fw __attribute__((ext_vector_type(W)));
                        fw v;
#pragma unroll
                        for (int i = 0; i < W; i++) v[i] = w[i];
                        *reinterpret_cast<fw *>(dst) = v;
                    } else {
#pragma unroll
                        for (int i = 0; i < W; i++) dst[i] = w[i];
                    }
                }
            }
        }
    }
}

// The source's own row, its key, and zeroed accumulators.
template <int LPH, int KT, bool FULL>
__device__ __forceinline__ void gat_src_begin(const GatSrcParams &p, int row, bool load,
                                              float (&xt)[KT][4], float (&acc)[KT][4],
                                              float (&kc)[KT], float (&gk)[KT]) {
    const int lane = lane_id();
#pragma unroll
    for (int t = 0; t < KT; t++) {
        kc[t] = gk[t] = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; i++) acc[t][i] = xt[t][i] = 0.0f;
        if (load) {
            RowLoad<4, float>::ld(p.x + (size_t)row * p.sp.L + t * 256 + lane * 4, xt[t]);
            if constexpr (FULL) kc[t] = p.key[(size_t)row * p.sp.H + t * (kWave / LPH) + lane / LPH];
        }
    }
}

// Writes the accumulated row to x_dst and (FULL) the head sums of gk to k_dst.
template <int LPH, int KT, bool FULL>
__device__ __forceinline__ void gat_src_end(float *x_dst, float *k_dst, const float (&acc)[KT][4],
                                            const float (&gk)[KT]) {
    const int lane = lane_id();
#pragma unroll
    for (int t = 0; t < KT; t++) {
        store_row_streaming<4>(x_dst + t * 256 + lane * 4, acc[t]);
        if constexpr (FULL) {
            float s = gk[t];
            s = group_sum<LPH>(s);
            if (lane % LPH == 0) k_dst[t * (kWave / LPH) + lane / LPH] = s;
        }
    }
}

template <int LPH, int KT, bool FULL>
__global__ __launch_bounds__(kBlock) void gat_src_rows_kernel(GatSrcParams p) {
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.sp.n_rows);
    const int r0 = (blockIdx.x * kWavesPerBlock + wave_id()) * rpw;
    if (r0 >= p.sp.n_rows) return;
    const int n_here = min(rpw, p.sp.n_rows - r0);
    const int my_ptr = p.sp.indptr[r0 + min(lane, n_here)];
    const int limit = __builtin_amdgcn_readlane(my_ptr, n_here);
    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;
    for (int i = 0; i < n_here; i++) {
        const int row = r0 + i;
        const int beg = __builtin_amdgcn_readlane(my_ptr, i), end = __builtin_amdgcn_readlane(my_ptr, i + 1);
        if (end - beg >= p.sp.plan.threshold) continue;  // a planned row: the item kernel
        float xt[KT][4], acc[KT][4], kc[KT], gk[KT];
        gat_src_begin<LPH, KT, FULL>(p, row, end > beg, xt, acc, kc, gk);
        for (int b = beg; b < end; b += kWave) {
            const int n = min(kWave, end - b);
            if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                load_window<W_EDGEHEAD>(win, p.sp, b, limit);
            gat_src_window<LPH, KT, FULL>(p, win, b - win.base, n, xt, acc, kc, gk);
        }
        gat_src_end<LPH, KT, FULL>(p.sp.out + (size_t)row * p.sp.L,
                                   FULL ? p.grad_k + (size_t)row * p.sp.H : nullptr, acc, gk);
    }
}

template <int LPH, int KT, bool FULL>
__global__ __launch_bounds__(kBlock) void gat_src_items_kernel(GatSrcParams p) {
    const int lane = lane_id();
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int L = p.sp.L, H = p.sp.H;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kSrcItems;
         pos0 < n_items; pos0 += n_waves * kSrcItems) {
        const int n_here = min(kSrcItems, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kSrcItems];
        int n_edges[kSrcItems], tag[kSrcItems], item[kSrcItems];
#pragma unroll
        for (int j = 0; j < kSrcItems; j++) {
            const int beg = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            item[j] = __builtin_amdgcn_readlane(my_rec.z, j);
            tag[j] = __builtin_amdgcn_readlane(my_rec.w, j);
            n_edges[j] = j < n_here ? end - beg : 0;
            if (n_edges[j] > 0) load_window<W_EDGEHEAD>(win[j], p.sp, beg, end);
        }
#pragma unroll
        for (int j = 0; j < kSrcItems; j++) {
            if (n_edges[j] <= 0) continue;
            const int row = tag[j] & 0x7fffffff;
            float xt[KT][4], acc[KT][4], kc[KT], gk[KT];
            gat_src_begin<LPH, KT, FULL>(p, row, true, xt, acc, kc, gk);
            gat_src_window<LPH, KT, FULL>(p, win[j], 0, n_edges[j], xt, acc, kc, gk);
            const bool single = tag[j] < 0;
            float *x_dst = single ? p.sp.out + (size_t)row * L : p.sp.partial + (size_t)item[j] * L;
            float *k_dst = nullptr;
            if constexpr (FULL)
                k_dst = single ? p.grad_k + (size_t)row * H : p.partial_k + (size_t)item[j] * H;
            gat_src_end<LPH, KT, FULL>(x_dst, k_dst, acc, gk);
        }
    }
}

// ---- head-mean gradient, rows of 256 floats: several edges per load -----------------
// When the gathered row is the F-float gradient of the head mean, a wave-wide load of
// the layout above fetches the same F floats once per head, and with F * 4 bytes per
// edge the pass is bound by the number of loads in flight, not by bandwidth. Here a
// load instruction fetches SLOTS = 64 / LPH = H different edges: lane (s, sub) holds
// floats [4 sub, +4) of the gradient row of the s-th edge of a group, and the source's
// own row as H slices x[c, h, 4 sub .. +4). Per group: H dots (one per head, reduced
// over the slot's LPH lanes), H x 4 FMAs into acc[h], and the epilogue on lanes
// sub < H (one head each). Slot sums are folded by a fixed butterfly at the end.
template <int LPH>
struct SlotRow {
    static constexpr int H = kWave / LPH;  // heads = slots (rows of 256 floats)
    float xh[H][4], acc[H][4];
    float kc, gk;  // lanes sub < H: key[c, sub] and this slot's share of grad_key[c, sub]
};

template <int LPH>
__device__ __forceinline__ void slot_begin(SlotRow<LPH> &row, const GatSrcParams &p, int c,
                                           bool load) {
    constexpr int H = SlotRow<LPH>::H;
    const int sub = lane_id() % LPH;
    row.kc = row.gk = 0.0f;
#pragma unroll
    for (int h = 0; h < H; h++) {
#pragma unroll
        for (int i = 0; i < 4; i++) row.acc[h][i] = row.xh[h][i] = 0.0f;
        if (load) RowLoad<4, float>::ld(p.x + (size_t)c * 256 + h * (4 * LPH) + sub * 4, row.xh[h]);
    }
    if (load && sub < H) row.kc = p.key[(size_t)c * H + sub];
}

template <int LPH>
__device__ __forceinline__ void slot_window(SlotRow<LPH> &row, const GatSrcParams &p,
                                            const EdgeWindow &win, int first, int n) {
    // U load groups in flight: 2 measured a little better than 4 (fewer registers)
    constexpr int H = SlotRow<LPH>::H, SLOTS = H, U = 2;
    const int lane = lane_id();
    const int s = lane / LPH, sub = lane % LPH;
    const float *__restrict__ g = static_cast<const float *>(p.sp.feat);
    const int F = 4 * LPH;
    for (int k0 = 0; k0 < n; k0 += SLOTS * U) {
        float v[U][4], a[U][H];
        float2 sq[U];
        int vr[U];
        bool valid[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (k0 + u * SLOTS < n) {  // wave-uniform
                const int k = k0 + u * SLOTS + s;
                valid[u] = k < n;
                const int src = first + min(k, n - 1);
                const int r = __shfl(win.col, src, kWave);
                vr[u] = __shfl(win.vrow, src, kWave);
                RowLoad<4, float>::ld(g + (size_t)r * F + sub * 4, v[u]);
                sq[u] = make_float2(0.0f, 0.0f);
                if (p.recompute) {
                    // no read of attn: lane sub < H makes the probability of (edge, head sub)
                    // from the destination's line, the slot's lanes then share the H values
                    float mine_a = 0.0f;
                    if (sub < H) {
                        const float4 t4 = p.row_sq[(size_t)r * H + sub];
                        sq[u] = make_float2(t4.x, t4.y);
                        mine_a = expf(leaky(t4.y + row.kc) - t4.z) * t4.w;
                    }
#pragma unroll
                    for (int h = 0; h < H; h++) a[u][h] = __shfl(mine_a, (lane - sub) + h, kWave);
                } else {
                    if constexpr (H == 8) {  // two 16-byte halves
                        float lo[4], hi[4];
                        RowLoad<4, float>::ld(p.sp.values + (size_t)vr[u] * 8, lo);
                        RowLoad<4, float>::ld(p.sp.values + (size_t)vr[u] * 8 + 4, hi);
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            a[u][i] = lo[i];
                            a[u][4 + i] = hi[i];
                        }
                    } else {
                        RowLoad<H, float>::ld(p.sp.values + (size_t)vr[u] * H, a[u]);
                    }
                    if (sub < H) {
                        const float4 t4 = p.row_sq[(size_t)r * H + sub];
                        sq[u] = make_float2(t4.x, t4.y);
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (k0 + u * SLOTS >= n) break;  // wave-uniform
            float mine = 0.0f;  // d_attn of (this slot's edge, head sub) on lanes sub < H
#pragma unroll
            for (int h = 0; h < H; h++) {
                float d = row.xh[h][0] * v[u][0] + row.xh[h][1] * v[u][1] + row.xh[h][2] * v[u][2] +
                          row.xh[h][3] * v[u][3];
                d = group_sum<LPH>(d);
                if (sub == h) mine = d;
                const float w = valid[u] ? a[u][h] * p.g_scale : 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) row.acc[h][i] += w * v[u][i];
            }
            if (valid[u] && sub < H) {
                float ah = 0.0f;
#pragma unroll
                for (int h = 0; h < H; h++)
                    if (sub == h) ah = a[u][h];
                const float gl = ah * (mine * p.g_scale - sq[u].x) *
                                 (sq[u].y + row.kc < 0.0f ? kSlope : 1.0f);
                p.grad_a[(size_t)vr[u] * H + sub] = gl;
                row.gk += gl;
            }
        }
    }
}

template <int LPH>
__device__ __forceinline__ void slot_end(SlotRow<LPH> &row, float *x_dst, float *k_dst) {
    constexpr int H = SlotRow<LPH>::H;
    const int lane = lane_id();
    const int s = lane / LPH, sub = lane % LPH;
#pragma unroll
    for (int o = kWave / 2; o >= LPH; o >>= 1) {
        row.gk += __shfl_xor(row.gk, o, kWave);
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int i = 0; i < 4; i++) row.acc[h][i] += __shfl_xor(row.acc[h][i], o, kWave);
    }
    if (s == 0) {
#pragma unroll
        for (int h = 0; h < H; h++) store_row_streaming<4>(x_dst + h * (4 * LPH) + sub * 4, row.acc[h]);
        if (sub < H) k_dst[sub] = row.gk;
    }
}

template <int LPH>
__global__ __launch_bounds__(kBlock) void gat_slot_rows_kernel(GatSrcParams p) {
    constexpr int H = kWave / LPH;
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.sp.n_rows);
    const int r0 = (blockIdx.x * kWavesPerBlock + wave_id()) * rpw;
    if (r0 >= p.sp.n_rows) return;
    const int n_here = min(rpw, p.sp.n_rows - r0);
    const int my_ptr = p.sp.indptr[r0 + min(lane, n_here)];
    const int limit = __builtin_amdgcn_readlane(my_ptr, n_here);
    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;
    for (int i = 0; i < n_here; i++) {
        const int row = r0 + i;
        const int beg = __builtin_amdgcn_readlane(my_ptr, i), end = __builtin_amdgcn_readlane(my_ptr, i + 1);
        if (end - beg >= p.sp.plan.threshold) continue;  // a planned row: the item kernel
        SlotRow<LPH> acc;
        slot_begin<LPH>(acc, p, row, end > beg);
        for (int b = beg; b < end; b += kWave) {
            const int n = min(kWave, end - b);
            if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                load_window<W_EDGEHEAD>(win, p.sp, b, limit);
            slot_window<LPH>(acc, p, win, b - win.base, n);
        }
        slot_end<LPH>(acc, p.sp.out + (size_t)row * 256, p.grad_k + (size_t)row * H);
    }
}

template <int LPH>
__global__ __launch_bounds__(kBlock) void gat_slot_items_kernel(GatSrcParams p) {
    constexpr int H = kWave / LPH;
    const int lane = lane_id();
    if (p.sp.plan.counters->overflow) return;
    const int n_items = min(p.sp.plan.counters->n_items, p.sp.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + wave_id()) * kSrcItems;
         pos0 < n_items; pos0 += n_waves * kSrcItems) {
        const int n_here = min(kSrcItems, n_items - pos0);
        const int4 my_rec = p.sp.plan.records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kSrcItems];
        int n_edges[kSrcItems], tag[kSrcItems], item[kSrcItems];
#pragma unroll
        for (int j = 0; j < kSrcItems; j++) {
            const int beg = __builtin_amdgcn_readlane(my_rec.x, j);
            const int end = __builtin_amdgcn_readlane(my_rec.y, j);
            item[j] = __builtin_amdgcn_readlane(my_rec.z, j);
            tag[j] = __builtin_amdgcn_readlane(my_rec.w, j);
            n_edges[j] = j < n_here ? end - beg : 0;
            if (n_edges[j] > 0) load_window<W_EDGEHEAD>(win[j], p.sp, beg, end);
        }
#pragma unroll
        for (int j = 0; j < kSrcItems; j++) {
            if (n_edges[j] <= 0) continue;
            const int row = tag[j] & 0x7fffffff;
            SlotRow<LPH> acc;
            slot_begin<LPH>(acc, p, row, true);
            slot_window<LPH>(acc, p, win[j], 0, n_edges[j]);
            const bool single = tag[j] < 0;
            slot_end<LPH>(acc,
                          single ? p.sp.out + (size_t)row * 256 : p.sp.partial + (size_t)item[j] * 256,
                          single ? p.grad_k + (size_t)row * H : p.partial_k + (size_t)item[j] * H);
        }
    }
}

template <int LPH, int KT, bool FULL>
static int gat_src_launch_shape(const GatSrcParams &p, bool has_items, const float *grad_out,
                                const float *out, const float *query, int n_dst,
                                hipStream_t stream) {
    if constexpr (FULL) {
        gat_row_dot_kernel<LPH, KT>
            <<<(int)ceil_div(n_dst, kWavesPerBlock * kRowsPerWave), kBlock, 0, stream>>>(
                const_cast<float4 *>(p.row_sq), grad_out, out, query, p.stats, n_dst, p.g_ld,
                p.head_mean, p.g_scale);
        YITU_LAUNCH_CHECK();
    }
    const int row_grid = (int)ceil_div(p.sp.n_rows, kWavesPerBlock * rows_per_wave(p.sp.n_rows));
    // enough workgroups to walk the item list once (a second turn would mix source bands)
    const int item_grid = (int)std::min<int64_t>(
        ceil_div(p.sp.plan.max_items, kWavesPerBlock * kSrcItems), 1 << 20);
    // a head-mean gradient of F < 256 floats per row: the several-edges-per-load kernels
    constexpr bool kSlots = FULL && KT == 1 && LPH < kWave;
    bool slots = false;
    if constexpr (kSlots) slots = p.head_mean != 0;
    if constexpr (kSlots) {
        if (slots) {
            gat_slot_rows_kernel<LPH><<<row_grid, kBlock, 0, stream>>>(p);
            YITU_LAUNCH_CHECK();
            if (has_items) {
                gat_slot_items_kernel<LPH><<<item_grid, kBlock, 0, stream>>>(p);
                YITU_LAUNCH_CHECK();
            }
        }
    }
    if (!slots) {
        gat_src_rows_kernel<LPH, KT, FULL><<<row_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        if (has_items) {
            gat_src_items_kernel<LPH, KT, FULL><<<item_grid, kBlock, 0, stream>>>(p);
            YITU_LAUNCH_CHECK();
        }
    }
    if (!has_items) return 0;
    const int red_grid = (int)std::min<int64_t>(p.sp.plan.max_rows, 1 << 16);
    spmm_reduce_kernel<W_NONE, 4><<<red_grid, kBlock, 0, stream>>>(p.sp);
    YITU_LAUNCH_CHECK();
    if constexpr (FULL) {
        // the item partials of grad_key, rows of H floats
        constexpr int H = kWave / LPH * KT;
        SpmmParams k = p.sp;
        k.L = k.F = H;
        k.H = 1;
        k.out = p.grad_k;
        k.partial = p.partial_k;
        spmm_reduce_kernel<W_NONE, (H % 4 == 0 ? 4 : H)><<<red_grid, kBlock, 0, stream>>>(k);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int LPH, bool FULL>
static int gat_src_launch_lph(const GatSrcParams &p, bool has_items, const float *grad_out,
                              const float *out, const float *query, int n_dst,
                              hipStream_t stream) {
    const int kt = p.sp.L / 256;
    if (kt == 1)
        return gat_src_launch_shape<LPH, 1, FULL>(p, has_items, grad_out, out, query, n_dst, stream);
    if (kt == 2)
        return gat_src_launch_shape<LPH, 2, FULL>(p, has_items, grad_out, out, query, n_dst, stream);
    if (kt == 4)
        return gat_src_launch_shape<LPH, 4, FULL>(p, has_items, grad_out, out, query, n_dst, stream);
    set_error("gat backward: unsupported row width %d", p.sp.L);
    return -1;
}

template <bool FULL>
static int gat_src_launch(const GatSrcParams &p, bool has_items, const float *grad_out,
                          const float *out, const float *query, int n_dst, hipStream_t stream) {
    switch (p.sp.F / 4) {
        case 8: return gat_src_launch_lph<8, FULL>(p, has_items, grad_out, out, query, n_dst, stream);
        case 16: return gat_src_launch_lph<16, FULL>(p, has_items, grad_out, out, query, n_dst, stream);
        case 32: return gat_src_launch_lph<32, FULL>(p, has_items, grad_out, out, query, n_dst, stream);
        case 64: return gat_src_launch_lph<64, FULL>(p, has_items, grad_out, out, query, n_dst, stream);
    }
    set_error("gat backward: unsupported head width %d", p.sp.F);
    return -1;
}

// ---- the by-source pass for a plain edge-weighted product -------------------------
// grad_a[e,h] = <grad_out[row_e,h,:], x[col_e,h,:]> and grad_x[c] = sum_e values[e,h]
// grad_out[row_e] from the same single gather of grad_out rows (rows of 256 floats, head
// width 32 to 256 a power of two): what yitu_spmm_backward otherwise does in two passes,
// one gathering x[col] by destination and one gathering grad_out[row] by source.
bool spmm_backward_one_gather_shape(int64_t n_heads, int64_t n_features, const float *features,
                                    const float *grad_out, const float *grad_x) {
    const int64_t lph = n_features / 4, L = n_heads * n_features;
    return (L == 256 || L == 512 || L == 1024) && n_features % 4 == 0 && lph >= 8 && lph <= 64 &&
           (lph & (lph - 1)) == 0 && aligned16(features) && aligned16(grad_out) &&
           aligned16(grad_x);
}

int spmm_backward_one_gather(float *grad_a, float *grad_x, const float *values,
                             const float *features, const float *grad_out,
                             const int32_t *t_indptr, const int32_t *t_rows, const int32_t *t_perm,
                             int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads,
                             int64_t n_features, int64_t max_degree_t, const void *plan_t,
                             void *workspace, size_t workspace_bytes, hipStream_t stream) {
    const int64_t L = n_heads * n_features;
    GatSrcParams p{};
    p.sp.indptr = t_indptr;
    p.sp.indices = t_rows;
    p.sp.eperm = t_perm;
    p.sp.values = values;
    p.sp.feat = grad_out;
    p.sp.out = grad_x;
    p.sp.n_rows = (int)n_src;
    p.sp.n_src = (int)n_dst;
    p.sp.L = (int)L;
    p.sp.F = (int)n_features;
    p.sp.H = (int)n_heads;
    p.sp.col_mask = 0x7fffffff;
    p.sp.alpha = 1.0f;
    p.x = features;
    p.grad_a = grad_a;
    p.grad_a_vec = aligned16(grad_a) ? 1 : 0;
    p.g_ld = (int)L;
    p.g_scale = 1.0f;
    bool has_items = false;
    void *rest = nullptr;
    size_t rest_bytes = 0;
    int rc = plan_resolve(p.sp.plan, has_items, plan_t, t_indptr, t_rows, n_src, n_dst, nnz,
                          0x7fffffff, max_degree_t, workspace, workspace_bytes, &rest, &rest_bytes,
                          stream);
    if (rc) return rc;
    const size_t part =
        has_items ? align_up(sizeof(float) * (size_t)p.sp.plan.max_items * (size_t)L, 256) : 0;
    YITU_REQUIRE(part == 0 || (rest && rest_bytes >= part),
                 "workspace too small: need %zu more bytes", part);
    if (has_items) p.sp.partial = static_cast<float *>(rest);
    return gat_src_launch<false>(p, has_items, grad_out, nullptr, nullptr, (int)n_dst, stream);
}

// ---- host side ----------------------------------------------------------------
// workspace beyond the plan: item statistics, row statistics, partial rows
static size_t gat_own_bytes(int64_t n_dst, int64_t nnz, int64_t H, int64_t L) {
    return align_up(sizeof(float) * 2 * (size_t)(plan_max_items(nnz) * H), 256) +
           align_up(sizeof(float) * 4 * (size_t)(n_dst * H), 256) +
           align_up(sizeof(float) * (size_t)(plan_max_items(nnz) * L), 256);
}

// every pointer aligned to a vector of hv floats
static bool vec_aligned(int hv, const void *a, const void *b, const void *c) {
    const uintptr_t m = (uintptr_t)hv * sizeof(float) - 1;
    return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
             reinterpret_cast<uintptr_t>(c)) & m) == 0;
}

template <int VEC, int G, int KT>
static int gat_fwd_launch(GatParams &p, bool has_items, hipStream_t stream) {
    const int hv = packed_head_vec(p.sp.H);
    if (G == kWave && VEC == 4 && p.sp.L <= 4 * kWave * KT && packed_heads_ok(p.sp.H) &&
        vec_aligned(hv, p.query, p.key, p.attn)) {
        // whole-wave rows: the short rows in the packed layout
        // fewer rows per wave than the attention-only kernels take (63): with a wave-wide
        // gather per edge, more waves in flight are worth more than longer chunk runs
        // (24 / 63 rows: 1.94 / 2.05 ms on a 2^21-node graph)
        const int R = std::min(packed_rows_per_wave(p.sp.n_rows), 24);
        const int grid = (int)ceil_div(p.sp.n_rows, (int64_t)kWavesPerBlock * R);
        if (hv == 4) gat_rows_packed_kernel<4, KT><<<grid, kBlock, 0, stream>>>(p, R);
        else if (hv == 2) gat_rows_packed_kernel<2, KT><<<grid, kBlock, 0, stream>>>(p, R);
        else gat_rows_packed_kernel<1, KT><<<grid, kBlock, 0, stream>>>(p, R);
    } else {
        gat_rows_kernel<VEC, G, KT>
            <<<(int)ceil_div(p.sp.n_rows, kWavesPerBlock * rows_per_wave(p.sp.n_rows)), kBlock, 0,
               stream>>>(p);
    }
    YITU_LAUNCH_CHECK();
    if (!has_items) return 0;
    const int item_grid = (int)std::min<int64_t>(
        ceil_div(p.sp.plan.max_items, kWavesPerBlock * kItemsPerWave), 1 << 16);
    const int combine_grid =
        (int)std::min<int64_t>(ceil_div(p.sp.plan.max_rows, kWavesPerBlock), 1 << 15);
    const int reduce_grid = (int)std::min<int64_t>(p.sp.plan.max_rows, 1 << 16);
    if (!p.attn && p.sp.F % 4 == 0) {
        // two items per wave and turn of the grid-stride loop: twice the workgroups
        const int hp_grid = (int)std::min<int64_t>(
            ceil_div(p.sp.plan.max_items, kWavesPerBlock * 1), 1 << 19);
        switch (p.HP) {
            case 1: gat_item_local_hp_kernel<VEC, G, KT, 1><<<hp_grid, kBlock, 0, stream>>>(p); break;
            case 2: gat_item_local_hp_kernel<VEC, G, KT, 2><<<hp_grid, kBlock, 0, stream>>>(p); break;
            case 4: gat_item_local_hp_kernel<VEC, G, KT, 4><<<hp_grid, kBlock, 0, stream>>>(p); break;
            case 8: gat_item_local_hp_kernel<VEC, G, KT, 8><<<hp_grid, kBlock, 0, stream>>>(p); break;
            default: gat_item_local_kernel<VEC, G, KT><<<item_grid, kBlock, 0, stream>>>(p);
        }
        YITU_LAUNCH_CHECK();
        gat_row_combine_kernel<<<combine_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        gat_scaled_reduce_kernel<<<reduce_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        return 0;
    }
    gat_item_stats_kernel<<<item_grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    gat_row_combine_kernel<<<combine_grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    gat_item_apply_kernel<VEC, G, KT><<<item_grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    p.sp.alpha = 1.0f;
    spmm_reduce_kernel<W_NONE, 4><<<reduce_grid, kBlock, 0, stream>>>(p.sp);
    YITU_LAUNCH_CHECK();
    return 0;
}

// ---- attention only: host side ---------------------------------------------------
size_t attn_workspace_bytes(int64_t n_dst, int64_t nnz, int64_t H) {
    return align_up(sizeof(float) * 3 * (size_t)(plan_max_items(nnz) * H), 256) +
           align_up(sizeof(float) * 2 * (size_t)(n_dst * H), 256);
}

int attn_forward_run(float *attn, const int32_t *indptr, const int32_t *indices,
                     const float *query, const float *key, int64_t n_dst, int64_t n_src,
                     int64_t nnz, int64_t n_heads, int64_t max_degree, const void *plan,
                     void *workspace, size_t workspace_bytes, hipStream_t stream) {
    GatParams p{};
    p.sp.indptr = indptr;
    p.sp.indices = indices;
    p.sp.n_rows = (int)n_dst;
    p.sp.n_src = (int)n_src;
    p.sp.H = (int)n_heads;
    p.sp.L = p.sp.F = (int)n_heads;
    p.sp.col_mask = kColMask;
    p.query = query;
    p.key = key;
    p.attn = attn;
    p.HP = 1;
    while (p.HP < p.sp.H) p.HP <<= 1;
    bool has_items = false;
    void *rest = nullptr;
    size_t rest_bytes = 0;
    int rc = plan_resolve(p.sp.plan, has_items, plan, indptr, indices, n_dst, n_src, nnz, kColMask,
                          max_degree, workspace, workspace_bytes, &rest, &rest_bytes, stream);
    if (rc) return rc;
    if (!has_items) p.sp.plan.threshold = 0x7fffffff;
    // one lane per edge whenever the heads of an edge are a few aligned vectors
    const int hv = packed_head_vec(p.sp.H);
    const bool packed = packed_heads_ok(p.sp.H) && vec_aligned(hv, query, key, attn);
    if (packed) {
        const int R = packed_rows_per_wave(p.sp.n_rows);
        const int grid = (int)ceil_div(p.sp.n_rows, (int64_t)kWavesPerBlock * R);
        if (hv == 4) attn_rows_packed_kernel<4><<<grid, kBlock, 0, stream>>>(p, R);
        else if (hv == 2) attn_rows_packed_kernel<2><<<grid, kBlock, 0, stream>>>(p, R);
        else attn_rows_packed_kernel<1><<<grid, kBlock, 0, stream>>>(p, R);
    } else {
        attn_rows_kernel<<<(int)ceil_div(p.sp.n_rows, kWavesPerBlock * rows_per_wave(p.sp.n_rows)),
                           kBlock, 0, stream>>>(p);
    }
    YITU_LAUNCH_CHECK();
    if (!has_items) return 0;
    const size_t need = attn_workspace_bytes(n_dst, nnz, n_heads);
    YITU_REQUIRE(rest && rest_bytes >= need, "workspace too small: need %zu more bytes", need);
    char *w = static_cast<char *>(rest);
    p.item_stats = reinterpret_cast<float *>(w);
    w += align_up(sizeof(float) * 3 * (size_t)(plan_max_items(nnz) * n_heads), 256);
    p.row_stats = reinterpret_cast<float *>(w);
    const int item_grid = (int)std::min<int64_t>(
        ceil_div(p.sp.plan.max_items, kWavesPerBlock * kItemsPerWave), 1 << 16);
    const int packed_grid = packed_item_grid(p.sp.plan.max_items);
    if (packed && hv == 4) attn_item_stats_packed_kernel<4><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed && hv == 2) attn_item_stats_packed_kernel<2><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed) attn_item_stats_packed_kernel<1><<<packed_grid, kBlock, 0, stream>>>(p);
    else gat_item_stats_kernel<<<item_grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    gat_row_combine_kernel<<<(int)std::min<int64_t>(
                                 ceil_div(p.sp.plan.max_rows, kWavesPerBlock), 1 << 15),
                             kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (packed && hv == 4) attn_item_write_packed_kernel<4><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed && hv == 2) attn_item_write_packed_kernel<2><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed) attn_item_write_packed_kernel<1><<<packed_grid, kBlock, 0, stream>>>(p);
    else attn_item_write_kernel<<<item_grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    return 0;
}

// grad_query and the per-edge logit gradient grad_edge [nnz, H]; the caller sums
// grad_edge into grad_key over the transposed structure.
int attn_backward_run(float *grad_query, float *grad_edge, const int32_t *indptr,
                      const int32_t *indices, const float *query, const float *key,
                      const float *attn, const float *grad_attn, int64_t n_dst, int64_t n_src,
                      int64_t nnz, int64_t n_heads, int64_t max_degree, const void *plan,
                      void *workspace, size_t workspace_bytes, hipStream_t stream) {
    GatBwdParams p{};
    p.sp.indptr = indptr;
    p.sp.indices = indices;
    p.sp.n_rows = (int)n_dst;
    p.sp.n_src = (int)n_src;
    p.sp.H = (int)n_heads;
    p.sp.L = p.sp.F = (int)n_heads;
    p.sp.col_mask = kColMask;
    p.query = query;
    p.key = key;
    p.attn = attn;
    p.grad_a = const_cast<float *>(grad_attn);
    p.grad_q = grad_query;
    p.grad_e = grad_edge;
    p.HP = 1;
    while (p.HP < p.sp.H) p.HP <<= 1;
    bool has_items = false;
    void *rest = nullptr;
    size_t rest_bytes = 0;
    int rc = plan_resolve(p.sp.plan, has_items, plan, indptr, indices, n_dst, n_src, nnz, kColMask,
                          max_degree, workspace, workspace_bytes, &rest, &rest_bytes, stream);
    if (rc) return rc;
    if (!has_items) p.sp.plan.threshold = 0x7fffffff;
    const int hv = packed_head_vec(p.sp.H);
    const bool packed = packed_heads_ok(p.sp.H) && vec_aligned(hv, query, key, attn) &&
                        vec_aligned(hv, grad_attn, grad_query, grad_edge);
    if (packed) {
        const int R = packed_rows_per_wave(p.sp.n_rows);
        const int grid = (int)ceil_div(p.sp.n_rows, (int64_t)kWavesPerBlock * R);
        if (hv == 4) attn_bwd_rows_packed_kernel<4><<<grid, kBlock, 0, stream>>>(p, R);
        else if (hv == 2) attn_bwd_rows_packed_kernel<2><<<grid, kBlock, 0, stream>>>(p, R);
        else attn_bwd_rows_packed_kernel<1><<<grid, kBlock, 0, stream>>>(p, R);
    } else {
        attn_bwd_rows_kernel<<<(int)ceil_div(p.sp.n_rows,
                                             kWavesPerBlock * rows_per_wave(p.sp.n_rows)),
                               kBlock, 0, stream>>>(p);
    }
    YITU_LAUNCH_CHECK();
    if (!has_items) return 0;
    const size_t need = attn_workspace_bytes(n_dst, nnz, n_heads);
    YITU_REQUIRE(rest && rest_bytes >= need, "workspace too small: need %zu more bytes", need);
    char *w = static_cast<char *>(rest);
    p.item_sums = reinterpret_cast<float *>(w);
    w += align_up(sizeof(float) * 3 * (size_t)(plan_max_items(nnz) * n_heads), 256);
    p.row_sum = reinterpret_cast<float *>(w);
    const int item_grid = (int)std::min<int64_t>(
        ceil_div(p.sp.plan.max_items, kWavesPerBlock * kItemsPerWave), 1 << 16);
    const int packed_grid = packed_item_grid(p.sp.plan.max_items);
    if (packed && hv == 4) attn_bwd_item_sums_packed_kernel<4><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed && hv == 2) attn_bwd_item_sums_packed_kernel<2><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed) attn_bwd_item_sums_packed_kernel<1><<<packed_grid, kBlock, 0, stream>>>(p);
    else attn_bwd_item_sums_kernel<<<item_grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    gat_bwd_combine_kernel<<<(int)std::min<int64_t>(ceil_div(p.sp.plan.max_rows, kWavesPerBlock),
                                                    1 << 15),
                             kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (packed && hv == 4) attn_bwd_apply_packed_kernel<4><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed && hv == 2) attn_bwd_apply_packed_kernel<2><<<packed_grid, kBlock, 0, stream>>>(p);
    else if (packed) attn_bwd_apply_packed_kernel<1><<<packed_grid, kBlock, 0, stream>>>(p);
    else gat_bwd_apply_kernel<<<item_grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    return 0;
}

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API size_t yitu_gat_workspace_bytes(int64_t n_dst, int64_t nnz, int64_t n_heads,
                                         int64_t n_features, int with_plans) {
    const int64_t L = n_heads * n_features;
    size_t b = gat_own_bytes(n_dst, nnz, n_heads, L) + (with_plans ? 0 : plan_temp_bytes(nnz));
    b = std::max(b, (size_t)yitu_spmm_workspace_bytes(nnz, L, with_plans));
    b = std::max(b, (size_t)yitu_sddmm_workspace_bytes(n_dst, nnz, n_heads, 1, with_plans));
    return b + 256;
}

YITU_API int yitu_gat_forward(float *out, float *attn, float *row_stats, const int32_t *indptr,
                              const int32_t *indices, const float *query, const float *key,
                              const float *features, int64_t n_dst, int64_t n_src, int64_t nnz,
                              int64_t n_heads, int64_t n_features, int64_t max_degree,
                              const void *plan, void *workspace, size_t workspace_bytes,
                              void *stream_) {
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
        YITU_REQUIRE(!row_stats, "row statistics are produced by the fused kernels only");
        int rc = yitu_sddmm_forward(attn, indptr, indices, query, key, n_dst, n_src, nnz, n_heads,
                                    1, max_degree, plan, workspace, workspace_bytes, stream_);
        if (rc) return rc;
        return yitu_spmm_forward(out, attn, indptr, indices, features, n_dst, n_src, nnz, n_heads,
                                 n_features, max_degree, plan, workspace, workspace_bytes,
                                 stream_);
    }
    GatParams p{};
    p.sp.indptr = indptr;
    p.sp.indices = indices;
    p.sp.feat = features;
    p.sp.out = out;
    p.sp.n_rows = (int)n_dst;
    p.sp.n_src = (int)n_src;
    p.sp.L = (int)L;
    p.sp.F = (int)n_features;
    p.sp.H = (int)n_heads;
    p.sp.col_mask = kColMask;
    p.sp.alpha = 1.0f;
    p.query = query;
    p.key = key;
    p.attn = attn;
    p.stats_out = row_stats;
    p.HP = 1;
    while (p.HP < p.sp.H) p.HP <<= 1;
    bool has_items = false;
    void *rest = nullptr;
    size_t rest_bytes = 0;
    int rc = plan_resolve(p.sp.plan, has_items, plan, indptr, indices, n_dst, n_src, nnz, kColMask,
                          max_degree, workspace, workspace_bytes, &rest, &rest_bytes, stream);
    if (rc) return rc;
    if (has_items) {
        const size_t need = gat_own_bytes(n_dst, nnz, n_heads, L);
        YITU_REQUIRE(rest && rest_bytes >= need, "workspace too small: need %zu more bytes", need);
        char *w = static_cast<char *>(rest);
        p.item_stats = reinterpret_cast<float *>(w);
        w += align_up(sizeof(float) * 2 * (size_t)(plan_max_items(nnz) * n_heads), 256);
        // the planned rows' statistics go straight to the caller's buffer when there is one
        p.row_stats = row_stats ? row_stats : reinterpret_cast<float *>(w);
        w += align_up(sizeof(float) * 4 * (size_t)(n_dst * n_heads), 256);
        p.sp.partial = reinterpret_cast<float *>(w);
    }
    const int lanes = (int)(L / 4);
    if (lanes <= 16) return gat_fwd_launch<4, 16, 1>(p, has_items, stream);
    if (lanes <= 32) return gat_fwd_launch<4, 32, 1>(p, has_items, stream);
    if (lanes <= 64) return gat_fwd_launch<4, 64, 1>(p, has_items, stream);
    if (lanes <= 128) return gat_fwd_launch<4, 64, 2>(p, has_items, stream);
    return gat_fwd_launch<4, 64, 4>(p, has_items, stream);
}

YITU_API int yitu_gat_backward(float *grad_query, float *grad_key, float *grad_features,
                               float *grad_attn_scratch, float *grad_edge_scratch,
                               const int32_t *indptr, const int32_t *indices, const float *query,
                               const float *key, const float *features, const float *attn,
                               const float *row_stats, const float *out, const float *grad_out,
                               const int32_t *t_indptr,
                               const int32_t *t_rows, const int32_t *t_perm, int64_t n_dst,
                               int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_features,
                               int64_t max_degree, int64_t max_degree_t, const void *plan,
                               const void *plan_t, int grad_out_is_head_mean, void *workspace,
                               size_t workspace_bytes, void *stream_) {
    YITU_REQUIRE(n_dst >= 0 && n_src >= 0 && nnz >= 0 && n_heads >= 0 && n_features >= 0,
                 "negative size");
    YITU_REQUIRE((grad_query || n_dst * n_heads == 0) && (grad_key || n_src * n_heads == 0) &&
                     (grad_features || n_src * n_heads * n_features == 0),
                 "null output");
    YITU_REQUIRE(nnz == 0 || attn || row_stats, "the backward needs attn or the row statistics");
    YITU_REQUIRE(nnz == 0 || (grad_attn_scratch && grad_edge_scratch),
                 "gat_backward needs two [nnz, H] scratch buffers");
    YITU_REQUIRE(t_indptr && (nnz == 0 || (t_rows && t_perm)),
                 "gat_backward needs the transposed structure (yitu_csr_transpose)");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    // Rows of 256, 512 or 1024 floats with a power-of-two head width of 32 to 256: one
    // pass over the transposed structure serves every gradient from a single gather.
    const int64_t L = n_heads * n_features;
    const int lph = (int)(n_features / 4);
    const bool one_gather = (L == 256 || L == 512 || L == 1024) && n_features % 4 == 0 && lph >= 8 &&
                            lph <= 64 &&
                            (lph & (lph - 1)) == 0 && n_dst > 0 && nnz > 0 && n_dst < INT32_MAX &&
                            n_src <= (1 << 24) && aligned16(features) && aligned16(grad_out) &&
                            aligned16(grad_features);
    YITU_REQUIRE(!grad_out_is_head_mean || aligned16(attn), "attn must be 16-byte aligned");
    YITU_REQUIRE(nnz == 0 || attn || (one_gather && out && aligned16(out)),
                 "without attn the backward needs a one-pass shape and the forward output");
    YITU_REQUIRE(!grad_out_is_head_mean || one_gather,
                 "a head-mean gradient is taken by the one-pass shapes only (rows of 256, 512 or "
                 "1024 floats, head width 32..256 a power of two); expand it to [n_dst, H, F] / H "
                 "for other shapes");
    if (one_gather) {
        GatSrcParams p{};
        p.sp.indptr = t_indptr;
        p.sp.indices = t_rows;
        p.sp.eperm = t_perm;
        p.sp.values = attn;
        p.sp.feat = grad_out;
        p.sp.out = grad_features;
        p.sp.n_rows = (int)n_src;
        p.sp.n_src = (int)n_dst;
        p.sp.L = (int)L;
        p.sp.F = (int)n_features;
        p.sp.H = (int)n_heads;
        p.sp.col_mask = 0x7fffffff;
        p.sp.alpha = 1.0f;
        p.x = features;
        p.grad_a = grad_attn_scratch;
        p.grad_a_vec = aligned16(grad_attn_scratch) ? 1 : 0;
        p.g_ld = grad_out_is_head_mean ? (int)n_features : (int)L;
        p.head_mean = grad_out_is_head_mean ? 1 : 0;
        p.g_scale = grad_out_is_head_mean ? 1.0f / (float)n_heads : 1.0f;
        bool has_items = false;
        void *rest = nullptr;
        size_t rest_bytes = 0;
        int rc = plan_resolve(p.sp.plan, has_items, plan_t, t_indptr, t_rows, n_src, n_dst, nnz,
                              0x7fffffff, max_degree_t, workspace, workspace_bytes, &rest,
                              &rest_bytes, stream);
        if (rc) return rc;
        const bool full = out != nullptr && aligned16(out);
        const size_t part = has_items ? align_up(sizeof(float) * (size_t)p.sp.plan.max_items *
                                                     (size_t)L, 256) : 0;
        const size_t part_k = has_items && full
                                  ? align_up(sizeof(float) * (size_t)p.sp.plan.max_items *
                                                 (size_t)n_heads, 256) : 0;
        const size_t dots = full ? sizeof(float4) * (size_t)(n_dst * n_heads) : 0;
        YITU_REQUIRE((part + part_k + dots == 0) || (rest && rest_bytes >= part + part_k + dots),
                     "workspace too small: need %zu more bytes", part + part_k + dots);
        char *w = static_cast<char *>(rest);
        if (has_items) p.sp.partial = reinterpret_cast<float *>(w);
        if (!full) {
            rc = gat_src_launch<false>(p, has_items, grad_out, nullptr, nullptr, (int)n_dst, stream);
            if (rc) return rc;
            // softmax + LeakyReLU backward from d_attn; grad_key over the transposed structure
            return sddmm_backward_run(grad_query, grad_key, grad_edge_scratch, indptr, indices,
                                      query, key, attn, grad_attn_scratch, t_indptr, t_perm, n_dst,
                                      n_src, nnz, n_heads, 1, max_degree, max_degree_t, plan,
                                      plan_t, workspace, workspace_bytes, 0, stream);
        }
        // With the forward output the softmax row sums are known up front and the pass
        // also finishes the per-edge logit gradient (left in grad_attn_scratch, CSR
        // order) and grad_key; grad_query is its sum over each destination row.
        p.partial_k = reinterpret_cast<float *>(w + part);
        p.row_sq = reinterpret_cast<float4 *>(w + part + part_k);
        p.stats = row_stats;
        p.recompute = row_stats != nullptr;
        p.key = key;
        p.grad_k = grad_key;
        rc = gat_src_launch<true>(p, has_items, grad_out, out, query, (int)n_dst, stream);
        if (rc) return rc;
        SpmmParams q{};
        q.indptr = indptr;
        q.indices = indices;
        q.cols_are_edges = 1;
        q.feat = grad_attn_scratch;
        q.out = grad_query;
        q.n_rows = (int)n_dst;
        q.n_src = (int)n_src;
        q.L = q.F = (int)n_heads;
        q.H = 1;
        q.col_mask = kColMask;
        q.alpha = 1.0f;
        return launch_spmm(q, W_NONE, false, nnz, max_degree, plan, workspace, workspace_bytes,
                           stream);
    }
    // d attn = <grad_out[row], x[col]> per edge and head; grad_x = attn-weighted
    // gather of grad_out over the transposed structure
    int rc = spmm_backward_run(grad_attn_scratch, grad_features, attn, indptr, indices, features,
                               grad_out, t_indptr, t_rows, t_perm, n_dst, n_src, nnz, n_heads,
                               n_features, max_degree, max_degree_t, plan, plan_t, workspace,
                               workspace_bytes, false, stream);
    if (rc) return rc;
    // softmax + LeakyReLU backward; grad_key gathered over the transposed structure
    return sddmm_backward_run(grad_query, grad_key, grad_edge_scratch, indptr, indices, query, key,
                              attn, grad_attn_scratch, t_indptr, t_perm, n_dst, n_src, nnz, n_heads,
                              1, max_degree, max_degree_t, plan, plan_t, workspace, workspace_bytes,
                              0, stream);
}
