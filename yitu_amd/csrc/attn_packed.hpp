// Attention-only kernels (SDDMM + LeakyReLU + edge softmax of one query block, forward
// and backward) in the packed layout of packed_rows.hpp: a lane owns an EDGE and HV
// heads of it, so keys, probabilities and gradients move as one 16-byte vector per edge.
//
// Short rows are walked in chunks of whole rows (packed_walk). Planned rows (64 edges
// and more) keep the three steps of the row plan (item statistics, per-row combine,
// item apply); an item is at most 64 edges, one per lane, and its reductions run on the
// vector ALU's data-parallel primitives.
//
// Included by gat.hip behind the parameter structs.
#pragma once
#include "packed_rows.hpp"

namespace yitu {

// Heads per lane and pass: the widest vector that divides the head count.
inline int packed_head_vec(int H) { return H % 4 == 0 ? 4 : (H % 2 == 0 ? 2 : 1); }
// The packed kernels make H / HV passes over a chunk; beyond 4 passes the
// (edge, head)-per-lane kernels are the better fit.
inline bool packed_heads_ok(int H) { return H >= 1 && H / packed_head_vec(H) <= 4; }

// ================================ forward ========================================

// Probabilities of one row of more than 64 edges by two walks over it (no plan).
template <int HV>
__device__ __forceinline__ void attn_big_row(const GatParams &p, int row, int beg, int end) {
    const int lane = lane_id();
    const int H = p.sp.H;
    for (int h0 = 0; h0 < H; h0 += HV) {
        float q[HV];
        RowLoad<HV, float>::ld(p.query + (size_t)row * H + h0, q);
        MaxSum a[HV];
#pragma unroll
        for (int h = 0; h < HV; h++) a[h] = ms_init();
        for (int e = beg + lane; e < end; e += kWave) {
            float k[HV];
            RowLoad<HV, float>::ld(p.key + (size_t)(p.sp.indices[e] & kColMask) * H + h0, k);
#pragma unroll
            for (int h = 0; h < HV; h++) a[h] = ms_push(a[h], leaky(q[h] + k[h]));
        }
#pragma unroll
        for (int h = 0; h < HV; h++) a[h] = ms_wave<1>(a[h]);
        for (int e = beg + lane; e < end; e += kWave) {
            float k[HV], o[HV];
            RowLoad<HV, float>::ld(p.key + (size_t)(p.sp.indices[e] & kColMask) * H + h0, k);
#pragma unroll
            for (int h = 0; h < HV; h++) o[h] = expf(leaky(q[h] + k[h]) - a[h].m) * (1.0f / a[h].s);
            store_row<HV>(p.attn + (size_t)e * H + h0, o);
        }
    }
}

template <int HV>
__global__ __launch_bounds__(kBlock) void attn_rows_packed_kernel(GatParams p, int R) {
    const int lane = lane_id();
    const int H = p.sp.H;
    packed_walk(
        p.sp, R, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave,
        [&](const PackedChunk &c) {
            // lanes past the chunk repeat its last edge: every load is unconditional
            const bool act = lane < c.n;
            const int e = c.base + min(lane, c.n - 1);
            const int col = p.sp.indices[e] & kColMask;
            for (int h0 = 0; h0 < H; h0 += HV) {
                float l[HV], m[HV], s[HV], q[HV], k[HV];
                RowLoad<HV, float>::ld(p.query + (size_t)(c.r0 + c.pos) * H + h0, q);
                RowLoad<HV, float>::ld(p.key + (size_t)col * H + h0, k);
#pragma unroll
                for (int h = 0; h < HV; h++) m[h] = l[h] = act ? leaky(q[h] + k[h]) : -FLT_MAX;
                seg_total<HV>(m, c, [](float a, float b) { return fmaxf(a, b); });
#pragma unroll
                for (int h = 0; h < HV; h++) l[h] = s[h] = act ? expf(l[h] - m[h]) : 0.0f;
                seg_total<HV>(s, c, [](float a, float b) { return a + b; });
                if (act) {
#pragma unroll
                    for (int h = 0; h < HV; h++) l[h] *= 1.0f / s[h];
                    store_row<HV>(p.attn + (size_t)e * H + h0, l);
                }
            }
        },
        [&](int row, int beg, int end) { attn_big_row<HV>(p, row, beg, end); },
        [](int, unsigned long long) {});
}

// ---- fused attention + aggregate on short rows, rows of 256 KT floats at most ------
// Phase A is the packed softmax above, kept in registers: lane e ends up with the
// probabilities of edge e for every head (H <= 4 HV). Phase B walks the rows of the chunk
// one after the other: an edge is one wave-wide gather of its source's feature row (a lane
// holds 4 floats of each of the KT tiles), weighted by the probability of the lane's head,
// which reaches the lane as a scalar read of the edge's lane. The (edge, head)-per-lane
// kernel did phase A row by row (a dependent load chain and several hundred instructions
// per row, whatever its length) and was bound by instruction issue, not by the gathers.
constexpr int kPackedGroups = 4;  // head groups of HV heads a lane can hold

template <int HV, int KT>
struct PackedGat {
    const GatParams &p;
    const float *__restrict__ feat;
    TileLanes<4, kWave, KT, W_EDGEHEAD> tl;
    int groups;

    __device__ __forceinline__ PackedGat(const GatParams &p_)
        : p(p_), feat(static_cast<const float *>(p_.sp.feat)), tl(p_.sp, 0),
          groups(p_.sp.H / HV) {}

    // acc += sum over the edges held by lanes [k, last] of prob[lane's head] * x[col]
    __device__ __forceinline__ void apply(float (&acc)[KT][4], int col,
                                          const float (&pr)[kPackedGroups][HV], int k,
                                          int last) const {
        constexpr int U = KT >= 4 ? 2 : 4;  // row gathers in flight
        const int L = p.sp.L;
        for (; k <= last; k += U) {
            float v[U][KT][4], w[U][KT];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const bool past = k + u > last;  // wave-uniform: no edge, no load
                const int ek = min(k + u, last);
                const int c = __builtin_amdgcn_readlane(col, ek);
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    if (!past) {
                        RowLoad<4, float>::ld(feat + (size_t)c * L + tl.off[t], v[u][t]);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; i++) v[u][t][i] = 0.0f;
                    }
                    w[u][t] = 0.0f;
                }
#pragma unroll
                for (int g = 0; g < kPackedGroups; g++) {
                    if (g >= groups) break;  // wave-uniform
#pragma unroll
                    for (int h = 0; h < HV; h++) {
                        const float ph = __int_as_float(
                            __builtin_amdgcn_readlane(__float_as_int(pr[g][h]), ek));
#pragma unroll
                        for (int t = 0; t < KT; t++)
                            if (tl.head[t] == g * HV + h) w[u][t] = ph;
                    }
                }
                if (past) {
#pragma unroll
                    for (int t = 0; t < KT; t++) w[u][t] = 0.0f;
                }
#pragma unroll
                for (int t = 0; t < KT; t++)
                    if (!tl.live[t]) w[u][t] = 0.0f;
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[t][i] += w[u][t] * v[u][t][i];
        }
    }

    __device__ __forceinline__ void store(int row, const float (&acc)[KT][4]) const {
#pragma unroll
        for (int t = 0; t < KT; t++) {
            const int o = (t * kWave + lane_id()) * 4;
            if (o < p.sp.L) store_row_streaming<4>(p.sp.out + (size_t)row * p.sp.L + o, acc[t]);
        }
    }
};

template <int HV, int KT>
__global__ __launch_bounds__(kBlock) void gat_rows_packed_kernel(GatParams p, int R) {
    const int lane = lane_id();
    const int H = p.sp.H;
    const PackedGat<HV, KT> pg(p);
    packed_walk(
        p.sp, R, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave,
        [&](const PackedChunk &c) {
            const bool act = lane < c.n;
            const int e = c.base + min(lane, c.n - 1);
            const int col = p.sp.indices[e] & kColMask;
            float pr[kPackedGroups][HV];
#pragma unroll
            for (int g = 0; g < kPackedGroups; g++) {
#pragma unroll
                for (int h = 0; h < HV; h++) pr[g][h] = 0.0f;
                if (g >= pg.groups) continue;  // wave-uniform
                const int h0 = g * HV;
                float l[HV], m[HV], s[HV], q[HV], k[HV];
                RowLoad<HV, float>::ld(p.query + (size_t)(c.r0 + c.pos) * H + h0, q);
                RowLoad<HV, float>::ld(p.key + (size_t)col * H + h0, k);
#pragma unroll
                for (int h = 0; h < HV; h++) m[h] = l[h] = act ? leaky(q[h] + k[h]) : -FLT_MAX;
                seg_total<HV>(m, c, [](float a, float b) { return fmaxf(a, b); });
#pragma unroll
                for (int h = 0; h < HV; h++) l[h] = s[h] = act ? expf(l[h] - m[h]) : 0.0f;
                seg_total<HV>(s, c, [](float a, float b) { return a + b; });
                if (act) {
#pragma unroll
                    for (int h = 0; h < HV; h++) {
                        s[h] = 1.0f / s[h];
                        pr[g][h] = l[h] * s[h];
                    }
                    if (p.attn) store_row<HV>(p.attn + (size_t)e * H + h0, pr[g]);
                    if (p.stats_out && lane == c.last) {
#pragma unroll
                        for (int h = 0; h < HV; h++) {
                            p.stats_out[((size_t)(c.r0 + c.pos) * H + h0 + h) * 2] = m[h];
                            p.stats_out[((size_t)(c.r0 + c.pos) * H + h0 + h) * 2 + 1] = s[h];
                        }
                    }
                }
            }
            for (int k = 0; k < c.n;) {  // the rows of the chunk, one after the other
                const int last = __builtin_amdgcn_readlane(c.last, k);
                const int row = c.r0 + __builtin_amdgcn_readlane(c.pos, k);
                float acc[KT][4];
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[t][i] = 0.0f;
                pg.apply(acc, col, pr, k, last);
                pg.store(row, acc);
                k = last + 1;
            }
        },
        [&](int row, int beg, int end) {  // more than 64 edges and no plan: two walks
            MaxSum a[kPackedGroups][HV];
#pragma unroll
            for (int g = 0; g < kPackedGroups; g++) {
#pragma unroll
                for (int h = 0; h < HV; h++) a[g][h] = ms_init();
                if (g >= pg.groups) continue;
                float q[HV];
                RowLoad<HV, float>::ld(p.query + (size_t)row * H + g * HV, q);
                for (int e = beg + lane; e < end; e += kWave) {
                    float k[HV];
                    RowLoad<HV, float>::ld(
                        p.key + (size_t)(p.sp.indices[e] & kColMask) * H + g * HV, k);
#pragma unroll
                    for (int h = 0; h < HV; h++) a[g][h] = ms_push(a[g][h], leaky(q[h] + k[h]));
                }
#pragma unroll
                for (int h = 0; h < HV; h++) {
                    a[g][h] = ms_wave<1>(a[g][h]);
                    a[g][h].s = 1.0f / a[g][h].s;
                    if (p.stats_out && lane == 0) {
                        p.stats_out[((size_t)row * H + g * HV + h) * 2] = a[g][h].m;
                        p.stats_out[((size_t)row * H + g * HV + h) * 2 + 1] = a[g][h].s;
                    }
                }
            }
            float acc[KT][4];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) acc[t][i] = 0.0f;
            for (int b = beg; b < end; b += kWave) {
                const int n = min(kWave, end - b);
                const int e = b + min(lane, n - 1);
                const int col = p.sp.indices[e] & kColMask;
                float pr[kPackedGroups][HV];
#pragma unroll
                for (int g = 0; g < kPackedGroups; g++) {
#pragma unroll
                    for (int h = 0; h < HV; h++) pr[g][h] = 0.0f;
                    if (g >= pg.groups) continue;
                    float q[HV], k[HV];
                    RowLoad<HV, float>::ld(p.query + (size_t)row * H + g * HV, q);
                    RowLoad<HV, float>::ld(p.key + (size_t)col * H + g * HV, k);
#pragma unroll
                    for (int h = 0; h < HV; h++)
                        pr[g][h] = expf(leaky(q[h] + k[h]) - a[g][h].m) * a[g][h].s;
                    if (p.attn && lane < n) store_row<HV>(p.attn + (size_t)e * H + g * HV, pr[g]);
                }
                pg.apply(acc, col, pr, 0, n - 1);
            }
            pg.store(row, acc);
        },
        [&](int r0, unsigned long long empty) {
            float z[KT][4];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) z[t][i] = 0.0f;
            while (empty) {  // wave-uniform: the whole wave clears one row per turn
                const int i = __ffsll((long long)empty) - 1;
                empty &= empty - 1;
                pg.store(r0 + i, z);
                if (p.stats_out && lane < H) {
                    p.stats_out[((size_t)(r0 + i) * H + lane) * 2] = 0.0f;
                    p.stats_out[((size_t)(r0 + i) * H + lane) * 2 + 1] = 0.0f;
                }
            }
        });
}

// ---- planned rows: a software-pipelined walk over the plan's items ---------------
// Every step of an item waits on the one before it (record -> edge indices -> keys), and
// a wave that takes one group of items and exits pays that chain, the kernel's start-up
// and the plan's counters once per group: measured, such kernels moved 1 to 3.5 TB/s.
// Here a modest grid of waves stays resident, a wave takes groups g, g + waves, ... and
// keeps three of them in flight: while it computes on group g, the indices of the next
// group and the records of the one after are already on their way. `issue` starts the
// gathers of a group and returns what it loaded, `finish` consumes it; the loads of the
// later groups are issued between the two, so waiting for the gathers does not wait for
// them (loads return in order).
constexpr int kPackedItems = 4;  // items of a group: their loads are in flight together

struct PackedItems {
    int beg[kPackedItems], n[kPackedItems], item[kPackedItems], row[kPackedItems];
    // this lane's edge and its source in every item; lanes past the item's end hold its last
    // edge, so that every load of a group is unconditional (loads under a lane mask of their
    // own are waited for one by one) and only the stores look at n
    int e[kPackedItems], col[kPackedItems];  // col: the packed index word, unmasked
};

template <int N, int HV>
struct ItemRegs {
    float v[N][kPackedItems][HV];
};

constexpr int kPackedItemBlocks = 2048;  // resident workgroups of the item kernels

inline int packed_item_grid(int64_t max_items) {
    return (int)std::min<int64_t>(ceil_div(max_items, kWavesPerBlock * kPackedItems),
                                  kPackedItemBlocks);
}

template <typename Issue, typename Finish>
__device__ __forceinline__ void packed_item_loop(const SpmmParams &sp, Issue issue, Finish finish) {
    const int lane = lane_id();
    if (sp.plan.counters->overflow) return;
    const int n_items = min(sp.plan.counters->n_items, sp.plan.max_items);
    const int n_groups = (n_items + kPackedItems - 1) / kPackedItems;
    const int n_waves = gridDim.x * kWavesPerBlock;
    int g = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (g >= n_groups) return;
    const auto record = [&](int grp) {
        return sp.plan.records[min(grp * kPackedItems + min(lane, kPackedItems - 1), n_items - 1)];
    };
    const auto unpack = [&](const int4 &rec, int grp) {
        PackedItems it;
        const int n_here = min(kPackedItems, n_items - grp * kPackedItems);
#pragma unroll
        for (int j = 0; j < kPackedItems; j++) {
            it.beg[j] = __builtin_amdgcn_readlane(rec.x, j);
            it.n[j] = j < n_here ? __builtin_amdgcn_readlane(rec.y, j) - it.beg[j] : 0;
            it.item[j] = __builtin_amdgcn_readlane(rec.z, j);
            it.row[j] = __builtin_amdgcn_readlane(rec.w, j) & 0x7fffffff;
        }
#pragma unroll
        for (int j = 0; j < kPackedItems; j++) {
            it.e[j] = it.beg[j] + min(lane, max(it.n[j], 1) - 1);
            it.col[j] = sp.indices[it.e[j]];  // masked where it is used: no wait here
        }
        return it;
    };
    PackedItems cur = unpack(record(g), g);
    int4 rec_next = record(min(g + n_waves, n_groups - 1));
    for (;;) {
        auto loaded = issue(cur);
        const int gn = g + n_waves;
        const bool more = gn < n_groups;
        PackedItems nxt = cur;
        if (more) nxt = unpack(rec_next, gn);
        const int4 rec_after = record(min(gn + n_waves, n_groups - 1));
        finish(cur, loaded);
        if (!more) break;
        cur = nxt;
        rec_next = rec_after;
        g = gn;
    }
}

// Planned rows, step 1: (max, sum) of every plan item, [item][H][2].
template <int HV>
__global__ __launch_bounds__(kBlock) void attn_item_stats_packed_kernel(GatParams p) {
    const int lane = lane_id();
    const int H = p.sp.H;
    for (int h0 = 0; h0 < H; h0 += HV) {
        packed_item_loop(
            p.sp,
            [&](const PackedItems &it) {
                ItemRegs<2, HV> r;  // query, key
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    RowLoad<HV, float>::ld(p.query + (size_t)it.row[j] * H + h0, r.v[0][j]);
                    RowLoad<HV, float>::ld(p.key + (size_t)(it.col[j] & kColMask) * H + h0, r.v[1][j]);
                }
                return r;
            },
            [&](const PackedItems &it, const ItemRegs<2, HV> &r) {
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    if (it.n[j] <= 0) continue;
                    const bool act = lane < it.n[j];
                    float l[HV], m[HV], s[HV];
#pragma unroll
                    for (int h = 0; h < HV; h++)
                        m[h] = l[h] = act ? leaky(r.v[0][j][h] + r.v[1][j][h]) : -FLT_MAX;
                    wave_max<HV>(m);
#pragma unroll
                    for (int h = 0; h < HV; h++) s[h] = act ? expf(l[h] - m[h]) : 0.0f;
                    wave_sum<HV>(s);
                    if (lane == 0) {
                        float st[2 * HV];
#pragma unroll
                        for (int h = 0; h < HV; h++) {
                            st[2 * h] = m[h];
                            st[2 * h + 1] = s[h];
                        }
                        float *dst = p.item_stats + ((size_t)it.item[j] * H + h0) * 2;
                        store_row<HV>(dst, *reinterpret_cast<const float(*)[HV]>(st));
                        store_row<HV>(dst + HV, *reinterpret_cast<const float(*)[HV]>(st + HV));
                    }
                }
            });
    }
}

// Planned rows, step 3: probabilities from the rows' (max, 1 / sum).
template <int HV>
__global__ __launch_bounds__(kBlock) void attn_item_write_packed_kernel(GatParams p) {
    const int lane = lane_id();
    const int H = p.sp.H;
    for (int h0 = 0; h0 < H; h0 += HV) {
        packed_item_loop(
            p.sp,
            [&](const PackedItems &it) {
                ItemRegs<4, HV> r;  // query, key, row statistics (2 HV floats)
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    const float *rs = p.row_stats + ((size_t)it.row[j] * H + h0) * 2;
                    RowLoad<HV, float>::ld(p.query + (size_t)it.row[j] * H + h0, r.v[0][j]);
                    RowLoad<HV, float>::ld(p.key + (size_t)(it.col[j] & kColMask) * H + h0, r.v[1][j]);
                    RowLoad<HV, float>::ld(rs, r.v[2][j]);
                    RowLoad<HV, float>::ld(rs + HV, r.v[3][j]);
                }
                return r;
            },
            [&](const PackedItems &it, const ItemRegs<4, HV> &r) {
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    if (lane >= it.n[j]) continue;
                    float o[HV];
#pragma unroll
                    for (int h = 0; h < HV; h++) {
                        // (max, 1 / sum) pairs of the HV heads lie interleaved in v[2], v[3]
                        const float mx = (2 * h < HV ? r.v[2][j] : r.v[3][j])[(2 * h) % HV];
                        const float inv = (2 * h + 1 < HV ? r.v[2][j] : r.v[3][j])[(2 * h + 1) % HV];
                        o[h] = expf(leaky(r.v[0][j][h] + r.v[1][j][h]) - mx) * inv;
                    }
                    store_row<HV>(p.attn + (size_t)(it.beg[j] + lane) * H + h0, o);
                }
            });
    }
}

// ================================ backward =======================================
// Per row and head S = sum a g, A1 = sum a g s, A2 = sum a s (a = attn, g = its gradient,
// s = LeakyReLU slope of the edge's logit); grad_query = A1 - S A2, and the logit
// gradient of an edge is a (g - S) s.

template <int HV>
__device__ __forceinline__ void attn_bwd_big_row(const GatBwdParams &p, int row, int beg, int end) {
    const int lane = lane_id();
    const int H = p.sp.H;
    for (int h0 = 0; h0 < H; h0 += HV) {
        float q[HV], S[HV], A1[HV], A2[HV];
        RowLoad<HV, float>::ld(p.query + (size_t)row * H + h0, q);
#pragma unroll
        for (int h = 0; h < HV; h++) S[h] = A1[h] = A2[h] = 0.0f;
        for (int e = beg + lane; e < end; e += kWave) {
            float k[HV], a[HV], g[HV];
            RowLoad<HV, float>::ld(p.key + (size_t)(p.sp.indices[e] & kColMask) * H + h0, k);
            RowLoad<HV, float>::ld(p.attn + (size_t)e * H + h0, a);
            RowLoad<HV, float>::ld(p.grad_a + (size_t)e * H + h0, g);
#pragma unroll
            for (int h = 0; h < HV; h++) {
                const float sl = q[h] + k[h] < 0.0f ? kSlope : 1.0f;
                S[h] += a[h] * g[h];
                A1[h] += a[h] * g[h] * sl;
                A2[h] += a[h] * sl;
            }
        }
        wave_sum<HV>(S);
        wave_sum<HV>(A1);
        wave_sum<HV>(A2);
        if (lane == 0) {
            float gq[HV];
#pragma unroll
            for (int h = 0; h < HV; h++) gq[h] = A1[h] - S[h] * A2[h];
            store_row<HV>(p.grad_q + (size_t)row * H + h0, gq);
        }
        for (int e = beg + lane; e < end; e += kWave) {
            float k[HV], a[HV], g[HV], o[HV];
            RowLoad<HV, float>::ld(p.key + (size_t)(p.sp.indices[e] & kColMask) * H + h0, k);
            RowLoad<HV, float>::ld(p.attn + (size_t)e * H + h0, a);
            RowLoad<HV, float>::ld(p.grad_a + (size_t)e * H + h0, g);
#pragma unroll
            for (int h = 0; h < HV; h++)
                o[h] = a[h] * (g[h] - S[h]) * (q[h] + k[h] < 0.0f ? kSlope : 1.0f);
            store_row<HV>(p.grad_e + (size_t)e * H + h0, o);
        }
    }
}

template <int HV>
__global__ __launch_bounds__(kBlock) void attn_bwd_rows_packed_kernel(GatBwdParams p, int R) {
    const int lane = lane_id();
    const int H = p.sp.H;
    packed_walk(
        p.sp, R, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave,
        [&](const PackedChunk &c) {
            const bool act = lane < c.n;
            const int e = c.base + min(lane, c.n - 1);
            const int col = p.sp.indices[e] & kColMask;
            for (int h0 = 0; h0 < H; h0 += HV) {
                float a[HV], g[HV], sl[HV], S[HV], A1[HV], A2[HV], q[HV], k[HV];
                RowLoad<HV, float>::ld(p.attn + (size_t)e * H + h0, a);
                RowLoad<HV, float>::ld(p.grad_a + (size_t)e * H + h0, g);
                RowLoad<HV, float>::ld(p.query + (size_t)(c.r0 + c.pos) * H + h0, q);
                RowLoad<HV, float>::ld(p.key + (size_t)col * H + h0, k);
#pragma unroll
                for (int h = 0; h < HV; h++) {
                    sl[h] = q[h] + k[h] < 0.0f ? kSlope : 1.0f;
                    if (!act) a[h] = 0.0f;  // adds nothing to the sums
                }
#pragma unroll
                for (int h = 0; h < HV; h++) {
                    S[h] = a[h] * g[h];
                    A1[h] = a[h] * g[h] * sl[h];
                    A2[h] = a[h] * sl[h];
                }
                const auto add = [](float x, float y) { return x + y; };
                seg_total<HV>(S, c, add);
                seg_total<HV>(A1, c, add);
                seg_total<HV>(A2, c, add);
                if (act) {
                    float o[HV];
#pragma unroll
                    for (int h = 0; h < HV; h++) o[h] = a[h] * (g[h] - S[h]) * sl[h];
                    store_row<HV>(p.grad_e + (size_t)e * H + h0, o);
                    if (lane == c.last) {
#pragma unroll
                        for (int h = 0; h < HV; h++) o[h] = A1[h] - S[h] * A2[h];
                        store_row<HV>(p.grad_q + (size_t)(c.r0 + c.pos) * H + h0, o);
                    }
                }
            }
        },
        [&](int row, int beg, int end) { attn_bwd_big_row<HV>(p, row, beg, end); },
        [&](int r0, unsigned long long empty) {
            if ((empty >> lane) & 1ull)
                for (int h = 0; h < H; h++) p.grad_q[(size_t)(r0 + lane) * H + h] = 0.0f;
        });
}

// Planned rows, step 1: (S, A1, A2) of every plan item, [item][H][3].
template <int HV>
__global__ __launch_bounds__(kBlock) void attn_bwd_item_sums_packed_kernel(GatBwdParams p) {
    const int lane = lane_id();
    const int H = p.sp.H;
    for (int h0 = 0; h0 < H; h0 += HV) {
        packed_item_loop(
            p.sp,
            [&](const PackedItems &it) {
                ItemRegs<4, HV> r;  // attn, its gradient, query, key
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    const size_t e = (size_t)it.e[j] * H + h0;
                    RowLoad<HV, float>::ld(p.attn + e, r.v[0][j]);
                    RowLoad<HV, float>::ld(p.grad_a + e, r.v[1][j]);
                    RowLoad<HV, float>::ld(p.query + (size_t)it.row[j] * H + h0, r.v[2][j]);
                    RowLoad<HV, float>::ld(p.key + (size_t)(it.col[j] & kColMask) * H + h0, r.v[3][j]);
                }
                return r;
            },
            [&](const PackedItems &it, const ItemRegs<4, HV> &r) {
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    if (it.n[j] <= 0) continue;
                    float S[HV], A1[HV], A2[HV];
#pragma unroll
                    for (int h = 0; h < HV; h++) {
                        S[h] = A1[h] = A2[h] = 0.0f;
                        if (lane < it.n[j]) {
                            const float sl = r.v[2][j][h] + r.v[3][j][h] < 0.0f ? kSlope : 1.0f;
                            S[h] = r.v[0][j][h] * r.v[1][j][h];
                            A1[h] = S[h] * sl;
                            A2[h] = r.v[0][j][h] * sl;
                        }
                    }
                    wave_sum<HV>(S);
                    wave_sum<HV>(A1);
                    wave_sum<HV>(A2);
                    if (lane == 0) {
#pragma unroll
                        for (int h = 0; h < HV; h++) {
                            float *st = p.item_sums + ((size_t)it.item[j] * H + h0 + h) * 3;
                            st[0] = S[h];
                            st[1] = A1[h];
                            st[2] = A2[h];
                        }
                    }
                }
            });
    }
}

// Planned rows, step 3: the per-edge logit gradient from the rows' S.
template <int HV>
__global__ __launch_bounds__(kBlock) void attn_bwd_apply_packed_kernel(GatBwdParams p) {
    const int lane = lane_id();
    const int H = p.sp.H;
    for (int h0 = 0; h0 < H; h0 += HV) {
        packed_item_loop(
            p.sp,
            [&](const PackedItems &it) {
                ItemRegs<5, HV> r;  // attn, its gradient, query, key, S of the row
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    const size_t e = (size_t)it.e[j] * H + h0;
                    RowLoad<HV, float>::ld(p.attn + e, r.v[0][j]);
                    RowLoad<HV, float>::ld(p.grad_a + e, r.v[1][j]);
                    RowLoad<HV, float>::ld(p.query + (size_t)it.row[j] * H + h0, r.v[2][j]);
                    RowLoad<HV, float>::ld(p.key + (size_t)(it.col[j] & kColMask) * H + h0, r.v[3][j]);
                    RowLoad<HV, float>::ld(p.row_sum + (size_t)it.row[j] * H + h0, r.v[4][j]);
                }
                return r;
            },
            [&](const PackedItems &it, const ItemRegs<5, HV> &r) {
#pragma unroll
                for (int j = 0; j < kPackedItems; j++) {
                    if (lane >= it.n[j]) continue;
                    float o[HV];
#pragma unroll
                    for (int h = 0; h < HV; h++)
                        o[h] = r.v[0][j][h] * (r.v[1][j][h] - r.v[4][j][h]) *
                               (r.v[2][j][h] + r.v[3][j][h] < 0.0f ? kSlope : 1.0f);
                    store_row<HV>(p.grad_e + (size_t)(it.beg[j] + lane) * H + h0, o);
                }
            });
    }
}

}  // namespace yitu
