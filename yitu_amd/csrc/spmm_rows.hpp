// Row-split CSR gather-accumulate, the one inner loop behind every SpMM in the
// library (GCN / GIN / SAG aggregation, multi-head edge-weighted SpMM, the
// transposed pass of its backward, and the aggregate step of the fused GAT).
//
// Mapping (wave64):
//   * the row vector of L = H*F floats is laid across G lanes x VEC elements x
//     KT tiles, so one wave-wide load instruction fetches 64/G ("slots")
//     neighbour rows at once;
//   * column ids (and per-edge scalars) of 64 consecutive CSR edges are fetched
//     with one coalesced load (an "edge window"), then broadcast lane-to-lane, so
//     the feature gathers of one round are independent and UNROLL of them are
//     in flight per wave;
//   * slots are folded in fixed pairs (lane swaps of the vector ALU, every slot keeping
//     its share of the row) and a row is written once, by all 64 lanes: no atomics,
//     bitwise reproducible;
//   * rows below the plan threshold (64 edges): a wave walks 4 consecutive rows
//     through a sliding window; longer rows: the row plan's items of at most 64
//     edges in band order, four per wave, whose partial rows a third kernel adds
//     in a fixed order.
#pragma once
#include "common.hpp"
#include "plan.hpp"

namespace yitu {

enum WeightMode : int {
    W_NONE = 0,      // w = 1
    W_DEGPROD = 1,   // w = s_row * s_col            (module-1 GCN norm)
    W_EDGEHEAD = 2,  // w = values[edge, head]       (module-2 SpMM)
};

struct SpmmParams {
    const int32_t *indptr;   // [n_rows + 1]
    const int32_t *indices;  // [nnz], column in the low bits selected by col_mask
    const void *feat;        // [n_src, L] fp32 or bf16
    float *out;              // [n_rows, L] fp32, or bf16 (see out_bf16)
    const float *scale_row;  // W_DEGPROD: s[n_rows]; otherwise unused
    const float *scale_col;  // W_DEGPROD: s[n_src]
    const float *edge_scale; // W_DEGPROD, optional: [nnz] = s[col of the edge], read in edge
                             // order instead of one random read of scale_col per edge
    const float *values;     // W_EDGEHEAD: [nnz, H]
    const int32_t *eperm;    // optional: values row of edge i is eperm[i] (transposed pass)
    int n_rows;
    int n_src;     // rows of feat (sets the width of the band-sort key)
    int L;         // floats per feature row (H * F)
    int F;         // floats per head
    int H;
    int col_mask;
    int cols_are_edges;  // nonzero: edge e reads feat row e (a segmented sum of per-edge rows)
    float alpha;   // output scale
    int out_bf16;  // nonzero: the output rows are bf16 (round to nearest even); partial rows
                   // stay fp32. Taken by the row / item / reduce kernels of this file.
    PlanView plan;   // long rows: band-ordered 64-edge items (plan.threshold = INT_MAX: none)
    float *partial;  // [plan item id, L] unscaled partial rows of multi-item rows
};

// Stores VEC consecutive elements of an output row, `elem` elements into the output:
// fp32 as they are, or rounded to bf16 when the caller asked for bf16 rows (a pipeline
// whose next product reads bf16 then needs no conversion pass of its own).
template <int VEC>
__device__ __forceinline__ void store_out(const SpmmParams &p, size_t elem, const float (&v)[VEC]) {
    if (!p.out_bf16) {  // same for the whole launch
        store_row_streaming<VEC>(p.out + elem, v);
        return;
    }
    uint16_t *dst = reinterpret_cast<uint16_t *>(p.out) + elem;
    if constexpr (VEC % 2 == 0) {
        typedef unsigned int uv __attribute__((ext_vector_type(VEC / 2)));
        uv w;
#pragma unroll
        for (int i = 0; i < VEC / 2; i++) {
            const __bf16 lo = static_cast<__bf16>(v[2 * i]), hi = static_cast<__bf16>(v[2 * i + 1]);
            w[i] = (unsigned)__builtin_bit_cast(uint16_t, lo) |
                   ((unsigned)__builtin_bit_cast(uint16_t, hi) << 16);
        }
        __builtin_nontemporal_store(w, reinterpret_cast<uv *>(dst));
    } else {
#pragma unroll
        for (int i = 0; i < VEC; i++)
            dst[i] = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v[i]));
    }
}

// A window is up to 64 consecutive CSR edges held one per lane: column id,
// per-edge scalar weight (W_NONE / W_DEGPROD) or the row of `values` to read
// (W_EDGEHEAD). It is loaded with one coalesced index load plus one gather and
// then serves every row that falls inside it, so short rows cost no dependent
// index loads of their own.
struct EdgeWindow {
    int base;  // CSR position held by lane 0; -1 = nothing loaded
    int col;
    float w;
    int vrow;
};

// Loads edges [base, base + 64) clipped to `limit` (exclusive). Lanes past the
// limit hold the clamped last edge; they are never selected by a valid step.
template <int WMODE>
__device__ __forceinline__ void load_window(EdgeWindow &win, const SpmmParams &p, int base,
                                            int limit) {
    const int e = min(base + lane_id(), limit - 1);
    win.base = base;
    // the edge arrays are read once per call: streaming loads leave the caches to the rows
    win.col = p.cols_are_edges ? e : (__builtin_nontemporal_load(p.indices + e) & p.col_mask);
    win.w = 1.0f;
    win.vrow = 0;
    if constexpr (WMODE == W_DEGPROD)
        win.w = p.edge_scale ? __builtin_nontemporal_load(p.edge_scale + e) : p.scale_col[win.col];
    if constexpr (WMODE == W_EDGEHEAD) win.vrow = p.eperm ? __builtin_nontemporal_load(p.eperm + e) : e;
}

// One step of the edge loop: every slot of the wave picks its edge
// (window lane first + step + slot) and loads that neighbour's row tile. Slots
// whose edge lies past the n edges of the range carry weight 0 and load the (valid)
// tile of the range's last edge, which the caller must drop (0 x inf is not 0).
// WHOLE: every slot of the step has an edge (step + SLOTS <= n): no clamp, no mask.
template <int VEC, int G, int KT, int WMODE, typename TIN, bool WHOLE = false>
__device__ __forceinline__ void gather_step(float (&v)[KT][VEC], float (&w)[KT],
                                            const SpmmParams &p, const TIN *__restrict__ feat,
                                            const EdgeWindow &win, int first, int step, int n,
                                            const int (&off)[KT], const int (&head)[KT],
                                            const bool (&live)[KT]) {
    constexpr int SLOTS = kWave / G;
    int c, vrow = 0;
    float ws = 0.0f;
    bool valid = true;
    if constexpr (SLOTS == 1) {
        // the edge is the same for the whole wave: scalar broadcast
        const int src = first + step;
        c = __builtin_amdgcn_readlane(win.col, src);
        if constexpr (WMODE == W_EDGEHEAD)
            vrow = __builtin_amdgcn_readlane(win.vrow, src);
        else
            ws = __builtin_bit_cast(float,
                                    __builtin_amdgcn_readlane(__builtin_bit_cast(int, win.w), src));
    } else {
        const int k = step + lane_id() / G;
        valid = WHOLE || k < n;
        const int src = WHOLE ? first + k : first + min(k, n - 1);
        c = __shfl(win.col, src, kWave);
        if constexpr (WMODE == W_EDGEHEAD)
            vrow = __shfl(win.vrow, src, kWave);
        else
            ws = __shfl(win.w, src, kWave);
    }
#pragma unroll
    for (int t = 0; t < KT; t++) {
        if constexpr (WMODE == W_EDGEHEAD)
            w[t] = (valid && live[t]) ? p.values[(size_t)vrow * p.H + head[t]] : 0.0f;
        else
            w[t] = (valid && live[t]) ? ws : 0.0f;
        RowLoad<VEC, TIN>::ld(feat + (size_t)c * p.L + off[t], v[t]);
    }
}

// Column-tile geometry of this lane for the tile that starts at element c0.
template <int VEC, int G, int KT, int WMODE>
struct TileLanes {
    int off[KT];
    int head[KT];
    bool live[KT];
    __device__ __forceinline__ TileLanes(const SpmmParams &p, int c0) {
        const int sub = lane_id() % G;
#pragma unroll
        for (int t = 0; t < KT; t++) {
            off[t] = c0 + (t * G + sub) * VEC;
            live[t] = off[t] < p.L;
            if (!live[t]) off[t] = 0;  // keep the address valid; the weight is forced to 0
            head[t] = WMODE == W_EDGEHEAD ? off[t] / p.F : 0;
        }
    }
};

// Accumulates the n (<= 64) edges that sit in window lanes [first, first + n)
// into acc. All lanes of the wave must call this together.
// UNROLL: load instructions in flight per wave. With 4 slots (G = 16) an instruction
// already fetches four rows and two of them measured best; wide rows keep registers low.
template <int VEC, int G, int KT, int WMODE, typename TIN,
          int UNROLL = ((KT >= 4 || G <= 16) ? 2 : ((G == kWave && KT == 1) ? 8 : 4))>
__device__ __forceinline__ void accumulate_window(float (&acc)[KT][VEC], const SpmmParams &p,
                                                  const EdgeWindow &win, int first, int n,
                                                  const TileLanes<VEC, G, KT, WMODE> &tl) {
    constexpr int SLOTS = kWave / G;
    const TIN *__restrict__ feat = static_cast<const TIN *>(p.feat);
    // full groups of UNROLL steps: all gathers of a group are issued before any FMA
    int s = 0;
    for (; s + SLOTS * UNROLL <= n; s += SLOTS * UNROLL) {
        float v[UNROLL][KT][VEC];
        float w[UNROLL][KT];
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
            gather_step<VEC, G, KT, WMODE, TIN, true>(v[u], w[u], p, feat, win, first,
                                                      s + u * SLOTS, n, tl.off, tl.head, tl.live);
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < VEC; i++) acc[t][i] += w[u][t] * v[u][t][i];
    }
    // the remaining steps (fewer than UNROLL) as one more group: their gathers go out
    // together as well, and the sums are added in the same order as one step at a time
    if (s < n) {
        float v[UNROLL][KT][VEC];
        float w[UNROLL][KT];
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
            if (s + u * SLOTS < n)  // wave-uniform
                gather_step<VEC, G, KT, WMODE, TIN>(v[u], w[u], p, feat, win, first, s + u * SLOTS,
                                                    n, tl.off, tl.head, tl.live);
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
            if (s + u * SLOTS < n) {
                // a slot without an edge has loaded the range's last row again: its values
                // must not reach the sum even as 0 x value. (Selected here, after all the
                // group's loads have been issued, not where the row is loaded.)
                const bool valid = SLOTS == 1 || s + u * SLOTS + lane_id() / G < n;
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < VEC; i++)
                        acc[t][i] += w[u][t] * (valid ? v[u][t][i] : 0.0f);
            }
    }
}

// Folds the SLOTS partial rows of a wave into slot 0 (fixed order).
template <int VEC, int G, int KT>
__device__ __forceinline__ void fold_slots(float (&acc)[KT][VEC]) {
#pragma unroll
    for (int o = 32; o >= G; o >>= 1)
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int i = 0; i < VEC; i++) acc[t][i] += __shfl_xor(acc[t][i], o, kWave);
}

// The same fold for one tile, shared out: the SLOTS partial rows are added in the same
// pairs as in fold_slots (the same bits), but every slot ends up with its own VEC / SLOTS
// consecutive elements of the lane's VEC, r[] = elements [slot * OUT, (slot + 1) * OUT).
// Half the exchanges and adds (two values per exchange), no LDS permutes, and the row is
// then stored by all 64 lanes.
template <int VEC, int G>
__device__ __forceinline__ void fold_scatter(const float (&a)[VEC],
                                             float (&r)[VEC / (kWave / G)]) {
    static_assert(G == 16 || G == 32 || G == kWave, "lanes per row");
    static_assert(VEC % (kWave / G) == 0, "every slot keeps a whole number of elements");
    if constexpr (G == kWave) {
#pragma unroll
        for (int i = 0; i < VEC; i++) r[i] = a[i];
    } else if constexpr (G == 32) {
#pragma unroll
        for (int i = 0; i < VEC / 2; i++) r[i] = pair_sum32(a[i], a[i + VEC / 2]);
    } else {
        float u[VEC / 2];
#pragma unroll
        for (int i = 0; i < VEC / 2; i++) u[i] = pair_sum32(a[i], a[i + VEC / 2]);
#pragma unroll
        for (int j = 0; j < VEC / 4; j++) r[j] = pair_sum16(u[j], u[j + VEC / 4]);
    }
}

constexpr int kRowsPerWave = 4;  // most consecutive rows one wave of a row kernel handles

// Rows per wave of the row kernels: 4 where that still leaves several thousand
// waves, fewer on small graphs (one root per wave at 2,048 sampled roots), so a
// small problem is spread over the chip instead of walked by a few waves. Host
// (grid size) and device (row range of a wave) both derive it from n_rows.
// Why not more: the rows that the resident waves of an XCD cover together are its
// working set. With 16 rows per wave 1,024 resident waves span 16 k rows, and on a
// graph whose rows share sources with their neighbours (communities of 512) the
// sources of 32 communities (8 MB) do not fit the 4 MB L2; with 4 rows they do.
// 2^21 vertices, 63 M edges, fp32 rows of 128 floats, per call: 16 / 8 / 4 / 2 / 1
// rows per wave = 2.69 / 2.15 / 2.07 / 2.06 / 2.09 ms on planted communities,
// 2.70 / 2.69 / 2.71 / 2.79 / 2.94 ms on a power-law graph without locality.
__host__ __device__ inline int rows_per_wave(int n_rows) {
    const int r = n_rows / 4096;
    return r < 1 ? 1 : (r > kRowsPerWave ? kRowsPerWave : r);
}

// Which block of rows a workgroup of the row kernel takes. The hardware deals
// consecutive workgroups to the 8 XCDs round robin. Taken as they come, the
// workgroups that run on one XCD at one time are spread over 8 times as many rows
// as they cover: right for graphs without locality, whose hot sources every L2
// holds anyway. When most sources of a row lie near the row's own id (community
// structure, a reordered graph), XCD k instead walks the k-th eighth of the rows,
// so that the rows in flight on an XCD are neighbours and share their sources in
// that XCD's L2. Which of the two a graph is, its row plan says (measured when the
// plan is built); launches of at least 64 workgroups come in multiples of 8, whose
// surplus workgroups find no rows.
__device__ __forceinline__ int row_block(const SpmmParams &p, int block, int n_blocks) {
    if (n_blocks < 64 || (n_blocks & 7) || !plan_says_local(p.plan)) return block;
    return (block & 7) * (n_blocks >> 3) + (block >> 3);
}

// Row kernel: a wave walks rows_per_wave consecutive rows. Their bounds come from
// one coalesced indptr load, their edges from a sliding 64-edge window, so a
// short row costs one round of feature gathers and nothing else that waits on
// memory. Rows that the plan covers are skipped.
template <int VEC, int G, int KT, int WMODE, typename TIN>
__device__ __forceinline__ void spmm_rows_body(const SpmmParams &p, int block, int n_blocks) {
    const int lane = lane_id();
    const int wave = wave_id();
    const int rpw = rows_per_wave(p.n_rows);
    const int r0 = (row_block(p, block, n_blocks) * kWavesPerBlock + wave) * rpw;
    if (r0 >= p.n_rows) return;
    const int n_here = min(rpw, p.n_rows - r0);
    const int my_ptr = p.indptr[r0 + min(lane, n_here)];
    // the rows' scales with the same round trip as their bounds (a load per row, placed
    // where the scale is first named, would be waited for before the row's gathers)
    float my_scale = 1.0f;
    if constexpr (WMODE == W_DEGPROD) my_scale = p.scale_row[r0 + min(lane, n_here - 1)];
    const int limit = __builtin_amdgcn_readlane(my_ptr, n_here);  // end of this wave's edges
    const int sub = lane % G;
    const int slot = lane / G;

    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;

    for (int i = 0; i < n_here; i++) {
        const int row = r0 + i;
        // (scalar reads: the row's bounds and loops stay off the vector ALU)
        const int beg = __builtin_amdgcn_readlane(my_ptr, i);
        const int end = __builtin_amdgcn_readlane(my_ptr, i + 1);
        const int deg = end - beg;
        if (deg >= p.plan.threshold) continue;  // a planned row: written by the item kernels
        const float sr = __builtin_bit_cast(float, __builtin_amdgcn_readlane(
                             __builtin_bit_cast(int, my_scale), i)) * p.alpha;
        for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
            const TileLanes<VEC, G, KT, WMODE> tl(p, c0);
            float acc[KT][VEC];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int k = 0; k < VEC; k++) acc[t][k] = 0.0f;
            for (int b = beg; b < end; b += kWave) {
                const int n = min(kWave, end - b);
                if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                    load_window<WMODE>(win, p, b, limit);
                accumulate_window<VEC, G, KT, WMODE, TIN>(acc, p, win, b - win.base, n, tl);
            }
            if constexpr (G < kWave && KT == 1) {
                constexpr int OUT = VEC / (kWave / G);
                float r[OUT];
#pragma unroll
                for (int k = 0; k < OUT; k++) r[k] = 0.0f;
                if (deg > 0) fold_scatter<VEC, G>(acc[0], r);
                if (c0 + sub * VEC < p.L) {
#pragma unroll
                    for (int k = 0; k < OUT; k++) r[k] *= sr;
                    store_out<OUT>(p, (size_t)row * p.L + c0 + sub * VEC + slot * OUT, r);
                }
            } else {
                if (deg > 0) fold_slots<VEC, G, KT>(acc);
                if (slot == 0) {
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        const int o = c0 + (t * G + sub) * VEC;
                        if (o < p.L) {
                            float r[VEC];
#pragma unroll
                            for (int k = 0; k < VEC; k++) r[k] = acc[t][k] * sr;
                            store_out<VEC>(p, (size_t)row * p.L + o, r);
                        }
                    }
                }
            }
        }
    }
}

template <int VEC, int G, int KT, int WMODE, typename TIN>
__global__ __launch_bounds__(kBlock) void spmm_rows_kernel(SpmmParams p) {
    spmm_rows_body<VEC, G, KT, WMODE, TIN>(p, blockIdx.x, gridDim.x);
}

constexpr int kItemsPerWave = 4;  // band-sorted items handled by one wave

// One group of up to IPW (items per wave) consecutive records [pos0, pos0 + n_here):
// the records come from one load, their edge windows are all fetched before the
// first feature gather, so the only waits per item are its own gathers. The
// unscaled partial row goes to partial[item id].
template <int VEC, int G, int KT, int WMODE, typename TIN, int IPW>
__device__ __forceinline__ void spmm_item_group(const SpmmParams &p, int pos0, int n_here) {
    const int lane = lane_id();
    const int sub = lane % G;
    const int slot = lane / G;
    const int4 my_rec = p.plan.records[pos0 + min(lane, n_here - 1)];
    EdgeWindow win[IPW];
    int item_id[IPW], n_edges[IPW], row_tag[IPW];
#pragma unroll
    for (int j = 0; j < IPW; j++) {
        const int beg = __builtin_amdgcn_readlane(my_rec.x, j);
        const int end = __builtin_amdgcn_readlane(my_rec.y, j);
        item_id[j] = __builtin_amdgcn_readlane(my_rec.z, j);
        row_tag[j] = __builtin_amdgcn_readlane(my_rec.w, j);
        n_edges[j] = j < n_here ? end - beg : 0;
        if (n_edges[j] > 0) load_window<WMODE>(win[j], p, beg, end);
    }
#pragma unroll
    for (int j = 0; j < IPW; j++) {
        if (n_edges[j] <= 0) continue;
        for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
            const TileLanes<VEC, G, KT, WMODE> tl(p, c0);
            float acc[KT][VEC];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < VEC; i++) acc[t][i] = 0.0f;
            accumulate_window<VEC, G, KT, WMODE, TIN>(acc, p, win[j], 0, n_edges[j], tl);
            const bool single = row_tag[j] < 0;
            const int row = row_tag[j] & 0x7fffffff;
            float *dst = p.partial + (size_t)item_id[j] * p.L;  // not for single items
            const float sr =
                single ? (WMODE == W_DEGPROD ? p.scale_row[row] : 1.0f) * p.alpha : 1.0f;
            if constexpr (G < kWave && KT == 1) {
                constexpr int OUT = VEC / (kWave / G);
                float r[OUT];
                fold_scatter<VEC, G>(acc[0], r);
                if (c0 + sub * VEC < p.L) {
                    const int o = c0 + sub * VEC + slot * OUT;
#pragma unroll
                    for (int i = 0; i < OUT; i++) r[i] *= sr;
                    if (single) store_out<OUT>(p, (size_t)row * p.L + o, r);
                    else store_row_streaming<OUT>(dst + o, r);
                }
                continue;
            }
            fold_slots<VEC, G, KT>(acc);
            if (slot == 0) {
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    const int o = c0 + (t * G + sub) * VEC;
                    if (o < p.L) {
                        float r[VEC];
#pragma unroll
                        for (int i = 0; i < VEC; i++) r[i] = acc[t][i] * sr;
                        if (single) store_out<VEC>(p, (size_t)row * p.L + o, r);
                        else store_row_streaming<VEC>(dst + o, r);
                    }
                }
            }
        }
    }
}

// Items of the plan in band order, IPW per wave. The order only
// affects cache behaviour: every item writes its own row.
template <int VEC, int G, int KT, int WMODE, typename TIN, int IPW = kItemsPerWave>
__global__ __launch_bounds__(kBlock) void spmm_items_kernel(SpmmParams p) {
    static_assert(kPlanChunk <= kWave, "an item must fit one edge window");
    if (p.plan.counters->overflow) return;
    const int n_items = min(p.plan.counters->n_items, p.plan.max_items);
    const int n_groups = (n_items + IPW - 1) / IPW;
    const int stride = gridDim.x * kWavesPerBlock;
    const int wave = wave_id();
    for (int grp = blockIdx.x * kWavesPerBlock + wave; grp < n_groups; grp += stride)
        spmm_item_group<VEC, G, KT, WMODE, TIN, IPW>(p, grp * IPW,
                                                min(IPW, n_items - grp * IPW));
}

// Adds the item partials of every planned row with more than one item and
// applies the row scale: the only writer of such a row of the output. The sum is
// a fixed function of the item count (bitwise reproducible):
//  * rows of up to kReduceWaveItems items: one wave per row. The row vector is
//    spread over `lanes` lanes, the wave's 64 / lanes slots add items slot,
//    slot + slots, ... and the slot sums are folded by a fixed butterfly;
//  * longer rows: one workgroup per row, its 256 / lanes teams add items
//    team, team + teams, ...; the team sums are then added in team order.
// Blocks [0, gridDim.x / 2) take the first kind, the others the second.
// s += src[c * L] for c = first, first + step, ... < n, added in that order;
// four loads are in flight at a time.
template <int VEC>
__device__ __forceinline__ void sum_partials(float (&s)[VEC], const float *src, int L, int first,
                                             int n, int step) {
    int c = first;
    for (; c + 3 * step < n; c += 4 * step) {
        float v[4][VEC];
#pragma unroll
        for (int u = 0; u < 4; u++) RowLoad<VEC, float>::ld(src + (size_t)(c + u * step) * L, v[u]);
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int i = 0; i < VEC; i++) s[i] += v[u][i];
    }
    for (; c < n; c += step) {
        float v[VEC];
        RowLoad<VEC, float>::ld(src + (size_t)c * L, v);
#pragma unroll
        for (int i = 0; i < VEC; i++) s[i] += v[i];
    }
}

constexpr int kReduceWaveItems = 32;

template <int WMODE, int VEC>
__global__ __launch_bounds__(kBlock) void spmm_reduce_kernel(SpmmParams p) {
    __shared__ float red[kBlock * VEC];
    if (p.plan.counters->overflow) return;
    const int n_hub = min(p.plan.counters->n_rows, p.plan.max_rows);
    const int lanes_total = p.L / VEC;  // VEC divides L (host picks VEC)
    const int half = gridDim.x / 2;
    if ((int)blockIdx.x < half) {
        const int lane = lane_id();
        // lanes per row vector: the power of two >= lanes_total, at most 64
        int lanes = 1;
        while (lanes < lanes_total && lanes < kWave) lanes <<= 1;
        const int slots = kWave / lanes;
        const int slot = lane / lanes, sub = lane % lanes;
        const int stride = half * kWavesPerBlock;
        for (int h = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave; h < n_hub; h += stride) {
            const int4 r = p.plan.rows[h];
            if (r.z <= 1 || r.z > kReduceWaveItems) continue;
            const float sr = (WMODE == W_DEGPROD ? p.scale_row[r.x] : 1.0f) * p.alpha;
            for (int l0 = 0; l0 < lanes_total; l0 += lanes) {
                const bool live = l0 + sub < lanes_total;
                float s[VEC];
#pragma unroll
                for (int i = 0; i < VEC; i++) s[i] = 0.0f;
                if (live) {
                    const float *src = p.partial + (size_t)r.y * p.L + (size_t)(l0 + sub) * VEC;
                    sum_partials<VEC>(s, src, p.L, slot, r.z, slots);
                }
                for (int o = kWave / 2; o >= lanes; o >>= 1)
#pragma unroll
                    for (int i = 0; i < VEC; i++) s[i] += __shfl_xor(s[i], o, kWave);
                if (live && slot == 0) {
#pragma unroll
                    for (int i = 0; i < VEC; i++) s[i] *= sr;
                    store_out<VEC>(p, (size_t)r.x * p.L + (size_t)(l0 + sub) * VEC, s);
                }
            }
        }
        return;
    }
    for (int h = blockIdx.x - half; h < n_hub; h += gridDim.x - half) {
        const int4 r = p.plan.rows[h];
        if (r.z <= kReduceWaveItems) continue;  // short rows: the wave path; single items: done
        const float sr = (WMODE == W_DEGPROD ? p.scale_row[r.x] : 1.0f) * p.alpha;
        for (int l0 = 0; l0 < lanes_total; l0 += kBlock) {
            const int lanes = min(kBlock, lanes_total - l0);
            const int groups = kBlock / lanes;
            const int g = threadIdx.x / lanes, l = threadIdx.x % lanes;
            float s[VEC];
#pragma unroll
            for (int i = 0; i < VEC; i++) s[i] = 0.0f;
            if (g < groups) {
                const float *src = p.partial + (size_t)r.y * p.L + (size_t)(l0 + l) * VEC;
                sum_partials<VEC>(s, src, p.L, g, r.z, groups);
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < VEC; i++) red[threadIdx.x * VEC + i] = s[i];
            __syncthreads();
            if (g == 0) {
                for (int gg = 1; gg < groups; gg++)
#pragma unroll
                    for (int i = 0; i < VEC; i++) s[i] += red[(gg * lanes + l) * VEC + i];
#pragma unroll
                for (int i = 0; i < VEC; i++) s[i] *= sr;
                store_out<VEC>(p, (size_t)r.x * p.L + (size_t)(l0 + l) * VEC, s);
            }
        }
    }
}


// ---- rows of at most 4 floats (one 16-byte vector or less) ------------------------
// The generic mapping would leave 15 of 16 lanes of a slot idle. Here a lane owns
// an EDGE: the window's 64 column ids and the 64 gathered vectors come from two
// load instructions, and every row that lies inside the window is then a masked
// full-wave butterfly sum: no further memory round trip per row. Unweighted sums
// only (the grad_key gather of the attention backward).
template <int VEC>
struct TinyWindow {
    int base;  // CSR position of lane 0; -1 = nothing loaded
    float v[VEC];
};

template <int VEC>
__device__ __forceinline__ void load_tiny_window(TinyWindow<VEC> &w, const SpmmParams &p, int base,
                                                 int limit) {
    const int e = min(base + lane_id(), limit - 1);
    const int c = p.cols_are_edges ? e : (p.indices[e] & p.col_mask);
    w.base = base;
    RowLoad<VEC, float>::ld(static_cast<const float *>(p.feat) + (size_t)c * VEC, w.v);
}

// sum of the window lanes [first, first + n) in every lane
template <int VEC>
__device__ __forceinline__ void tiny_sum(float (&acc)[VEC], const TinyWindow<VEC> &w, int first,
                                         int n) {
    const int lane = lane_id();
    const bool in = lane >= first && lane < first + n;
    float t[VEC];
#pragma unroll
    for (int i = 0; i < VEC; i++) t[i] = in ? w.v[i] : 0.0f;
#pragma unroll
    for (int o = kWave / 2; o >= 1; o >>= 1)
#pragma unroll
        for (int i = 0; i < VEC; i++) t[i] += __shfl_xor(t[i], o, kWave);
#pragma unroll
    for (int i = 0; i < VEC; i++) acc[i] += t[i];
}

template <int VEC>
__device__ __forceinline__ void tiny_rows_body(const SpmmParams &p, int block) {
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.n_rows);
    const int r0 = (block * kWavesPerBlock + threadIdx.x / kWave) * rpw;
    if (r0 >= p.n_rows) return;
    const int n_here = min(rpw, p.n_rows - r0);
    const int my_ptr = p.indptr[r0 + min(lane, n_here)];
    const int limit = __shfl(my_ptr, n_here, kWave);
    TinyWindow<VEC> win;
    win.base = -1;
#pragma unroll
    for (int i = 0; i < VEC; i++) win.v[i] = 0.0f;
    for (int i = 0; i < n_here; i++) {
        const int beg = __shfl(my_ptr, i, kWave), end = __shfl(my_ptr, i + 1, kWave);
        if (end - beg >= p.plan.threshold) continue;  // a planned row: the item kernel
        float acc[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) acc[k] = 0.0f;
        for (int b = beg; b < end; b += kWave) {
            const int n = min(kWave, end - b);
            if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                load_tiny_window<VEC>(win, p, b, limit);
            tiny_sum<VEC>(acc, win, b - win.base, n);
        }
        if (lane == 0) {
#pragma unroll
            for (int k = 0; k < VEC; k++) acc[k] *= p.alpha;
            store_row<VEC>(p.out + (size_t)(r0 + i) * VEC, acc);
        }
    }
}

template <int VEC>
__global__ __launch_bounds__(kBlock) void tiny_items_kernel(SpmmParams p) {
    const int lane = lane_id();
    if (p.plan.counters->overflow) return;
    const int n_items = min(p.plan.counters->n_items, p.plan.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = p.plan.records[pos0 + min(lane, n_here - 1)];
        TinyWindow<VEC> win[kItemsPerWave];
        int n[kItemsPerWave], item[kItemsPerWave], tag[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            const int beg = __shfl(my_rec.x, j, kWave), end = __shfl(my_rec.y, j, kWave);
            item[j] = __shfl(my_rec.z, j, kWave);
            tag[j] = __shfl(my_rec.w, j, kWave);
            n[j] = j < n_here ? end - beg : 0;
            if (n[j] > 0) load_tiny_window<VEC>(win[j], p, beg, end);
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            if (n[j] <= 0) continue;
            float acc[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) acc[k] = 0.0f;
            tiny_sum<VEC>(acc, win[j], 0, n[j]);
            if (lane == 0) {
                const bool single = tag[j] < 0;
                if (single) {
#pragma unroll
                    for (int k = 0; k < VEC; k++) acc[k] *= p.alpha;
                }
                store_row<VEC>(single ? p.out + (size_t)(tag[j] & 0x7fffffff) * VEC
                                      : p.partial + (size_t)item[j] * VEC,
                               acc);
            }
        }
    }
}

// Planned rows of a segmented sum of per-edge rows (cols_are_edges): the edges of a
// row are contiguous, so no items are needed. Rows of up to kEdgeSumWave edges: one
// wave per row, lanes stride the edges, four loads in flight, one butterfly at the
// end. Longer rows: one workgroup per row, thread sums added in thread order.
// Blocks [0, gridDim.x / 2) take the first kind. Bitwise reproducible.
constexpr int kEdgeSumWave = 4096;

template <int VEC>
__global__ __launch_bounds__(kBlock) void edge_sum_long_kernel(SpmmParams p) {
    __shared__ float red[kBlock * VEC];
    if (p.plan.counters->overflow) return;
    const int n_long = min(p.plan.counters->n_rows, p.plan.max_rows);
    const float *__restrict__ feat = static_cast<const float *>(p.feat);
    const int half = gridDim.x / 2;
    if ((int)blockIdx.x < half) {
        const int lane = lane_id();
        const int stride = half * kWavesPerBlock;
        for (int i = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave; i < n_long; i += stride) {
            const int row = p.plan.rows[i].x;
            const int beg = p.indptr[row], n = p.indptr[row + 1] - beg;
            if (n > kEdgeSumWave) continue;
            float s[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) s[k] = 0.0f;
            sum_partials<VEC>(s, feat + (size_t)beg * VEC, VEC, lane, n, kWave);
#pragma unroll
            for (int o = kWave / 2; o >= 1; o >>= 1)
#pragma unroll
                for (int k = 0; k < VEC; k++) s[k] += __shfl_xor(s[k], o, kWave);
            if (lane == 0) {
#pragma unroll
                for (int k = 0; k < VEC; k++) s[k] *= p.alpha;
                store_row<VEC>(p.out + (size_t)row * VEC, s);
            }
        }
        return;
    }
    for (int i = blockIdx.x - half; i < n_long; i += gridDim.x - half) {
        const int row = p.plan.rows[i].x;
        const int beg = p.indptr[row], n = p.indptr[row + 1] - beg;
        if (n <= kEdgeSumWave) continue;
        float s[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) s[k] = 0.0f;
        sum_partials<VEC>(s, feat + (size_t)beg * VEC, VEC, threadIdx.x, n, kBlock);
        __syncthreads();  // red[] may still be read for the previous row
#pragma unroll
        for (int k = 0; k < VEC; k++) red[threadIdx.x * VEC + k] = s[k];
        __syncthreads();
        if (threadIdx.x < kWave) {
            // 64 lanes add four thread sums each in thread order, then a fixed butterfly
            float t[VEC];
#pragma unroll
            for (int k = 0; k < VEC; k++) t[k] = 0.0f;
            for (int q = 0; q < kBlock / kWave; q++)
#pragma unroll
                for (int k = 0; k < VEC; k++) t[k] += red[(threadIdx.x * (kBlock / kWave) + q) * VEC + k];
#pragma unroll
            for (int o = kWave / 2; o >= 1; o >>= 1)
#pragma unroll
                for (int k = 0; k < VEC; k++) t[k] += __shfl_xor(t[k], o, kWave);
            if (threadIdx.x == 0) {
#pragma unroll
                for (int k = 0; k < VEC; k++) t[k] *= p.alpha;
                store_row<VEC>(p.out + (size_t)row * VEC, t);
            }
        }
    }
}

// Picks the instantiation for (element type, L) and launches the row, item and reduce kernels.
// max_degree_hint < 0 means unknown; plan may be null (a temporary one is then
// built in the workspace). p.n_src and p.col_mask must be set.
int launch_spmm(SpmmParams &p, int wmode, bool bf16_in, int64_t nnz, int64_t max_degree_hint,
                const void *plan, void *workspace, size_t workspace_bytes, hipStream_t stream);
// Workspace of launch_spmm: partial rows, plus the temporary plan when none is given.
size_t spmm_workspace_bytes(int64_t nnz, int64_t L, bool with_plan);
// Both gradients of an edge-weighted product from one gather over the by-source
// structure (gat.hip), for the shapes spmm_backward_one_gather_shape accepts.
bool spmm_backward_one_gather_shape(int64_t n_heads, int64_t n_features, const float *features,
                                    const float *grad_out, const float *grad_x);
int spmm_backward_one_gather(float *grad_a, float *grad_x, const float *values,
                             const float *features, const float *grad_out,
                             const int32_t *t_indptr, const int32_t *t_rows, const int32_t *t_perm,
                             int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads,
                             int64_t n_features, int64_t max_degree_t, const void *plan_t,
                             void *workspace, size_t workspace_bytes, hipStream_t stream);
// The body of yitu_spmm_backward (spmm_bwd.hip).
int spmm_backward_run(float *grad_a, float *grad_x, const float *values, const int32_t *indptr,
                      const int32_t *indices, const float *features, const float *grad_out,
                      const int32_t *t_indptr, const int32_t *t_rows, const int32_t *t_perm,
                      int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads,
                      int64_t n_features, int64_t max_degree, int64_t max_degree_t,
                      const void *plan, const void *plan_t, void *workspace,
                      size_t workspace_bytes, bool long_rows_only, hipStream_t stream);
// w[e] = scale[indices[e] & col_mask] for every edge.
int edge_scale_fill(float *w, const int32_t *indices, const float *scale, int64_t nnz, int col_mask,
                    hipStream_t stream);
const char *last_error();
// Zero-fill by kernel (safe to record into a captured graph, unlike a memset node).
int fill_zero(float *p, int64_t n, hipStream_t stream);

}  // namespace yitu
