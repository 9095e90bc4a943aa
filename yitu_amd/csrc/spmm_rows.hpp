// Row-split CSR gather-accumulate, the one inner loop behind every SpMM in the
// library (GCN / GIN / SAG aggregation, multi-head edge-weighted SpMM, the
// transposed pass of its backward, and the aggregate step of the fused GAT).
//
// Mapping (wave64):
//   * one wave owns one output row; the row vector of L = H*F floats is laid
//     across G lanes x VEC elements x KT tiles, so one wave-wide load
//     instruction fetches 64/G ("slots") neighbour rows at once;
//   * column ids (and per-edge scalars) of up to 64 edges are fetched with one
//     coalesced load, then broadcast lane-to-lane, so the feature gathers of
//     one batch are independent and UNROLL of them are in flight per wave;
//   * slots are folded with a fixed butterfly and the row is written once:
//     no atomics, bitwise reproducible.
//   * rows with at least hub_threshold edges are not processed here but queued
//     (row, chunk) for the workgroup-per-chunk kernel, whose partial sums are
//     combined in chunk order by a third kernel.
#pragma once
#include "common.hpp"

namespace yitu {

enum WeightMode : int {
    W_NONE = 0,      // w = 1
    W_DEGPROD = 1,   // w = s_row * s_col            (module-1 GCN norm)
    W_EDGEHEAD = 2,  // w = values[edge, head]       (module-2 SpMM)
};

constexpr int kHubChunk = 512;      // edges per hub work item (SDDMM / GAT / dot kernels)
constexpr int kHubThreshold = 512;  // rows with >= this many edges go to the hub path there
// The SpMM splits much finer: rows with >= 64 edges become items of 64 edges
// (one wave each) that are processed in ascending order of their median source
// id, so that at any moment the whole chip gathers from one narrow band of the
// feature table and the hot sources of that band stay in every XCD's L2.
constexpr int kAggChunk = 64;
constexpr int kAggThreshold = 64;

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
    int32_t *order;         // SpMM: item ids sorted by median source id
    int max_rows;
    int max_items;
    int chunk;              // edges per item
};

struct SpmmParams {
    const int32_t *indptr;   // [n_rows + 1]
    const int32_t *indices;  // [nnz], column in the low bits selected by col_mask
    const void *feat;        // [n_src, L] fp32 or bf16
    float *out;              // [n_rows, L]
    const float *scale_row;  // W_DEGPROD: s[n_rows]; otherwise unused
    const float *scale_col;  // W_DEGPROD: s[n_src]
    const float *values;     // W_EDGEHEAD: [nnz, H]
    const int32_t *eperm;    // optional: values row of edge i is eperm[i] (transposed pass)
    int n_rows;
    int n_src;     // rows of feat (sets the width of the band-sort key)
    int L;         // floats per feature row (H * F)
    int F;         // floats per head
    int H;
    int col_mask;
    float alpha;   // output scale
    int hub_threshold;
    int xcd_remap;
    HubQueue hub;
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
    win.col = p.indices[e] & p.col_mask;
    win.w = 1.0f;
    win.vrow = 0;
    if constexpr (WMODE == W_DEGPROD) win.w = p.scale_col[win.col];
    if constexpr (WMODE == W_EDGEHEAD) win.vrow = p.eperm ? p.eperm[e] : e;
}

// One step of the edge loop: every slot of the wave picks its edge
// (window lane first + step + slot) and loads that neighbour's row tile. Slots
// whose edge lies past the n edges of the range carry weight 0 and load the
// (valid) tile of the range's last edge.
template <int VEC, int G, int KT, int WMODE, typename TIN>
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
        valid = k < n;
        const int src = first + min(k, n - 1);
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
template <int VEC, int G, int KT, int WMODE, typename TIN, int UNROLL = (KT >= 4 ? 2 : 4)>
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
            gather_step<VEC, G, KT, WMODE, TIN>(v[u], w[u], p, feat, win, first, s + u * SLOTS, n,
                                                tl.off, tl.head, tl.live);
#pragma unroll
        for (int u = 0; u < UNROLL; u++)
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < VEC; i++) acc[t][i] += w[u][t] * v[u][t][i];
    }
    // remaining steps one at a time
    for (; s < n; s += SLOTS) {
        float v[KT][VEC];
        float w[KT];
        gather_step<VEC, G, KT, WMODE, TIN>(v, w, p, feat, win, first, s, n, tl.off, tl.head,
                                            tl.live);
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int i = 0; i < VEC; i++) acc[t][i] += w[t] * v[t][i];
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

constexpr int kRowsPerWave = 16;  // consecutive rows handled by one wave of the row kernel

// Row kernel: a wave walks kRowsPerWave consecutive rows. Their bounds come from
// one coalesced indptr load, their edges from a sliding 64-edge window, so a
// short row costs one round of feature gathers and nothing else that waits on
// memory. Rows at or above the hub threshold are queued instead.
template <int VEC, int G, int KT, int WMODE, typename TIN>
__global__ __launch_bounds__(kBlock) void spmm_rows_kernel(SpmmParams p) {
    __shared__ int wave_rows[kWavesPerBlock], wave_items[kWavesPerBlock];
    __shared__ int block_first_row, block_first_item;
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    int blk = blockIdx.x;
    if (p.xcd_remap) blk = xcd_contiguous_block(blk, gridDim.x);
    const int r0 = (blk * kWavesPerBlock + wave) * kRowsPerWave;
    const int n_here = max(0, min(kRowsPerWave, p.n_rows - r0));
    const int my_ptr = n_here > 0 ? p.indptr[r0 + min(lane, n_here)] : 0;
    const int limit = __shfl(my_ptr, n_here, kWave);  // end of this wave's edges
    const int sub = lane % G;
    const int slot = lane / G;

    // ---- queue this workgroup's hub rows with ONE atomic --------------------
    // (hundreds of thousands of same-address atomics would serialise in L2)
    const int my_deg = __shfl_down(my_ptr, 1, kWave) - my_ptr;  // lane i: degree of row r0 + i
    const bool my_hub = lane < n_here && my_deg >= p.hub_threshold;
    const int my_chunks = my_hub ? (my_deg + p.hub.chunk - 1) / p.hub.chunk : 0;
    if (p.hub.counters != nullptr) {  // block-uniform: the queue exists
        // exclusive prefix sums over the (at most 16) row lanes
        int pre_rows = my_hub ? 1 : 0, pre_items = my_chunks;
#pragma unroll
        for (int o = 1; o < kRowsPerWave; o <<= 1) {
            const int a = __shfl_up(pre_rows, o, kWave), b = __shfl_up(pre_items, o, kWave);
            if (lane >= o) {
                pre_rows += a;
                pre_items += b;
            }
        }
        const int tot_rows = __shfl(pre_rows, kRowsPerWave - 1, kWave);
        const int tot_items = __shfl(pre_items, kRowsPerWave - 1, kWave);
        pre_rows -= my_hub ? 1 : 0;
        pre_items -= my_chunks;
        if (lane == 0) {
            wave_rows[wave] = tot_rows;
            wave_items[wave] = tot_items;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int br = 0, bi = 0;
            for (int w = 0; w < kWavesPerBlock; w++) {
                br += wave_rows[w];
                bi += wave_items[w];
            }
            unsigned long long old = 0;
            if (br > 0)
                old = atomicAdd(reinterpret_cast<unsigned long long *>(p.hub.counters),
                                ((unsigned long long)(unsigned)br << 32) | (unsigned)bi);
            block_first_item = (int)(old & 0xffffffffu);  // HubCounters: n_items then n_rows
            block_first_row = (int)(old >> 32);
        }
        __syncthreads();
        if (tot_rows > 0) {
            int first_row = block_first_row, first_item = block_first_item;
            for (int w = 0; w < wave; w++) {
                first_row += wave_rows[w];
                first_item += wave_items[w];
            }
            const bool fits = first_row + tot_rows <= p.hub.max_rows &&
                              first_item + tot_items <= p.hub.max_items;
            if (!fits) {
                if (lane == 0) atomicExch(&p.hub.counters->overflow, 1);
            } else {
                if (my_hub)
                    p.hub.rows[first_row + pre_rows] =
                        make_int4(r0 + lane, first_item + pre_items, my_chunks, 0);
                // the chunk items of each hub row, written by the whole wave
                unsigned long long hubs = __ballot(my_hub);
                while (hubs) {
                    const int i = __builtin_ctzll(hubs);
                    hubs &= hubs - 1;
                    const int n_c = __shfl(my_chunks, i, kWave);
                    const int it0 = first_item + __shfl(pre_items, i, kWave);
                    const int rs = first_row + __shfl(pre_rows, i, kWave);
                    for (int c = lane; c < n_c; c += kWave)
                        p.hub.items[it0 + c] = make_int4(r0 + i, c, rs, 0);
                }
            }
        }
    }
    if (n_here == 0) return;

    EdgeWindow win;
    win.base = -1;
    win.col = 0;
    win.w = 0.0f;
    win.vrow = 0;

    for (int i = 0; i < n_here; i++) {
        const int row = r0 + i;
        const int beg = __shfl(my_ptr, i, kWave);
        const int end = __shfl(my_ptr, i + 1, kWave);
        const int deg = end - beg;
        if (deg >= p.hub_threshold) continue;  // queued above; written by the hub kernels
        const float sr = (WMODE == W_DEGPROD ? p.scale_row[row] : 1.0f) * p.alpha;
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
            if (deg > 0) fold_slots<VEC, G, KT>(acc);
            if (slot == 0) {
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    const int o = c0 + (t * G + sub) * VEC;
                    if (o < p.L) {
                        float r[VEC];
#pragma unroll
                        for (int k = 0; k < VEC; k++) r[k] = acc[t][k] * sr;
                        store_row<VEC>(p.out + (size_t)row * p.L + o, r);
                    }
                }
            }
        }
    }
}

// Band-sort key of every queued item: the source id in the middle of its chunk,
// reduced to 16 bits. Slots past the item count get the largest key.
static __global__ __launch_bounds__(kBlock) void spmm_hub_keys_kernel(SpmmParams p, uint32_t *keys,
                                                                      int32_t *vals, int shift) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= p.hub.max_items) return;
    const int n_items = p.hub.counters->overflow ? 0 : min(p.hub.counters->n_items, p.hub.max_items);
    uint32_t key = 0xffffu;
    if (i < n_items) {
        const int4 it = p.hub.items[i];
        const int beg = p.indptr[it.x] + it.y * p.hub.chunk;
        const int end = min(p.indptr[it.x + 1], beg + p.hub.chunk);
        key = min(0xffffu, (uint32_t)(p.indices[(beg + end) >> 1] & p.col_mask) >> shift);
    }
    keys[i] = key;
    vals[i] = i;
}

// After the sort: position -> {first edge, end edge, item id, row}, so the item
// kernel needs one load per item to know its work.
static __global__ __launch_bounds__(kBlock) void spmm_hub_records_kernel(SpmmParams p,
                                                                         int4 *records) {
    const int pos = blockIdx.x * kBlock + threadIdx.x;
    if (pos >= p.hub.max_items) return;
    const int n_items = p.hub.counters->overflow ? 0 : min(p.hub.counters->n_items, p.hub.max_items);
    const int item = p.hub.order[pos];
    int4 rec = make_int4(0, 0, 0, 0);
    if (pos < n_items && item < n_items) {
        const int4 it = p.hub.items[item];
        const int beg = p.indptr[it.x] + it.y * p.hub.chunk;
        rec = make_int4(beg, min(p.indptr[it.x + 1], beg + p.hub.chunk), item, it.x);
    }
    records[pos] = rec;
}

constexpr int kItemsPerWave = 4;  // band-sorted items handled by one wave

// Items in band order, kItemsPerWave per wave: the records of a wave's items
// come from one load, their edge windows are all fetched before the first
// feature gather, so the only waits per item are its own gathers. The unscaled
// partial row goes to partial[item id]; the order only affects cache behaviour.
template <int VEC, int G, int KT, int WMODE, typename TIN>
__global__ __launch_bounds__(kBlock) void spmm_hub_items_kernel(SpmmParams p,
                                                                const int4 *__restrict__ records) {
    static_assert(kAggChunk <= kWave, "an item must fit one edge window");
    const int lane = lane_id();
    const int sub = lane % G;
    const int slot = lane / G;
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);
    const int n_waves = gridDim.x * kWavesPerBlock;
    for (int pos0 = (blockIdx.x * kWavesPerBlock + threadIdx.x / kWave) * kItemsPerWave;
         pos0 < n_items; pos0 += n_waves * kItemsPerWave) {
        const int n_here = min(kItemsPerWave, n_items - pos0);
        const int4 my_rec = records[pos0 + min(lane, n_here - 1)];
        EdgeWindow win[kItemsPerWave];
        int item_id[kItemsPerWave], n_edges[kItemsPerWave];
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            const int beg = __shfl(my_rec.x, j, kWave);
            const int end = __shfl(my_rec.y, j, kWave);
            item_id[j] = __shfl(my_rec.z, j, kWave);
            n_edges[j] = j < n_here ? end - beg : 0;
            if (n_edges[j] > 0) load_window<WMODE>(win[j], p, beg, end);
        }
#pragma unroll
        for (int j = 0; j < kItemsPerWave; j++) {
            if (n_edges[j] <= 0) continue;
            for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
                const TileLanes<VEC, G, KT, WMODE> tl(p, c0);
                float acc[KT][VEC];
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < VEC; i++) acc[t][i] = 0.0f;
                accumulate_window<VEC, G, KT, WMODE, TIN>(acc, p, win[j], 0, n_edges[j], tl);
                fold_slots<VEC, G, KT>(acc);
                if (slot == 0) {
#pragma unroll
                    for (int t = 0; t < KT; t++) {
                        const int o = c0 + (t * G + sub) * VEC;
                        if (o < p.L)
                            store_row<VEC>(p.hub.partial + (size_t)item_id[j] * p.L + o, acc[t]);
                    }
                }
            }
        }
    }
}

// Adds the chunk partials of every queued row and applies the row scale: the
// only writer of a hub row of the output. The 256 threads form `groups` teams of
// `lanes` threads; team g adds chunks g, g + groups, ... and the team sums are
// then added in team order, so the result is a fixed function of the chunk count.
template <int WMODE, int VEC>
__global__ __launch_bounds__(kBlock) void spmm_hub_reduce_kernel(SpmmParams p) {
    __shared__ float red[kBlock * VEC];
    if (p.hub.counters->overflow) return;
    const int n_hub = min(p.hub.counters->n_rows, p.hub.max_rows);
    const int lanes_total = p.L / VEC;  // VEC divides L (host picks VEC)
    for (int h = blockIdx.x; h < n_hub; h += gridDim.x) {
        const int4 r = p.hub.rows[h];
        const float sr = (WMODE == W_DEGPROD ? p.scale_row[r.x] : 1.0f) * p.alpha;
        for (int l0 = 0; l0 < lanes_total; l0 += kBlock) {
            const int lanes = min(kBlock, lanes_total - l0);
            const int groups = kBlock / lanes;
            const int g = threadIdx.x / lanes, l = threadIdx.x % lanes;
            float s[VEC];
#pragma unroll
            for (int i = 0; i < VEC; i++) s[i] = 0.0f;
            if (g < groups) {
                for (int c = g; c < r.z; c += groups) {
                    float v[VEC];
                    RowLoad<VEC, float>::ld(
                        p.hub.partial + (size_t)(r.y + c) * p.L + (size_t)(l0 + l) * VEC, v);
#pragma unroll
                    for (int i = 0; i < VEC; i++) s[i] += v[i];
                }
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
                store_row<VEC>(p.out + (size_t)r.x * p.L + (size_t)(l0 + l) * VEC, s);
            }
        }
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

// Host side: carve the queue out of a caller-provided workspace.
size_t hub_workspace_bytes(int64_t nnz, int64_t L);
int hub512_queue_init(HubQueue &q, void *workspace, size_t workspace_bytes, int64_t nnz);

// Picks the instantiation for (element type, L) and launches the 1 + 3 kernels.
// max_degree_hint < 0 means unknown.
int launch_spmm(SpmmParams &p, int wmode, bool bf16_in, int64_t nnz, int64_t max_degree_hint,
                void *workspace, size_t workspace_bytes, hipStream_t stream);
const char *last_error();
// Zero-fill by kernel (safe to record into a captured graph, unlike a memset node).
int fill_zero(float *p, int64_t n, hipStream_t stream);

}  // namespace yitu
