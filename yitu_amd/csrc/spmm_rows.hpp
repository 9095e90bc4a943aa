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

constexpr int kHubChunk = 512;      // edges per hub work item
constexpr int kHubThreshold = 512;  // rows with >= this many edges go to the hub path

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
    const int n_chunks = (deg + kHubChunk - 1) / kHubChunk;
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

// One step of the edge loop: every slot of the wave picks its edge (step + slot)
// out of the batch held one-per-lane in my_col / my_w / my_vrow and loads that
// neighbour's row tile. Lanes whose edge lies past the batch load the (valid)
// clamped column of the last edge with weight 0.
template <int VEC, int G, int KT, int WMODE, typename TIN>
__device__ __forceinline__ void gather_step(float (&v)[KT][VEC], float (&w)[KT],
                                            const SpmmParams &p, const TIN *__restrict__ feat,
                                            int my_col, float my_w, int my_vrow, int step, int n,
                                            const int (&off)[KT], const int (&head)[KT],
                                            const bool (&live)[KT]) {
    constexpr int SLOTS = kWave / G;
    int c, vrow = 0;
    float ws = 0.0f;
    bool valid = true;
    if constexpr (SLOTS == 1) {
        // the edge is the same for the whole wave: scalar broadcast
        c = __builtin_amdgcn_readlane(my_col, step);
        if constexpr (WMODE == W_EDGEHEAD)
            vrow = __builtin_amdgcn_readlane(my_vrow, step);
        else
            ws = __builtin_bit_cast(float,
                                    __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_w), step));
    } else {
        const int src = step + lane_id() / G;  // < 64: steps advance in multiples of SLOTS
        valid = src < n;
        c = __shfl(my_col, src, kWave);
        if constexpr (WMODE == W_EDGEHEAD)
            vrow = __shfl(my_vrow, src, kWave);
        else
            ws = __shfl(my_w, src, kWave);
    }
#pragma unroll
    for (int t = 0; t < KT; t++) {
        if constexpr (WMODE == W_EDGEHEAD)
            w[t] = (valid && live[t]) ? p.values[(size_t)vrow * p.H + head[t]] : 0.0f;
        else
            w[t] = live[t] ? ws : 0.0f;
        RowLoad<VEC, TIN>::ld(feat + (size_t)c * p.L + off[t], v[t]);
    }
}

// Accumulates edges [e_beg, e_end) of one row into acc for the column tile
// starting at element c0. All lanes of the wave must call this together.
template <int VEC, int G, int KT, int WMODE, typename TIN, int UNROLL = (KT >= 4 ? 2 : 4)>
__device__ __forceinline__ void accumulate_edges(float (&acc)[KT][VEC], const SpmmParams &p,
                                                 int e_beg, int e_end, int c0) {
    constexpr int SLOTS = kWave / G;
    const int lane = lane_id();
    const int sub = lane % G;
    const TIN *__restrict__ feat = static_cast<const TIN *>(p.feat);

    int off[KT];
    int head[KT];
    bool live[KT];
#pragma unroll
    for (int t = 0; t < KT; t++) {
        off[t] = c0 + (t * G + sub) * VEC;
        live[t] = off[t] < p.L;
        if (!live[t]) off[t] = 0;  // keep the address valid; the weight is forced to 0
        head[t] = WMODE == W_EDGEHEAD ? off[t] / p.F : 0;
    }

    for (int base = e_beg; base < e_end; base += kWave) {
        const int n = min(kWave, e_end - base);
        const int my_e = base + min(lane, n - 1);
        const int my_col = p.indices[my_e] & p.col_mask;
        float my_w = 0.0f;
        int my_vrow = 0;
        if constexpr (WMODE == W_DEGPROD) {
            if (lane < n) my_w = p.scale_col[my_col];
        } else if constexpr (WMODE == W_NONE) {
            if (lane < n) my_w = 1.0f;
        } else {
            my_vrow = p.eperm ? p.eperm[my_e] : my_e;
        }

        // full groups of UNROLL steps: all gathers of a group are issued before any FMA
        int s = 0;
        for (; s + SLOTS * UNROLL <= n; s += SLOTS * UNROLL) {
            float v[UNROLL][KT][VEC];
            float w[UNROLL][KT];
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
                gather_step<VEC, G, KT, WMODE, TIN>(v[u], w[u], p, feat, my_col, my_w, my_vrow,
                                                    s + u * SLOTS, n, off, head, live);
#pragma unroll
            for (int u = 0; u < UNROLL; u++)
#pragma unroll
                for (int t = 0; t < KT; t++)
#pragma unroll
                    for (int i = 0; i < VEC; i++) acc[t][i] += w[u][t] * v[u][t][i];
        }
        // remaining steps one at a time; lanes past the end carry weight 0
        for (; s < n; s += SLOTS) {
            float v[KT][VEC];
            float w[KT];
            gather_step<VEC, G, KT, WMODE, TIN>(v, w, p, feat, my_col, my_w, my_vrow, s, n, off,
                                                head, live);
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < VEC; i++) acc[t][i] += w[t] * v[t][i];
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

template <int VEC, int G, int KT, int WMODE, typename TIN>
__global__ __launch_bounds__(kBlock) void spmm_rows_kernel(SpmmParams p) {
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    int blk = blockIdx.x;
    if (p.xcd_remap) blk = xcd_contiguous_block(blk, gridDim.x);
    const int row = blk * kWavesPerBlock + wave;
    if (row >= p.n_rows) return;

    const int beg = p.indptr[row];
    const int end = p.indptr[row + 1];
    const int deg = end - beg;

    if (deg >= p.hub_threshold) {
        // queue the row for the chunked kernels; nothing is written here
        queue_hub_row(p.hub, row, deg);
        return;
    }

    const int sub = lane % G;
    const int slot = lane / G;
    const float sr = (WMODE == W_DEGPROD ? p.scale_row[row] : 1.0f) * p.alpha;

    for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
        float acc[KT][VEC];
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int i = 0; i < VEC; i++) acc[t][i] = 0.0f;

        if (deg > 0) {
            accumulate_edges<VEC, G, KT, WMODE, TIN>(acc, p, beg, end, c0);
            fold_slots<VEC, G, KT>(acc);
        }
        if (slot == 0) {
#pragma unroll
            for (int t = 0; t < KT; t++) {
                const int o = c0 + (t * G + sub) * VEC;
                if (o < p.L) {
                    float r[VEC];
#pragma unroll
                    for (int i = 0; i < VEC; i++) r[i] = acc[t][i] * sr;
                    store_row<VEC>(p.out + (size_t)row * p.L + o, r);
                }
            }
        }
    }
}

// One workgroup per (hub row, chunk of kHubChunk edges): each of the 4 waves
// takes a contiguous quarter of the chunk, the four partial rows are added in
// wave order through LDS and the unscaled sum goes to partial[item].
template <int VEC, int G, int KT, int WMODE, typename TIN>
__global__ __launch_bounds__(kBlock) void spmm_hub_items_kernel(SpmmParams p) {
    __shared__ float red[kWavesPerBlock][G * VEC * KT];
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int sub = lane % G;
    const int slot = lane / G;
    if (p.hub.counters->overflow) return;
    const int n_items = min(p.hub.counters->n_items, p.hub.max_items);

    for (int item = blockIdx.x; item < n_items; item += gridDim.x) {
        const int4 it = p.hub.items[item];
        const int row = it.x;
        const int beg = p.indptr[row] + it.y * kHubChunk;
        const int end = min(p.indptr[row + 1], beg + kHubChunk);
        constexpr int kPerWave = kHubChunk / kWavesPerBlock;
        const int wbeg = min(end, beg + wave * kPerWave);
        const int wend = min(end, wbeg + kPerWave);

        for (int c0 = 0; c0 < p.L; c0 += G * VEC * KT) {
            float acc[KT][VEC];
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < VEC; i++) acc[t][i] = 0.0f;
            if (wend > wbeg) {
                accumulate_edges<VEC, G, KT, WMODE, TIN>(acc, p, wbeg, wend, c0);
                fold_slots<VEC, G, KT>(acc);
            }
            __syncthreads();  // previous tile's readers are done with red[]
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

// Adds the chunk partials of every queued row in chunk order and applies the
// row scale: the only writer of a hub row of the output.
template <int WMODE>
__global__ __launch_bounds__(kBlock) void spmm_hub_reduce_kernel(SpmmParams p) {
    if (p.hub.counters->overflow) return;
    const int n_hub = min(p.hub.counters->n_rows, p.hub.max_rows);
    for (int h = blockIdx.x; h < n_hub; h += gridDim.x) {
        const int4 r = p.hub.rows[h];
        const float sr = (WMODE == W_DEGPROD ? p.scale_row[r.x] : 1.0f) * p.alpha;
        for (int e = threadIdx.x; e < p.L; e += kBlock) {
            float s = 0.0f;
            for (int c = 0; c < r.z; c++) s += p.hub.partial[(size_t)(r.y + c) * p.L + e];
            p.out[(size_t)r.x * p.L + e] = s * sr;
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
int hub_queue_init(HubQueue &q, void *workspace, size_t workspace_bytes, int64_t nnz, int64_t L);

// Picks the instantiation for (element type, L) and launches the 1 + 3 kernels.
// max_degree_hint < 0 means unknown.
int launch_spmm(SpmmParams &p, int wmode, bool bf16_in, int64_t nnz, int64_t max_degree_hint,
                void *workspace, size_t workspace_bytes, hipStream_t stream);
const char *last_error();
// Zero-fill by kernel (safe to record into a captured graph, unlike a memset node).
int fill_zero(float *p, int64_t n, hipStream_t stream);

}  // namespace yitu
