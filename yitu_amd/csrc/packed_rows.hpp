// Short rows in the packed layout: a lane owns an EDGE, and a wave handles every row
// that fits its 64 lanes at once.
//
// A wave owns up to 63 consecutive rows; their bounds sit one per lane. It walks them in
// chunks of whole rows that hold at most 64 edges together. Inside a chunk a lane finds
// its row by bisection over the bounds (lane shuffles), per-row maxima and sums are
// segmented scans over the lanes (an add or max with the lane 1, 2, 4, ... 32 places
// down when that lane belongs to the same row), and the row's last lane hands the total
// back. A row therefore costs no memory round trip of its own: kernels that walk their
// rows one after the other spend one to two microseconds per row on dependent loads and
// a full-wave butterfly, whatever the row's length, which bounds them on graphs whose
// rows average a handful of edges.
#pragma once
#include <cfloat>

#include "spmm_rows.hpp"

namespace yitu {

constexpr int kPackedRows = 63;  // rows of a wave: bounds [0, 63] fill the 64 lanes

// Enough waves to fill the chip several times over before a wave takes more rows.
__host__ __device__ inline int packed_rows_per_wave(int n_rows) {
    const int r = n_rows / 16384;
    return r < 1 ? 1 : (r > kPackedRows ? kPackedRows : r);
}

struct PackedChunk {
    int r0;        // first row of the wave
    int base;      // first edge of the chunk
    int n;         // edges in the chunk (1 .. 64); lane < n is live
    int pos;       // this lane's row, relative to r0
    int last;      // lane that holds the last edge of this lane's row
    unsigned same; // bit k: the lane 2^k places down is live and in the same row
};

// Inclusive segmented scan over the lanes of a chunk, then every lane takes its row's total.
template <int HV, typename Op>
__device__ __forceinline__ void seg_total(float (&v)[HV], const PackedChunk &c, Op op) {
#pragma unroll
    for (int k = 0; k < 6; k++) {
#pragma unroll
        for (int h = 0; h < HV; h++) {
            const float t = __shfl_up(v[h], 1 << k, kWave);
            if ((c.same >> k) & 1u) v[h] = op(v[h], t);
        }
    }
#pragma unroll
    for (int h = 0; h < HV; h++) v[h] = __shfl(v[h], c.last, kWave);
}

// Full-wave reductions on the data-parallel-primitive path of the vector ALU (no LDS
// round trip per step, which is what a lane shuffle costs): two quad permutes and two
// rotations inside the rows of 16 lanes leave every lane with its row's total, two row
// broadcasts carry the totals of rows 0 .. 2 into row 3, and lane 63 is read back as a
// scalar. The order of the additions is fixed.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float identity, float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(identity), __float_as_int(v),
                                                      CTRL, ROW_MASK, 0xf, false));
}

template <typename Op>
__device__ __forceinline__ float wave_reduce(float v, float identity, Op op) {
    v = op(v, dpp_move<0xb1, 0xf>(identity, v));   // quad_perm [1,0,3,2]
    v = op(v, dpp_move<0x4e, 0xf>(identity, v));   // quad_perm [2,3,0,1]
    v = op(v, dpp_move<0x124, 0xf>(identity, v));  // row_ror 4
    v = op(v, dpp_move<0x128, 0xf>(identity, v));  // row_ror 8
    v = op(v, dpp_move<0x142, 0xa>(identity, v));  // row_bcast 15 into rows 1 and 3
    v = op(v, dpp_move<0x143, 0xc>(identity, v));  // row_bcast 31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), kWave - 1));
}

template <int HV>
__device__ __forceinline__ void wave_max(float (&v)[HV]) {
#pragma unroll
    for (int h = 0; h < HV; h++)
        v[h] = wave_reduce(v[h], -FLT_MAX, [](float a, float b) { return fmaxf(a, b); });
}

template <int HV>
__device__ __forceinline__ void wave_sum(float (&v)[HV]) {
#pragma unroll
    for (int h = 0; h < HV; h++)
        v[h] = wave_reduce(v[h], 0.0f, [](float a, float b) { return a + b; });
}

// Walks the short rows of wave `wave_id`: chunk(c) for every chunk of whole rows,
// big(row, beg, end) for a row of more than 64 edges that no plan covers (a caller's
// max-degree hint that was too small), empties(r0, mask) once with the mask of the rows
// r0 + i that have no edges. Rows that the plan covers are skipped. Every call is made by
// the whole wave.
template <typename Chunk, typename Big, typename Empty>
__device__ __forceinline__ void packed_walk(const SpmmParams &sp, int R, int wave_id, Chunk chunk,
                                            Big big, Empty empty) {
    const int lane = lane_id();
    wave_id = __builtin_amdgcn_readfirstlane(wave_id);  // what follows from it stays scalar
    const long long first = (long long)wave_id * R;
    if (first >= sp.n_rows) return;
    const int r0 = (int)first;
    const int n_here = min(R, sp.n_rows - r0);
    const int my_ptr = sp.indptr[r0 + min(lane, n_here)];
    const int next_ptr = __shfl_down(my_ptr, 1, kWave);
    const bool is_row = lane < n_here;
    const int deg = is_row ? next_ptr - my_ptr : 0;
    const bool planned = deg >= sp.plan.threshold;
    const unsigned long long planned_mask = __ballot(planned);
    const unsigned long long stop =
        planned_mask | __ballot(!planned && deg > kWave) | (1ull << n_here);
    empty(r0, __ballot(is_row && deg == 0));
    int cur = 0;
    while (cur < n_here) {
        const int base = __builtin_amdgcn_readlane(my_ptr, cur);
        const bool over = is_row && lane >= cur && next_ptr - base > kWave;
        const unsigned long long m = (__ballot(over) | stop) & (~0ull << cur);
        const int r_end = __ffsll((long long)m) - 1;  // the chunk is rows [cur, r_end)
        if (r_end == cur) {
            if (!((planned_mask >> cur) & 1ull))
                big(r0 + cur, base, __builtin_amdgcn_readlane(my_ptr, cur + 1));
            cur++;
            continue;
        }
        PackedChunk c;
        c.r0 = r0;
        c.base = base;
        c.n = __builtin_amdgcn_readlane(my_ptr, r_end) - base;
        if (c.n > 0) {
            const int e = base + lane;
            int pos = cur;  // the largest row index whose first edge is <= e
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) {
                const int cand = pos + step;
                const int v = __shfl(my_ptr, min(cand, kWave - 1), kWave);
                if (cand < r_end && v <= e) pos = cand;
            }
            c.pos = pos;
            c.last = __shfl(my_ptr, pos + 1, kWave) - base - 1;
            c.same = 0;
#pragma unroll
            for (int k = 0; k < 6; k++) {
                const int up = __shfl_up(pos, 1 << k, kWave);
                if (lane < c.n && lane >= (1 << k) && up == pos) c.same |= 1u << k;
            }
            chunk(c);
        }
        cur = r_end;
    }
}

// Segmented sum of gathered edge rows of VEC <= 4 floats (unweighted; the grad_key and
// grad_query sums of the attention backward): out[row] = alpha * sum of feat[col(e)].
template <int VEC>
__global__ __launch_bounds__(kBlock) void tiny_rows_packed_kernel(SpmmParams p, int R) {
    const int lane = lane_id();
    const float *__restrict__ feat = static_cast<const float *>(p.feat);
    const auto source = [&](int e) { return p.cols_are_edges ? e : (p.indices[e] & p.col_mask); };
    packed_walk(
        p, R, blockIdx.x * kWavesPerBlock + threadIdx.x / kWave,
        [&](const PackedChunk &c) {
            float v[VEC];
            RowLoad<VEC, float>::ld(feat + (size_t)source(c.base + min(lane, c.n - 1)) * VEC, v);
            if (lane >= c.n) {
#pragma unroll
                for (int i = 0; i < VEC; i++) v[i] = 0.0f;
            }
            seg_total<VEC>(v, c, [](float a, float b) { return a + b; });
            if (lane < c.n && lane == c.last) {
#pragma unroll
                for (int i = 0; i < VEC; i++) v[i] *= p.alpha;
                store_row<VEC>(p.out + (size_t)(c.r0 + c.pos) * VEC, v);
            }
        },
        [&](int row, int beg, int end) {  // more than 64 edges and no plan
            float v[VEC];
#pragma unroll
            for (int i = 0; i < VEC; i++) v[i] = 0.0f;
            for (int e = beg + lane; e < end; e += kWave) {
                float t[VEC];
                RowLoad<VEC, float>::ld(feat + (size_t)source(e) * VEC, t);
#pragma unroll
                for (int i = 0; i < VEC; i++) v[i] += t[i];
            }
            wave_sum<VEC>(v);
            if (lane == 0) {
#pragma unroll
                for (int i = 0; i < VEC; i++) v[i] *= p.alpha;
                store_row<VEC>(p.out + (size_t)row * VEC, v);
            }
        },
        [&](int r0, unsigned long long empty) {
            if ((empty >> lane) & 1ull) {
                float z[VEC];
#pragma unroll
                for (int i = 0; i < VEC; i++) z[i] = 0.0f;
                store_row<VEC>(p.out + (size_t)(r0 + lane) * VEC, z);
            }
        });
}

}  // namespace yitu
