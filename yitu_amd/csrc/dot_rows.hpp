// Per-edge dot products grad_a[i,h] = <grad_out[row_i,h,:], feat[col_i,h,:]> of the
// multi-head SpMM backward (spmm_cuda.cu:27-32), for the rows below the plan
// threshold: shared by the SpMM backward and the horizontally fused backward.
#pragma once
#include "spmm_rows.hpp"

namespace yitu {

struct DotParams {
    SpmmParams sp;          // indptr, indices, feat, n_rows, L, F, H, col_mask, plan
    const float *grad_out;  // [n_dst, L]
    float *grad_a;          // [nnz, H]
    int lph;  // lanes per head (F / VEC) when that is a power of two <= G, else 0
    int long_rows_only;  // the rows below the plan threshold were handled by another kernel
};

// Dot products of the row's grad_out tile `gt` with the n edges in window lanes
// [first, first + n); edge k of them is CSR edge e0 + k.
template <int VEC, int G, int KT, int UNROLL = (KT >= 4 ? 2 : 4)>
__device__ __forceinline__ void dot_window(const DotParams &p, const float (&gt)[KT][VEC],
                                           const TileLanes<VEC, G, KT, W_EDGEHEAD> &tl,
                                           const EdgeWindow &win, int first, int n, int e0,
                                           int c0) {
    constexpr int SLOTS = kWave / G;
    const int lane = lane_id();
    const int slot = lane / G, sub = lane % G;
    const float *__restrict__ feat = static_cast<const float *>(p.sp.feat);
    const int L = p.sp.L, F = p.sp.F, H = p.sp.H;
    // heads present in this column tile, for the generic reduction
    const int h_lo = c0 / F;
    const int h_hi = min(H - 1, (min(L, c0 + G * VEC * KT) - 1) / F);

    for (int s0 = 0; s0 < n; s0 += SLOTS * UNROLL) {
        float v[UNROLL][KT][VEC];
        // all gathers of the group first
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int k = min(s0 + u * SLOTS + slot, n - 1);
            const int c = __shfl(win.col, first + k, kWave);
            if (s0 + u * SLOTS < n) {  // wave-uniform
#pragma unroll
                for (int t = 0; t < KT; t++)
                    RowLoad<VEC, float>::ld(feat + (size_t)c * L + tl.off[t], v[u][t]);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            if (s0 + u * SLOTS >= n) break;  // wave-uniform
            const int k = s0 + u * SLOTS + slot;
            const bool valid = k < n;
            const size_t e = (size_t)(e0 + min(k, n - 1));
            float part[KT];
#pragma unroll
            for (int t = 0; t < KT; t++) {
                float d = 0.0f;
#pragma unroll
                for (int i = 0; i < VEC; i++) d += gt[t][i] * v[u][t][i];
                part[t] = d;
            }
            if (p.lph > 0) {
                // a head is lph consecutive lanes of one tile
#pragma unroll
                for (int t = 0; t < KT; t++) {
                    float d = part[t];
                    for (int o = p.lph >> 1; o >= 1; o >>= 1) d += __shfl_xor(d, o, kWave);
                    if (valid && tl.live[t] && (sub & (p.lph - 1)) == 0)
                        p.grad_a[e * H + tl.head[t]] = d;
                }
            } else {
                // generic shapes: one masked reduction per head present in the tile
                for (int h = h_lo; h <= h_hi; h++) {
                    float d = 0.0f;
#pragma unroll
                    for (int t = 0; t < KT; t++)
                        if (tl.live[t] && tl.head[t] == h) d += part[t];
                    d = group_sum<G>(d);
                    if (valid && sub == 0) {
                        float *dst = p.grad_a + e * H + h;
                        // a head that started in an earlier column pass keeps its partial
                        if (h * F < c0)
                            *dst += d;
                        else
                            *dst = d;
                    }
                }
            }
        }
    }
}

template <int VEC, int G, int KT>
__device__ __forceinline__ void load_grad_tile(float (&gt)[KT][VEC], const DotParams &p,
                                               const TileLanes<VEC, G, KT, W_EDGEHEAD> &tl,
                                               int row) {
#pragma unroll
    for (int t = 0; t < KT; t++) {
        RowLoad<VEC, float>::ld(p.grad_out + (size_t)row * p.sp.L + tl.off[t], gt[t]);
        if (!tl.live[t])
#pragma unroll
            for (int i = 0; i < VEC; i++) gt[t][i] = 0.0f;
    }
}

// Short rows: a wave walks rows_per_wave consecutive rows through a sliding edge window.
template <int VEC, int G, int KT>
__device__ __forceinline__ void dot_rows_body(const DotParams &p, int block) {
    const int lane = lane_id();
    const int rpw = rows_per_wave(p.sp.n_rows);
    const int r0 = (block * kWavesPerBlock + wave_id()) * rpw;
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
        const int beg = __builtin_amdgcn_readlane(my_ptr, i), end = __builtin_amdgcn_readlane(my_ptr, i + 1);
        if (end == beg || end - beg >= p.sp.plan.threshold) continue;
        for (int c0 = 0; c0 < p.sp.L; c0 += G * VEC * KT) {
            const TileLanes<VEC, G, KT, W_EDGEHEAD> tl(p.sp, c0);
            float gt[KT][VEC];
            load_grad_tile<VEC, G, KT>(gt, p, tl, r0 + i);
            for (int b = beg; b < end; b += kWave) {
                const int n = min(kWave, end - b);
                if (win.base < 0 || b < win.base || b + n > win.base + kWave)
                    load_window<W_NONE>(win, p.sp, b, limit);
                dot_window<VEC, G, KT>(p, gt, tl, win, b - win.base, n, b, c0);
            }
        }
    }
}

template <int VEC, int G, int KT>
__global__ __launch_bounds__(kBlock) void dot_rows_kernel(DotParams p) {
    dot_rows_body<VEC, G, KT>(p, blockIdx.x);
}

}  // namespace yitu
