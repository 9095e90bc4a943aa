// Temporal neighbour attention (YiTu_GNN/YiTu_T/layers.py:75-142, the non-combined
// branches) as a handful of launches around three dense products.
//
// The layer is  out = LayerNorm(ReLU(W_out [agg | h_root] + b_out))  with
//   agg[r] = sum_e softmax_r(LeakyReLU_0.2(<Q[r], K[e]>)) V[e]   per head,
//   Q = W_q [h_root | cos(b_t)] + b_q,   K, V = W_{k,v} [h_nbr | f | cos(w_t dt + b_t)] + b_{k,v}.
// Written with torch ops it is some forty launches of a few microseconds each on a
// batch of 2,048 roots x 20 neighbours, and the host cannot issue them as fast as the
// GPU runs them. Here:
//  * tattn_prepare_kernel builds the inputs of the three products in one pass: the
//    concatenations, the time encoding, and every weight matrix with its bias as one
//    more column against a column of ones in the input, so the products carry the
//    biases and their transposed forms give the bias gradients for nothing;
//  * tattn_forward_kernel: one wave per root, dot + LeakyReLU + softmax + weighted sum
//    in registers, online over chunks of 64 neighbours, written straight into the
//    input of the output product;
//  * relu_layernorm kernels; tattn_backward_kernel (softmax, LeakyReLU and both dot
//    gradients per root); tattn_finalize_kernel (feature gradients and the time
//    encoder's frequency / phase gradients); every column sum in two stages with a
//    fixed order, so results are bitwise reproducible and the step can be captured.
// All augmented matrices share one row length LD (a multiple of 4, column LD-1 =
// ones / bias, columns between the payload and LD-1 zero), so that products of
// different height go into one grouped launch.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../../include/yitu_hip.h"
#include "common.hpp"

namespace yitu {

namespace {

constexpr int kTattnMaxOut = 256;            // dim_out (and dim_time) <= 4 elements per lane
constexpr int kT = kTattnMaxOut / kWave;
constexpr int kTattnMaxHeads = 8;
constexpr int kEdgesInFlight = 4;            // neighbour rows a wave requests at a time
constexpr int kRowsPerWaveReduce = 8;        // rows a wave folds before the per-workgroup partial

struct TattnDims {
    int n_dst, n_edges;
    int Dn, De, Dt;  // node / edge / time feature widths
    int O, H;        // dim_out, heads
    int LD;          // row length of every augmented matrix
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}

// The time encoder's argument, rounded like a Linear(1, dim) evaluates it: the product
// first, then the bias. A fused multiply-add differs by up to an ulp of dt * w, which at
// dt = 10^6 is 0.06 radians; hipcc contracts a * b + c by default (also when written
// with __fmul_rn / __fadd_rn, which are plain operators here), hence the pragma.
__device__ __forceinline__ float time_arg(float dt, float w, float b) {
#pragma clang fp contract(off)
    const float product = dt * w;
    return product + b;
}

struct PrepareArgs {
    float *x_kv, *x_q, *x_r, *w_kv, *w_q2, *w_r;
    const float *h, *f, *dt, *time_w, *time_b;
    const float *wq, *bq, *wk, *bk, *wv, *bv, *wo, *bo;
};

// One wave per row of: x_kv [E], x_q [B], x_r [B] (columns O.. only; the attention
// writes 0..O-1), w_kv [2 O], w_q2 [2 O] (rows O.. zero), w_r [O].
__global__ __launch_bounds__(kBlock) void tattn_prepare_kernel(TattnDims d, PrepareArgs a) {
    const int lane = lane_id();
    const int64_t row = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int E = d.n_edges, B = d.n_dst, O = d.O, LD = d.LD;
    const int Dkv = d.Dn + d.De + d.Dt, Dq = d.Dn + d.Dt, Dr = O + d.Dn;
    int64_t r = row;
    if (r < E) {
        const float t = a.dt[r];
        float *out = a.x_kv + r * LD;
        for (int c = lane; c < LD; c += kWave) {
            float v = c == LD - 1 ? 1.0f : 0.0f;
            if (c < d.Dn) v = a.h[(B + r) * d.Dn + c];
            else if (c < d.Dn + d.De) v = a.f[r * d.De + (c - d.Dn)];
            else if (c < Dkv) v = cosf(time_arg(t, a.time_w[c - d.Dn - d.De], a.time_b[c - d.Dn - d.De]));
            out[c] = v;
        }
        return;
    }
    r -= E;
    if (r < B) {
        float *out = a.x_q + r * LD;
        for (int c = lane; c < LD; c += kWave) {
            float v = c == LD - 1 ? 1.0f : 0.0f;
            if (c < d.Dn) v = a.h[r * d.Dn + c];
            else if (c < Dq) v = cosf(a.time_b[c - d.Dn]);
            out[c] = v;
        }
        return;
    }
    r -= B;
    if (r < B) {
        float *out = a.x_r + r * LD;
        for (int c = O + lane; c < LD; c += kWave) {
            float v = c == LD - 1 ? 1.0f : 0.0f;
            if (c < Dr) v = a.h[r * d.Dn + (c - O)];
            out[c] = v;
        }
        return;
    }
    r -= B;
    if (r < 2 * O) {
        const bool is_k = r < O;
        const float *w = (is_k ? a.wk : a.wv) + (is_k ? r : r - O) * Dkv;
        const float bias = is_k ? a.bk[r] : a.bv[r - O];
        float *out = a.w_kv + r * LD;
        for (int c = lane; c < LD; c += kWave)
            out[c] = c < Dkv ? w[c] : (c == LD - 1 ? bias : 0.0f);
        return;
    }
    r -= 2 * O;
    if (r < 2 * O) {
        float *out = a.w_q2 + r * LD;
        for (int c = lane; c < LD; c += kWave) {
            float v = 0.0f;
            if (r < O) v = c < Dq ? a.wq[r * Dq + c] : (c == LD - 1 ? a.bq[r] : 0.0f);
            out[c] = v;
        }
        return;
    }
    r -= 2 * O;
    if (r < O) {
        float *out = a.w_r + r * LD;
        for (int c = lane; c < LD; c += kWave)
            out[c] = c < Dr ? a.wo[r * Dr + c] : (c == LD - 1 ? a.bo[r] : 0.0f);
    }
}

// One wave per root. Lane l holds elements l, l + 64, ... of the O-wide rows; element i
// belongs to head i / D. Neighbours go through in chunks of 64: lane j of a chunk keeps
// the logits of its j-th edge, running (max, sum) per head are rescaled between chunks.
// attn [E, H] receives the probabilities, x_r[r, 0..O) the aggregate (zero for a root
// without neighbours).
__global__ __launch_bounds__(kBlock) void tattn_forward_kernel(
    TattnDims d, float *__restrict__ x_r, float *__restrict__ attn, const float *__restrict__ q2,
    const float *__restrict__ kv, const int32_t *__restrict__ indptr) {
    const int lane = lane_id();
    const int r = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (r >= d.n_dst) return;
    const int O = d.O, H = d.H, D = O / H;
    const int beg = indptr[r], end = indptr[r + 1];
    float q[kT], acc[kT];
    int head[kT];
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        q[t] = i < O ? q2[(int64_t)r * 2 * O + i] : 0.0f;
        head[t] = i < O ? i / D : -1;
        acc[t] = 0.0f;
    }
    float run_max[kTattnMaxHeads], run_sum[kTattnMaxHeads];
#pragma unroll
    for (int h = 0; h < kTattnMaxHeads; h++) {
        run_max[h] = -INFINITY;
        run_sum[h] = 0.0f;
    }
    for (int c0 = beg; c0 < end; c0 += kWave) {
        const int n = min(kWave, end - c0);
        float mine[kTattnMaxHeads];  // logits of edge c0 + lane
#pragma unroll
        for (int h = 0; h < kTattnMaxHeads; h++) mine[h] = -INFINITY;
        for (int j = 0; j < n; j += kEdgesInFlight) {
            // the rows of several edges are requested before the first reduction waits
            float prod[kEdgesInFlight][kT];
#pragma unroll
            for (int u = 0; u < kEdgesInFlight; u++) {
                const float *krow = kv + (int64_t)(c0 + min(j + u, n - 1)) * 2 * O;
#pragma unroll
                for (int t = 0; t < kT; t++) {
                    const int i = lane + t * kWave;
                    prod[u][t] = i < O ? q[t] * krow[i] : 0.0f;
                }
            }
#pragma unroll
            for (int h = 0; h < kTattnMaxHeads; h++) {
                if (h < H) {
#pragma unroll
                    for (int u = 0; u < kEdgesInFlight; u++) {
                        float part = 0.0f;
#pragma unroll
                        for (int t = 0; t < kT; t++) part += head[t] == h ? prod[u][t] : 0.0f;
                        float l = wave_sum(part);
                        l = l > 0.0f ? l : 0.2f * l;
                        if (j + u < n && lane == j + u) mine[h] = l;
                    }
                }
            }
        }
        float p[kTattnMaxHeads];
#pragma unroll
        for (int h = 0; h < kTattnMaxHeads; h++) {
            p[h] = 0.0f;
            if (h < H) {
                const float m_new = fmaxf(run_max[h], wave_max(mine[h]));
                const float rescale = expf(run_max[h] - m_new);  // first chunk: exp(-inf) = 0
                p[h] = lane < n ? expf(mine[h] - m_new) : 0.0f;
                run_sum[h] = run_sum[h] * rescale + wave_sum(p[h]);
                run_max[h] = m_new;
#pragma unroll
                for (int t = 0; t < kT; t++)
                    if (head[t] == h) acc[t] *= rescale;
                // logits are parked in attn; every lane rereads only what it wrote itself
                if (lane < n) attn[(int64_t)(c0 + lane) * H + h] = mine[h];
            }
        }
        for (int j = 0; j < n; j += kEdgesInFlight) {
            float v[kEdgesInFlight][kT];
#pragma unroll
            for (int u = 0; u < kEdgesInFlight; u++) {
                const float *vrow = kv + (int64_t)(c0 + min(j + u, n - 1)) * 2 * O + O;
#pragma unroll
                for (int t = 0; t < kT; t++) {
                    const int i = lane + t * kWave;
                    v[u][t] = i < O ? vrow[i] : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < kEdgesInFlight; u++) {
#pragma unroll
                for (int h = 0; h < kTattnMaxHeads; h++) {
                    if (h < H) {
                        const float pj = j + u < n ? __shfl(p[h], (j + u) & (kWave - 1), kWave) : 0.0f;
#pragma unroll
                        for (int t = 0; t < kT; t++)
                            if (head[t] == h) acc[t] += pj * v[u][t];
                    }
                }
            }
        }
    }
    for (int c0 = beg; c0 < end; c0 += kWave) {
        const int e = c0 + lane;
        if (e < end) {
#pragma unroll
            for (int h = 0; h < kTattnMaxHeads; h++)
                if (h < H) attn[(int64_t)e * H + h] = expf(attn[(int64_t)e * H + h] - run_max[h]) / run_sum[h];
        }
    }
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        if (i < O) {
            float s = 1.0f;
#pragma unroll
            for (int h = 0; h < kTattnMaxHeads; h++)
                if (head[t] == h) s = run_sum[h];
            x_r[(int64_t)r * d.LD + i] = end > beg ? acc[t] / s : 0.0f;
        }
    }
}

// One wave per root: from d_agg (columns 0..O-1 of dx_r) to dq2 [B, 2 O] (columns
// 0..O-1) and dkv [E, 2 O]. Phase A finds d_attn and the sign of the raw logit per edge
// and head (parked in `scratch` [E, H, 2], each lane rereading its own words) and the
// softmax row sums; phase B writes the three gradients.
__global__ __launch_bounds__(kBlock) void tattn_backward_kernel(
    TattnDims d, float *__restrict__ dq2, float *__restrict__ dkv, float *__restrict__ scratch,
    const float *__restrict__ dx_r, const float *__restrict__ q2, const float *__restrict__ kv,
    const float *__restrict__ attn, const int32_t *__restrict__ indptr) {
    const int lane = lane_id();
    const int r = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (r >= d.n_dst) return;
    const int O = d.O, H = d.H, D = O / H;
    const int beg = indptr[r], end = indptr[r + 1];
    float q[kT], g[kT], dq[kT];
    int head[kT];
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        q[t] = i < O ? q2[(int64_t)r * 2 * O + i] : 0.0f;
        g[t] = i < O ? dx_r[(int64_t)r * d.LD + i] : 0.0f;
        head[t] = i < O ? i / D : -1;
        dq[t] = 0.0f;
    }
    float row_s[kTattnMaxHeads];
#pragma unroll
    for (int h = 0; h < kTattnMaxHeads; h++) row_s[h] = 0.0f;
    for (int c0 = beg; c0 < end; c0 += kWave) {
        const int n = min(kWave, end - c0);
        float d_att[kTattnMaxHeads], slope[kTattnMaxHeads];
#pragma unroll
        for (int h = 0; h < kTattnMaxHeads; h++) d_att[h] = slope[h] = 0.0f;
        for (int j = 0; j < n; j += kEdgesInFlight) {
            float qk[kEdgesInFlight][kT], gv[kEdgesInFlight][kT];
#pragma unroll
            for (int u = 0; u < kEdgesInFlight; u++) {
                const float *row = kv + (int64_t)(c0 + min(j + u, n - 1)) * 2 * O;
#pragma unroll
                for (int t = 0; t < kT; t++) {
                    const int i = lane + t * kWave;
                    qk[u][t] = i < O ? q[t] * row[i] : 0.0f;
                    gv[u][t] = i < O ? g[t] * row[O + i] : 0.0f;
                }
            }
#pragma unroll
            for (int h = 0; h < kTattnMaxHeads; h++) {
                if (h < H) {
#pragma unroll
                    for (int u = 0; u < kEdgesInFlight; u++) {
                        float a = 0.0f, b = 0.0f;
#pragma unroll
                        for (int t = 0; t < kT; t++) {
                            a += head[t] == h ? qk[u][t] : 0.0f;
                            b += head[t] == h ? gv[u][t] : 0.0f;
                        }
                        a = wave_sum(a);
                        b = wave_sum(b);
                        if (j + u < n && lane == j + u) {
                            slope[h] = a > 0.0f ? 1.0f : 0.2f;
                            d_att[h] = b;
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int h = 0; h < kTattnMaxHeads; h++) {
            if (h < H) {
                const int64_t e = c0 + lane;
                const float a = lane < n ? attn[e * H + h] : 0.0f;
                row_s[h] += wave_sum(a * d_att[h]);
                if (lane < n) {
                    scratch[(e * H + h) * 2] = d_att[h];
                    scratch[(e * H + h) * 2 + 1] = slope[h];
                }
            }
        }
    }
    for (int c0 = beg; c0 < end; c0 += kWave) {
        const int n = min(kWave, end - c0);
        float a[kTattnMaxHeads], dl[kTattnMaxHeads];
#pragma unroll
        for (int h = 0; h < kTattnMaxHeads; h++) {
            a[h] = dl[h] = 0.0f;
            if (h < H && lane < n) {
                const int64_t e = c0 + lane;
                a[h] = attn[e * H + h];
                dl[h] = a[h] * (scratch[(e * H + h) * 2] - row_s[h]) * scratch[(e * H + h) * 2 + 1];
            }
        }
#pragma unroll 2
        for (int j = 0; j < n; j++) {
            const float *row = kv + (int64_t)(c0 + j) * 2 * O;
            float *drow = dkv + (int64_t)(c0 + j) * 2 * O;
            // broadcasts with every lane active; the selection per element comes after
            float a_j[kTattnMaxHeads], dl_j[kTattnMaxHeads];
#pragma unroll
            for (int h = 0; h < kTattnMaxHeads; h++) {
                a_j[h] = dl_j[h] = 0.0f;
                if (h < H) {
                    a_j[h] = __shfl(a[h], j, kWave);
                    dl_j[h] = __shfl(dl[h], j, kWave);
                }
            }
#pragma unroll
            for (int t = 0; t < kT; t++) {
                const int i = lane + t * kWave;
                if (i < O) {
                    float aj = 0.0f, dlj = 0.0f;
#pragma unroll
                    for (int h = 0; h < kTattnMaxHeads; h++) {
                        if (head[t] == h) {
                            aj = a_j[h];
                            dlj = dl_j[h];
                        }
                    }
                    dq[t] += dlj * row[i];
                    drow[i] = dlj * q[t];
                    drow[O + i] = aj * g[t];
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        if (i < O) dq2[(int64_t)r * 2 * O + i] = dq[t];
    }
}

// out = LayerNorm(ReLU(pre)) per row, biased variance, like torch.nn.LayerNorm.
__global__ __launch_bounds__(kBlock) void relu_layernorm_fwd_kernel(
    float *__restrict__ out, const float *__restrict__ pre, const float *__restrict__ gamma,
    const float *__restrict__ beta, int n, int O, float eps) {
    const int lane = lane_id();
    const int r = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (r >= n) return;
    float a[kT], s = 0.0f;
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        a[t] = i < O ? fmaxf(pre[(int64_t)r * O + i], 0.0f) : 0.0f;
        s += a[t];
    }
    const float mean = wave_sum(s) / O;
    float v = 0.0f;
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        const float c = i < O ? a[t] - mean : 0.0f;
        v += c * c;
    }
    const float rstd = rsqrtf(wave_sum(v) / O + eps);
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        if (i < O) out[(int64_t)r * O + i] = (a[t] - mean) * rstd * gamma[i] + beta[i];
    }
}

// d_pre (row stride ld) and, per workgroup, the partial column sums of g * xhat (gamma's
// gradient) and of g (beta's): partial [n_blocks, 2 O].
__global__ __launch_bounds__(kBlock) void relu_layernorm_bwd_kernel(
    float *__restrict__ d_pre, float *__restrict__ partial, const float *__restrict__ g,
    const float *__restrict__ pre, const float *__restrict__ gamma, int n, int O, int ld,
    float eps) {
    __shared__ float fold[kWavesPerBlock][2][kTattnMaxOut];
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int r0 = (blockIdx.x * kWavesPerBlock + wave) * kRowsPerWaveReduce;
    float dgam[kT], dbet[kT];
#pragma unroll
    for (int t = 0; t < kT; t++) dgam[t] = dbet[t] = 0.0f;
    for (int r = r0; r < min(n, r0 + kRowsPerWaveReduce); r++) {
        float a[kT], gy[kT], gr[kT], s = 0.0f;
        bool pos[kT];
#pragma unroll
        for (int t = 0; t < kT; t++) {
            const int i = lane + t * kWave;
            const float p = i < O ? pre[(int64_t)r * O + i] : 0.0f;
            pos[t] = p > 0.0f;
            a[t] = fmaxf(p, 0.0f);
            gr[t] = i < O ? g[(int64_t)r * O + i] : 0.0f;
            gy[t] = i < O ? gr[t] * gamma[i] : 0.0f;
            s += a[t];
        }
        const float mean = wave_sum(s) / O;
        float v = 0.0f;
#pragma unroll
        for (int t = 0; t < kT; t++) {
            const int i = lane + t * kWave;
            const float c = i < O ? a[t] - mean : 0.0f;
            v += c * c;
        }
        const float rstd = rsqrtf(wave_sum(v) / O + eps);
        float m1 = 0.0f, m2 = 0.0f;
        float xh[kT];
#pragma unroll
        for (int t = 0; t < kT; t++) {
            const int i = lane + t * kWave;
            xh[t] = i < O ? (a[t] - mean) * rstd : 0.0f;
            m1 += gy[t];
            m2 += gy[t] * xh[t];
        }
        m1 = wave_sum(m1) / O;
        m2 = wave_sum(m2) / O;
#pragma unroll
        for (int t = 0; t < kT; t++) {
            const int i = lane + t * kWave;
            if (i < O) {
                const float da = rstd * (gy[t] - m1 - xh[t] * m2);
                d_pre[(int64_t)r * ld + i] = pos[t] ? da : 0.0f;
                dgam[t] += gr[t] * xh[t];
                dbet[t] += gr[t];
            }
        }
    }
#pragma unroll
    for (int t = 0; t < kT; t++) {
        fold[wave][0][lane + t * kWave] = dgam[t];
        fold[wave][1][lane + t * kWave] = dbet[t];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * O; i += kBlock) {
        const int which = i / O, c = i % O;
        float s = 0.0f;
        for (int w = 0; w < kWavesPerBlock; w++) s += fold[w][which][c];
        partial[(int64_t)blockIdx.x * 2 * O + i] = s;
    }
}

// Rows 0..E-1: edges, rows E..E+B-1: roots. Writes grad_h / grad_f and, per workgroup, the
// partial sums of the time encoder's gradients: partial [n_blocks, 2 Dt] (frequency, phase).
__global__ __launch_bounds__(kBlock) void tattn_finalize_kernel(
    TattnDims d, float *__restrict__ grad_h, float *__restrict__ grad_f,
    float *__restrict__ partial, const float *__restrict__ dx_kv, const float *__restrict__ dx_q,
    const float *__restrict__ dx_r, const float *__restrict__ dt, const float *__restrict__ time_w,
    const float *__restrict__ time_b) {
    __shared__ float fold[kWavesPerBlock][2][kTattnMaxOut];
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int E = d.n_edges, B = d.n_dst, LD = d.LD, O = d.O;
    const int64_t r0 = ((int64_t)blockIdx.x * kWavesPerBlock + wave) * kRowsPerWaveReduce;
    float dw[kT], db[kT], tw[kT], tb[kT];
#pragma unroll
    for (int t = 0; t < kT; t++) {
        const int i = lane + t * kWave;
        dw[t] = db[t] = 0.0f;
        tw[t] = i < d.Dt ? time_w[i] : 0.0f;
        tb[t] = i < d.Dt ? time_b[i] : 0.0f;
    }
    for (int64_t r = r0; r < min((int64_t)E + B, r0 + kRowsPerWaveReduce); r++) {
        if (r < E) {
            const float *row = dx_kv + r * LD;
            if (grad_h)
                for (int c = lane; c < d.Dn; c += kWave) grad_h[(B + r) * d.Dn + c] = row[c];
            if (grad_f)
                for (int c = lane; c < d.De; c += kWave) grad_f[r * d.De + c] = row[d.Dn + c];
            const float tt = dt[r];
#pragma unroll
            for (int t = 0; t < kT; t++) {
                const int i = lane + t * kWave;
                if (i < d.Dt) {
                    const float s = -sinf(time_arg(tt, tw[t], tb[t])) * row[d.Dn + d.De + i];
                    dw[t] += s * tt;
                    db[t] += s;
                }
            }
        } else {
            const int64_t q = r - E;
            const float *rq = dx_q + q * LD, *rr = dx_r + q * LD;
            if (grad_h)
                for (int c = lane; c < d.Dn; c += kWave) grad_h[q * d.Dn + c] = rq[c] + rr[O + c];
#pragma unroll
            for (int t = 0; t < kT; t++) {
                const int i = lane + t * kWave;
                if (i < d.Dt) db[t] += -sinf(tb[t]) * rq[d.Dn + i];
            }
        }
    }
#pragma unroll
    for (int t = 0; t < kT; t++) {
        fold[wave][0][lane + t * kWave] = dw[t];
        fold[wave][1][lane + t * kWave] = db[t];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2 * d.Dt; i += kBlock) {
        const int which = i / d.Dt, c = i % d.Dt;
        float s = 0.0f;
        for (int w = 0; w < kWavesPerBlock; w++) s += fold[w][which][c];
        partial[(int64_t)blockIdx.x * 2 * d.Dt + i] = s;
    }
}

// Column sums of a table of partial rows, 64 columns per workgroup: wave w adds the rows
// w, w + 4, ... (four independent chains, so the loads overlap), the four waves' sums are
// added in wave order. The order of additions is fixed by the table's height alone.
__device__ __forceinline__ void column_sums_block(float *__restrict__ out,
                                                  const float *__restrict__ part, int n, int cols,
                                                  int block) {
    __shared__ float fold[kWavesPerBlock][kWave];
    const int lane = lane_id(), wave = threadIdx.x / kWave;
    const int c = block * kWave + lane;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
    if (c < cols) {
        int r = wave;
        for (; r + 3 * kWavesPerBlock < n; r += 4 * kWavesPerBlock) {
            s0 += part[(int64_t)r * cols + c];
            s1 += part[(int64_t)(r + kWavesPerBlock) * cols + c];
            s2 += part[(int64_t)(r + 2 * kWavesPerBlock) * cols + c];
            s3 += part[(int64_t)(r + 3 * kWavesPerBlock) * cols + c];
        }
        for (; r < n; r += kWavesPerBlock) s0 += part[(int64_t)r * cols + c];
    }
    fold[wave][lane] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (wave == 0 && c < cols) out[c] = (fold[0][lane] + fold[1][lane]) + (fold[2][lane] + fold[3][lane]);
}

// out_x[c] = sum over the n_x rows of partial_x[., c]; two tables in one launch (x = a for
// the first blocks_a workgroups).
__global__ __launch_bounds__(kBlock) void partial_sums_kernel(
    float *__restrict__ out_a, const float *__restrict__ part_a, int n_a, int cols_a, int blocks_a,
    float *__restrict__ out_b, const float *__restrict__ part_b, int n_b, int cols_b) {
    if ((int)blockIdx.x < blocks_a)
        column_sums_block(out_a, part_a, n_a, cols_a, blockIdx.x);
    else
        column_sums_block(out_b, part_b, n_b, cols_b, blockIdx.x - blocks_a);
}

struct CollectArgs {
    float *out_ln, *out_time;
    const float *part_ln, *part_t;
    int rows_ln, rows_t;
    float *g_wq, *g_bq, *g_wk, *g_bk, *g_wv, *g_bv, *g_wo, *g_bo;
    const float *dw_kv, *dw_q, *dw_r;
};

// The last launch of the backward: the two tables of partial sums (LayerNorm affine,
// time encoder) and the weight gradients out of their bias-augmented rows into one
// contiguous tensor per parameter (one wave per row).
__global__ __launch_bounds__(kBlock) void tattn_collect_kernel(TattnDims d, CollectArgs a,
                                                               int blocks_ln, int blocks_t) {
    int block = blockIdx.x;
    if (block < blocks_ln) {
        column_sums_block(a.out_ln, a.part_ln, a.rows_ln, 2 * d.O, block);
        return;
    }
    block -= blocks_ln;
    if (block < blocks_t) {
        column_sums_block(a.out_time, a.part_t, a.rows_t, 2 * d.Dt, block);
        return;
    }
    block -= blocks_t;
    const int lane = lane_id();
    const int O = d.O, LD = d.LD;
    const int Dkv = d.Dn + d.De + d.Dt, Dq = d.Dn + d.Dt, Dr = O + d.Dn;
    int r = block * kWavesPerBlock + threadIdx.x / kWave;
    const float *src;
    float *w, *bias;
    int width;
    if (r < 2 * O) {
        const bool is_k = r < O;
        src = a.dw_kv + (int64_t)r * LD;
        r = is_k ? r : r - O;
        w = (is_k ? a.g_wk : a.g_wv) + (int64_t)r * Dkv;
        bias = (is_k ? a.g_bk : a.g_bv) + r;
        width = Dkv;
    } else if (r < 3 * O) {
        r -= 2 * O;
        src = a.dw_q + (int64_t)r * LD;
        w = a.g_wq + (int64_t)r * Dq;
        bias = a.g_bq + r;
        width = Dq;
    } else if (r < 4 * O) {
        r -= 3 * O;
        src = a.dw_r + (int64_t)r * LD;
        w = a.g_wo + (int64_t)r * Dr;
        bias = a.g_bo + r;
        width = Dr;
    } else {
        return;
    }
    for (int c = lane; c < width; c += kWave) w[c] = src[c];
    if (lane == 0) *bias = src[LD - 1];
}

int check_dims(TattnDims &d, int64_t n_dst, int64_t n_edges, int64_t dim_node, int64_t dim_edge,
               int64_t dim_time, int64_t dim_out, int64_t n_heads, int64_t ld) {
    YITU_REQUIRE(n_dst >= 0 && n_edges >= 0 && dim_node >= 0 && dim_edge >= 0 && dim_time >= 0,
                 "negative size");
    YITU_REQUIRE(n_dst + n_edges < ((int64_t)1 << 30), "too many rows");
    YITU_REQUIRE(dim_out >= 1 && dim_out <= kTattnMaxOut, "dim_out must be 1..%d", kTattnMaxOut);
    YITU_REQUIRE(dim_time <= kTattnMaxOut, "dim_time must be at most %d", kTattnMaxOut);
    YITU_REQUIRE(n_heads >= 1 && n_heads <= kTattnMaxHeads && dim_out % n_heads == 0,
                 "n_heads must be 1..%d and divide dim_out", kTattnMaxHeads);
    YITU_REQUIRE(ld == yitu_tattn_row_length(dim_node, dim_edge, dim_time, dim_out),
                 "row length must be yitu_tattn_row_length(...) = %lld",
                 (long long)yitu_tattn_row_length(dim_node, dim_edge, dim_time, dim_out));
    d = TattnDims{(int)n_dst, (int)n_edges, (int)dim_node, (int)dim_edge, (int)dim_time,
                  (int)dim_out, (int)n_heads, (int)ld};
    return 0;
}

}  // namespace

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API int64_t yitu_tattn_row_length(int64_t dim_node, int64_t dim_edge, int64_t dim_time,
                                       int64_t dim_out) {
    const int64_t widest = std::max(dim_node + dim_edge + dim_time, dim_out + dim_node);
    return (widest + 1 + 3) / 4 * 4;
}

YITU_API int64_t yitu_tattn_partial_rows(int64_t n_rows) {
    return std::max<int64_t>(1, ceil_div(n_rows, kWavesPerBlock * kRowsPerWaveReduce));
}

YITU_API int yitu_tattn_prepare(float *x_kv, float *x_q, float *x_r, float *w_kv, float *w_q2,
                                float *w_r, const float *h, const float *f, const float *dt,
                                const float *time_w, const float *time_b, const float *wq,
                                const float *bq, const float *wk, const float *bk, const float *wv,
                                const float *bv, const float *wo, const float *bo, int64_t n_dst,
                                int64_t n_edges, int64_t dim_node, int64_t dim_edge,
                                int64_t dim_time, int64_t dim_out, int64_t ld, void *stream) {
    TattnDims d;
    if (int rc = check_dims(d, n_dst, n_edges, dim_node, dim_edge, dim_time, dim_out, 1, ld)) return rc;
    YITU_REQUIRE(x_kv && x_q && x_r && w_kv && w_q2 && w_r, "null output");
    YITU_REQUIRE((dim_node == 0 || h) && (dim_edge == 0 || f) &&
                     (dim_time == 0 || (time_w && time_b && (n_edges == 0 || dt))),
                 "null feature input");
    YITU_REQUIRE(dim_node + dim_time > 0, "the query needs node or time features");
    YITU_REQUIRE(wq && bq && wk && bk && wv && bv && wo && bo, "null parameter");
    PrepareArgs a{x_kv, x_q, x_r, w_kv, w_q2, w_r, h, f, dt, time_w, time_b,
                  wq, bq, wk, bk, wv, bv, wo, bo};
    const int64_t rows = n_edges + 2 * n_dst + 5 * dim_out;
    tattn_prepare_kernel<<<(int)ceil_div(rows, kWavesPerBlock), kBlock, 0,
                           static_cast<hipStream_t>(stream)>>>(d, a);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_tattn_forward(float *x_r, float *attn, const float *q2, const float *kv,
                                const int32_t *indptr, int64_t n_dst, int64_t n_edges,
                                int64_t dim_out, int64_t n_heads, int64_t ld, void *stream) {
    YITU_REQUIRE(n_dst >= 0 && n_edges >= 0, "negative size");
    YITU_REQUIRE(dim_out >= 1 && dim_out <= kTattnMaxOut && n_heads >= 1 &&
                     n_heads <= kTattnMaxHeads && dim_out % n_heads == 0 && ld >= dim_out,
                 "dim_out must be 1..%d, n_heads 1..%d and divide it", kTattnMaxOut,
                 kTattnMaxHeads);
    if (n_dst == 0) return 0;
    YITU_REQUIRE(x_r && q2 && indptr && (n_edges == 0 || (attn && kv)), "null operand");
    TattnDims d{(int)n_dst, (int)n_edges, 0, 0, 0, (int)dim_out, (int)n_heads, (int)ld};
    tattn_forward_kernel<<<(int)ceil_div(n_dst, kWavesPerBlock), kBlock, 0,
                           static_cast<hipStream_t>(stream)>>>(d, x_r, attn, q2, kv, indptr);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_tattn_backward(float *dq2, float *dkv, float *scratch, const float *dx_r,
                                 const float *q2, const float *kv, const float *attn,
                                 const int32_t *indptr, int64_t n_dst, int64_t n_edges,
                                 int64_t dim_out, int64_t n_heads, int64_t ld, void *stream) {
    YITU_REQUIRE(n_dst >= 0 && n_edges >= 0, "negative size");
    YITU_REQUIRE(dim_out >= 1 && dim_out <= kTattnMaxOut && n_heads >= 1 &&
                     n_heads <= kTattnMaxHeads && dim_out % n_heads == 0 && ld >= dim_out,
                 "dim_out must be 1..%d, n_heads 1..%d and divide it", kTattnMaxOut,
                 kTattnMaxHeads);
    if (n_dst == 0) return 0;
    YITU_REQUIRE(dq2 && dx_r && q2 && indptr && (n_edges == 0 || (dkv && scratch && kv && attn)),
                 "null operand");
    TattnDims d{(int)n_dst, (int)n_edges, 0, 0, 0, (int)dim_out, (int)n_heads, (int)ld};
    tattn_backward_kernel<<<(int)ceil_div(n_dst, kWavesPerBlock), kBlock, 0,
                            static_cast<hipStream_t>(stream)>>>(d, dq2, dkv, scratch, dx_r, q2, kv,
                                                                attn, indptr);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_relu_layernorm_forward(float *out, const float *pre, const float *gamma,
                                         const float *beta, int64_t n_rows, int64_t n_cols,
                                         float eps, void *stream) {
    YITU_REQUIRE(n_rows >= 0 && n_cols >= 1 && n_cols <= kTattnMaxOut && n_rows < INT32_MAX,
                 "n_cols must be 1..%d", kTattnMaxOut);
    if (n_rows == 0) return 0;
    YITU_REQUIRE(out && pre && gamma && beta, "null operand");
    relu_layernorm_fwd_kernel<<<(int)ceil_div(n_rows, kWavesPerBlock), kBlock, 0,
                                static_cast<hipStream_t>(stream)>>>(out, pre, gamma, beta,
                                                                    (int)n_rows, (int)n_cols, eps);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_relu_layernorm_backward(float *d_pre, float *partial, const float *grad_out,
                                          const float *pre, const float *gamma, int64_t n_rows,
                                          int64_t n_cols, int64_t d_pre_row_stride, float eps,
                                          void *stream) {
    YITU_REQUIRE(n_rows >= 0 && n_cols >= 1 && n_cols <= kTattnMaxOut && n_rows < INT32_MAX &&
                     d_pre_row_stride >= n_cols,
                 "n_cols must be 1..%d and the row stride at least n_cols", kTattnMaxOut);
    YITU_REQUIRE(d_pre && partial && (n_rows == 0 || (grad_out && pre && gamma)), "null operand");
    relu_layernorm_bwd_kernel<<<(int)yitu_tattn_partial_rows(n_rows), kBlock, 0,
                                static_cast<hipStream_t>(stream)>>>(
        d_pre, partial, grad_out, pre, gamma, (int)n_rows, (int)n_cols, (int)d_pre_row_stride, eps);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_tattn_finalize(float *grad_h, float *grad_f, float *partial, const float *dx_kv,
                                 const float *dx_q, const float *dx_r, const float *dt,
                                 const float *time_w, const float *time_b, int64_t n_dst,
                                 int64_t n_edges, int64_t dim_node, int64_t dim_edge,
                                 int64_t dim_time, int64_t dim_out, int64_t ld, void *stream) {
    TattnDims d;
    if (int rc = check_dims(d, n_dst, n_edges, dim_node, dim_edge, dim_time, dim_out, 1, ld)) return rc;
    YITU_REQUIRE(partial && dx_q && dx_r && (n_edges == 0 || dx_kv), "null operand");
    YITU_REQUIRE(dim_time == 0 || (time_w && time_b && (n_edges == 0 || dt)), "null time input");
    tattn_finalize_kernel<<<(int)yitu_tattn_partial_rows(n_dst + n_edges), kBlock, 0,
                            static_cast<hipStream_t>(stream)>>>(d, grad_h, grad_f, partial, dx_kv,
                                                                dx_q, dx_r, dt, time_w, time_b);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_partial_sums(float *out_a, const float *partial_a, int64_t rows_a, int64_t cols_a,
                               float *out_b, const float *partial_b, int64_t rows_b, int64_t cols_b,
                               void *stream) {
    YITU_REQUIRE(rows_a >= 0 && cols_a >= 0 && rows_b >= 0 && cols_b >= 0 && cols_a < INT32_MAX &&
                     cols_b < INT32_MAX && rows_a < INT32_MAX && rows_b < INT32_MAX,
                 "size out of range");
    YITU_REQUIRE((cols_a == 0 || (out_a && (rows_a == 0 || partial_a))) &&
                     (cols_b == 0 || (out_b && (rows_b == 0 || partial_b))),
                 "null operand");
    const int blocks_a = (int)ceil_div(cols_a, kWave), blocks_b = (int)ceil_div(cols_b, kWave);
    if (blocks_a + blocks_b == 0) return 0;
    partial_sums_kernel<<<blocks_a + blocks_b, kBlock, 0, static_cast<hipStream_t>(stream)>>>(
        out_a, partial_a, (int)rows_a, (int)cols_a, blocks_a, out_b, partial_b, (int)rows_b,
        (int)cols_b);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_tattn_collect(float *grad_ln, float *grad_time, float *grad_w_q, float *grad_b_q,
                                float *grad_w_k, float *grad_b_k, float *grad_w_v, float *grad_b_v,
                                float *grad_w_out, float *grad_b_out, const float *partial_ln,
                                int64_t rows_ln, const float *partial_time, int64_t rows_time,
                                const float *dw_kv, const float *dw_q, const float *dw_r,
                                int64_t dim_node, int64_t dim_edge, int64_t dim_time,
                                int64_t dim_out, int64_t ld, void *stream) {
    TattnDims d;
    if (int rc = check_dims(d, 0, 0, dim_node, dim_edge, dim_time, dim_out, 1, ld)) return rc;
    YITU_REQUIRE(rows_ln >= 0 && rows_time >= 0 && rows_ln < INT32_MAX && rows_time < INT32_MAX,
                 "size out of range");
    YITU_REQUIRE(grad_ln && (rows_ln == 0 || partial_ln) &&
                     (dim_time == 0 || (grad_time && (rows_time == 0 || partial_time))),
                 "null partial table");
    YITU_REQUIRE(grad_w_q && grad_b_q && grad_w_k && grad_b_k && grad_w_v && grad_b_v &&
                     grad_w_out && grad_b_out && dw_kv && dw_q && dw_r,
                 "null gradient");
    CollectArgs a{grad_ln, grad_time, partial_ln, partial_time, (int)rows_ln, (int)rows_time,
                  grad_w_q, grad_b_q, grad_w_k, grad_b_k, grad_w_v, grad_b_v, grad_w_out,
                  grad_b_out, dw_kv, dw_q, dw_r};
    const int blocks_ln = (int)ceil_div(2 * dim_out, kWave);
    const int blocks_t = (int)ceil_div(2 * dim_time, kWave);
    const int blocks_w = (int)ceil_div(4 * dim_out, kWavesPerBlock);
    tattn_collect_kernel<<<blocks_ln + blocks_t + blocks_w, kBlock, 0,
                           static_cast<hipStream_t>(stream)>>>(d, a, blocks_ln, blocks_t);
    YITU_LAUNCH_CHECK();
    return 0;
}
