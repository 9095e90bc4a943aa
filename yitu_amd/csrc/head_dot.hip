// Row-wise dense helpers around the sparse ops, three families in this file:
//   1. per-head projections of a GAT layer (yitu_head_dot*),
//   2. Linear layers with a handful of outputs (yitu_skinny_linear*),
//   3. column sums = bias gradients, replayable from a HIP graph (yitu_column_sum).
// They share the row layout (tiles of 256 floats over the wave, 4 per lane) and the
// fixed-order two-stage sums.
//
// 1. Per-head projections of a GAT layer with attention vectors:
//   q[n,h] = <a_dst[h,:], x[n,h,:]>,   k[n,h] = <a_src[h,:], x[n,h,:]>
// and their backward. The reference's example layer uses dense H*F -> H Linears
// for the two (test/common/model.py:70-71); the per-head vectors a_src / a_dst
// [H, F] are their block-diagonal, bias-free special case and the form GAT is
// usually stated in. As torch ops ((x * a).sum(-1) twice, and the broadcast
// products and sums of its backward) they take ten passes over x; here the
// forward reads x once and the backward reads x once and updates grad_x once.
//
// Layout: a row of L = H * F floats is spread over the wave in tiles of 256
// floats, 4 per lane; F = 4 * LPH with LPH a power of two <= 64, so a head is LPH
// consecutive lanes of one tile and its dot is a butterfly inside the group.
#include "../../include/yitu_hip.h"
#include "spmm_rows.hpp"

namespace yitu {

namespace {

constexpr int kMaxTiles = 4;      // rows of up to 1024 floats
constexpr int kRowsInFlight = 4;  // rows a wave loads before it reduces

struct HeadDotParams {
    const float *x;        // [n, L]
    const float *a1, *a2;  // [L] each (a2 may be null)
    float *o1, *o2;        // [n, H]
    const float *g1, *g2;  // backward: gradients of o1, o2 [n, H]
    float *grad_x;         // backward: [n, L], written or accumulated into
    float *partial;        // backward: [workgroups][2][L] partial sums for the vector gradients
    int accumulate;
    int n, L, H, lph;
};

__device__ __forceinline__ float group_sum_rt(float v, int lph) {
    for (int o = lph >> 1; o >= 1; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

template <int KT, bool TWO>
__global__ __launch_bounds__(kBlock) void head_dot_kernel(HeadDotParams p) {
    const int lane = lane_id();
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int wave = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    float a1[KT][4], a2[KT][4];
    bool live[KT];
#pragma unroll
    for (int t = 0; t < KT; t++) {
        const int col = t * 256 + lane * 4;
        live[t] = col < p.L;
#pragma unroll
        for (int i = 0; i < 4; i++) a1[t][i] = a2[t][i] = 0.0f;
        if (live[t]) {
            RowLoad<4, float>::ld(p.a1 + col, a1[t]);
            if constexpr (TWO) RowLoad<4, float>::ld(p.a2 + col, a2[t]);
        }
    }
    for (int r0 = wave * kRowsInFlight; r0 < p.n; r0 += n_waves * kRowsInFlight) {
        float x[kRowsInFlight][KT][4];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; u++) {
            const int r = min(r0 + u, p.n - 1);
#pragma unroll
            for (int t = 0; t < KT; t++)
                if (live[t]) RowLoad<4, float>::ld(p.x + (size_t)r * p.L + t * 256 + lane * 4, x[u][t]);
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; u++) {
            const int r = r0 + u;
#pragma unroll
            for (int t = 0; t < KT; t++) {
                float d1 = 0.0f, d2 = 0.0f;
                if (live[t]) {
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        d1 += x[u][t][i] * a1[t][i];
                        if constexpr (TWO) d2 += x[u][t][i] * a2[t][i];
                    }
                }
                d1 = group_sum_rt(d1, p.lph);
                if constexpr (TWO) d2 = group_sum_rt(d2, p.lph);
                const int head = (t * 256 + lane * 4) / (4 * p.lph);
                if (live[t] && r < p.n && lane % p.lph == 0) {
                    p.o1[(size_t)r * p.H + head] = d1;
                    if constexpr (TWO) p.o2[(size_t)r * p.H + head] = d2;
                }
            }
        }
    }
}

// grad_x[n,h,:] (+)= g1[n,h] a1[h,:] + g2[n,h] a2[h,:]; the workgroup's sums of
// g1[n,h] x[n,h,:] and g2[n,h] x[n,h,:] go to partial[workgroup][0 / 1][:], added up by
// the kernel below.
template <int KT, bool TWO>
__global__ __launch_bounds__(kBlock) void head_dot_bwd_kernel(HeadDotParams p) {
    const int lane = lane_id();
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int wave = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    float a1[KT][4], a2[KT][4], s1[KT][4], s2[KT][4];
    bool live[KT];
    int head[KT];
#pragma unroll
    for (int t = 0; t < KT; t++) {
        const int col = t * 256 + lane * 4;
        live[t] = col < p.L;
        head[t] = live[t] ? col / (4 * p.lph) : 0;
#pragma unroll
        for (int i = 0; i < 4; i++) a1[t][i] = a2[t][i] = s1[t][i] = s2[t][i] = 0.0f;
        if (live[t]) {
            RowLoad<4, float>::ld(p.a1 + col, a1[t]);
            if constexpr (TWO) RowLoad<4, float>::ld(p.a2 + col, a2[t]);
        }
    }
    for (int r0 = wave * kRowsInFlight; r0 < p.n; r0 += n_waves * kRowsInFlight) {
        float x[kRowsInFlight][KT][4], gx[kRowsInFlight][KT][4];
        float g1[kRowsInFlight][KT], g2[kRowsInFlight][KT];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; u++) {
            const int r = min(r0 + u, p.n - 1);
#pragma unroll
            for (int t = 0; t < KT; t++) {
                g1[u][t] = g2[u][t] = 0.0f;
                if (live[t]) {
                    const size_t off = (size_t)r * p.L + t * 256 + lane * 4;
                    RowLoad<4, float>::ld(p.x + off, x[u][t]);
                    if (p.accumulate) RowLoad<4, float>::ld(p.grad_x + off, gx[u][t]);
                    g1[u][t] = p.g1[(size_t)r * p.H + head[t]];
                    if constexpr (TWO) g2[u][t] = p.g2[(size_t)r * p.H + head[t]];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; u++) {
            if (r0 + u >= p.n) break;  // wave-uniform
#pragma unroll
            for (int t = 0; t < KT; t++) {
                if (!live[t]) continue;
                float out[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float v = g1[u][t] * a1[t][i];
                    s1[t][i] += g1[u][t] * x[u][t][i];
                    if constexpr (TWO) {
                        v += g2[u][t] * a2[t][i];
                        s2[t][i] += g2[u][t] * x[u][t][i];
                    }
                    out[i] = p.accumulate ? gx[u][t][i] + v : v;
                }
                store_row<4>(p.grad_x + (size_t)(r0 + u) * p.L + t * 256 + lane * 4, out);
            }
        }
    }
    // the four waves of the workgroup are added in wave order; one partial row per workgroup
    __shared__ float red[kWavesPerBlock][2][256 * KT];
    const int w = threadIdx.x / kWave;
#pragma unroll
    for (int t = 0; t < KT; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            red[w][0][t * 256 + lane * 4 + i] = s1[t][i];
            red[w][1][t * 256 + lane * 4 + i] = s2[t][i];
        }
    __syncthreads();
    for (int j = threadIdx.x; j < 2 * p.L; j += kBlock) {
        const int which = j / p.L, col = j % p.L;
        float s = 0.0f;
#pragma unroll
        for (int q = 0; q < kWavesPerBlock; q++) s += red[q][which][col];
        p.partial[(size_t)blockIdx.x * 2 * p.L + j] = s;
    }
}

// grad_a[j] = sum over the workgroups' partial rows. A workgroup takes 16 columns;
// its 16 thread groups add rows g, g + 16, ... and the group sums are added in order.
constexpr int kSumCols = 16, kSumGroups = kBlock / kSumCols;

__global__ __launch_bounds__(kBlock) void head_dot_sum_kernel(float *__restrict__ grad_a1,
                                                              float *__restrict__ grad_a2,
                                                              const float *__restrict__ partial,
                                                              int n_rows, int L) {
    __shared__ float red[kSumGroups][kSumCols];
    const int c = threadIdx.x % kSumCols, g = threadIdx.x / kSumCols;
    const int j = blockIdx.x * kSumCols + c;
    float s = 0.0f;
    if (j < 2 * L)
        for (int r = g; r < n_rows; r += kSumGroups) s += partial[(size_t)r * 2 * L + j];
    red[g][c] = s;
    __syncthreads();
    if (g == 0 && j < 2 * L) {
        float t = 0.0f;
#pragma unroll
        for (int q = 0; q < kSumGroups; q++) t += red[q][c];
        if (j < L)
            grad_a1[j] = t;
        else if (grad_a2)
            grad_a2[j - L] = t;
    }
}

// workgroups of the forward (enough to fill the chip) and of the backward (each leaves
// one partial row for the attention-vector gradients)
int head_dot_grid(int64_t n) {
    return (int)std::min<int64_t>(ceil_div(n, kWavesPerBlock * kRowsInFlight), 4096);
}
int head_dot_bwd_grid(int64_t n) {
    return (int)std::min<int64_t>(ceil_div(n, kWavesPerBlock * kRowsInFlight), 1024);
}

int check_shape(int64_t n, int64_t n_heads, int64_t n_features) {
    YITU_REQUIRE(n >= 0 && n_heads > 0 && n_features > 0 && n < INT32_MAX, "size out of range");
    const int64_t lph = n_features / 4;
    YITU_REQUIRE(n_features % 4 == 0 && lph <= 64 && (lph & (lph - 1)) == 0 &&
                     n_heads * n_features <= 256 * kMaxTiles,
                 "head_dot: head width must be 4 * a power of two up to 256 and rows at most %d "
                 "floats (got H=%lld F=%lld)",
                 256 * kMaxTiles, (long long)n_heads, (long long)n_features);
    return 0;
}

template <bool BWD, bool TWO>
int launch_tiles(const HeadDotParams &p, int grid, hipStream_t stream) {
    switch ((p.L + 255) / 256) {
        case 1:
            if constexpr (BWD) head_dot_bwd_kernel<1, TWO><<<grid, kBlock, 0, stream>>>(p);
            else head_dot_kernel<1, TWO><<<grid, kBlock, 0, stream>>>(p);
            break;
        case 2:
            if constexpr (BWD) head_dot_bwd_kernel<2, TWO><<<grid, kBlock, 0, stream>>>(p);
            else head_dot_kernel<2, TWO><<<grid, kBlock, 0, stream>>>(p);
            break;
        default:
            if constexpr (BWD) head_dot_bwd_kernel<4, TWO><<<grid, kBlock, 0, stream>>>(p);
            else head_dot_kernel<4, TWO><<<grid, kBlock, 0, stream>>>(p);
    }
    YITU_LAUNCH_CHECK();
    return 0;
}

}  // namespace

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API int yitu_head_dot(float *out_a, float *out_b, const float *x, const float *vec_a,
                           const float *vec_b, int64_t n, int64_t n_heads, int64_t n_features,
                           void *stream) {
    if (int rc = check_shape(n, n_heads, n_features)) return rc;
    if (n == 0) return 0;
    YITU_REQUIRE(out_a && x && vec_a && (!vec_b == !out_b), "null pointer");
    YITU_REQUIRE(aligned16(x) && aligned16(vec_a) && aligned16(vec_b), "pointers must be 16-byte aligned");
    HeadDotParams p{};
    p.x = x;
    p.a1 = vec_a;
    p.a2 = vec_b;
    p.o1 = out_a;
    p.o2 = out_b;
    p.n = (int)n;
    p.L = (int)(n_heads * n_features);
    p.H = (int)n_heads;
    p.lph = (int)(n_features / 4);
    const int grid = head_dot_grid(n);
    return vec_b ? launch_tiles<false, true>(p, grid, static_cast<hipStream_t>(stream))
                 : launch_tiles<false, false>(p, grid, static_cast<hipStream_t>(stream));
}

YITU_API size_t yitu_head_dot_workspace_bytes(int64_t n, int64_t n_heads, int64_t n_features) {
    return sizeof(float) * 2 * (size_t)(n_heads * n_features) *
           (size_t)head_dot_bwd_grid(std::max<int64_t>(n, 1));
}

YITU_API int yitu_head_dot_backward(float *grad_x, int accumulate, float *grad_vec_a,
                                    float *grad_vec_b, const float *x, const float *vec_a,
                                    const float *vec_b, const float *grad_a, const float *grad_b,
                                    int64_t n, int64_t n_heads, int64_t n_features, void *workspace,
                                    size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_shape(n, n_heads, n_features)) return rc;
    const int64_t L = n_heads * n_features;
    YITU_REQUIRE(grad_x && grad_vec_a && x && vec_a && grad_a, "null pointer");
    YITU_REQUIRE(!vec_b == !grad_b && !vec_b == !grad_vec_b,
                 "the second vector, its output gradient and its gradient go together");
    YITU_REQUIRE(aligned16(x) && aligned16(grad_x) && aligned16(vec_a) && aligned16(vec_b),
                 "pointers must be 16-byte aligned");
    if (n == 0) {
        int rc = fill_zero(grad_vec_a, L, stream);
        if (!rc && grad_vec_b) rc = fill_zero(grad_vec_b, L, stream);
        return rc;
    }
    YITU_REQUIRE(workspace && workspace_bytes >= yitu_head_dot_workspace_bytes(n, n_heads, n_features) &&
                     aligned16(workspace),
                 "workspace too small: need %zu bytes",
                 yitu_head_dot_workspace_bytes(n, n_heads, n_features));
    HeadDotParams p{};
    p.x = x;
    p.a1 = vec_a;
    p.a2 = vec_b;
    p.g1 = grad_a;
    p.g2 = grad_b;
    p.grad_x = grad_x;
    p.partial = static_cast<float *>(workspace);
    p.accumulate = accumulate;
    p.n = (int)n;
    p.L = (int)L;
    p.H = (int)n_heads;
    p.lph = (int)(n_features / 4);
    const int grid = head_dot_bwd_grid(n);
    int rc = vec_b ? launch_tiles<true, true>(p, grid, stream) : launch_tiles<true, false>(p, grid, stream);
    if (rc) return rc;
    head_dot_sum_kernel<<<(int)ceil_div(2 * L, kSumCols), kBlock, 0, stream>>>(
        grad_vec_a, grad_vec_b, p.partial, grid, (int)L);
    YITU_LAUNCH_CHECK();
    return 0;
}

// ---- skinny Linear: y[n, J] = x[n, K] . w[J, K]^T (+ b), J small ---------------------
// The dense query / key projections of the reference's GATLayer (H*F -> H Linears with
// bias, test/common/model.py:70-71) have a handful of outputs per row: as GEMMs they
// are one read of x each with a tile that is almost empty. Here a wave takes rows of
// K floats (4 per lane and tile), the J weight rows sit in LDS, and each output is a
// full-wave butterfly; two Linears that read the same x are one call with their
// weights stacked. Backward: grad_x (+)= grad_y . w in place, grad_w and grad_b as
// per-workgroup partial sums added in a fixed order.
namespace yitu {
namespace {

constexpr int kSkinnyMaxJ = 16;

struct SkinnyParams {
    const float *x, *w, *b;  // [n, K], [J, K], [J] or null
    float *y;                // [n, J]
    const float *gy;         // backward: [n, J]
    float *grad_x;           // backward: [n, K]
    float *partial;          // backward: [workgroups][J * K + J]
    int accumulate;
    int n, K, J;
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = kWave / 2; o >= 1; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

template <int KT>
__global__ __launch_bounds__(kBlock) void skinny_linear_kernel(SkinnyParams p) {
    extern __shared__ __align__(16) float w_lds[];  // [J][256 * KT]
    constexpr int KP = 256 * KT;
    for (int i = threadIdx.x; i < p.J * KP; i += kBlock) {
        const int j = i / KP, c = i % KP;
        w_lds[i] = c < p.K ? p.w[(size_t)j * p.K + c] : 0.0f;
    }
    __syncthreads();
    const int lane = lane_id();
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int wave = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    for (int r0 = wave * kRowsInFlight; r0 < p.n; r0 += n_waves * kRowsInFlight) {
        float x[kRowsInFlight][KT][4];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; u++) {
            const int r = min(r0 + u, p.n - 1);
#pragma unroll
            for (int t = 0; t < KT; t++) {
                const int c = t * 256 + lane * 4;
#pragma unroll
                for (int i = 0; i < 4; i++) x[u][t][i] = 0.0f;
                if (c < p.K) RowLoad<4, float>::ld(p.x + (size_t)r * p.K + c, x[u][t]);
            }
        }
        for (int j = 0; j < p.J; j++) {
            float d[kRowsInFlight];
#pragma unroll
            for (int u = 0; u < kRowsInFlight; u++) d[u] = 0.0f;
#pragma unroll
            for (int t = 0; t < KT; t++) {
                const float4 w4 = *reinterpret_cast<const float4 *>(&w_lds[j * KP + t * 256 + lane * 4]);
#pragma unroll
                for (int u = 0; u < kRowsInFlight; u++)
                    d[u] += x[u][t][0] * w4.x + x[u][t][1] * w4.y + x[u][t][2] * w4.z + x[u][t][3] * w4.w;
            }
            const float bj = p.b ? p.b[j] : 0.0f;
#pragma unroll
            for (int u = 0; u < kRowsInFlight; u++) {
                const float s = wave_sum(d[u]);
                if (lane == 0 && r0 + u < p.n) p.y[(size_t)(r0 + u) * p.J + j] = s + bj;
            }
        }
    }
}

// JT = outputs whose weight-gradient accumulators a lane keeps (J <= JT).
template <int KT, int JT>
__global__ __launch_bounds__(kBlock) void skinny_linear_bwd_kernel(SkinnyParams p) {
    extern __shared__ __align__(16) float lds[];  // [J][256 * KT] weights, then the workgroup reduction
    constexpr int KP = 256 * KT;
    for (int i = threadIdx.x; i < p.J * KP; i += kBlock) {
        const int j = i / KP, c = i % KP;
        lds[i] = c < p.K ? p.w[(size_t)j * p.K + c] : 0.0f;
    }
    __syncthreads();
    const int lane = lane_id();
    const int w_id = threadIdx.x / kWave;
    const int n_waves = gridDim.x * kWavesPerBlock;
    const int wave = blockIdx.x * kWavesPerBlock + w_id;
    float gw[JT][KT][4], gb[JT];
#pragma unroll
    for (int j = 0; j < JT; j++) {
        gb[j] = 0.0f;
#pragma unroll
        for (int t = 0; t < KT; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) gw[j][t][i] = 0.0f;
    }
    for (int r = wave; r < p.n; r += n_waves) {
        float x[KT][4], out[KT][4];
#pragma unroll
        for (int t = 0; t < KT; t++) {
            const int c = t * 256 + lane * 4;
#pragma unroll
            for (int i = 0; i < 4; i++) x[t][i] = out[t][i] = 0.0f;
            if (c < p.K) {
                RowLoad<4, float>::ld(p.x + (size_t)r * p.K + c, x[t]);
                if (p.accumulate) RowLoad<4, float>::ld(p.grad_x + (size_t)r * p.K + c, out[t]);
            }
        }
        const float g_lane = lane < p.J ? p.gy[(size_t)r * p.J + lane] : 0.0f;
#pragma unroll
        for (int j = 0; j < JT; j++) {
            if (j >= p.J) break;
            const float g = __shfl(g_lane, j, kWave);
            gb[j] += g;
#pragma unroll
            for (int t = 0; t < KT; t++) {
                const float4 w4 = *reinterpret_cast<const float4 *>(&lds[j * KP + t * 256 + lane * 4]);
                out[t][0] += g * w4.x;
                out[t][1] += g * w4.y;
                out[t][2] += g * w4.z;
                out[t][3] += g * w4.w;
#pragma unroll
                for (int i = 0; i < 4; i++) gw[j][t][i] += g * x[t][i];
            }
        }
#pragma unroll
        for (int t = 0; t < KT; t++) {
            const int c = t * 256 + lane * 4;
            if (c < p.K) store_row<4>(p.grad_x + (size_t)r * p.K + c, out[t]);
        }
    }
    // workgroup partial: the four waves added in wave order, one output row at a time
    float *dst = p.partial + (size_t)blockIdx.x * (p.J * p.K + p.J);
    for (int j = 0; j < p.J; j++) {
        __syncthreads();  // the weights (first pass) or the previous row are no longer needed
#pragma unroll
        for (int jj = 0; jj < JT; jj++) {
            if (jj != j) continue;
#pragma unroll
            for (int t = 0; t < KT; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) lds[w_id * KP + t * 256 + lane * 4 + i] = gw[jj][t][i];
            if (lane == 0) lds[kWavesPerBlock * KP + w_id] = gb[jj];
        }
        __syncthreads();
        for (int c = threadIdx.x; c < p.K; c += kBlock) {
            float s = 0.0f;
#pragma unroll
            for (int q = 0; q < kWavesPerBlock; q++) s += lds[q * KP + c];
            dst[(size_t)j * p.K + c] = s;
        }
        if (threadIdx.x == 0) {
            float s = 0.0f;
#pragma unroll
            for (int q = 0; q < kWavesPerBlock; q++) s += lds[kWavesPerBlock * KP + q];
            dst[(size_t)p.J * p.K + j] = s;
        }
    }
}

// out[j] = sum over partial rows of partial[row][j], rows added by kSumGroups thread
// groups and the group sums in order (the same scheme as head_dot_sum_kernel).
__global__ __launch_bounds__(kBlock) void partial_sum_kernel(float *__restrict__ out_a, int n_a,
                                                             float *__restrict__ out_b, int n_b,
                                                             const float *__restrict__ partial,
                                                             int n_rows) {
    __shared__ float red[kSumGroups][kSumCols];
    const int width = n_a + n_b;
    const int c = threadIdx.x % kSumCols, g = threadIdx.x / kSumCols;
    const int j = blockIdx.x * kSumCols + c;
    float s = 0.0f;
    if (j < width)
#pragma unroll 8
        for (int r = g; r < n_rows; r += kSumGroups) s += partial[(size_t)r * width + j];
    red[g][c] = s;
    __syncthreads();
    if (g == 0 && j < width) {
        float t = 0.0f;
#pragma unroll
        for (int q = 0; q < kSumGroups; q++) t += red[q][c];
        if (j < n_a)
            out_a[j] = t;
        else if (out_b)
            out_b[j - n_a] = t;
    }
}

int skinny_check(int64_t n, int64_t k, int64_t j) {
    YITU_REQUIRE(n >= 0 && n < INT32_MAX && k > 0 && j > 0, "size out of range");
    const int64_t tiles = k <= 256 ? 1 : (k <= 512 ? 2 : 4);  // the kernels' tile counts
    YITU_REQUIRE(k % 4 == 0 && k <= 256 * kMaxTiles && j <= kSkinnyMaxJ && j * tiles <= 16,
                 "skinny linear: in_features a multiple of 4 up to %d, out_features up to %d with "
                 "out_features * tiles(in_features) <= 16, tiles = 1, 2, 4 for up to 256, 512, 1024 "
                 "(got %lld -> %lld)",
                 256 * kMaxTiles, kSkinnyMaxJ, (long long)k, (long long)j);
    return 0;
}

int skinny_bwd_grid(int64_t n) {
    return (int)std::min<int64_t>(ceil_div(std::max<int64_t>(n, 1), kWavesPerBlock * 8), 1024);
}

template <int KT>
int skinny_bwd_launch(const SkinnyParams &p, int grid, size_t lds_bytes, hipStream_t stream) {
    if (p.J <= 4) skinny_linear_bwd_kernel<KT, 4><<<grid, kBlock, lds_bytes, stream>>>(p);
    else if (p.J <= 8) {
        if constexpr (KT <= 2) skinny_linear_bwd_kernel<KT, 8><<<grid, kBlock, lds_bytes, stream>>>(p);
    } else {
        if constexpr (KT == 1) skinny_linear_bwd_kernel<KT, 16><<<grid, kBlock, lds_bytes, stream>>>(p);
    }
    YITU_LAUNCH_CHECK();
    return 0;
}

}  // namespace
}  // namespace yitu

YITU_API int yitu_skinny_linear(float *y, const float *x, const float *w, const float *bias,
                                int64_t n, int64_t in_features, int64_t out_features,
                                void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = skinny_check(n, in_features, out_features)) return rc;
    if (n == 0) return 0;
    YITU_REQUIRE(y && x && w && aligned16(x), "null or misaligned pointer");
    SkinnyParams p{};
    p.x = x;
    p.w = w;
    p.b = bias;
    p.y = y;
    p.n = (int)n;
    p.K = (int)in_features;
    p.J = (int)out_features;
    const int kt = (int)((in_features + 255) / 256);
    const int grid = head_dot_grid(n);
    switch (kt) {
        case 1: skinny_linear_kernel<1><<<grid, kBlock, sizeof(float) * p.J * 256, stream>>>(p); break;
        case 2: skinny_linear_kernel<2><<<grid, kBlock, sizeof(float) * p.J * 512, stream>>>(p); break;
        default: skinny_linear_kernel<4><<<grid, kBlock, sizeof(float) * p.J * 1024, stream>>>(p);
    }
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API size_t yitu_skinny_linear_workspace_bytes(int64_t n, int64_t in_features,
                                                   int64_t out_features) {
    return sizeof(float) * (size_t)(out_features * in_features + out_features) *
           (size_t)skinny_bwd_grid(n);
}

YITU_API int yitu_skinny_linear_backward(float *grad_x, int accumulate, float *grad_w,
                                         float *grad_bias, const float *x, const float *w,
                                         const float *grad_y, int64_t n, int64_t in_features,
                                         int64_t out_features, void *workspace,
                                         size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = skinny_check(n, in_features, out_features)) return rc;
    YITU_REQUIRE(grad_x && grad_w && x && w && grad_y && aligned16(x) && aligned16(grad_x),
                 "null or misaligned pointer");
    YITU_REQUIRE(workspace && aligned16(workspace) &&
                     workspace_bytes >= yitu_skinny_linear_workspace_bytes(n, in_features, out_features),
                 "workspace too small: need %zu bytes",
                 yitu_skinny_linear_workspace_bytes(n, in_features, out_features));
    SkinnyParams p{};
    p.x = x;
    p.w = w;
    p.gy = grad_y;
    p.grad_x = grad_x;
    p.partial = static_cast<float *>(workspace);
    p.accumulate = accumulate;
    p.n = (int)n;
    p.K = (int)in_features;
    p.J = (int)out_features;
    const int kt = (int)((in_features + 255) / 256);
    const int grid = skinny_bwd_grid(n);
    // LDS: the weights, later per-wave rows of one output plus the four bias sums
    const size_t kp = 256 * (kt == 3 ? 4 : kt);
    const size_t lds_bytes = sizeof(float) * std::max<size_t>(p.J * kp, kWavesPerBlock * kp + kWavesPerBlock);
    int rc;
    switch (kt) {
        case 1: rc = skinny_bwd_launch<1>(p, grid, lds_bytes, stream); break;
        case 2: rc = skinny_bwd_launch<2>(p, grid, lds_bytes, stream); break;
        default: rc = skinny_bwd_launch<4>(p, grid, lds_bytes, stream);
    }
    if (rc) return rc;
    const int width = p.J * p.K + p.J;
    partial_sum_kernel<<<(int)ceil_div(width, kSumCols), kBlock, 0, stream>>>(
        grad_w, p.J * p.K, grad_bias, p.J, p.partial, grid);
    YITU_LAUNCH_CHECK();
    return 0;
}

// ---- column sums: out[j] = sum_r x[r, j] -----------------------------------------------
// The bias gradient of a Linear layer. Two stages with a fixed order of additions and no
// cleared accumulator (library reductions clear one with a memset node, which makes them
// unsafe to replay from a captured graph): workgroups sum row chunks into partial rows,
// partial_sum_kernel adds those.
namespace yitu {
namespace {

// rows per workgroup: about a thousand workgroups on large inputs (all resident at once, a few
// hundred KB of row data each, and a thousand partial rows for the second step), 8 rows on
// small ones (a function of n_rows alone: the workspace size and the summation order follow
// from it)
inline int col_sum_chunk(int64_t n_rows) {
    const int64_t c = ceil_div(n_rows, 1024);
    return c < 8 ? 8 : (int)c;
}

__global__ __launch_bounds__(kBlock) void column_chunk_sum_kernel(float *__restrict__ partial,
                                                                  const float *__restrict__ x,
                                                                  int n_rows, int n_cols, int chunk) {
    const int r0 = blockIdx.x * chunk, r1 = min(r0 + chunk, n_rows);
    for (int c = threadIdx.x; c < n_cols; c += kBlock) {
        float s = 0.0f;
#pragma unroll 8
        for (int r = r0; r < r1; r++) s += x[(size_t)r * n_cols + c];
        partial[(size_t)blockIdx.x * n_cols + c] = s;
    }
}

// The same for rows of up to 1024 columns, a multiple of 4: a thread reads 16 bytes of a row,
// 256 / (n_cols / 4) rows are read side by side, and their sums are added in row-group order.
__global__ __launch_bounds__(kBlock) void column_chunk_sum4_kernel(float *__restrict__ partial,
                                                                   const float *__restrict__ x,
                                                                   int n_rows, int n_cols, int chunk) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ f4 red[kBlock];
    const int vc = n_cols / 4, side = kBlock / vc;
    const int c4 = threadIdx.x % vc, rg = threadIdx.x / vc;
    const int r0 = blockIdx.x * chunk, r1 = min(r0 + chunk, n_rows);
    f4 s = {0.0f, 0.0f, 0.0f, 0.0f};
    if (rg < side) {
        const f4 *__restrict__ src = reinterpret_cast<const f4 *>(x) + c4;
#pragma unroll 8
        for (int r = r0 + rg; r < r1; r += side)
            s += __builtin_nontemporal_load(src + (size_t)r * vc);
    }
    red[threadIdx.x] = s;
    __syncthreads();
    if (rg == 0) {
        for (int q = 1; q < side; q++) s += red[q * vc + c4];
        reinterpret_cast<f4 *>(partial + (size_t)blockIdx.x * n_cols)[c4] = s;
    }
}

}  // namespace
}  // namespace yitu

namespace yitu {
namespace {
// Column sums of up to 32 short matrices in one launch (blockIdx.y = matrix, blockIdx.x =
// block of CB columns): the bias gradients of the per-relation Linears of a small
// heterogeneous graph, where one launch pair per Linear costs more than the sums. A
// thread adds every (256 / CB)-th row of its column, the thread sums are added in order.
constexpr int kColSumGroup = 32;
struct ColSumGroup {
    const float *src[kColSumGroup];
    float *out[kColSumGroup];
    int rows[kColSumGroup];
    int n_cols;
    int64_t ld;
};

template <int CB>
__global__ __launch_bounds__(kBlock) void column_sum_group_kernel(ColSumGroup g) {
    constexpr int RG = kBlock / CB;
    __shared__ float red[RG][CB];
    const int q = blockIdx.y, c = threadIdx.x % CB, rg = threadIdx.x / CB;
    const int j = blockIdx.x * CB + c;
    const float *__restrict__ src = g.src[q];
    float s = 0.0f;
    if (j < g.n_cols)
        for (int r = rg; r < g.rows[q]; r += RG) s += src[(size_t)r * g.ld + j];
    red[rg][c] = s;
    __syncthreads();
    if (rg == 0 && j < g.n_cols) {
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < RG; k++) t += red[k][c];
        g.out[q][j] = t;
    }
}
}  // namespace
}  // namespace yitu

YITU_API int yitu_column_sum_typed(float *const *out, const float *const *x, const int64_t *n_rows,
                                   int64_t n_problems, int64_t n_cols, int64_t ld, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_problems >= 0 && n_cols >= 0 && n_cols < (1 << 24) && ld >= n_cols,
                 "size out of range");
    if (n_problems == 0 || n_cols == 0) return 0;
    YITU_REQUIRE(out && x && n_rows, "null problem table");
    for (int64_t first = 0; first < n_problems; first += kColSumGroup) {
        ColSumGroup g{};
        const int count = (int)std::min<int64_t>(kColSumGroup, n_problems - first);
        for (int i = 0; i < count; i++) {
            const int64_t m = n_rows[first + i];
            YITU_REQUIRE(m >= 0 && m < INT32_MAX && out[first + i] && (m == 0 || x[first + i]),
                         "problem %d: null pointer or size out of range", (int)(first + i));
            g.src[i] = x[first + i];
            g.out[i] = out[first + i];
            g.rows[i] = (int)m;
        }
        g.n_cols = (int)n_cols;
        g.ld = ld;
        if (n_cols <= 32)
            column_sum_group_kernel<32><<<dim3((unsigned)ceil_div(n_cols, 32), (unsigned)count),
                                          kBlock, 0, stream>>>(g);
        else
            column_sum_group_kernel<64><<<dim3((unsigned)ceil_div(n_cols, 64), (unsigned)count),
                                          kBlock, 0, stream>>>(g);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

YITU_API size_t yitu_column_sum_workspace_bytes(int64_t n_rows, int64_t n_cols) {
    return sizeof(float) * (size_t)std::max<int64_t>(ceil_div(n_rows, col_sum_chunk(n_rows)), 1) *
           (size_t)n_cols;
}

YITU_API int yitu_column_sum(float *out, const float *x, int64_t n_rows, int64_t n_cols,
                             void *workspace, size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_rows >= 0 && n_cols >= 0 && n_rows < INT32_MAX && n_cols < (1 << 24),
                 "size out of range");
    if (n_cols == 0) return 0;
    YITU_REQUIRE(out && (n_rows == 0 || x), "null pointer");
    if (n_rows == 0) return fill_zero(out, n_cols, stream);
    YITU_REQUIRE(workspace && workspace_bytes >= yitu_column_sum_workspace_bytes(n_rows, n_cols),
                 "workspace too small: need %zu bytes",
                 yitu_column_sum_workspace_bytes(n_rows, n_cols));
    const int chunk = col_sum_chunk(n_rows);
    const int chunks = (int)ceil_div(n_rows, chunk);
    float *partial = static_cast<float *>(workspace);
    if (n_cols % 4 == 0 && n_cols <= 4 * kBlock && aligned16(x) && aligned16(partial))
        column_chunk_sum4_kernel<<<chunks, kBlock, 0, stream>>>(partial, x, (int)n_rows,
                                                                (int)n_cols, chunk);
    else
        column_chunk_sum_kernel<<<chunks, kBlock, 0, stream>>>(partial, x, (int)n_rows,
                                                               (int)n_cols, chunk);
    YITU_LAUNCH_CHECK();
    partial_sum_kernel<<<(int)ceil_div(n_cols, kSumCols), kBlock, 0, stream>>>(
        out, (int)n_cols, nullptr, 0, partial, chunks);
    YITU_LAUNCH_CHECK();
    return 0;
}
