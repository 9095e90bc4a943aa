// bf16 GEMM with fp32 accumulation on the CDNA4 matrix cores
// (v_mfma_f32_32x32x16_bf16) for the per-type / per-relation feature
// transforms of the heterogeneous path when features are kept in bf16:
//
//   C[M,N] = A[M,K] . B,   A row-major bf16 (K contiguous),
//                          B given as Bt[N,K] (trans_b = 1, the layout of an
//                          nn.Linear weight) or as [K,N] (trans_b = 0: it is
//                          transposed into the workspace first; weights are small),
//                          C row-major fp32 or bf16 (round to nearest even).
//
// With K = N = 256 the product moves 0.4 bytes per flop-pair less than the
// matrix cores need to be busy (128 flop/B against a ridge of about 310), so
// the kernel is built to stream A and C at memory speed: a workgroup owns 128
// rows x 256 columns, reads its rows of A exactly once, and takes the weight
// from L2. K advances in steps of 32 through double-buffered LDS tiles whose
// rows are padded to 80 bytes, so the 16-byte operand reads of 8 consecutive
// lanes fall into different banks; the global loads run four steps ahead.
// Each of the 4 waves owns all 128 rows of 64 columns: 4 x 2 MFMA tiles, 128
// accumulator registers.
#include "../../include/yitu_hip.h"
#include "common.hpp"

#include <algorithm>

namespace yitu {

namespace {

constexpr int HM = 128, HN = 256, HK = 32, HLD = 40;  // HLD: padded LDS row, bf16 elements

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct HGemmParams {
    const uint16_t *A;   // [M, lda]
    const uint16_t *Bt;  // [N, ldbt]
    void *C;             // [M, ldc] fp32 or bf16
    int M, N, K;
    int64_t lda, ldbt, ldc;
};

// round to nearest even; gfx950 converts in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    const __bf16 h = static_cast<__bf16>(f);
    return __builtin_bit_cast(uint16_t, h);
}

template <bool OUT_BF16>
__global__ __launch_bounds__(256, 2) void hgemm_mfma_kernel(HGemmParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t As[2][HM][HLD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[2][HN][HLD];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int m0 = blockIdx.x * HM, n0 = blockIdx.y * HN;  // rows on x: no 65,535 limit
    const int l32 = lane & 31, lk = lane >> 5;
    const int wn = wave * 64;
    const int lrow = t >> 2, lkof = (t & 3) * 8;  // loader: 4 threads cover the 32 k of one row

    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // Global loads run D K-steps ahead of the MFMAs through a ring of registers
    // (one step ahead keeps too few bytes in flight to fill the memory pipe).
    constexpr int D = 4;
    static_assert(D % 2 == 0, "the LDS buffer index must be static inside the unrolled ring");
    constexpr int DB = 2;  // the weight comes from L2: two steps ahead are enough
    uint4 ra[D][2], rb[DB][4];
    auto gload_a = [&](int slot, int k0) {
        const int k = k0 + lkof;  // K is a multiple of 8: k < K means the 8 elements exist
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int row = m0 + lrow + 64 * i;
            ra[slot][i] = (row < p.M && k < p.K)
                              ? *reinterpret_cast<const uint4 *>(p.A + (int64_t)row * p.lda + k)
                              : make_uint4(0, 0, 0, 0);
        }
    };
    auto gload_b = [&](int slot, int k0) {
        const int k = k0 + lkof;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int col = n0 + lrow + 64 * i;
            rb[slot][i] = (col < p.N && k < p.K)
                              ? *reinterpret_cast<const uint4 *>(p.Bt + (int64_t)col * p.ldbt + k)
                              : make_uint4(0, 0, 0, 0);
        }
    };
    auto lstore = [&](int slot, int buf) {
#pragma unroll
        for (int i = 0; i < 2; i++)
            *reinterpret_cast<uint4 *>(&As[buf][lrow + 64 * i][lkof]) = ra[slot][i];
#pragma unroll
        for (int i = 0; i < 4; i++)
            *reinterpret_cast<uint4 *>(&Bs[buf][lrow + 64 * i][lkof]) = rb[slot % DB][i];
    };

#pragma unroll
    for (int u = 0; u < D; u++) gload_a(u, u * HK);
#pragma unroll
    for (int u = 0; u < DB; u++) gload_b(u, u * HK);
    lstore(0, 0);
    __syncthreads();
    const int n_steps = (p.K + HK - 1) / HK;
    for (int s0 = 0; s0 < n_steps; s0 += D) {
#pragma unroll
        for (int u = 0; u < D; u++) {
            const int s = s0 + u;
            if (s < n_steps) {  // same for the whole workgroup
                const int cur = u & 1;        // == s & 1
                // the slots of step s were stored to LDS in step s - 1
                gload_a(u, (s + D) * HK);
                gload_b(u % DB, (s + DB) * HK);
#pragma unroll
                for (int kk = 0; kk < HK; kk += 16) {
                    bf16x8 a[4], b[2];
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        a[i] = *reinterpret_cast<const bf16x8 *>(&As[cur][32 * i + l32][kk + 8 * lk]);
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        b[j] = *reinterpret_cast<const bf16x8 *>(
                            &Bs[cur][wn + 32 * j + l32][kk + 8 * lk]);
#pragma unroll
                    for (int i = 0; i < 4; i++)
#pragma unroll
                        for (int j = 0; j < 2; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j],
                                                                               0, 0, 0);
                }
                // the other buffer was last read in step s-1, before the barrier below
                if (s + 1 < n_steps) lstore((u + 1) % D, cur ^ 1);
                __syncthreads();
            }
        }
    }

    // accumulator element 4*jj + ii of tile (i, j) is C[32i + 8jj + 4*(lane/32) + ii][32j + lane%32]
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = n0 + wn + 32 * j + l32;
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    const int row = m0 + 32 * i + 8 * jj + 4 * lk + ii;
                    if (row < p.M && col < p.N) {
                        const float v = acc[i][j][4 * jj + ii];
                        if constexpr (OUT_BF16)
                            static_cast<uint16_t *>(p.C)[(int64_t)row * p.ldc + col] = f32_to_bf16_rne(v);
                        else
                            static_cast<float *>(p.C)[(int64_t)row * p.ldc + col] = v;
                    }
                }
        }
}

// Inner dimension of at most 256 and many rows: the weight stays in registers. A
// workgroup of 4 waves holds all of Bt[n0 .. n0 + 256, 0 .. K) as MFMA operands (wave w
// keeps 64 columns: 16 K-steps x 2 column tiles x 4 registers), walks row tiles of 32
// rows and reads every one as whole rows: the tile is one contiguous piece of memory when
// lda = K, requested RPF tiles ahead through a ring of registers and passed through a
// double-buffered LDS tile, one barrier per tile. The kernel above asks for 64 bytes of
// every row per K-step and writes its outputs two bytes at a time. Rows of the LDS tile
// are padded to 528 bytes: the 16-byte operand reads of 16 consecutive lanes (16 rows, one
// piece) then cover every bank once, at one address register and an immediate offset per
// K-step. The inner dimension is a template parameter (64, 128 or 256), so the K loop has
// no branch. The weight is the first MFMA operand, so a lane ends up with four consecutive columns of one row;
// a wave passes them through an LDS area of its own and stores 128-byte row segments:
// stores of 8 or 16 bytes per row cost the L2 one request each and ran at half the rate.
constexpr int RM = 32, RPF = 2, RA_LD = 264;
constexpr int RC_LD = 144;  // staged output row: 128 bytes + 16 of padding
constexpr int kRowsProblems = 8;

// Up to 8 products of one width (node types: C_q = A_q . Bt_q^T) share the launch. Their
// row tiles form one list, tile_start[q] is the first tile of problem q; a workgroup
// takes every gridDim.x-th tile and reloads the weight when the problem changes.
struct HRowsParams {
    const uint16_t *A[kRowsProblems];   // [M_q, lda]
    const uint16_t *Bt[kRowsProblems];  // [N, ldbt]
    void *C[kRowsProblems];             // [M_q, ldc] fp32 or bf16
    int M[kRowsProblems];
    int tile_start[kRowsProblems + 1];
    int n_problems, N;
    int64_t lda, ldbt, ldc;
};

template <bool OUT_BF16, int KS>
__global__ __launch_bounds__(256, 2) void hgemm_rows_kernel(HRowsParams p) {
    constexpr int K = 16 * KS;        // inner dimension: KS steps of 16
    constexpr int TPR = K / 8;        // threads that cover one row with 16 bytes each
    constexpr int RPS = 256 / TPR;    // rows the workgroup covers at a time
    constexpr int LR = RM / RPS;      // 16-byte pieces of the tile per thread
    __shared__ __attribute__((aligned(16))) uint16_t As[2][RM][RA_LD];
    __shared__ __attribute__((aligned(16))) unsigned char Cs[4][RM * RC_LD];
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int wn = blockIdx.y * HN + wave * 64;
    unsigned char *stage = Cs[wave];
    // A workgroup takes a run of consecutive tiles of the list of all problems: it then
    // crosses from one problem into the next once at most (and loads a weight once or
    // twice), where every gridDim.x-th tile took it through all of them.
    constexpr int stride = 1;
    const int n_all = p.tile_start[p.n_problems];
    const int per_wg = (n_all + (int)gridDim.x - 1) / (int)gridDim.x;
    const int my_lo = blockIdx.x * per_wg, my_hi = min(my_lo + per_wg, n_all);
    // per wave: its 64 columns lie wholly inside the output (vector stores through the
    // staging area), partly (element by element), or not at all (nothing to compute)
    const bool whole_cols = wn + 64 <= p.N, no_cols = wn >= p.N;
    // loader: TPR threads cover one row, the workgroup RPS rows at a time. Rows past the
    // end are read from the last row (their outputs are never stored) and tiles past the
    // end from the last tile: no load of the ring is conditional.
    const int lrow = t / TPR, lk_ld = (t % TPR) * 8;

    for (int q = 0; q < p.n_problems; q++) {
    const int lo = p.tile_start[q];
    // this workgroup's tiles of the problem
    const int tile0 = max(lo, my_lo), hi = min(p.tile_start[q + 1], my_hi);
    if (tile0 >= hi) continue;  // same for the whole workgroup
    const uint16_t *a_q = p.A[q], *bt = p.Bt[q];
    void *c_q = p.C[q];
    const int m_q = p.M[q];
    bf16x8 b[KS][2];
#pragma unroll
    for (int s = 0; s < KS; s++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = min(wn + 32 * j + l32, p.N - 1);  // columns past N: never stored
            b[s][j] = __builtin_bit_cast(
                bf16x8,
                *reinterpret_cast<const uint4 *>(bt + (int64_t)col * p.ldbt + 16 * s + 8 * lk));
        }
    u32x4 ra[RPF][LR];
    auto gload = [&](int slot, int64_t tile64) {
        const int tile = (int)std::min<int64_t>(tile64, hi - 1);
        const int r0 = (tile - lo) * RM + lrow;
#pragma unroll
        for (int i = 0; i < LR; i++) {
            const int64_t row = min(r0 + RPS * i, m_q - 1);
            ra[slot][i] = __builtin_nontemporal_load(
                reinterpret_cast<const u32x4 *>(a_q + row * p.lda + lk_ld));
        }
    };
#pragma unroll
    for (int u = 0; u < RPF; u++) {
        gload(u, tile0 + (int64_t)u * stride);
        __builtin_amdgcn_sched_barrier(0);  // oldest first
    }
    for (int it0 = 0; tile0 + (int64_t)it0 * stride < hi; it0 += RPF) {
#pragma unroll
        for (int u = 0; u < RPF; u++) {
            const int it = it0 + u;
            const int64_t tile64 = tile0 + (int64_t)it * stride;
            if (tile64 >= hi) break;  // same for the whole workgroup
            const int tile = (int)tile64, buf = it & 1;
            // this buffer was last read two tiles ago, before the previous barrier
#pragma unroll
            for (int i = 0; i < LR; i++)
                *reinterpret_cast<u32x4 *>(&As[buf][lrow + RPS * i][lk_ld]) = ra[u][i];
            __syncthreads();
            gload(u, tile64 + (int64_t)RPF * stride);
            f32x16 acc[2];
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[j][e] = 0.0f;
            if (no_cols) continue;  // (after the barrier and the loads that every wave shares)
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const bf16x8 a =
                    *reinterpret_cast<const bf16x8 *>(&As[buf][l32][16 * s + 8 * lk]);
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[s][j], a, acc[j], 0, 0, 0);
                // operand reads stay at most four steps ahead of their products: hoisted
                // all the way they would not fit beside the weight
                if (s % 4 == 3) __builtin_amdgcn_sched_barrier(0);
            }
            // accumulator element 4 jj + ii of column tile j is
            // C[32 tile + lane % 32][wn + 32 j + 8 jj + 4 (lane / 32) + ii]
            const int row0 = (tile - lo) * RM;
            if (whole_cols && row0 + RM <= m_q) {  // same for the whole wave
                if constexpr (OUT_BF16) {
#pragma unroll
                    for (int j = 0; j < 2; j++)
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) {
                            u32x2 w;
                            w[0] = (unsigned)f32_to_bf16_rne(acc[j][4 * jj]) |
                                   ((unsigned)f32_to_bf16_rne(acc[j][4 * jj + 1]) << 16);
                            w[1] = (unsigned)f32_to_bf16_rne(acc[j][4 * jj + 2]) |
                                   ((unsigned)f32_to_bf16_rne(acc[j][4 * jj + 3]) << 16);
                            *reinterpret_cast<u32x2 *>(stage + l32 * RC_LD + 64 * j + 16 * jj +
                                                       8 * lk) = w;
                        }
#pragma unroll
                    for (int r = 0; r < RM / 8; r++) {
                        const int row = 8 * r + (lane >> 3);
                        const u32x4 w = *reinterpret_cast<const u32x4 *>(stage + row * RC_LD +
                                                                         16 * (lane & 7));
                        __builtin_nontemporal_store(
                            w, reinterpret_cast<u32x4 *>(static_cast<uint16_t *>(c_q) +
                                                         (int64_t)(row0 + row) * p.ldc + wn +
                                                         8 * (lane & 7)));
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 2; j++) {
#pragma unroll
                        for (int jj = 0; jj < 4; jj++) {
                            const f4 w = {acc[j][4 * jj], acc[j][4 * jj + 1], acc[j][4 * jj + 2],
                                          acc[j][4 * jj + 3]};
                            *reinterpret_cast<f4 *>(stage + l32 * RC_LD + 32 * jj + 16 * lk) = w;
                        }
#pragma unroll
                        for (int r = 0; r < RM / 8; r++) {
                            const int row = 8 * r + (lane >> 3);
                            const f4 w = *reinterpret_cast<const f4 *>(stage + row * RC_LD +
                                                                       16 * (lane & 7));
                            *reinterpret_cast<f4 *>(static_cast<float *>(c_q) +
                                                    (int64_t)(row0 + row) * p.ldc + wn + 32 * j +
                                                    4 * (lane & 7)) = w;
                        }
                    }
                }
            } else if (row0 + l32 < m_q) {
                const int64_t row = row0 + l32;
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int e = 0; e < 16; e++) {
                        const int col = wn + 32 * j + 8 * (e / 4) + 4 * lk + e % 4;
                        if (col < p.N) {
                            if constexpr (OUT_BF16)
                                static_cast<uint16_t *>(c_q)[row * p.ldc + col] =
                                    f32_to_bf16_rne(acc[j][e]);
                            else
                                static_cast<float *>(c_q)[row * p.ldc + col] = acc[j][e];
                        }
                    }
            }
        }
    }
    __syncthreads();  // the next problem starts over with the first LDS buffer
    }
}

// Launches the kernel above for problems of one width; false when the shape is not one
// of its own (the caller then takes the general kernel per problem).
bool rows_kernel_takes(int64_t total_rows, int64_t k, const void *const *c, int n_problems,
                       int c_is_bf16, int64_t ldc) {
    if (!(k == 64 || k == 128 || k == 256) || total_rows < 4096) return false;
    // the staged stores write 16 bytes at a time: C rows must keep them aligned
    if (ldc % (c_is_bf16 ? 8 : 4) != 0) return false;
    for (int q = 0; q < n_problems; q++)
        if (!aligned16(c[q])) return false;
    return true;
}

int rows_kernel_launch(const HRowsParams &p, int k, int c_is_bf16, hipStream_t stream) {
    const int n_tiles = p.tile_start[p.n_problems];
    dim3 grid((unsigned)std::min(n_tiles, 512), (unsigned)ceil_div(p.N, HN));
    if (k == 256) {
        if (c_is_bf16) hgemm_rows_kernel<true, 16><<<grid, 256, 0, stream>>>(p);
        else hgemm_rows_kernel<false, 16><<<grid, 256, 0, stream>>>(p);
    } else if (k == 128) {
        if (c_is_bf16) hgemm_rows_kernel<true, 8><<<grid, 256, 0, stream>>>(p);
        else hgemm_rows_kernel<false, 8><<<grid, 256, 0, stream>>>(p);
    } else {
        if (c_is_bf16) hgemm_rows_kernel<true, 4><<<grid, 256, 0, stream>>>(p);
        else hgemm_rows_kernel<false, 4><<<grid, 256, 0, stream>>>(p);
    }
    YITU_LAUNCH_CHECK();
    return 0;
}

// dst[n][k] = src[k][n] for a [K, N] matrix of 16-bit elements (32 x 32 tiles through LDS)
struct Transpose16Params {
    uint16_t *dst[kRowsProblems];        // [N, ld_dst]
    const uint16_t *src[kRowsProblems];  // [K, ld_src]
};

__global__ __launch_bounds__(256) void transpose16_kernel(Transpose16Params tp, int K, int N,
                                                          int64_t ld_src, int64_t ld_dst) {
    __shared__ uint16_t tile[32][33];
    uint16_t *__restrict__ dst = tp.dst[blockIdx.z];
    const uint16_t *__restrict__ src = tp.src[blockIdx.z];
    const int k0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8)
        tile[r][tx] = (k0 + r < K && n0 + tx < N) ? src[(int64_t)(k0 + r) * ld_src + n0 + tx] : 0;
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (n0 + r < N && k0 + tx < K) dst[(int64_t)(n0 + r) * ld_dst + k0 + tx] = tile[tx][r];
}


// ---- C[Ki, No] = A^T . B : the weight gradient dW = X^T . dY ------------------------
// A [M, lda] and B [M, ldb] are row-major bf16, the sum runs over their (many) rows,
// the output is small. The matrix instruction wants each lane to hold 8 consecutive
// elements ALONG the summed index, which in memory are a row stride apart. A
// workgroup therefore stages 32 rows x 128 columns of both operands in LDS as they
// lie in memory (16-byte global loads, one stage ahead in registers); a lane then
// reads one dword = two neighbouring columns from each of its 8 rows and splits them
// with byte permutes into the operand of the even column and the operand of the odd
// column. Output tile rows are thereby interleaved (even columns, then odd ones),
// which only matters when the tile is written. Each wave owns 64 x 64 of the
// workgroup's 128 x 128 tile. The rows are split over the grid; every workgroup
// writes its partial tile and a second kernel adds the partials in chunk order
// (bitwise reproducible).
constexpr int TN_TILE = 128, TN_ROWS = 32, TN_LD = TN_TILE + 4;  // padded LDS row (bf16)

// Up to 8 products of one shape share the launch: their row chunks form one list,
// chunk_start[q] is the first chunk of problem q.
struct TnParams {
    const uint16_t *A[kRowsProblems], *B[kRowsProblems];
    float *C[kRowsProblems];  // [Ki, ldc]
    int M[kRowsProblems];
    int chunk_start[kRowsProblems + 1];
    int n_problems;
    float *partial;  // [chunks of all problems, Ki, No]
    int Ki, No;
    int64_t lda, ldb, ldc;
    int rows_per_chunk;  // multiple of TN_ROWS
    int accumulate;
};

constexpr int TN_DEPTH = 3;  // row stages requested ahead of the products

__global__ __launch_bounds__(256, 3) void hgemm_tn_kernel(TnParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t As[2][TN_ROWS][TN_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[2][TN_ROWS][TN_LD];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    // Workgroups go to the 8 XCDs in turn. The output tiles of one row chunk read the same
    // rows, so they are given ids that differ by multiples of 8: they run on one XCD, close
    // in time, and all but the first find the rows in that XCD's L2. Spread over the XCDs
    // every row crossed the fabric once per tile that reads it.
    const int tiles_j = (p.No + TN_TILE - 1) / TN_TILE;
    const int n_tiles = tiles_j * ((p.Ki + TN_TILE - 1) / TN_TILE);
    const int tile = (blockIdx.x / 8) % n_tiles;
    const int chunk = (blockIdx.x / 8 / n_tiles) * 8 + blockIdx.x % 8;
    if (chunk >= p.chunk_start[p.n_problems]) return;  // same for the whole workgroup
    const int i0 = (tile / tiles_j) * TN_TILE, j0 = (tile % tiles_j) * TN_TILE;
    const int wi = (wave >> 1) * 64, wj = (wave & 1) * 64;
    int q = 0;  // the chunk's problem (same for the whole workgroup)
#pragma unroll
    for (int k = 1; k < kRowsProblems; k++)
        q += (k < p.n_problems && chunk >= p.chunk_start[k]) ? 1 : 0;
    const uint16_t *__restrict__ A = p.A[q], *__restrict__ B = p.B[q];
    const int m_beg = (chunk - p.chunk_start[q]) * p.rows_per_chunk;
    const int m_end = min(p.M[q], m_beg + p.rows_per_chunk);
    // loader: thread -> (row, 8 columns); 16 threads cover the 128 columns of a row
    const int lrow = t >> 4, lcol = (t & 15) * 8;

    f32x16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[a][b][e] = 0.0f;

    // Rows are requested TN_DEPTH stages ahead through a ring of registers: one stage
    // ahead left 16 KB per workgroup in flight, too little to cover the memory latency.
    uint4 ra[TN_DEPTH][2], rb[TN_DEPTH][2];
    const bool a_cols = i0 + lcol < p.Ki, b_cols = j0 + lcol < p.No;
    auto gload = [&](int slot, int m0) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int row = m0 + lrow + 16 * h;
            const bool in = row < m_end;
            // Ki, No are multiples of 8: a column below the bound has its 8 elements
            ra[slot][h] = (in && a_cols)
                              ? *reinterpret_cast<const uint4 *>(A + (int64_t)row * p.lda + i0 + lcol)
                              : make_uint4(0, 0, 0, 0);
            rb[slot][h] = (in && b_cols)
                              ? *reinterpret_cast<const uint4 *>(B + (int64_t)row * p.ldb + j0 + lcol)
                              : make_uint4(0, 0, 0, 0);
        }
    };
    auto lstore = [&](int slot, int buf) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            *reinterpret_cast<uint2 *>(&As[buf][lrow + 16 * h][lcol]) =
                make_uint2(ra[slot][h].x, ra[slot][h].y);
            *reinterpret_cast<uint2 *>(&As[buf][lrow + 16 * h][lcol + 4]) =
                make_uint2(ra[slot][h].z, ra[slot][h].w);
            *reinterpret_cast<uint2 *>(&Bs[buf][lrow + 16 * h][lcol]) =
                make_uint2(rb[slot][h].x, rb[slot][h].y);
            *reinterpret_cast<uint2 *>(&Bs[buf][lrow + 16 * h][lcol + 4]) =
                make_uint2(rb[slot][h].z, rb[slot][h].w);
        }
    };
    // operand pair (even column, odd column) of the 8 rows kk + 8 * lk .. + 7
    auto fragments = [&](const uint16_t (*tile)[TN_LD], int col0, int kk, bf16x8 &even, bf16x8 &odd) {
        uint32_t raw[8];
#pragma unroll
        for (int k = 0; k < 8; k++)
            raw[k] = *reinterpret_cast<const uint32_t *>(&tile[kk + 8 * lk + k][col0 + 2 * l32]);
        uint32_t e[4], o[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            e[q] = __builtin_amdgcn_perm(raw[2 * q + 1], raw[2 * q], 0x05040100u);
            o[q] = __builtin_amdgcn_perm(raw[2 * q + 1], raw[2 * q], 0x07060302u);
        }
        even = __builtin_bit_cast(bf16x8, make_uint4(e[0], e[1], e[2], e[3]));
        odd = __builtin_bit_cast(bf16x8, make_uint4(o[0], o[1], o[2], o[3]));
    };

    if (m_beg < m_end) {
        const int n_steps = (m_end - m_beg + TN_ROWS - 1) / TN_ROWS;
#pragma unroll
        for (int u = 0; u < TN_DEPTH; u++) gload(u, m_beg + u * TN_ROWS);  // past the end: zeros
        lstore(0, 0);
        __syncthreads();
        for (int s0 = 0; s0 < n_steps; s0 += TN_DEPTH) {
#pragma unroll
            for (int u = 0; u < TN_DEPTH; u++) {
                const int st = s0 + u;
                if (st >= n_steps) break;  // same for the whole workgroup
                const int buf = st & 1;
                // stage st went to LDS during stage st - 1: its slot takes stage st + TN_DEPTH
                gload(u, m_beg + (st + TN_DEPTH) * TN_ROWS);
#pragma unroll
                for (int kk = 0; kk < TN_ROWS; kk += 16) {
                    bf16x8 a[2], b[2];
                    fragments(As[buf], wi, kk, a[0], a[1]);
                    fragments(Bs[buf], wj, kk, b[0], b[1]);
#pragma unroll
                    for (int x = 0; x < 2; x++)
#pragma unroll
                        for (int y = 0; y < 2; y++)
                            acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[x], b[y], acc[x][y],
                                                                               0, 0, 0);
                }
                if (st + 1 < n_steps) lstore((u + 1) % TN_DEPTH, buf ^ 1);
                __syncthreads();
            }
        }
    }
    // accumulator element 4*jj + ii of tile (x, y) is row 8jj + 4lk + ii, column l32 of the
    // MFMA tile; MFMA row r of parity x is output row wi + 2r + x, column c of parity y is
    // output column wj + 2c + y
    float *dst = p.partial + (int64_t)chunk * p.Ki * p.No;
#pragma unroll
    for (int x = 0; x < 2; x++)
#pragma unroll
        for (int y = 0; y < 2; y++) {
            const int col = j0 + wj + 2 * l32 + y;
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    const int row = i0 + wi + 2 * (8 * jj + 4 * lk + ii) + x;
                    if (row < p.Ki && col < p.No) dst[(int64_t)row * p.No + col] = acc[x][y][4 * jj + ii];
                }
        }
}

// C_q (+)= sum over the problem's chunks of its partial products, in a fixed order. A
// workgroup takes 64 consecutive outputs; its four 64-thread groups each add a quarter of
// the chunks with four independent running sums and the quarters are combined through
// LDS (one thread per output walking every chunk is a chain of dependent loads).
__global__ __launch_bounds__(256) void hgemm_tn_reduce_kernel(TnParams p) {
    __shared__ float red[4][64];
    const int q = blockIdx.y;
    const int c0 = p.chunk_start[q], n_chunks = p.chunk_start[q + 1] - c0;
    if (p.M[q] == 0 && p.accumulate) return;
    const int64_t total = (int64_t)p.Ki * p.No;
    const int e_lane = threadIdx.x & 63, zg = threadIdx.x >> 6;
    const int per = (n_chunks + 3) / 4;
    const int zb = min(zg * per, n_chunks), ze = min(zb + per, n_chunks);
    float *__restrict__ c = p.C[q];
    for (int64_t e0 = (int64_t)blockIdx.x * 64; e0 < total; e0 += (int64_t)gridDim.x * 64) {
        const int64_t e = e0 + e_lane;
        const bool live = e < total;
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
        if (live) {
            const float *src = p.partial + (size_t)c0 * total + e;
            int z = zb;
            for (; z + 4 <= ze; z += 4) {
                a0 += src[(size_t)z * total];
                a1 += src[(size_t)(z + 1) * total];
                a2 += src[(size_t)(z + 2) * total];
                a3 += src[(size_t)(z + 3) * total];
            }
            for (; z < ze; z++) a0 += src[(size_t)z * total];
        }
        red[zg][e_lane] = (a0 + a1) + (a2 + a3);
        __syncthreads();
        if (zg == 0 && live) {
            const float sum = ((red[0][e_lane] + red[1][e_lane]) + red[2][e_lane]) + red[3][e_lane];
            float *out = c + (e / p.No) * p.ldc + e % p.No;
            *out = p.accumulate ? *out + sum : sum;
        }
        __syncthreads();
    }
}

// Row chunks of the A^T.B products: as many workgroups as the chip holds at once (three
// per CU) over all the problems of a launch and no more, since a few left over would run
// alone for as long again; chunks a multiple of the stage height. Every problem may add a
// chunk by rounding, and the chunk count is rounded up to a multiple of 8.
inline int tn_chunk_rows(int64_t total_rows, int64_t ki, int64_t no, int count) {
    const int64_t tiles = ceil_div(ki, TN_TILE) * ceil_div(no, TN_TILE);
    const int64_t want_chunks = std::max<int64_t>(1, 768 / tiles - count - 7);
    int64_t rows = ceil_div(ceil_div(total_rows, want_chunks), TN_ROWS) * TN_ROWS;
    return (int)std::max<int64_t>(rows, 4 * TN_ROWS);
}

// chunks of a group of problems that share one launch (an empty problem keeps one chunk
// of zeros, so that its output is written)
inline int64_t tn_group_chunks(const int64_t *m, int count, int rows) {
    int64_t chunks = 0;
    for (int q = 0; q < count; q++) chunks += std::max<int64_t>(1, ceil_div(m[q], rows));
    return chunks;
}

inline int64_t tn_group_rows(const int64_t *m, int count) {
    int64_t total = 0;
    for (int q = 0; q < count; q++) total += m[q];
    return total;
}

}  // namespace

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API size_t yitu_gemm_bf16_workspace_bytes(int64_t n, int64_t k, int trans_b) {
    return trans_b ? 256 : align_up((size_t)(n * k) * sizeof(uint16_t), 256) + 256;
}

YITU_API int yitu_gemm_bf16(void *c, int c_is_bf16, const void *a, const void *b, int64_t m,
                            int64_t n, int64_t k, int trans_b, int64_t lda, int64_t ldb,
                            int64_t ldc, void *workspace, size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(m >= 0 && n >= 0 && k >= 0, "negative size");
    if (m == 0 || n == 0) return 0;
    YITU_REQUIRE(c && (k == 0 || (a && b)), "null operand");
    YITU_REQUIRE(m < INT32_MAX && n < INT32_MAX && k < INT32_MAX && ldc >= n, "size out of range");
    YITU_REQUIRE(k % 8 == 0 && lda % 8 == 0 && lda >= k && aligned16(a),
                 "bf16 GEMM needs K and lda to be multiples of 8 and A 16-byte aligned");
    YITU_REQUIRE(ldb >= (trans_b ? k : n), "leading dimension of B too small");
    HGemmParams p{};
    p.A = static_cast<const uint16_t *>(a);
    p.C = c;
    p.M = (int)m;
    p.N = (int)n;
    p.K = (int)k;
    p.lda = lda;
    p.ldc = ldc;
    if (trans_b) {
        YITU_REQUIRE(ldb % 8 == 0 && aligned16(b),
                     "bf16 GEMM needs ldb to be a multiple of 8 and B 16-byte aligned");
        p.Bt = static_cast<const uint16_t *>(b);
        p.ldbt = ldb;
    } else if (k > 0) {
        const size_t need = (size_t)(n * k) * sizeof(uint16_t);
        YITU_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace),
                     "workspace too small for the transposed weight: need %zu bytes", need);
        dim3 tg((unsigned)ceil_div(n, 32), (unsigned)ceil_div(k, 32));
        Transpose16Params tp{};
        tp.dst[0] = static_cast<uint16_t *>(workspace);
        tp.src[0] = static_cast<const uint16_t *>(b);
        transpose16_kernel<<<tg, 256, 0, stream>>>(tp, (int)k, (int)n, ldb, k);
        YITU_LAUNCH_CHECK();
        p.Bt = static_cast<const uint16_t *>(workspace);
        p.ldbt = k;
    }
    if (rows_kernel_takes(m, k, &c, 1, c_is_bf16, ldc)) {
        HRowsParams r{};
        r.A[0] = p.A;
        r.Bt[0] = p.Bt;
        r.C[0] = c;
        r.M[0] = (int)m;
        r.tile_start[1] = (int)ceil_div(m, RM);
        r.n_problems = 1;
        r.N = (int)n;
        r.lda = lda;
        r.ldbt = p.ldbt;
        r.ldc = ldc;
        return rows_kernel_launch(r, (int)k, c_is_bf16, stream);
    }
    dim3 grid((unsigned)ceil_div(m, HM), (unsigned)ceil_div(n, HN));
    if (c_is_bf16)
        hgemm_mfma_kernel<true><<<grid, 256, 0, stream>>>(p);
    else
        hgemm_mfma_kernel<false><<<grid, 256, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    return 0;
}


YITU_API size_t yitu_gemm_bf16_typed_workspace_bytes(int64_t n_problems, int64_t n, int64_t k,
                                                     int trans_b) {
    if (trans_b) return 256;
    const int64_t group = std::min<int64_t>(std::max<int64_t>(n_problems, 1), kRowsProblems);
    return (size_t)group * align_up((size_t)(n * k) * sizeof(uint16_t), 256) + 256;
}

YITU_API int yitu_gemm_bf16_typed(void *const *c, int c_is_bf16, const void *const *a,
                                  const void *const *b, const int64_t *m, int64_t n_problems,
                                  int64_t n, int64_t k, int trans_b, int64_t lda, int64_t ldb,
                                  int64_t ldc, void *workspace, size_t workspace_bytes,
                                  void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_problems >= 0 && n >= 0 && k >= 0, "negative size");
    if (n_problems == 0 || n == 0) return 0;
    YITU_REQUIRE(c && a && b && m, "null pointer list");
    YITU_REQUIRE(n < INT32_MAX && k < INT32_MAX && ldc >= n, "size out of range");
    YITU_REQUIRE(k % 8 == 0 && lda % 8 == 0 && lda >= k,
                 "bf16 GEMM needs K and lda to be multiples of 8");
    YITU_REQUIRE(ldb >= (trans_b ? k : n), "leading dimension of B too small");
    int64_t total = 0;
    bool aligned = trans_b ? ldb % 8 == 0 : true;
    for (int64_t q = 0; q < n_problems; q++) {
        YITU_REQUIRE(m[q] >= 0 && m[q] < INT32_MAX, "row count out of range");
        YITU_REQUIRE(m[q] == 0 || (c[q] && (k == 0 || (a[q] && b[q]))), "null operand");
        total += m[q];
        aligned = aligned && aligned16(a[q]) && (!trans_b || aligned16(b[q]));
    }
    const size_t slot = align_up((size_t)(n * k) * sizeof(uint16_t), 256);
    const bool fits = trans_b || (workspace && aligned16(workspace) &&
                                  workspace_bytes >= yitu_gemm_bf16_typed_workspace_bytes(
                                                         n_problems, n, k, trans_b));
    if (!(aligned && fits && total < INT32_MAX &&
          rows_kernel_takes(total, k, c, (int)n_problems, c_is_bf16, ldc))) {
        for (int64_t q = 0; q < n_problems; q++) {
            const int rc = yitu_gemm_bf16(c[q], c_is_bf16, a[q], b[q], m[q], n, k, trans_b, lda,
                                          ldb, ldc, workspace, workspace_bytes, stream_);
            if (rc) return rc;
        }
        return 0;
    }
    for (int64_t g0 = 0; g0 < n_problems; g0 += kRowsProblems) {
        const int cnt = (int)std::min<int64_t>(kRowsProblems, n_problems - g0);
        HRowsParams r{};
        Transpose16Params tp{};
        for (int q = 0; q < cnt; q++) {
            r.A[q] = static_cast<const uint16_t *>(a[g0 + q]);
            r.C[q] = c[g0 + q];
            r.M[q] = (int)m[g0 + q];
            r.tile_start[q + 1] = r.tile_start[q] + (int)ceil_div(m[g0 + q], RM);
            if (trans_b) {
                r.Bt[q] = static_cast<const uint16_t *>(b[g0 + q]);
            } else {
                tp.dst[q] = reinterpret_cast<uint16_t *>(static_cast<char *>(workspace) + q * slot);
                tp.src[q] = static_cast<const uint16_t *>(b[g0 + q]);
                r.Bt[q] = tp.dst[q];
            }
        }
        r.n_problems = cnt;
        r.N = (int)n;
        r.lda = lda;
        r.ldbt = trans_b ? ldb : k;
        r.ldc = ldc;
        if (r.tile_start[cnt] == 0) continue;
        if (!trans_b) {
            dim3 tg((unsigned)ceil_div(n, 32), (unsigned)ceil_div(k, 32), (unsigned)cnt);
            transpose16_kernel<<<tg, 256, 0, stream>>>(tp, (int)k, (int)n, ldb, k);
            YITU_LAUNCH_CHECK();
        }
        const int rc = rows_kernel_launch(r, (int)k, c_is_bf16, stream);
        if (rc) return rc;
    }
    return 0;
}


YITU_API size_t yitu_gemm_bf16_tn_typed_workspace_bytes(const int64_t *m, int64_t n_problems,
                                                        int64_t ki, int64_t no) {
    int64_t most = 1;
    for (int64_t g0 = 0; m && g0 < n_problems; g0 += kRowsProblems) {
        const int cnt = (int)std::min<int64_t>(kRowsProblems, n_problems - g0);
        const int rows = tn_chunk_rows(tn_group_rows(m + g0, cnt), ki, no, cnt);
        most = std::max(most, tn_group_chunks(m + g0, cnt, rows));
    }
    return align_up((size_t)(most * ki * no) * sizeof(float), 256) + 256;
}

YITU_API int yitu_gemm_bf16_tn_typed(float *const *c, const void *const *a, const void *const *b,
                                     const int64_t *m, int64_t n_problems, int64_t ki, int64_t no,
                                     int64_t lda, int64_t ldb, int64_t ldc, int accumulate,
                                     void *workspace, size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_problems >= 0 && ki >= 0 && no >= 0, "negative size");
    if (n_problems == 0 || ki == 0 || no == 0) return 0;
    YITU_REQUIRE(c && a && b && m, "null pointer list");
    YITU_REQUIRE(ki < (1 << 20) && no < (1 << 20) && ldc >= no, "size out of range");
    YITU_REQUIRE(ki % 8 == 0 && no % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && lda >= ki &&
                     ldb >= no,
                 "bf16 A^T.B needs both widths and leading dimensions to be multiples of 8");
    for (int64_t q = 0; q < n_problems; q++) {
        YITU_REQUIRE(m[q] >= 0 && m[q] < INT32_MAX, "row count out of range");
        YITU_REQUIRE(c[q] && (m[q] == 0 || (a[q] && b[q])), "null operand");
        YITU_REQUIRE(aligned16(a[q]) && aligned16(b[q]), "bf16 A^T.B needs 16-byte aligned operands");
    }
    const size_t need = yitu_gemm_bf16_tn_typed_workspace_bytes(m, n_problems, ki, no) - 256;
    YITU_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace),
                 "workspace too small for the partial products: need %zu bytes", need);
    for (int64_t g0 = 0; g0 < n_problems; g0 += kRowsProblems) {
        const int cnt = (int)std::min<int64_t>(kRowsProblems, n_problems - g0);
        TnParams p{};
        p.rows_per_chunk = tn_chunk_rows(tn_group_rows(m + g0, cnt), ki, no, cnt);
        for (int q = 0; q < cnt; q++) {
            p.A[q] = static_cast<const uint16_t *>(a[g0 + q]);
            p.B[q] = static_cast<const uint16_t *>(b[g0 + q]);
            p.C[q] = c[g0 + q];
            p.M[q] = (int)m[g0 + q];
            p.chunk_start[q + 1] =
                p.chunk_start[q] +
                (int)std::max<int64_t>(1, ceil_div(m[g0 + q], (int64_t)p.rows_per_chunk));
        }
        p.n_problems = cnt;
        p.partial = static_cast<float *>(workspace);
        p.Ki = (int)ki;
        p.No = (int)no;
        p.lda = lda;
        p.ldb = ldb;
        p.ldc = ldc;
        p.accumulate = accumulate;
        const int64_t wgs = ceil_div((int64_t)p.chunk_start[cnt], 8) * 8 * ceil_div(ki, TN_TILE) *
                            ceil_div(no, TN_TILE);
        hgemm_tn_kernel<<<(unsigned)wgs, 256, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        dim3 rgrid((unsigned)std::min<int64_t>(ceil_div(ki * no, 64), 4096), (unsigned)cnt);
        hgemm_tn_reduce_kernel<<<rgrid, 256, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

YITU_API size_t yitu_gemm_bf16_tn_workspace_bytes(int64_t m, int64_t ki, int64_t no) {
    return yitu_gemm_bf16_tn_typed_workspace_bytes(&m, 1, ki, no);
}

YITU_API int yitu_gemm_bf16_tn(float *c, const void *a, const void *b, int64_t m, int64_t ki,
                               int64_t no, int64_t lda, int64_t ldb, int64_t ldc, int accumulate,
                               void *workspace, size_t workspace_bytes, void *stream_) {
    YITU_REQUIRE(m >= 0, "negative size");
    if (ki == 0 || no == 0) return 0;
    YITU_REQUIRE(c && (m == 0 || (a && b)), "null operand");
    return yitu_gemm_bf16_tn_typed(&c, &a, &b, &m, 1, ki, no, lda, ldb, ldc, accumulate, workspace,
                                   workspace_bytes, stream_);
}
