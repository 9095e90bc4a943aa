// fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x2_f32) for the dense
// products of the heterogeneous path (two Linear layers sharing one input,
// fc_cuda.cu) and the X.W / G.W^T / X^T.G products around the GCN / GIN
// aggregation (YiTu_GNN_kernel.cu:276,471-472,606,715-716).
//
//   C[M,N] (+)= A[M,K] . B[K,N],  element (i,k) of A at A + i*a_si + k*a_sk,
//                                  element (k,j) of B at B + k*b_sk + j*b_sj,
// one of each stride pair being 1, C row-major. Up to 32 problems that share
// N and the strides, each with its own M and K, are grouped into one launch
// (blockIdx.z walks the problems and their K splits).
//
// Tiling: 128x128 output tile per 256-thread workgroup, each of the 4 waves
// owns 64x64 = 2x2 MFMA tiles (64 accumulator registers); K advances in steps
// of 16 through double-buffered LDS tiles stored K-major, so an MFMA operand
// read is 32 consecutive floats per half wave (conflict free). Operands that
// are K-contiguous in memory are transposed on their way into LDS. The next
// K-step's global loads are issued before the current step's MFMAs.
#include "../../include/yitu_hip.h"
#include "spmm_rows.hpp"

namespace yitu {

constexpr int BK = 16;  // K-step
constexpr int kMaxGroup = 32;  // problems per launch (their table travels as kernel arguments)
constexpr int kMinSplitK = 128;  // shortest K range worth a workgroup of its own

typedef float float16v __attribute__((ext_vector_type(16)));

struct GemmProblem {
    const float *A;
    const float *B;
    float *C;
    int M, K;
    // split-K: this problem owns blockIdx.z in [z0, z0 + n_split); split s covers
    // the K range [s * k_chunk, min(K, (s+1) * k_chunk)) and, when n_split > 1,
    // writes its own [M, N] slab of `partial` (slab index = blockIdx.z)
    int z0, n_split, k_chunk;
    const float *bias = nullptr;  // [N], added to every row (the many-rows kernel only)
};

struct GemmParams {
    GemmProblem prob[kMaxGroup];
    int n_prob;
    int N;
    int64_t a_si, a_sk, b_sk, b_sj;
    int ldc;
    int accumulate;  // C += A.B instead of C = A.B
    int a_vec4, b_vec4;  // bounds-checked tiles: 16-byte loads are all-or-nothing for this operand
    int max_m;       // slabs of `partial` are [max_m, N]
    float *partial;
};

__device__ __forceinline__ int problem_of(const GemmParams &p, int z) {
    int i = 0;
    while (i + 1 < p.n_prob && z >= p.prob[i + 1].z0) i++;
    return i;
}

// Tile geometry: a workgroup of 4 waves (2 x 2) owns a square tile of 64 * TM rows
// and columns, each wave TM x TM MFMA tiles. TM = 2 (128 x 128) is the shape for
// large products; TM = 1 (64 x 64, a quarter of the MFMAs per K-step and four
// times the workgroups) is taken when the larger tiles would leave most CUs idle.
template <int TM>
struct TileGeom {
    static constexpr int R = 64 * TM;       // rows (and columns) per workgroup tile
    static constexpr int PER = 4 * TM;      // elements per thread and operand tile
    static constexpr int LD = R + 4;        // padded LDS row, floats
};

// Loads this thread's PER elements of an [R x 16] operand tile into regs.
// KCONT: the operand is contiguous along K (thread owns PER consecutive k of one row),
// otherwise contiguous along the row dimension (PER consecutive rows of one k).
template <int TM, bool KCONT, bool FAST>
__device__ __forceinline__ void load_tile(float (&r)[4 * TM], const float *__restrict__ base,
                                          int64_t s_row, int64_t s_k, int row0, int k0, int n_rows,
                                          int K, bool vec4) {
    constexpr int PER = TileGeom<TM>::PER;
    const int t = threadIdx.x;
    if constexpr (KCONT) {
        constexpr int TPR = BK / PER;  // threads per row
        const int row = row0 + t / TPR, k = k0 + (t % TPR) * PER;
        const float *p = base + (int64_t)row * s_row + k;
        if constexpr (FAST) {
#pragma unroll
            for (int h = 0; h < TM; h++) {
                const float4 v = *reinterpret_cast<const float4 *>(p + 4 * h);
                r[4 * h] = v.x; r[4 * h + 1] = v.y; r[4 * h + 2] = v.z; r[4 * h + 3] = v.w;
            }
        } else if (vec4) {  // K and the row stride are multiples of 4: whole float4 or nothing
#pragma unroll
            for (int h = 0; h < TM; h++) {
                const float4 v = (row < n_rows && k + 4 * h + 4 <= K)
                                     ? *reinterpret_cast<const float4 *>(p + 4 * h)
                                     : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                r[4 * h] = v.x; r[4 * h + 1] = v.y; r[4 * h + 2] = v.z; r[4 * h + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < PER; i++) r[i] = (row < n_rows && k + i < K) ? p[i] : 0.0f;
        }
    } else {
        const int k = k0 + (t >> 4), row = row0 + (t & 15) * PER;
        const float *p = base + (int64_t)k * s_k + row;
        if constexpr (FAST) {
#pragma unroll
            for (int h = 0; h < TM; h++) {
                const float4 v = *reinterpret_cast<const float4 *>(p + 4 * h);
                r[4 * h] = v.x; r[4 * h + 1] = v.y; r[4 * h + 2] = v.z; r[4 * h + 3] = v.w;
            }
        } else if (vec4) {  // the row count and the k stride are multiples of 4
#pragma unroll
            for (int h = 0; h < TM; h++) {
                const float4 v = (k < K && row + 4 * h + 4 <= n_rows)
                                     ? *reinterpret_cast<const float4 *>(p + 4 * h)
                                     : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                r[4 * h] = v.x; r[4 * h + 1] = v.y; r[4 * h + 2] = v.z; r[4 * h + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < PER; i++) r[i] = (k < K && row + i < n_rows) ? p[i] : 0.0f;
        }
    }
}

template <int TM, bool KCONT>
__device__ __forceinline__ void store_tile(float (*tile)[TileGeom<TM>::LD], const float (&r)[4 * TM]) {
    constexpr int PER = TileGeom<TM>::PER;
    const int t = threadIdx.x;
    if constexpr (KCONT) {
        constexpr int TPR = BK / PER;
        const int row = t / TPR, k = (t % TPR) * PER;
#pragma unroll
        for (int i = 0; i < PER; i++) tile[k + i][row] = r[i];
    } else {
        const int k = t >> 4, row = (t & 15) * PER;
#pragma unroll
        for (int h = 0; h < TM; h++)
            *reinterpret_cast<float4 *>(&tile[k][row + 4 * h]) =
                make_float4(r[4 * h], r[4 * h + 1], r[4 * h + 2], r[4 * h + 3]);
    }
}

template <int TM, bool A_KCONT, bool B_KCONT, bool FAST>
__global__ __launch_bounds__(256) void sgemm_mfma_kernel(GemmParams p) {
    constexpr int R = TileGeom<TM>::R, LD = TileGeom<TM>::LD, PER = TileGeom<TM>::PER;
    __shared__ float As[2][BK][LD];
    __shared__ float Bs[2][BK][LD];
    const GemmProblem pr = p.prob[problem_of(p, blockIdx.z)];
    const int split = blockIdx.z - pr.z0;
    const int kb = split * pr.k_chunk, ke = min(pr.K, kb + pr.k_chunk);
    const int m0 = blockIdx.y * R, n0 = blockIdx.x * R;
    if (m0 >= pr.M) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = (wave >> 1) * 32 * TM, wn = (wave & 1) * 32 * TM;
    const int l32 = lane & 31, lk = lane >> 5;

    float16v acc[TM][TM];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    float ra[PER], rb[PER];
    load_tile<TM, A_KCONT, FAST>(ra, pr.A, p.a_si, p.a_sk, m0, kb, pr.M, ke, p.a_vec4 != 0);
    load_tile<TM, B_KCONT, FAST>(rb, pr.B, p.b_sj, p.b_sk, n0, kb, p.N, ke, p.b_vec4 != 0);
    store_tile<TM, A_KCONT>(As[0], ra);
    store_tile<TM, B_KCONT>(Bs[0], rb);
    __syncthreads();

    const int n_steps = (ke - kb + BK - 1) / BK;
    for (int s = 0; s < n_steps; s++) {
        const int cur = s & 1;
        if (s + 1 < n_steps) {
            load_tile<TM, A_KCONT, FAST>(ra, pr.A, p.a_si, p.a_sk, m0, kb + (s + 1) * BK, pr.M, ke,
                                         p.a_vec4 != 0);
            load_tile<TM, B_KCONT, FAST>(rb, pr.B, p.b_sj, p.b_sk, n0, kb + (s + 1) * BK, p.N, ke,
                                         p.b_vec4 != 0);
        }
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float a[TM], b[TM];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = As[cur][kk + lk][wm + 32 * i + l32];
#pragma unroll
            for (int j = 0; j < TM; j++) b[j] = Bs[cur][kk + lk][wn + 32 * j + l32];
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (s + 1 < n_steps) {
            // the other buffer was last read in step s-1, before the barrier below
            store_tile<TM, A_KCONT>(As[cur ^ 1], ra);
            store_tile<TM, B_KCONT>(Bs[cur ^ 1], rb);
        }
        __syncthreads();
    }

    // accumulator element 4*jj + ii of tile (i, j) is C[8*jj + 4*(lane/32) + ii][lane % 32]
    float *cbase = pr.C;
    int ldc = p.ldc;
    bool accumulate = p.accumulate != 0;
    if (pr.n_split > 1) {
        cbase = p.partial + (size_t)blockIdx.z * p.max_m * p.N;
        ldc = p.N;
        accumulate = false;
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TM; j++) {
            const int col = n0 + wn + 32 * j + l32;
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    const int row = m0 + wm + 32 * i + 8 * jj + 4 * lk + ii;
                    if (FAST || (row < pr.M && col < p.N)) {
                        float *c = cbase + (int64_t)row * ldc + col;
                        const float v = acc[i][j][4 * jj + ii];
                        *c = accumulate ? *c + v : v;
                    }
                }
        }
}

// C (+)= sum over splits of the partial slabs, in a fixed order (reproducible). A
// workgroup takes 64 consecutive outputs; its four 64-thread groups each add a quarter of
// the splits with four independent running sums (the loads of a thread do not wait for
// each other), and the quarters are combined through LDS. One thread per output walking
// all splits left a 256 x 256 product with 256 splits at one workgroup per CU and 256
// dependent steps: 88 us.
constexpr int kSplitReduceCols = 64;
constexpr int kSplitReduceGroups = 256 / kSplitReduceCols;

__global__ __launch_bounds__(256) void sgemm_splitk_reduce_kernel(GemmParams p) {
    __shared__ float red[kSplitReduceGroups][kSplitReduceCols];
    const GemmProblem pr = p.prob[blockIdx.y];
    if (pr.n_split <= 1) return;  // written in place by the product kernel
    const int64_t total = (int64_t)pr.M * p.N;
    const int lane_e = threadIdx.x % kSplitReduceCols, zg = threadIdx.x / kSplitReduceCols;
    const int chunk = (pr.n_split + kSplitReduceGroups - 1) / kSplitReduceGroups;
    const int zb = min(zg * chunk, pr.n_split), ze = min(zb + chunk, pr.n_split);
    const size_t slab = (size_t)p.max_m * p.N;
    for (int64_t e0 = (int64_t)blockIdx.x * kSplitReduceCols; e0 < total;
         e0 += (int64_t)gridDim.x * kSplitReduceCols) {
        const int64_t e = e0 + lane_e;
        const bool live = e < total;
        const int row = live ? (int)(e / p.N) : 0, col = live ? (int)(e % p.N) : 0;
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
        if (live) {
            const float *src = p.partial + (size_t)pr.z0 * slab + (size_t)row * p.N + col;
            int z = zb;
            for (; z + 4 <= ze; z += 4) {
                a0 += src[(size_t)z * slab];
                a1 += src[(size_t)(z + 1) * slab];
                a2 += src[(size_t)(z + 2) * slab];
                a3 += src[(size_t)(z + 3) * slab];
            }
            for (; z < ze; z++) a0 += src[(size_t)z * slab];
        }
        red[zg][lane_e] = (a0 + a1) + (a2 + a3);
        __syncthreads();
        if (zg == 0 && live) {
            float s = red[0][lane_e];
#pragma unroll
            for (int g = 1; g < kSplitReduceGroups; g++) s += red[g][lane_e];
            float *c = pr.C + (int64_t)row * p.ldc + col;
            *c = p.accumulate ? *c + s : s;
        }
        __syncthreads();
    }
}

// Few output tiles and a long inner dimension (dW = X^T.G with K = number of
// nodes): split K so the whole chip works, partials summed by a second kernel.
// Returns the number of blockIdx.z values.
static int choose_split(GemmParams &p, int max_m, size_t workspace_bytes, int tile) {
    p.max_m = max_m;
    int64_t tiles = 0;
    for (int i = 0; i < p.n_prob; i++) tiles += ceil_div(p.N, tile) * ceil_div(p.prob[i].M, tile);
    const int64_t slab = (int64_t)max_m * p.N * sizeof(float);
    const int64_t slab_cap = slab > 0 ? (int64_t)(workspace_bytes / slab) / p.n_prob : 0;
    int z = 0;
    for (int i = 0; i < p.n_prob; i++) {
        GemmProblem &pr = p.prob[i];
        pr.z0 = z;
        pr.n_split = 1;
        pr.k_chunk = (int)(ceil_div(pr.K, BK) * BK);
        if (tiles < 256 && pr.K >= 2 * kMinSplitK && pr.M > 0) {
            int64_t want = std::min<int64_t>(ceil_div(pr.K, kMinSplitK), ceil_div(1024, tiles));
            want = std::min<int64_t>(want, slab_cap);
            if (want > 1) {
                pr.k_chunk = (int)(ceil_div(ceil_div(pr.K, want), BK) * BK);
                pr.n_split = (int)ceil_div(pr.K, pr.k_chunk);
            }
        }
        z += pr.n_split;
    }
    return z;
}

// 128 x 128 tiles when they, times the K splits a long inner dimension allows, fill every
// CU to the kernel's occupancy (3 workgroups each); 64 x 64 tiles otherwise
constexpr int kFillTiles = 768;
static int pick_tile(int64_t n, const int64_t *m, int n_prob, int64_t same_m, int64_t k_max) {
    int64_t tiles = 0;
    for (int i = 0; i < n_prob; i++) tiles += ceil_div(n, 128) * ceil_div(m ? m[i] : same_m, 128);
    if (tiles <= 0) return 64;
    if (n <= 64) return 64;  // half of every 128-column tile would be empty
    int64_t splits = 1;
    if (k_max >= 2 * kMinSplitK)
        splits = std::max<int64_t>(1, std::min<int64_t>(ceil_div(k_max, kMinSplitK),
                                                        ceil_div(1024, tiles)));
    return tiles * splits >= kFillTiles ? 128 : 64;
}

template <int TM, bool A_KCONT, bool B_KCONT>
static int sgemm_launch_tile(const GemmParams &p, int max_m, int n_z, hipStream_t stream) {
    constexpr int R = TileGeom<TM>::R;
    bool fast = p.N % R == 0, any_split = false;
    for (int i = 0; i < p.n_prob; i++) {
        const GemmProblem &pr = p.prob[i];
        fast = fast && pr.M % R == 0 && pr.K % BK == 0 && pr.K > 0 && aligned16(pr.A) &&
               aligned16(pr.B);
        any_split = any_split || pr.n_split > 1;
    }
    // vector loads also need every row / k-line to start 16-byte aligned
    fast = fast && (A_KCONT ? p.a_si % 4 == 0 : p.a_sk % 4 == 0) &&
           (B_KCONT ? p.b_sj % 4 == 0 : p.b_sk % 4 == 0);
    dim3 grid((unsigned)ceil_div(p.N, R), (unsigned)ceil_div(max_m, R), (unsigned)n_z);
    if (fast) {
        sgemm_mfma_kernel<TM, A_KCONT, B_KCONT, true><<<grid, 256, 0, stream>>>(p);
    } else {
        // ragged tiles: 16-byte loads still work where each one lies wholly inside or
        // wholly outside the operand (contiguous extent a multiple of 4, aligned lines)
        GemmParams q = p;
        bool a4 = A_KCONT ? p.a_si % 4 == 0 : p.a_sk % 4 == 0;
        bool b4 = (B_KCONT ? p.b_sj % 4 == 0 : p.b_sk % 4 == 0) && (B_KCONT || p.N % 4 == 0);
        for (int i = 0; i < p.n_prob; i++) {
            const GemmProblem &pr = p.prob[i];
            a4 = a4 && aligned16(pr.A) && (A_KCONT ? pr.K % 4 == 0 : pr.M % 4 == 0);
            b4 = b4 && aligned16(pr.B) && (!B_KCONT || pr.K % 4 == 0);
        }
        q.a_vec4 = a4;
        q.b_vec4 = b4;
        sgemm_mfma_kernel<TM, A_KCONT, B_KCONT, false><<<grid, 256, 0, stream>>>(q);
    }
    YITU_LAUNCH_CHECK();
    if (any_split) {
        dim3 rg((unsigned)std::min<int64_t>(ceil_div((int64_t)max_m * p.N, kSplitReduceCols), 4096),
                (unsigned)p.n_prob);
        sgemm_splitk_reduce_kernel<<<rg, 256, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <bool A_KCONT, bool B_KCONT>
static int sgemm_launch(const GemmParams &p, int tile, int max_m, int n_z, hipStream_t stream) {
    if (tile == 128) return sgemm_launch_tile<2, A_KCONT, B_KCONT>(p, max_m, n_z, stream);
    return sgemm_launch_tile<1, A_KCONT, B_KCONT>(p, max_m, n_z, stream);
}

// ---- many rows, inner dimension 64 / 128 / 256: the weight stays in registers -------
// C_q[M_q, N] = A_q[M_q, K] . B_q for up to 32 problems (node types, relations). The 8 waves of a
// workgroup hold all of B_q[0 .. K, n0 .. n0 + 256) as MFMA operands (wave w keeps 32
// columns: K / 2 steps x 1 register), the workgroup walks 32-row tiles of A and reads each
// as whole rows, two tiles ahead through a ring of registers into a double-buffered LDS
// tile, one barrier per tile; no operand of the inner loop comes from memory. The MFMA
// step s of lane (i, half) takes k = half * K / 2 + s, so a lane's A operands of four
// consecutive steps are 16 contiguous bytes of its row (the weight registers are loaded in
// the same order, once). LDS rows are padded by 16 bytes: 16 consecutive lanes read 16
// different banks groups. The weight is the first MFMA operand, so a lane ends up with
// four consecutive columns of one row; a wave passes its 32 x 32 outputs through an LDS
// area of its own and stores whole 128-byte row segments.
constexpr int SR_M = 32;      // rows of a tile
constexpr int SR_C_LD = 144;  // staged output row: 128 bytes + 16 of padding
constexpr int SR_PF = 2;      // tiles requested ahead

struct SRowsParams {
    const float *A[kMaxGroup];
    const float *B[kMaxGroup];
    float *C[kMaxGroup];
    const float *bias[kMaxGroup];  // [N] added to every row of the problem, or null
    int M[kMaxGroup];
    int tile_start[kMaxGroup + 1];
    int n_problems, N;
    int64_t lda, ldb, ldc;
};

template <int K>
constexpr size_t sgemm_rows_lds_bytes() {
    return (size_t)2 * SR_M * (K + 4) * sizeof(float) + (size_t)8 * SR_M * SR_C_LD;
}

template <int K, bool B_KCONT>
__global__ __launch_bounds__(512, 1) void sgemm_rows_kernel(SRowsParams p) {
    constexpr int KS = K / 2;        // MFMA steps of 2
    constexpr int A_LD = K + 4;      // padded LDS row, floats
    constexpr int TPR = K / 4;       // threads that cover one row with 16 bytes each
    constexpr int RPS = 512 / TPR;   // rows the workgroup covers at a time
    constexpr int LR = SR_M / RPS;   // 16-byte pieces of the tile per thread
    static_assert(LR >= 1, "a pass of the loader must not exceed the tile");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int wn = blockIdx.y * 256 + wave * 32;
    float *As = reinterpret_cast<float *>(smem);  // [2][SR_M][A_LD]
    unsigned char *stage = smem + (size_t)2 * SR_M * A_LD * sizeof(float) + wave * (SR_M * SR_C_LD);
    // A workgroup takes a run of consecutive tiles of the list of all problems: it then
    // crosses from one problem into the next once at most (and loads a weight once or
    // twice), where every gridDim.x-th tile took it through all of them.
    constexpr int stride = 1;
    const int n_all = p.tile_start[p.n_problems];
    const int per_wg = (n_all + (int)gridDim.x - 1) / (int)gridDim.x;
    const int my_lo = blockIdx.x * per_wg, my_hi = min(my_lo + per_wg, n_all);
    // per wave: its 32 columns lie wholly inside the output (vector stores through the
    // staging area), partly (element by element), or not at all (nothing to compute)
    const bool whole_cols = wn + 32 <= p.N, no_cols = wn >= p.N;
    const int lrow = t / TPR, lcol = (t % TPR) * 4;

    for (int q = 0; q < p.n_problems; q++) {
        const int lo = p.tile_start[q];
        // this workgroup's tiles of the problem
        const int tile0 = max(lo, my_lo), hi = min(p.tile_start[q + 1], my_hi);
        if (tile0 >= hi) continue;  // same for the whole workgroup
        const float *__restrict__ a_q = p.A[q];
        const float *__restrict__ b_q = p.B[q];
        float *__restrict__ c_q = p.C[q];
        const float *__restrict__ bias_q = p.bias[q];
        const int m_q = p.M[q];
        float b[KS];
        {
            const int col = min(wn + l32, p.N - 1);  // columns past N: never stored
            const float *bp = B_KCONT ? b_q + (int64_t)col * p.ldb + KS * lk
                                      : b_q + (int64_t)(KS * lk) * p.ldb + col;
#pragma unroll
            for (int s = 0; s < KS; s++) {
                b[s] = *bp;
                bp += B_KCONT ? 1 : p.ldb;
                // (addresses made as they are needed: all at once they crowd out the weight)
                if (s % 32 == 31) __builtin_amdgcn_sched_barrier(0);
            }
        }
        f4 ra[SR_PF][LR];
        auto gload = [&](int slot, int64_t tile64) {
            const int tile = (int)min(tile64, (int64_t)hi - 1);
            const int r0 = (tile - lo) * SR_M + lrow;
#pragma unroll
            for (int i = 0; i < LR; i++) {
                const int64_t row = min(r0 + RPS * i, m_q - 1);
                ra[slot][i] = __builtin_nontemporal_load(
                    reinterpret_cast<const f4 *>(a_q + row * p.lda + lcol));
            }
        };
#pragma unroll
        for (int u = 0; u < SR_PF; u++) {
            gload(u, tile0 + (int64_t)u * stride);
            __builtin_amdgcn_sched_barrier(0);  // oldest first
        }
        for (int it0 = 0; tile0 + (int64_t)it0 * stride < hi; it0 += SR_PF) {
#pragma unroll
            for (int u = 0; u < SR_PF; u++) {
                const int it = it0 + u;
                const int64_t tile64 = tile0 + (int64_t)it * stride;
                if (tile64 >= hi) break;  // same for the whole workgroup
                const int tile = (int)tile64;
                float *At = As + (size_t)(it & 1) * SR_M * A_LD;
                // this buffer was last read two tiles ago, before the previous barrier
#pragma unroll
                for (int i = 0; i < LR; i++)
                    *reinterpret_cast<f4 *>(At + (lrow + RPS * i) * A_LD + lcol) = ra[u][i];
                __syncthreads();
                gload(u, tile64 + (int64_t)SR_PF * stride);
                float16v acc;
#pragma unroll
                for (int e = 0; e < 16; e++) acc[e] = 0.0f;
                if (no_cols) continue;  // (after the barrier and the loads that every wave shares)
                const float *arow = At + l32 * A_LD + KS * lk;
#pragma unroll
                for (int s4 = 0; s4 < KS; s4 += 4) {
                    const f4 a = *reinterpret_cast<const f4 *>(arow + s4);
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b[s4 + e], a[e], acc, 0, 0, 0);
                    // operand reads stay a few steps ahead of their products: hoisted all the
                    // way they would not fit beside the weight
                    if (s4 % 16 == 12) __builtin_amdgcn_sched_barrier(0);
                }
                // accumulator element 4 jj + ii is C[32 tile + lane % 32][wn + 8 jj + 4 (lane / 32) + ii]
                const int row0 = (tile - lo) * SR_M;
                if (whole_cols && row0 + SR_M <= m_q) {  // same for the whole wave
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) {
                        f4 w = {acc[4 * jj], acc[4 * jj + 1], acc[4 * jj + 2], acc[4 * jj + 3]};
                        if (bias_q)  // same for the whole launch of the problem
                            w += *reinterpret_cast<const f4 *>(bias_q + wn + 8 * jj + 4 * lk);
                        *reinterpret_cast<f4 *>(stage + l32 * SR_C_LD + 32 * jj + 16 * lk) = w;
                    }
#pragma unroll
                    for (int r = 0; r < SR_M / 8; r++) {
                        const int row = 8 * r + (lane >> 3);
                        const f4 w = *reinterpret_cast<const f4 *>(stage + row * SR_C_LD +
                                                                   16 * (lane & 7));
                        *reinterpret_cast<f4 *>(c_q + (int64_t)(row0 + row) * p.ldc + wn +
                                                4 * (lane & 7)) = w;
                    }
                } else if (row0 + l32 < m_q) {
                    const int64_t row = row0 + l32;
#pragma unroll
                    for (int e = 0; e < 16; e++) {
                        const int col = wn + 8 * (e / 4) + 4 * lk + e % 4;
                        if (col < p.N) c_q[row * p.ldc + col] = acc[e] + (bias_q ? bias_q[col] : 0.0f);
                    }
                }
            }
        }
        __syncthreads();  // the next problem starts over with the first LDS buffer
    }
}

template <int K, bool B_KCONT>
static int sgemm_rows_launch_k(const SRowsParams &r, hipStream_t stream) {
    constexpr size_t lds = sgemm_rows_lds_bytes<K>();
    // more LDS than the default limit: asked for once per device
    static bool prepared_on[64] = {};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) device = 0;
    bool &prepared = prepared_on[device];
    if (!prepared) {
        hipError_t e = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&sgemm_rows_kernel<K, B_KCONT>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            set_error("hipFuncSetAttribute(dynamic LDS %zu): %s", lds, hipGetErrorString(e));
            return -1;
        }
        prepared = true;
    }
    const int n_tiles = r.tile_start[r.n_problems];
    dim3 grid((unsigned)std::min(n_tiles, 256), (unsigned)ceil_div(r.N, 256));
    sgemm_rows_kernel<K, B_KCONT><<<grid, 512, lds, stream>>>(r);
    YITU_LAUNCH_CHECK();
    return 0;
}

// dst_q[n][k] = src_q[k][n] for the weights of a group (blockIdx.z = problem): a weight
// stored [K, N] is read by the kernel above with one 4-byte load per element and lane,
// and a load of 4 bytes takes the address path as long as one of 16; from the [N, K]
// copy the same registers are filled with a quarter of the loads.
struct TransposeParams {
    float *dst[kMaxGroup];
    const float *src[kMaxGroup];
};

__global__ __launch_bounds__(256) void transpose32_kernel(TransposeParams tp, int K, int N,
                                                          int64_t ld_src) {
    __shared__ float tile[32][33];
    float *__restrict__ dst = tp.dst[blockIdx.z];
    const float *__restrict__ src = tp.src[blockIdx.z];
    const int k0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8)
        tile[r][tx] = (k0 + r < K && n0 + tx < N) ? src[(int64_t)(k0 + r) * ld_src + n0 + tx] : 0.0f;
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (n0 + r < N && k0 + tx < K) dst[(int64_t)(n0 + r) * K + k0 + tx] = tile[tx][r];
}

static size_t sgemm_rows_workspace_bytes(int64_t n, int64_t k, int64_t n_problems) {
    if (!(k == 64 || k == 128 || k == 256)) return 0;
    return (size_t)std::min<int64_t>(std::max<int64_t>(n_problems, 1), kMaxGroup) *
           align_up((size_t)(n * k) * sizeof(float), 256);
}

// Takes the group when it is one of the kernel's shapes; *taken says whether it did.
static int sgemm_rows_try(const GemmParams &p, bool trans_a, bool trans_b, int lda, int ldb,
                          void *workspace, size_t workspace_bytes, hipStream_t stream,
                          bool *taken) {
    *taken = false;
    if (trans_a || p.accumulate || p.n_prob < 1 || p.ldc % 4 != 0 || lda % 4 != 0) return 0;
    const int k = p.prob[0].K;
    if (!(k == 64 || k == 128 || k == 256)) return 0;
    int64_t total = 0;
    SRowsParams r{};
    for (int i = 0; i < p.n_prob; i++) {
        const GemmProblem &pr = p.prob[i];
        if (pr.K != k || !aligned16(pr.A) || !aligned16(pr.C) || !aligned16(pr.bias) || pr.M < 0)
            return 0;
        r.bias[i] = pr.bias;
        r.A[i] = pr.A;
        r.B[i] = pr.B;
        r.C[i] = pr.C;
        r.M[i] = pr.M;
        r.tile_start[i + 1] = r.tile_start[i] + (int)ceil_div(pr.M, SR_M);
        total += pr.M;
    }
    // Eight waves side by side cover 256 columns: with fewer than 192 in the last block most
    // of them would idle (N = 64: 279 us against 154 us for the tiled kernel at 2^18 rows),
    // and a workgroup has to walk a few dozen tiles to pay for loading the weight
    // (2^15 rows: 46 against 44 us).
    const int last = p.N % 256;
    if (total < 49152 || (last != 0 && last < 192)) return 0;
    r.n_problems = p.n_prob;
    r.N = p.N;
    r.lda = lda;
    r.ldb = ldb;
    r.ldc = p.ldc;
    *taken = true;
    if (!trans_b && workspace && aligned16(workspace) &&
        workspace_bytes >= sgemm_rows_workspace_bytes(p.N, k, p.n_prob)) {
        // (weights are small: the copies cost a few microseconds for the whole group)
        TransposeParams tp{};
        const size_t slot = align_up((size_t)p.N * k * sizeof(float), 256);
        for (int i = 0; i < p.n_prob; i++) {
            tp.src[i] = r.B[i];
            tp.dst[i] = reinterpret_cast<float *>(static_cast<char *>(workspace) + i * slot);
            r.B[i] = tp.dst[i];
        }
        dim3 tg((unsigned)ceil_div(p.N, 32), (unsigned)ceil_div(k, 32), (unsigned)p.n_prob);
        transpose32_kernel<<<tg, 256, 0, stream>>>(tp, k, p.N, ldb);
        YITU_LAUNCH_CHECK();
        r.ldb = k;
        trans_b = true;
    }
    if (trans_b) {
        if (k == 256) return sgemm_rows_launch_k<256, true>(r, stream);
        if (k == 128) return sgemm_rows_launch_k<128, true>(r, stream);
        return sgemm_rows_launch_k<64, true>(r, stream);
    }
    if (k == 256) return sgemm_rows_launch_k<256, false>(r, stream);
    if (k == 128) return sgemm_rows_launch_k<128, false>(r, stream);
    return sgemm_rows_launch_k<64, false>(r, stream);
}

// ---- weight gradients C_q[KI, NO] = A_q^T . B_q over many rows (KI, NO = 64, 128 or 256):
// the output stays in registers. A workgroup of 8 waves owns a chunk of the rows of one
// problem and the whole KI x NO product of that chunk (256 x 256: wave (wi, wj) the block
// of rows 64 wi, columns 128 wj, 2 x 4 MFMA tiles, 128 accumulator registers), so every
// row of A and B is read once, whole, two 16-row stages ahead through a ring of registers
// into a double-buffered LDS stage, one barrier per stage. Both MFMA operands are columns
// of the row-major stage (lane = column, the two halves of the wave take the two rows of
// the step), with stage rows padded by 128 bytes so that the halves fall into different
// banks. The chunk products go to the slabs of `partial` and are added by
// sgemm_splitk_reduce_kernel in a fixed order.
constexpr int TR_STAGE = 16;  // rows per stage

// KI x NO = (32 TX WI) x (32 TY WJ): WI x WJ = 8 waves, each TX x TY MFMA tiles.
template <int WI, int WJ, int TX, int TY>
struct TnRowsGeom {
    static_assert(WI * WJ == 8 && TX * TY <= 8, "8 waves, at most 128 accumulator registers");
    static constexpr int KI = 32 * TX * WI, NO = 32 * TY * WJ;
    static constexpr int LDA = KI + 32, LDB = NO + 32;  // padded stage rows, floats
    static constexpr size_t kLds = (size_t)2 * TR_STAGE * (LDA + LDB) * sizeof(float);
};

template <int WI, int WJ, int TX, int TY>
__global__ __launch_bounds__(512, 1) void sgemm_tn_rows_kernel(GemmParams p) {
    using G = TnRowsGeom<WI, WJ, TX, TY>;
    constexpr int KI = G::KI, NO = G::NO, LDA = G::LDA, LDB = G::LDB;
    constexpr int PA = (TR_STAGE * KI / 4 + 511) / 512, PB = (TR_STAGE * NO / 4 + 511) / 512;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef float f4 __attribute__((ext_vector_type(4)));
    float *stage_mem = reinterpret_cast<float *>(smem);  // [2 buffers][A stage, B stage]
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int i0 = (wave / WJ) * 32 * TX, j0 = (wave % WJ) * 32 * TY;
    const GemmProblem pr = p.prob[problem_of(p, blockIdx.x)];
    const int split = blockIdx.x - pr.z0;
    const int m_beg = split * pr.k_chunk, m_end = min(pr.K, m_beg + pr.k_chunk);
    const int n_stages = (m_end - m_beg + TR_STAGE - 1) / TR_STAGE;

    float16v acc[TX][TY];
#pragma unroll
    for (int a = 0; a < TX; a++)
#pragma unroll
        for (int b = 0; b < TY; b++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[a][b][e] = 0.0f;

    // loader: thread t takes the 16-byte pieces t, t + 512, ... of a stage of A and of B
    f4 ra[2][PA], rb[2][PB];
    auto gload = [&](int slot, int st) {
        const int r0 = m_beg + st * TR_STAGE;
#pragma unroll
        for (int h = 0; h < PA; h++) {
            const int piece = t + 512 * h, row = r0 + piece / (KI / 4);
            f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (piece < TR_STAGE * KI / 4 && row < m_end)  // rows past the chunk add nothing
                v = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(
                    pr.A + (int64_t)row * p.a_sk + (piece % (KI / 4)) * 4));
            ra[slot][h] = v;
        }
#pragma unroll
        for (int h = 0; h < PB; h++) {
            const int piece = t + 512 * h, row = r0 + piece / (NO / 4);
            f4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (piece < TR_STAGE * NO / 4 && row < m_end)
                v = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(
                    pr.B + (int64_t)row * p.b_sk + (piece % (NO / 4)) * 4));
            rb[slot][h] = v;
        }
    };
    gload(0, 0);
    __builtin_amdgcn_sched_barrier(0);  // oldest first
    gload(1, 1);
    for (int s0 = 0; s0 < n_stages; s0 += 2) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int st = s0 + u;
            if (st >= n_stages) break;  // same for the whole workgroup
            float *As = stage_mem + (size_t)(st & 1) * TR_STAGE * (LDA + LDB);
            float *Bs = As + TR_STAGE * LDA;
            // this buffer was last read two stages ago, before the previous barrier
#pragma unroll
            for (int h = 0; h < PA; h++) {
                const int piece = t + 512 * h;
                if (piece < TR_STAGE * KI / 4)
                    *reinterpret_cast<f4 *>(As + (piece / (KI / 4)) * LDA + (piece % (KI / 4)) * 4) =
                        ra[u][h];
            }
#pragma unroll
            for (int h = 0; h < PB; h++) {
                const int piece = t + 512 * h;
                if (piece < TR_STAGE * NO / 4)
                    *reinterpret_cast<f4 *>(Bs + (piece / (NO / 4)) * LDB + (piece % (NO / 4)) * 4) =
                        rb[u][h];
            }
            __syncthreads();
            gload(u, st + 2);
#pragma unroll
            for (int k2 = 0; k2 < TR_STAGE; k2 += 2) {
                float a[TX], b[TY];
#pragma unroll
                for (int x = 0; x < TX; x++) a[x] = As[(k2 + lk) * LDA + i0 + 32 * x + l32];
#pragma unroll
                for (int y = 0; y < TY; y++) b[y] = Bs[(k2 + lk) * LDB + j0 + 32 * y + l32];
#pragma unroll
                for (int x = 0; x < TX; x++)
#pragma unroll
                    for (int y = 0; y < TY; y++)
                        acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[x], b[y], acc[x][y], 0, 0, 0);
            }
        }
    }
    // accumulator element 4 jj + ii of tile (x, y) is row i0 + 32 x + 8 jj + 4 (lane / 32) + ii,
    // column j0 + 32 y + lane % 32 of this chunk's slab
    float *dst = p.partial + (size_t)blockIdx.x * p.max_m * p.N;
#pragma unroll
    for (int x = 0; x < TX; x++)
#pragma unroll
        for (int y = 0; y < TY; y++)
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int ii = 0; ii < 4; ii++) {
                    const int row = i0 + 32 * x + 8 * jj + 4 * lk + ii;
                    __builtin_nontemporal_store(acc[x][y][4 * jj + ii],
                                                dst + (size_t)row * p.N + j0 + 32 * y + l32);
                }
}

template <int WI, int WJ, int TX, int TY>
static int sgemm_tn_rows_launch(const GemmParams &p, int z, hipStream_t stream) {
    constexpr size_t lds = TnRowsGeom<WI, WJ, TX, TY>::kLds;
    static bool prepared_on[64] = {};  // more LDS than the default limit: once per device
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) device = 0;
    if (lds > 65536 && !prepared_on[device]) {
        hipError_t e = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&sgemm_tn_rows_kernel<WI, WJ, TX, TY>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            set_error("hipFuncSetAttribute(dynamic LDS %zu): %s", lds, hipGetErrorString(e));
            return -1;
        }
        prepared_on[device] = true;
    }
    sgemm_tn_rows_kernel<WI, WJ, TX, TY><<<z, 512, lds, stream>>>(p);
    YITU_LAUNCH_CHECK();
    return 0;
}

// widths the kernel is built for: 64, 128 or 256 on either side, at least 8 MFMA tiles
static bool tn_rows_shape(int64_t ki, int64_t no) {
    const bool ok_i = ki == 64 || ki == 128 || ki == 256, ok_j = no == 64 || no == 128 || no == 256;
    return ok_i && ok_j && ki * no >= 64 * 128;
}

// chunks of all problems together: a workgroup per CU when the products keep the matrix
// pipes busy (256 x 256), two when the rows are narrow and the kernel waits for memory
static int tn_rows_chunks(int64_t ki, int64_t no) { return ki * no >= 256 * 256 ? 256 : 512; }

// Takes a group of weight-gradient products [rows, KI]^T . [rows, NO] with many rows in
// all; *taken says whether it did.
static int sgemm_tn_rows_try(GemmParams &p, bool trans_a, bool trans_b, int lda, int ldb,
                             void *workspace, size_t workspace_bytes, hipStream_t stream,
                             bool *taken) {
    *taken = false;
    if (!trans_a || trans_b || p.n_prob < 1 || lda % 4 != 0 || ldb % 4 != 0 || !workspace) return 0;
    const int ki = p.prob[0].M, no = p.N;
    if (!tn_rows_shape(ki, no)) return 0;
    int64_t total = 0;
    for (int i = 0; i < p.n_prob; i++) {
        const GemmProblem &pr = p.prob[i];
        if (pr.M != ki || !aligned16(pr.A) || !aligned16(pr.B)) return 0;
        total += pr.K;
    }
    if (total < 49152) return 0;
    // every problem gets at least two chunks (its slabs are then always summed by the
    // reduce kernel)
    const size_t slab = (size_t)ki * no * sizeof(float);
    const int64_t chunks = tn_rows_chunks(ki, no);
    int z = 0;
    GemmProblem saved[kMaxGroup];
    for (int i = 0; i < p.n_prob; i++) saved[i] = p.prob[i];
    for (int i = 0; i < p.n_prob; i++) {
        GemmProblem &pr = p.prob[i];
        int64_t want = std::max<int64_t>(2, (chunks * (int64_t)pr.K + total / 2) / total);
        want = std::min<int64_t>(want, std::max<int64_t>(2, ceil_div(pr.K, TR_STAGE)));
        pr.k_chunk = (int)(ceil_div(ceil_div(pr.K, want), TR_STAGE) * TR_STAGE);
        pr.n_split = (int)std::max<int64_t>(2, ceil_div(pr.K, pr.k_chunk));
        pr.z0 = z;
        z += pr.n_split;
    }
    if ((size_t)z * slab > workspace_bytes || !aligned16(workspace)) {
        for (int i = 0; i < p.n_prob; i++) p.prob[i] = saved[i];
        return 0;
    }
    *taken = true;
    p.max_m = ki;
    p.partial = static_cast<float *>(workspace);
    p.a_sk = lda;
    p.a_si = 1;
    p.b_sk = ldb;
    p.b_sj = 1;
    int rc = -1;
    if (ki == 256 && no == 256) rc = sgemm_tn_rows_launch<4, 2, 2, 4>(p, z, stream);
    else if (ki == 256 && no == 128) rc = sgemm_tn_rows_launch<4, 2, 2, 2>(p, z, stream);
    else if (ki == 128 && no == 256) rc = sgemm_tn_rows_launch<2, 4, 2, 2>(p, z, stream);
    else if (ki == 256 && no == 64) rc = sgemm_tn_rows_launch<8, 1, 1, 2>(p, z, stream);
    else if (ki == 64 && no == 256) rc = sgemm_tn_rows_launch<1, 8, 2, 1>(p, z, stream);
    else if (ki == 128 && no == 128) rc = sgemm_tn_rows_launch<2, 4, 2, 1>(p, z, stream);
    else if (ki == 128 && no == 64) rc = sgemm_tn_rows_launch<4, 2, 1, 1>(p, z, stream);
    else if (ki == 64 && no == 128) rc = sgemm_tn_rows_launch<2, 4, 1, 1>(p, z, stream);
    if (rc) return rc;
    dim3 rg((unsigned)std::min<int64_t>(ceil_div((int64_t)ki * no, kSplitReduceCols), 4096),
            (unsigned)p.n_prob);
    sgemm_splitk_reduce_kernel<<<rg, 256, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    return 0;
}

// trans_a: A is given as [K, M] row-major (else [M, K]); trans_b: B is given as
// [N, K] row-major (else [K, N]).
int sgemm_grouped(GemmParams &p, bool trans_a, bool trans_b, int lda, int ldb, void *workspace,
                  size_t workspace_bytes, hipStream_t stream) {
    // problems with an empty inner dimension: C = 0 (or unchanged); they leave the group
    int kept = 0;
    for (int i = 0; i < p.n_prob; i++) {
        const GemmProblem pr = p.prob[i];
        if (pr.M == 0) continue;
        if (pr.K > 0) {
            p.prob[kept++] = pr;
            continue;
        }
        if (p.accumulate) continue;
        if (p.ldc == p.N) {
            int rc = fill_zero(pr.C, (int64_t)pr.M * p.N, stream);
            if (rc) return rc;
        } else {
            for (int r = 0; r < pr.M; r++) {
                int rc = fill_zero(pr.C + (int64_t)r * p.ldc, p.N, stream);
                if (rc) return rc;
            }
        }
    }
    p.n_prob = kept;
    {
        bool taken = false;
        const int rc = sgemm_rows_try(p, trans_a, trans_b, lda, ldb, workspace, workspace_bytes,
                                      stream, &taken);
        if (taken) return rc;
        const int rc2 = sgemm_tn_rows_try(p, trans_a, trans_b, lda, ldb, workspace, workspace_bytes,
                                          stream, &taken);
        if (taken) return rc2;
    }
    int max_m = 0;
    for (int i = 0; i < p.n_prob; i++) max_m = std::max(max_m, p.prob[i].M);
    if (max_m == 0 || p.N == 0) return 0;
    int64_t heights[kMaxGroup];
    int64_t k_max = 0;
    for (int i = 0; i < p.n_prob; i++) {
        heights[i] = p.prob[i].M;
        k_max = std::max<int64_t>(k_max, p.prob[i].K);
    }
    // (without a workspace there are no splits to count on)
    const int tile = pick_tile(p.N, heights, p.n_prob, 0, workspace ? k_max : 0);
    const int n_z = choose_split(p, max_m, workspace ? workspace_bytes : 0, tile);
    p.partial = static_cast<float *>(workspace);
    if (trans_a) {  // element (i,k) at A[k*lda + i]: contiguous along rows
        p.a_si = 1;
        p.a_sk = lda;
    } else {
        p.a_si = lda;
        p.a_sk = 1;
    }
    if (trans_b) {  // element (k,j) at B[j*ldb + k]: contiguous along K
        p.b_sk = 1;
        p.b_sj = ldb;
    } else {
        p.b_sk = ldb;
        p.b_sj = 1;
    }
    if (!trans_a && trans_b) return sgemm_launch<true, true>(p, tile, max_m, n_z, stream);
    if (!trans_a && !trans_b) return sgemm_launch<true, false>(p, tile, max_m, n_z, stream);
    if (trans_a && !trans_b) return sgemm_launch<false, false>(p, tile, max_m, n_z, stream);
    return sgemm_launch<false, true>(p, tile, max_m, n_z, stream);
}

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

// Enough for the widest split the policy picks: 1024 / tiles slabs of [m, n].
YITU_API size_t yitu_sgemm_workspace_bytes(int64_t m, int64_t n, int64_t k, int64_t n_problems) {
    const int tile = pick_tile(n, nullptr, (int)std::min<int64_t>(n_problems, kMaxGroup), m, k);
    const int64_t tiles = ceil_div(n, tile) * ceil_div(m, tile) * n_problems;
    // (or room for the [N, K] copies of the weights that the many-rows kernel reads, or for
    // the chunk products of the weight-gradient kernel: a chunk per CU and two per problem)
    size_t rows_ws = std::max<size_t>(sgemm_rows_workspace_bytes(n, k, n_problems), 256);
    if (tn_rows_shape(m, n))
        rows_ws = std::max(rows_ws, (size_t)(tn_rows_chunks(m, n) + 2 * kMaxGroup) * m * n *
                                        sizeof(float));
    if (tiles <= 0 || tiles >= 256 || k < 2 * kMinSplitK) return rows_ws;
    const int64_t splits = std::min<int64_t>(ceil_div(k, kMinSplitK), ceil_div(1024, tiles));
    return std::max(rows_ws, align_up((size_t)(splits * m * n * n_problems) * sizeof(float), 256));
}

YITU_API int yitu_sgemm(float *c, const float *a, const float *b, int64_t m, int64_t n, int64_t k,
                        int trans_a, int trans_b, int64_t lda, int64_t ldb, int64_t ldc,
                        int accumulate, void *workspace, size_t workspace_bytes, void *stream) {
    YITU_REQUIRE(m >= 0 && n >= 0 && k >= 0, "negative size");
    if (m == 0 || n == 0) return 0;
    YITU_REQUIRE(c && (k == 0 || (a && b)), "null operand");
    YITU_REQUIRE(m < INT32_MAX && n < INT32_MAX && k < INT32_MAX && ldc >= n, "size out of range");
    YITU_REQUIRE(lda >= (trans_a ? m : k) && ldb >= (trans_b ? k : n), "leading dimension too small");
    GemmParams p{};
    p.prob[0] = GemmProblem{a, b, c, (int)m, (int)k};
    p.n_prob = 1;
    p.N = (int)n;
    p.ldc = (int)ldc;
    p.accumulate = accumulate;
    return sgemm_grouped(p, trans_a != 0, trans_b != 0, (int)lda, (int)ldb, workspace,
                         workspace_bytes, static_cast<hipStream_t>(stream));
}

namespace yitu {
// y[i, j] += bias[j]: the bias of a Linear whose product did not run on the kernel that adds it
__global__ __launch_bounds__(256) void bias_add_kernel(float *__restrict__ y,
                                                       const float *__restrict__ bias, int64_t m,
                                                       int n, int64_t ldy) {
    const int64_t total = m * n, stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
        y[(i / n) * ldy + i % n] += bias[i % n];
}
// The same for every problem of a group in one launch (blockIdx.y = problem): the per-relation
// Linears of a small heterogeneous graph are dozens of products of a few hundred rows.
__global__ __launch_bounds__(256) void bias_add_group_kernel(GemmParams p) {
    const GemmProblem &pr = p.prob[blockIdx.y];
    if (!pr.bias) return;
    const int n = p.N;
    const int64_t total = (int64_t)pr.M * n, stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride)
        pr.C[(i / n) * p.ldc + i % n] += pr.bias[i % n];
}
}  // namespace yitu

YITU_API int yitu_linear_forward(float *y, const float *x, const float *w, const float *bias,
                                 int64_t m, int64_t n, int64_t k, void *workspace,
                                 size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(m >= 0 && n >= 0 && k >= 0, "negative size");
    if (m == 0 || n == 0) return 0;
    YITU_REQUIRE(y && (k == 0 || (x && w)), "null operand");
    YITU_REQUIRE(m < INT32_MAX && n < INT32_MAX && k < INT32_MAX, "size out of range");
    GemmParams p{};
    p.prob[0] = GemmProblem{x, w, y, (int)m, (int)k};
    p.prob[0].bias = bias;
    p.n_prob = 1;
    p.N = (int)n;
    p.ldc = (int)n;
    if (k > 0) {
        bool taken = false;
        const int rc = sgemm_rows_try(p, false, true, (int)k, (int)k, workspace, workspace_bytes,
                                      stream, &taken);
        if (taken) return rc;
    }
    p.prob[0].bias = nullptr;
    const int rc = sgemm_grouped(p, false, true, (int)k, (int)k, workspace, workspace_bytes, stream);
    if (rc || !bias) return rc;
    const int grid = (int)std::min<int64_t>(ceil_div(m * n, 256), 16384);
    bias_add_kernel<<<grid, 256, 0, stream>>>(y, bias, m, (int)n, n);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_linear_forward_typed(float *const *y, const float *const *x,
                                       const float *const *w, const float *const *bias,
                                       const int64_t *m, int64_t n_problems, int64_t n, int64_t k,
                                       void *workspace, size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_problems >= 0 && n >= 0 && k >= 0, "negative size");
    if (n_problems == 0 || n == 0) return 0;
    YITU_REQUIRE(y && x && w && m, "null problem table");
    YITU_REQUIRE(n < INT32_MAX && k < INT32_MAX, "size out of range");
    for (int64_t first = 0; first < n_problems; first += kMaxGroup) {
        GemmParams p{};
        p.N = (int)n;
        p.ldc = (int)n;
        const int count = (int)std::min<int64_t>(kMaxGroup, n_problems - first);
        for (int i = 0; i < count; i++) {
            const int64_t mi = m[first + i];
            YITU_REQUIRE(mi >= 0 && mi < INT32_MAX, "problem %d: size out of range",
                         (int)(first + i));
            if (mi == 0) continue;
            YITU_REQUIRE(y[first + i] && (k == 0 || (x[first + i] && w[first + i])),
                         "problem %d: null operand", (int)(first + i));
            GemmProblem pr{x[first + i], w[first + i], y[first + i], (int)mi, (int)k};
            pr.bias = bias ? bias[first + i] : nullptr;
            p.prob[p.n_prob++] = pr;
        }
        if (p.n_prob == 0) continue;
        if (k > 0) {
            bool taken = false;
            const int rc = sgemm_rows_try(p, false, true, (int)k, (int)k, workspace,
                                          workspace_bytes, stream, &taken);
            if (rc) return rc;
            if (taken) continue;
        }
        // (the grouped call drops problems from its table: keep what the bias pass needs)
        const GemmParams all = p;
        for (int i = 0; i < p.n_prob; i++) p.prob[i].bias = nullptr;
        const int rc = sgemm_grouped(p, false, true, (int)k, (int)k, workspace, workspace_bytes,
                                     stream);
        if (rc) return rc;
        int64_t most = 0;
        for (int i = 0; i < all.n_prob; i++)
            if (all.prob[i].bias) most = std::max<int64_t>(most, (int64_t)all.prob[i].M * n);
        if (most > 0) {
            const dim3 grid((unsigned)std::min<int64_t>(ceil_div(most, 256), 16384),
                            (unsigned)all.n_prob);
            bias_add_group_kernel<<<grid, 256, 0, stream>>>(all);
            YITU_LAUNCH_CHECK();
        }
    }
    return 0;
}

YITU_API int yitu_sgemm_typed(float *const *c, const float *const *a, const float *const *b,
                              const int64_t *m, const int64_t *k, int64_t n_problems, int64_t n,
                              int trans_a, int trans_b, int64_t lda, int64_t ldb, int64_t ldc,
                              int accumulate, void *workspace, size_t workspace_bytes,
                              void *stream) {
    YITU_REQUIRE(n_problems >= 0 && n >= 0, "negative size");
    if (n_problems == 0 || n == 0) return 0;
    YITU_REQUIRE(c && a && b && m && k, "null problem table");
    YITU_REQUIRE(n < INT32_MAX && ldc >= n, "size out of range");
    for (int64_t first = 0; first < n_problems; first += kMaxGroup) {
        GemmParams p{};
        p.n_prob = (int)std::min<int64_t>(kMaxGroup, n_problems - first);
        p.N = (int)n;
        p.ldc = (int)ldc;
        p.accumulate = accumulate;
        for (int i = 0; i < p.n_prob; i++) {
            const int64_t mi = m[first + i], ki = k[first + i];
            YITU_REQUIRE(mi >= 0 && ki >= 0 && mi < INT32_MAX && ki < INT32_MAX,
                         "problem %d: size out of range", (int)(first + i));
            YITU_REQUIRE(mi == 0 || (c[first + i] && (ki == 0 || (a[first + i] && b[first + i]))),
                         "problem %d: null operand", (int)(first + i));
            YITU_REQUIRE(lda >= (trans_a ? mi : ki) && ldb >= (trans_b ? ki : n),
                         "problem %d: leading dimension too small", (int)(first + i));
            p.prob[i] = GemmProblem{a[first + i], b[first + i], c[first + i], (int)mi, (int)ki};
        }
        int rc = sgemm_grouped(p, trans_a != 0, trans_b != 0, (int)lda, (int)ldb, workspace,
                               workspace_bytes, static_cast<hipStream_t>(stream));
        if (rc) return rc;
    }
    return 0;
}

YITU_API int yitu_b2gemm(float *y_a, float *y_b, const float *x, const float *w_a,
                         const float *w_b, int64_t n, int64_t k, int64_t m, void *stream) {
    YITU_REQUIRE(n >= 0 && k >= 0 && m >= 0, "negative size");
    if (n == 0 || m == 0) return 0;
    YITU_REQUIRE(y_a && y_b && (k == 0 || (x && w_a && w_b)), "null operand");
    YITU_REQUIRE(n < INT32_MAX && k < INT32_MAX && m < INT32_MAX, "size out of range");
    GemmParams p{};
    p.prob[0] = GemmProblem{x, w_a, y_a, (int)n, (int)k};
    p.prob[1] = GemmProblem{x, w_b, y_b, (int)n, (int)k};
    p.n_prob = 2;
    p.N = (int)m;
    p.ldc = (int)m;
    return sgemm_grouped(p, false, true, (int)k, (int)k, nullptr, 0,
                         static_cast<hipStream_t>(stream));
}

YITU_API int yitu_b2gemm_backward(float *dx, float *dw_a, float *dw_b, const float *x,
                                  const float *w_a, const float *w_b, const float *grad_a,
                                  const float *grad_b, int64_t n, int64_t k, int64_t m,
                                  void *workspace, size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n >= 0 && k >= 0 && m >= 0, "negative size");
    YITU_REQUIRE(n < INT32_MAX && k < INT32_MAX && m < INT32_MAX, "size out of range");
    YITU_REQUIRE(dx && dw_a && dw_b, "null output");
    // dw_* [m,k] = grad_*^T [m,n] . x [n,k]: one grouped launch of two problems
    if (m > 0 && k > 0) {
        GemmParams p{};
        p.prob[0] = GemmProblem{grad_a, x, dw_a, (int)m, (int)n};
        p.prob[1] = GemmProblem{grad_b, x, dw_b, (int)m, (int)n};
        p.n_prob = 2;
        p.N = (int)k;
        p.ldc = (int)k;
        int rc = sgemm_grouped(p, true, false, (int)m, (int)k, workspace, workspace_bytes, stream);
        if (rc) return rc;
    }
    // dx [n,k] = grad_a [n,m] . w_a [m,k] + grad_b . w_b
    if (n > 0 && k > 0) {
        for (int pass = 0; pass < 2; pass++) {
            GemmParams p{};
            p.prob[0] = GemmProblem{pass ? grad_b : grad_a, pass ? w_b : w_a, dx, (int)n, (int)m};
            p.n_prob = 1;
            p.N = (int)k;
            p.ldc = (int)k;
            p.accumulate = pass;
            int rc = sgemm_grouped(p, false, false, (int)m, (int)k, nullptr, 0, stream);
            if (rc) return rc;
        }
    }
    return 0;
}
