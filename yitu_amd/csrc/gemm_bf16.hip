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

// dst[n][k] = src[k][n] for a [K, N] matrix of 16-bit elements (32 x 32 tiles through LDS)
__global__ __launch_bounds__(256) void transpose16_kernel(uint16_t *__restrict__ dst,
                                                          const uint16_t *__restrict__ src, int K,
                                                          int N, int64_t ld_src, int64_t ld_dst) {
    __shared__ uint16_t tile[32][33];
    const int k0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8)
        tile[r][tx] = (k0 + r < K && n0 + tx < N) ? src[(int64_t)(k0 + r) * ld_src + n0 + tx] : 0;
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (n0 + r < N && k0 + tx < K) dst[(int64_t)(n0 + r) * ld_dst + k0 + tx] = tile[tx][r];
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
        transpose16_kernel<<<tg, 256, 0, stream>>>(static_cast<uint16_t *>(workspace),
                                                   static_cast<const uint16_t *>(b), (int)k, (int)n,
                                                   ldb, k);
        YITU_LAUNCH_CHECK();
        p.Bt = static_cast<const uint16_t *>(workspace);
        p.ldbt = k;
    }
    dim3 grid((unsigned)ceil_div(m, HM), (unsigned)ceil_div(n, HN));
    if (c_is_bf16)
        hgemm_mfma_kernel<true><<<grid, 256, 0, stream>>>(p);
    else
        hgemm_mfma_kernel<false><<<grid, 256, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    return 0;
}
