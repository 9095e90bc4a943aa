// extern "C" surface of libyitu_hip.so (declared in include/yitu_hip.h).
#include "../../include/yitu_hip.h"

#include "spmm_rows.hpp"

#include <mutex>

using namespace yitu;

#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API const char *yitu_last_error(void) { return last_error(); }
YITU_API int yitu_abi_version(void) { return 4; }

YITU_API size_t yitu_spmm_workspace_bytes(int64_t nnz, int64_t row_len, int with_plan) {
    return spmm_workspace_bytes(nnz, row_len, with_plan != 0);
}

YITU_API int yitu_agg_csr(float *out, const void *x, int x_is_bf16, const int32_t *row_pointers,
                          const int32_t *column_index, const float *degrees, int64_t n_rows,
                          int64_t n_src, int64_t nnz, int64_t dim, float alpha,
                          int64_t max_degree, const void *plan, const float *edge_scale,
                          void *workspace, size_t workspace_bytes, void *stream) {
    YITU_REQUIRE(n_rows >= 0 && n_src >= 0 && nnz >= 0 && dim >= 0, "negative size");
    if (n_rows == 0 || dim == 0) return 0;
    YITU_REQUIRE(out && row_pointers, "null output or row_pointers");
    YITU_REQUIRE(nnz == 0 || (x && column_index), "null input with nnz > 0");
    YITU_REQUIRE(n_rows < INT32_MAX && n_src < INT32_MAX && dim < (1 << 20), "size out of range");
    SpmmParams p{};
    p.indptr = row_pointers;
    p.indices = column_index;
    p.feat = x;
    p.out = out;
    p.scale_row = degrees;
    p.scale_col = degrees;
    p.edge_scale = degrees ? edge_scale : nullptr;
    p.n_rows = (int)n_rows;
    p.n_src = (int)n_src;
    p.L = (int)dim;
    p.F = (int)dim;
    p.H = 1;
    p.col_mask = 0x7fffffff;
    p.alpha = alpha;
    return launch_spmm(p, degrees ? W_DEGPROD : W_NONE, x_is_bf16 != 0, nnz, max_degree, plan,
                       workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

YITU_API int yitu_edge_scale(float *edge_scale, const int32_t *column_index, const float *degrees,
                            int64_t nnz, int64_t n_src, void *stream) {
    YITU_REQUIRE(nnz >= 0 && nnz < INT32_MAX && n_src >= 0, "size out of range");
    if (nnz == 0) return 0;
    YITU_REQUIRE(edge_scale && column_index && degrees, "null pointer");
    return edge_scale_fill(edge_scale, column_index, degrees, nnz, 0x7fffffff,
                           static_cast<hipStream_t>(stream));
}

// ---- aggregation without any allocation ------------------------------------------
// The scratch of yitu_agg_csr (temporary row plan + partial rows) taken from a
// file-scope device array instead of a caller's workspace. Every GPU the library
// runs on holds its own copy of the array, at its own address, until the process
// ends; the name below is only a host-side handle, the address on the current
// device comes from hipGetSymbolAddress, once per device.
namespace {
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int static_scratch(void **ptr) {
    int dev = 0;
    YITU_HIP(hipGetDevice(&dev));
    YITU_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        YITU_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        YITU_REQUIRE(p != nullptr, "no device address for the static scratch array");
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}
}  // namespace

YITU_API size_t yitu_agg_csr_noalloc_max_bytes(void) { return kStaticScratchBytes; }

YITU_API int yitu_agg_csr_noalloc_init(void) {
    void *ws = nullptr;
    return static_scratch(&ws);
}

YITU_API int yitu_agg_csr_noalloc(float *out, const void *x, int x_is_bf16,
                                  const int32_t *row_pointers, const int32_t *column_index,
                                  const float *degrees, int64_t n_rows, int64_t n_src,
                                  int64_t nnz, int64_t dim, float alpha, int64_t max_degree,
                                  void *stream) {
    YITU_REQUIRE(n_rows >= 0 && n_src >= 0 && nnz >= 0 && dim >= 0, "negative size");
    // no row can reach the planning threshold: no temporary plan, no partial rows, no scratch
    if (nnz < kPlanThreshold || (max_degree >= 0 && max_degree < kPlanThreshold))
        return yitu_agg_csr(out, x, x_is_bf16, row_pointers, column_index, degrees, n_rows, n_src,
                            nnz, dim, alpha, max_degree, nullptr, nullptr, nullptr, 0, stream);
    const size_t need = spmm_workspace_bytes(nnz, dim, false);
    YITU_REQUIRE(need <= kStaticScratchBytes,
                 "problem needs %zu bytes of scratch, the static array holds %zu: use "
                 "yitu_agg_csr with a workspace",
                 need, kStaticScratchBytes);
    void *ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc) return rc;
    return yitu_agg_csr(out, x, x_is_bf16, row_pointers, column_index, degrees, n_rows, n_src, nnz,
                        dim, alpha, max_degree, nullptr, nullptr, ws, kStaticScratchBytes, stream);
}

static int spmm_forward_any(void *out, bool bf16_out, const float *values, const int32_t *indptr,
                            const int32_t *indices, const void *features, bool bf16_in,
                            int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads,
                            int64_t n_features, int64_t max_degree, const void *plan,
                            void *workspace, size_t workspace_bytes, void *stream) {
    YITU_REQUIRE(n_dst >= 0 && n_src >= 0 && nnz >= 0 && n_heads >= 0 && n_features >= 0,
                 "negative size");
    if (n_dst == 0 || n_heads * n_features == 0) return 0;
    YITU_REQUIRE(out && indptr, "null output or indptr");
    YITU_REQUIRE(nnz == 0 || (values && indices && features), "null input with nnz > 0");
    YITU_REQUIRE(n_dst < INT32_MAX && n_src <= (1 << 24) && n_heads * n_features < (1 << 20),
                 "size out of range (columns are 24-bit)");
    YITU_REQUIRE(!bf16_out || (bf16_in && n_features % 8 == 0 && aligned16(features) &&
                               aligned16(out)),
                 "bf16 output rows need bf16 feature rows, a head width that is a multiple of 8 "
                 "and 16-byte aligned buffers");
    SpmmParams p{};
    p.indptr = indptr;
    p.indices = indices;
    p.feat = features;
    p.out = static_cast<float *>(out);
    p.out_bf16 = bf16_out ? 1 : 0;
    p.values = values;
    p.n_rows = (int)n_dst;
    p.n_src = (int)n_src;
    p.L = (int)(n_heads * n_features);
    p.F = (int)n_features;
    p.H = (int)n_heads;
    p.col_mask = 0xffffff;
    p.alpha = 1.0f;
    return launch_spmm(p, W_EDGEHEAD, bf16_in, nnz, max_degree, plan, workspace, workspace_bytes,
                       static_cast<hipStream_t>(stream));
}

YITU_API int yitu_spmm_forward(float *out, const float *values, const int32_t *indptr,
                               const int32_t *indices, const float *features, int64_t n_dst,
                               int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_features,
                               int64_t max_degree, const void *plan, void *workspace,
                               size_t workspace_bytes, void *stream) {
    return spmm_forward_any(out, false, values, indptr, indices, features, false, n_dst, n_src, nnz,
                            n_heads, n_features, max_degree, plan, workspace, workspace_bytes,
                            stream);
}

YITU_API int yitu_spmm_forward_bf16(float *out, const float *values, const int32_t *indptr,
                                    const int32_t *indices, const void *features_bf16,
                                    int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads,
                                    int64_t n_features, int64_t max_degree, const void *plan,
                                    void *workspace, size_t workspace_bytes, void *stream) {
    return spmm_forward_any(out, false, values, indptr, indices, features_bf16, true, n_dst, n_src,
                            nnz, n_heads, n_features, max_degree, plan, workspace, workspace_bytes,
                            stream);
}

YITU_API int yitu_spmm_forward_bf16_rows(void *out_bf16, const float *values, const int32_t *indptr,
                                         const int32_t *indices, const void *features_bf16,
                                         int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads,
                                         int64_t n_features, int64_t max_degree, const void *plan,
                                         void *workspace, size_t workspace_bytes, void *stream) {
    return spmm_forward_any(out_bf16, true, values, indptr, indices, features_bf16, true, n_dst,
                            n_src, nnz, n_heads, n_features, max_degree, plan, workspace,
                            workspace_bytes, stream);
}


// Plain streaming copy (16 bytes per lane), used to calibrate the HBM traffic
// counters and as the achievable-bandwidth reference of the benchmark.
namespace yitu {
__global__ __launch_bounds__(kBlock) void stream_copy_kernel(const uint4 *__restrict__ src,
                                                             uint4 *__restrict__ dst, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (; i < n; i += stride) dst[i] = src[i];
}
}  // namespace yitu

YITU_API int yitu_stream_copy(void *dst, const void *src, int64_t n_bytes, void *stream) {
    YITU_REQUIRE(n_bytes >= 0 && n_bytes % 16 == 0, "size must be a multiple of 16 bytes");
    YITU_REQUIRE(n_bytes == 0 || (dst && src && aligned16(dst) && aligned16(src)),
                 "null or unaligned buffer");
    if (n_bytes == 0) return 0;
    const int64_t n = n_bytes / 16;
    const int grid = (int)std::min<int64_t>(ceil_div(n, kBlock), 32768);
    stream_copy_kernel<<<grid, kBlock, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint4 *>(src), static_cast<uint4 *>(dst), n);
    YITU_LAUNCH_CHECK();
    return 0;
}
