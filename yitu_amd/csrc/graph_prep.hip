// One-time integer graph preparation on the device: the transposed (by-source)
// view of a CSR with the edge permutation that links the two orders. The
// backward kernels use it to turn scatter-adds into gathers.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "../../include/yitu_hip.h"
#include "common.hpp"

namespace yitu {

__global__ __launch_bounds__(kBlock) void transpose_keys_kernel(const int32_t *__restrict__ indices,
                                                                int32_t *__restrict__ keys,
                                                                int32_t *__restrict__ vals,
                                                                int64_t nnz, int col_mask) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < nnz) {
        keys[i] = indices[i] & col_mask;
        vals[i] = (int32_t)i;
    }
}

// sorted keys -> indptr of the transposed matrix; position j closes every
// column in (keys[j-1], keys[j]] (empty columns included).
__global__ __launch_bounds__(kBlock) void transpose_bounds_kernel(
    const int32_t *__restrict__ keys_sorted, int32_t *__restrict__ t_indptr, int64_t nnz,
    int32_t n_cols) {
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j > nnz) return;
    const int32_t prev = j == 0 ? -1 : keys_sorted[j - 1];
    const int32_t cur = j == nnz ? n_cols : keys_sorted[j];
    for (int32_t c = prev + 1; c <= cur && c <= n_cols; c++) t_indptr[c] = (int32_t)j;
}

// row of CSR edge e = last r with indptr[r] <= e
__global__ __launch_bounds__(kBlock) void transpose_rows_kernel(const int32_t *__restrict__ indptr,
                                                                const int32_t *__restrict__ t_perm,
                                                                int32_t *__restrict__ t_rows,
                                                                int64_t nnz, int32_t n_rows) {
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= nnz) return;
    const int32_t e = t_perm[j];
    int32_t lo = 0, hi = n_rows;  // invariant: indptr[lo] <= e < indptr[hi]
    while (hi - lo > 1) {
        const int32_t mid = lo + ((hi - lo) >> 1);
        if (indptr[mid] <= e)
            lo = mid;
        else
            hi = mid;
    }
    t_rows[j] = lo;
}

static int key_bits(int64_t n_cols) {
    int b = 1;
    while (((int64_t)1 << b) < n_cols) b++;
    return b;
}

static size_t sort_temp_bytes(int64_t nnz, int bits) {
    size_t bytes = 0;
    int32_t *k = nullptr;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, k, k, k, k, (size_t)nnz, 0, bits);
    return bytes;
}

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API size_t yitu_csr_transpose_workspace_bytes(int64_t nnz, int64_t n_cols) {
    if (nnz <= 0) return 256;
    return align_up(sort_temp_bytes(nnz, key_bits(n_cols)), 256) +
           3 * align_up(sizeof(int32_t) * (size_t)nnz, 256);
}

YITU_API int yitu_csr_transpose(int32_t *t_indptr, int32_t *t_rows, int32_t *t_perm,
                                const int32_t *indptr, const int32_t *indices, int64_t n_rows,
                                int64_t n_cols, int64_t nnz, int32_t col_mask, void *workspace,
                                size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_rows >= 0 && n_cols >= 0 && nnz >= 0, "negative size");
    YITU_REQUIRE(t_indptr && indptr, "null indptr");
    YITU_REQUIRE(n_rows < INT32_MAX && n_cols < INT32_MAX && nnz < INT32_MAX, "size out of range");
    const int grid_c = (int)ceil_div(nnz + 1, kBlock);
    if (nnz == 0) {
        // all columns empty
        transpose_bounds_kernel<<<(int)ceil_div(1, kBlock), kBlock, 0, stream>>>(nullptr, t_indptr,
                                                                                 0, (int32_t)n_cols);
        YITU_LAUNCH_CHECK();
        return 0;
    }
    YITU_REQUIRE(t_rows && t_perm && indices, "null edge array");
    YITU_REQUIRE(workspace && workspace_bytes >= yitu_csr_transpose_workspace_bytes(nnz, n_cols),
                 "workspace too small: need %zu bytes",
                 yitu_csr_transpose_workspace_bytes(nnz, n_cols));
    const int bits = key_bits(n_cols);
    char *w = static_cast<char *>(workspace);
    const size_t arr = align_up(sizeof(int32_t) * (size_t)nnz, 256);
    int32_t *keys = reinterpret_cast<int32_t *>(w);
    int32_t *keys_sorted = reinterpret_cast<int32_t *>(w + arr);
    int32_t *vals = reinterpret_cast<int32_t *>(w + 2 * arr);
    void *temp = w + 3 * arr;
    size_t temp_bytes = sort_temp_bytes(nnz, bits);

    const int grid = (int)ceil_div(nnz, kBlock);
    transpose_keys_kernel<<<grid, kBlock, 0, stream>>>(indices, keys, vals, nnz, col_mask);
    YITU_LAUNCH_CHECK();
    // stable: inside one source column the edges keep CSR order, i.e. ascending row
    YITU_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys, keys_sorted, vals, t_perm,
                                       (size_t)nnz, 0, bits, stream));
    transpose_bounds_kernel<<<grid_c, kBlock, 0, stream>>>(keys_sorted, t_indptr, nnz,
                                                           (int32_t)n_cols);
    YITU_LAUNCH_CHECK();
    transpose_rows_kernel<<<grid, kBlock, 0, stream>>>(indptr, t_perm, t_rows, nnz,
                                                       (int32_t)n_rows);
    YITU_LAUNCH_CHECK();
    return 0;
}
