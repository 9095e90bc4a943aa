// One-time integer graph preparation on the device: edge list -> canonical CSR,
// and the transposed (by-source) view of a CSR with the edge permutation that
// links the two orders. The backward kernels use the latter to turn
// scatter-adds into gathers.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>
#include <rocprim/device/device_select.hpp>

#include "../../include/yitu_hip.h"
#include "spmm_rows.hpp"

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


// ---- edge list -> canonical CSR ---------------------------------------------------
__global__ __launch_bounds__(kBlock) void coo_keys_kernel(const int32_t *__restrict__ rows,
                                                          const int32_t *__restrict__ cols,
                                                          unsigned long long *__restrict__ keys,
                                                          int64_t n_edges, int32_t n_rows,
                                                          int32_t n_cols, int *__restrict__ bad) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_edges) return;
    const int32_t r = rows[i], c = cols[i];
    if (r < 0 || r >= n_rows || c < 0 || c >= n_cols) {
        atomicExch(bad, 1);
        keys[i] = ~0ull;  // sorts last; the count below excludes it
    } else {
        keys[i] = ((unsigned long long)(uint32_t)r << 32) | (uint32_t)c;
    }
}

// unique sorted keys -> indices; indptr[r] = first position whose key is >= (r, 0)
__global__ __launch_bounds__(kBlock) void coo_finish_kernel(
    const unsigned long long *__restrict__ uniq, const size_t *__restrict__ n_unique,
    const int *__restrict__ bad, int32_t *__restrict__ indptr, int32_t *__restrict__ indices,
    long long *__restrict__ nnz_out, int32_t n_rows, int64_t n_edges) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    // an out-of-range edge leaves one ~0 key at the end of the unique list
    const int64_t nnz = (int64_t)*n_unique - (*bad ? 1 : 0);
    if (i == 0) *nnz_out = *bad ? -1 : nnz;
    if (i < nnz) indices[i] = (int32_t)(uniq[i] & 0xffffffffull);
    if (i <= n_rows) {
        const unsigned long long first = (unsigned long long)i << 32;
        int64_t lo = 0, hi = nnz;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (uniq[mid] < first) lo = mid + 1; else hi = mid;
        }
        indptr[i] = (int32_t)lo;
    }
}

static int coo_key_bits(int64_t n_rows) {
    int b = 1;
    while (((int64_t)1 << b) < n_rows) b++;
    return 32 + b;
}

struct CooTemp {
    size_t sort_bytes, unique_bytes;
};
static CooTemp coo_temp(int64_t n_edges, int bits) {
    CooTemp t{};
    unsigned long long *k = nullptr;
    size_t *cnt = nullptr;
    (void)bits;  // all 64 bits are sorted: an out-of-range edge carries the ~0 key
    (void)rocprim::radix_sort_keys(nullptr, t.sort_bytes, k, k, (size_t)n_edges, 0, 64);
    (void)rocprim::unique(nullptr, t.unique_bytes, k, k, cnt, (size_t)n_edges);
    return t;
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

namespace yitu {
namespace {

// groups of row r = ceil(deg / part_size)
__global__ __launch_bounds__(kBlock) void part_count_kernel(int32_t *__restrict__ count,
                                                            const int32_t *__restrict__ indptr,
                                                            int n_rows, int part_size) {
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r < n_rows) count[r] = (indptr[r + 1] - indptr[r] + part_size - 1) / part_size;
}

// One wave per row: group g of row r starts at edge indptr[r] + g part_size. The entry
// behind the last group is the number of edges when the last row has edges and 0
// otherwise, as the reference leaves it (YiTu_GNN.cpp:240-241).
__global__ __launch_bounds__(kBlock) void part_fill_kernel(
    int32_t *__restrict__ part_ptr, int32_t *__restrict__ part2node, long long *__restrict__ n_parts,
    const int32_t *__restrict__ first, const int32_t *__restrict__ count,
    const int32_t *__restrict__ indptr, int n_rows, int part_size, long long capacity) {
    const int lane = threadIdx.x & (kWave - 1);
    const int r = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (r >= n_rows) return;
    const int base = first[r], n = count[r], beg = indptr[r];
    for (int g = lane; g < n; g += kWave) {
        if (base + g < capacity) {
            part_ptr[base + g] = beg + g * part_size;
            part2node[base + g] = r;
        }
    }
    if (r == n_rows - 1 && lane == 0) {
        const long long total = (long long)base + n;
        *n_parts = total;
        if (total < capacity + 1) part_ptr[total] = n > 0 ? indptr[n_rows] : 0;
    }
}

size_t part_scan_bytes(int64_t n_rows) {
    size_t bytes = 0;
    int32_t *p = nullptr;
    (void)rocprim::exclusive_scan(nullptr, bytes, p, p, 0, (size_t)std::max<int64_t>(n_rows, 1),
                                  rocprim::plus<int32_t>());
    return bytes;
}

}  // namespace
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

YITU_API size_t yitu_coo_to_csr_workspace_bytes(int64_t n_edges, int64_t n_rows) {
    if (n_edges <= 0) return 256;
    const CooTemp t = coo_temp(n_edges, coo_key_bits(n_rows));
    return 256 + 2 * align_up(sizeof(unsigned long long) * (size_t)n_edges, 256) +
           align_up(std::max(t.sort_bytes, t.unique_bytes), 256);
}

YITU_API int yitu_coo_to_csr(int32_t *indptr, int32_t *indices, long long *nnz_out,
                             const int32_t *rows, const int32_t *cols, int64_t n_edges,
                             int64_t n_rows, int64_t n_cols, void *workspace,
                             size_t workspace_bytes, void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_edges >= 0 && n_rows >= 0 && n_cols >= 0, "negative size");
    YITU_REQUIRE(n_rows < INT32_MAX && n_cols < INT32_MAX && n_edges < INT32_MAX,
                 "size out of range");
    YITU_REQUIRE(indptr && nnz_out, "null output");
    YITU_REQUIRE(n_edges == 0 || (indices && rows && cols), "null edge array");
    YITU_REQUIRE(workspace && workspace_bytes >= yitu_coo_to_csr_workspace_bytes(n_edges, n_rows) &&
                     (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "workspace too small or not 256-byte aligned: need %zu bytes",
                 yitu_coo_to_csr_workspace_bytes(n_edges, n_rows));
    char *w = static_cast<char *>(workspace);
    size_t *n_unique = reinterpret_cast<size_t *>(w);
    int *bad = reinterpret_cast<int *>(w + 64);
    w += 256;
    const size_t arr = align_up(sizeof(unsigned long long) * (size_t)n_edges, 256);
    unsigned long long *keys = reinterpret_cast<unsigned long long *>(w);
    unsigned long long *sorted = reinterpret_cast<unsigned long long *>(w + arr);
    void *temp = w + 2 * arr;
    int rc = fill_zero(reinterpret_cast<float *>(workspace), 64, stream);  // count and flag
    if (rc) return rc;
    const int grid = (int)ceil_div(std::max<int64_t>(std::max(n_edges, n_rows + 1), 1), kBlock);
    if (n_edges > 0) {
        const int bits = coo_key_bits(n_rows);
        const CooTemp t = coo_temp(n_edges, bits);
        coo_keys_kernel<<<(int)ceil_div(n_edges, kBlock), kBlock, 0, stream>>>(
            rows, cols, keys, n_edges, (int32_t)n_rows, (int32_t)n_cols, bad);
        YITU_LAUNCH_CHECK();
        size_t bytes = t.sort_bytes;
        // all 64 bits when an out-of-range edge may carry the ~0 key
        YITU_HIP(rocprim::radix_sort_keys(temp, bytes, keys, sorted, (size_t)n_edges, 0, 64, stream));
        bytes = t.unique_bytes;
        YITU_HIP(rocprim::unique(temp, bytes, sorted, keys, n_unique, (size_t)n_edges,
                                 rocprim::equal_to<unsigned long long>(), stream));
    }
    // after unique, `keys` holds the distinct (row, col) pairs in ascending order
    coo_finish_kernel<<<grid, kBlock, 0, stream>>>(keys, n_unique, bad, indptr, indices, nnz_out,
                                                   (int32_t)n_rows, n_edges);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API size_t yitu_build_part_workspace_bytes(int64_t n_rows) {
    return 2 * align_up(sizeof(int32_t) * (size_t)std::max<int64_t>(n_rows, 1), 256) +
           align_up(part_scan_bytes(n_rows), 256);
}

namespace yitu {
__global__ void part_empty_kernel(int32_t *part_ptr, long long *n_parts_out) {
    *n_parts_out = 0;
    part_ptr[0] = 0;
}
}  // namespace yitu

YITU_API int yitu_build_part(int32_t *part_ptr, int32_t *part2node, long long *n_parts_out,
                             const int32_t *indptr, int64_t n_rows, int64_t part_size,
                             int64_t capacity, void *workspace, size_t workspace_bytes,
                             void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_rows >= 0 && n_rows < INT32_MAX, "row count out of range");
    YITU_REQUIRE(part_size > 0 && part_size < INT32_MAX, "partSize must be positive");
    YITU_REQUIRE(capacity >= 0 && part_ptr && n_parts_out && (capacity == 0 || part2node),
                 "null output");
    YITU_REQUIRE(indptr, "null indptr");
    YITU_REQUIRE(workspace && workspace_bytes >= yitu_build_part_workspace_bytes(n_rows) &&
                     (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "workspace too small or misaligned: need %zu bytes, 256-byte aligned",
                 yitu_build_part_workspace_bytes(n_rows));
    if (n_rows == 0) {
        // one thread writes the two words: no memset node, so the call may be captured
        part_empty_kernel<<<1, 1, 0, stream>>>(part_ptr, n_parts_out);
        YITU_LAUNCH_CHECK();
        return 0;
    }
    char *w = static_cast<char *>(workspace);
    const size_t arr = align_up(sizeof(int32_t) * (size_t)n_rows, 256);
    int32_t *count = reinterpret_cast<int32_t *>(w);
    int32_t *first = reinterpret_cast<int32_t *>(w + arr);
    void *temp = w + 2 * arr;
    size_t temp_bytes = part_scan_bytes(n_rows);
    part_count_kernel<<<(int)ceil_div(n_rows, kBlock), kBlock, 0, stream>>>(count, indptr,
                                                                           (int)n_rows, (int)part_size);
    YITU_LAUNCH_CHECK();
    YITU_HIP(rocprim::exclusive_scan(temp, temp_bytes, count, first, 0, (size_t)n_rows,
                                     rocprim::plus<int32_t>(), stream));
    part_fill_kernel<<<(int)ceil_div(n_rows, kWavesPerBlock), kBlock, 0, stream>>>(
        part_ptr, part2node, n_parts_out, first, count, indptr, (int)n_rows, (int)part_size,
        (long long)capacity);
    YITU_LAUNCH_CHECK();
    return 0;
}
