// Builds the row plan on the device: queue the long rows and their 64-edge
// items (one atomic per workgroup), key every item by its middle source id,
// stable radix sort, write the band-ordered records.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "../../include/yitu_hip.h"
#include "plan.hpp"

namespace yitu {

namespace {

constexpr int kQueueRowsPerWave = 64;  // one row per lane

struct BuildBuffers {
    PlanCounters *counters;
    int4 *rows;
    int4 *records;
    int4 *items;  // {row, chunk, index into rows[], 0} in queue order
    uint32_t *keys_in, *keys_out;
    int32_t *vals_in, *order;
    void *sort_temp;
    size_t sort_temp_bytes;
    int max_rows, max_items;
};

__global__ void plan_zero_kernel(PlanCounters *c) {
    if (threadIdx.x == 0) {
        c->n_items = 0;
        c->n_rows = 0;
        c->overflow = 0;
        c->pad = 0;
    }
}

// Every lane owns one row. Long rows get consecutive item ids; a workgroup's
// rows are numbered with a block-level prefix sum and ONE 64-bit atomic on the
// two counters (hundreds of thousands of same-address atomics serialise in L2).
__global__ __launch_bounds__(kBlock) void plan_queue_kernel(BuildBuffers b,
                                                            const int32_t *__restrict__ indptr,
                                                            int n_rows) {
    __shared__ int wave_rows[kWavesPerBlock], wave_items[kWavesPerBlock];
    __shared__ int block_first_row, block_first_item;
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int row = blockIdx.x * kBlock + threadIdx.x;
    int deg = 0;
    if (row < n_rows) deg = indptr[row + 1] - indptr[row];
    const bool longrow = deg >= kPlanThreshold;
    const int chunks = longrow ? (deg + kPlanChunk - 1) / kPlanChunk : 0;
    int pre_rows = longrow ? 1 : 0, pre_items = chunks;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int x = __shfl_up(pre_rows, o, kWave), y = __shfl_up(pre_items, o, kWave);
        if (lane >= o) {
            pre_rows += x;
            pre_items += y;
        }
    }
    if (lane == kWave - 1) {
        wave_rows[wave] = pre_rows;
        wave_items[wave] = pre_items;
    }
    pre_rows -= longrow ? 1 : 0;
    pre_items -= chunks;
    __syncthreads();
    if (threadIdx.x == 0) {
        int br = 0, bi = 0;
        for (int w = 0; w < kWavesPerBlock; w++) {
            br += wave_rows[w];
            bi += wave_items[w];
        }
        unsigned long long old = 0;
        if (br > 0)  // PlanCounters starts with n_items (low word) then n_rows (high word)
            old = atomicAdd(reinterpret_cast<unsigned long long *>(b.counters),
                            ((unsigned long long)(unsigned)br << 32) | (unsigned)bi);
        block_first_item = (int)(old & 0xffffffffu);
        block_first_row = (int)(old >> 32);
    }
    __syncthreads();
    if (!longrow) return;
    int first_row = block_first_row + pre_rows, first_item = block_first_item + pre_items;
    for (int w = 0; w < wave; w++) {
        first_row += wave_rows[w];
        first_item += wave_items[w];
    }
    if (first_row >= b.max_rows || first_item + chunks > b.max_items) {
        atomicExch(&b.counters->overflow, 1);
        return;
    }
    b.rows[first_row] = make_int4(row, first_item, chunks, 0);
    for (int c = 0; c < chunks; c++) b.items[first_item + c] = make_int4(row, c, first_row, 0);
}

// Band key of every queued item: the source id in the middle of the item,
// reduced to 16 bits. Slots past the item count get the largest key.
__global__ __launch_bounds__(kBlock) void plan_keys_kernel(BuildBuffers b,
                                                           const int32_t *__restrict__ indptr,
                                                           const int32_t *__restrict__ indices,
                                                           int col_mask, int shift) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= b.max_items) return;
    const int n_items = b.counters->overflow ? 0 : min(b.counters->n_items, b.max_items);
    uint32_t key = 0xffffu;
    if (i < n_items) {
        const int4 it = b.items[i];
        const int beg = indptr[it.x] + it.y * kPlanChunk;
        const int end = min(indptr[it.x + 1], beg + kPlanChunk);
        key = min(0xffffu, (uint32_t)(indices[(beg + end) >> 1] & col_mask) >> shift);
    }
    b.keys_in[i] = key;
    b.vals_in[i] = i;
}

__global__ __launch_bounds__(kBlock) void plan_records_kernel(BuildBuffers b,
                                                              const int32_t *__restrict__ indptr) {
    const int pos = blockIdx.x * kBlock + threadIdx.x;
    if (pos >= b.max_items) return;
    const int n_items = b.counters->overflow ? 0 : min(b.counters->n_items, b.max_items);
    int4 rec = make_int4(0, 0, 0, 0);
    if (pos < n_items) {
        const int item = b.order[pos];  // stable sort: real items precede the padding
        const int4 it = b.items[item];
        const int row_beg = indptr[it.x], row_end = indptr[it.x + 1];
        const int beg = row_beg + it.y * kPlanChunk;
        // a row that is a single item is finished by the item kernel itself
        const int single = (row_end - row_beg <= kPlanChunk) ? (int)0x80000000 : 0;
        rec = make_int4(beg, min(row_end, beg + kPlanChunk), item, it.x | single);
    }
    b.records[pos] = rec;
}

size_t sort_temp_bytes(int64_t n) {
    size_t bytes = 0;
    uint32_t *k = nullptr;
    int32_t *v = nullptr;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, k, k, v, v, (size_t)n, 0, 16);
    return bytes;
}

}  // namespace

size_t plan_bytes(int64_t nnz) {
    return 256 + align_up(sizeof(int4) * (size_t)plan_max_rows(nnz), 256) +
           align_up(sizeof(int4) * (size_t)plan_max_items(nnz), 256);
}

size_t plan_build_workspace_bytes(int64_t nnz) {
    const size_t items = (size_t)plan_max_items(nnz);
    return align_up(sizeof(int4) * items, 256) + 4 * align_up(sizeof(int32_t) * items, 256) +
           align_up(sort_temp_bytes((int64_t)items), 256);
}

size_t plan_temp_bytes(int64_t nnz) { return plan_bytes(nnz) + plan_build_workspace_bytes(nnz); }

PlanView plan_view(const void *plan, int64_t nnz) {
    PlanView v{};
    const char *w = static_cast<const char *>(plan);
    v.counters = reinterpret_cast<const PlanCounters *>(w);
    w += 256;
    v.max_rows = (int)plan_max_rows(nnz);
    v.max_items = (int)plan_max_items(nnz);
    v.rows = reinterpret_cast<const int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)v.max_rows, 256);
    v.records = reinterpret_cast<const int4 *>(w);
    v.threshold = kPlanThreshold;
    return v;
}

int plan_build(void *plan, size_t plan_size, const int32_t *indptr, const int32_t *indices,
               int64_t n_rows, int64_t n_src, int64_t nnz, int32_t col_mask, void *workspace,
               size_t workspace_bytes, hipStream_t stream) {
    YITU_REQUIRE(plan && plan_size >= plan_bytes(nnz), "plan buffer too small: need %zu bytes",
                 plan_bytes(nnz));
    YITU_REQUIRE(workspace && workspace_bytes >= plan_build_workspace_bytes(nnz),
                 "workspace too small: need %zu bytes", plan_build_workspace_bytes(nnz));
    YITU_REQUIRE((reinterpret_cast<uintptr_t>(plan) & 255u) == 0 &&
                     (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "plan and workspace must be 256-byte aligned");
    YITU_REQUIRE(n_rows < INT32_MAX && nnz < INT32_MAX, "size out of range");
    const PlanView v = plan_view(plan, nnz);
    BuildBuffers b{};
    b.counters = const_cast<PlanCounters *>(v.counters);
    b.rows = const_cast<int4 *>(v.rows);
    b.records = const_cast<int4 *>(v.records);
    b.max_rows = v.max_rows;
    b.max_items = v.max_items;
    char *w = static_cast<char *>(workspace);
    b.items = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)b.max_items, 256);
    const size_t arr = align_up(sizeof(int32_t) * (size_t)b.max_items, 256);
    b.keys_in = reinterpret_cast<uint32_t *>(w);
    b.keys_out = reinterpret_cast<uint32_t *>(w + arr);
    b.vals_in = reinterpret_cast<int32_t *>(w + 2 * arr);
    b.order = reinterpret_cast<int32_t *>(w + 3 * arr);
    w += 4 * arr;
    b.sort_temp = w;
    b.sort_temp_bytes = sort_temp_bytes(b.max_items);

    plan_zero_kernel<<<1, kWave, 0, stream>>>(b.counters);
    YITU_LAUNCH_CHECK();
    if (n_rows > 0) {
        plan_queue_kernel<<<(int)ceil_div(n_rows, kBlock), kBlock, 0, stream>>>(b, indptr,
                                                                                (int)n_rows);
        YITU_LAUNCH_CHECK();
    }
    int bits = 1;
    while (((int64_t)1 << bits) < n_src) bits++;
    const int grid = (int)ceil_div(b.max_items, kBlock);
    plan_keys_kernel<<<grid, kBlock, 0, stream>>>(b, indptr, indices, col_mask,
                                                  std::max(0, bits - 16));
    YITU_LAUNCH_CHECK();
    size_t temp_bytes = b.sort_temp_bytes;
    YITU_HIP(rocprim::radix_sort_pairs(b.sort_temp, temp_bytes, b.keys_in, b.keys_out, b.vals_in,
                                       b.order, (size_t)b.max_items, 0, 16, stream));
    plan_records_kernel<<<grid, kBlock, 0, stream>>>(b, indptr);
    YITU_LAUNCH_CHECK();
    return 0;
}

int plan_resolve(PlanView &view, bool &has_items, const void *plan, const int32_t *indptr,
                 const int32_t *indices, int64_t n_rows, int64_t n_src, int64_t nnz,
                 int32_t col_mask, int64_t max_degree_hint, void *workspace,
                 size_t workspace_bytes, void **rest, size_t *rest_bytes, hipStream_t stream) {
    *rest = workspace;
    *rest_bytes = workspace_bytes;
    has_items = nnz >= kPlanThreshold && !(max_degree_hint >= 0 && max_degree_hint < kPlanThreshold);
    if (!has_items) {
        view = plan_none();
        return 0;
    }
    if (plan) {
        view = plan_view(plan, nnz);
        return 0;
    }
    const size_t pb = plan_bytes(nnz), bw = plan_build_workspace_bytes(nnz);
    YITU_REQUIRE(workspace && workspace_bytes >= pb + bw,
                 "workspace too small for a temporary row plan: need %zu bytes, got %zu", pb + bw,
                 workspace_bytes);
    char *w = static_cast<char *>(workspace);
    int rc = plan_build(w, pb, indptr, indices, n_rows, n_src, nnz, col_mask, w + pb, bw, stream);
    if (rc) return rc;
    view = plan_view(w, nnz);
    // the build scratch is dead once the records are written: hand it back
    *rest = w + pb;
    *rest_bytes = workspace_bytes - pb;
    return 0;
}

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API size_t yitu_plan_bytes(int64_t nnz) { return plan_bytes(nnz); }
YITU_API size_t yitu_plan_workspace_bytes(int64_t nnz) { return plan_build_workspace_bytes(nnz); }

YITU_API int yitu_plan_build(void *plan, size_t plan_size, const int32_t *indptr,
                             const int32_t *indices, int64_t n_rows, int64_t n_src, int64_t nnz,
                             int32_t col_mask, void *workspace, size_t workspace_bytes,
                             void *stream) {
    YITU_REQUIRE(n_rows >= 0 && n_src >= 0 && nnz >= 0, "negative size");
    YITU_REQUIRE(indptr && (nnz == 0 || indices), "null CSR");
    return plan_build(plan, plan_size, indptr, indices, n_rows, n_src, nnz, col_mask, workspace,
                      workspace_bytes, static_cast<hipStream_t>(stream));
}
