// Builds the row plan on the device: queue the long rows (one atomic per
// workgroup), cut every long row where its sorted columns cross the boundaries
// of its source bands and into items of at most 64 edges, key every item by its
// middle source id, stable radix sort, write the records.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "../../include/yitu_hip.h"
#include "plan.hpp"

namespace yitu {

namespace {

constexpr int kBandBits = 16;  // sort key = middle source id reduced to this many bits

struct BuildBuffers {
    PlanCounters *counters;
    int4 *rows;
    int4 *records;
    int *band_info;   // {log2 of the band width, number of bands, local edges, sampled edges}, in the plan header
    int4 *items;      // {first edge, end edge, index into rows[], row} in queue order
    uint32_t *keys_in, *keys_out;
    int32_t *vals_in, *order;
    void *sort_temp;
    size_t sort_temp_bytes;
    int key_shift;    // sort key = middle source id >> key_shift (16 bits)
    int band_shift;   // band of a source = id >> band_shift
    int n_bands;      // 1 = no cuts
    int max_rows, max_items;
};

__global__ __launch_bounds__(kBlock) void plan_init_kernel(BuildBuffers b) {
    const int64_t i0 = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    if (i0 == 0) {
        b.counters->n_items = 0;
        b.counters->n_rows = 0;
        b.counters->overflow = 0;
        b.counters->pad = 0;
    }
    if (i0 == 0) {
        b.band_info[0] = b.band_shift;
        b.band_info[1] = b.n_bands;
        b.band_info[kPlanInfoLocal] = 0;
        b.band_info[kPlanInfoSampled] = 0;
    }
    // slots that get no item sort behind every real key
    for (int64_t i = i0; i < b.max_items; i += stride) {
        b.keys_in[i] = 0xffffu;
        b.vals_in[i] = (int32_t)i;
    }
}

// Every lane owns one row; the long rows of a workgroup are numbered with a
// block-level prefix sum and ONE atomic (hundreds of thousands of same-address
// atomics serialise in L2).
__device__ __forceinline__ int block_rank(bool flag, int *wave_sums, int *block_base, int *counter) {
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    int pre = flag ? 1 : 0;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const int x = __shfl_up(pre, o, kWave);
        if (lane >= o) pre += x;
    }
    if (lane == kWave - 1) wave_sums[wave] = pre;
    pre -= flag ? 1 : 0;
    __syncthreads();
    if (threadIdx.x == 0) {
        int br = 0;
        for (int w = 0; w < kWavesPerBlock; w++) br += wave_sums[w];
        *block_base = br > 0 ? atomicAdd(counter, br) : 0;
    }
    __syncthreads();
    int slot = *block_base + pre;
    for (int w = 0; w < wave; w++) slot += wave_sums[w];
    __syncthreads();  // the shared words are reused by the next call
    return slot;
}

// The same pass measures whether the graph is local, on the rows that the row
// kernels walk (fewer than 64 edges): up to 4 edges of every such row, evenly
// spaced, are sampled, and an edge counts as local when its source lies within
// 1/64 of the id space (at least 1,024 ids) of the row's own relative position.
// One add per workgroup and counter.
__global__ __launch_bounds__(kBlock) void plan_queue_kernel(BuildBuffers b,
                                                            const int32_t *__restrict__ indptr,
                                                            const int32_t *__restrict__ indices,
                                                            int n_rows, int n_src, int col_mask) {
    __shared__ int wave_sums[kWavesPerBlock];
    __shared__ int block_base;
    const int row = blockIdx.x * kBlock + threadIdx.x;
    int deg = 0, beg = 0;
    if (row < n_rows) {
        beg = indptr[row];
        deg = indptr[row + 1] - beg;
    }
    int sampled = 0, local = 0;
    if (deg < kPlanThreshold) {
        sampled = min(deg, 4);
        const long long own = (long long)row * n_src / n_rows;
        const long long reach = max((long long)n_src >> 6, 1024ll);
        for (int k = 0; k < sampled; k++) {
            const long long c = indices[beg + deg * k / sampled] & col_mask;
            local += c - own <= reach && own - c <= reach;
        }
    }
    __shared__ int seen[2];  // sampled edges, local ones
    if (threadIdx.x == 0) seen[0] = seen[1] = 0;
    __syncthreads();
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
        sampled += __shfl_xor(sampled, o, kWave);
        local += __shfl_xor(local, o, kWave);
    }
    if (lane_id() == 0 && sampled) {
        atomicAdd(&seen[0], sampled);
        atomicAdd(&seen[1], local);
    }
    __syncthreads();
    if (threadIdx.x == 0 && seen[0]) {
        atomicAdd(&b.band_info[kPlanInfoSampled], seen[0]);
        if (seen[1]) atomicAdd(&b.band_info[kPlanInfoLocal], seen[1]);
    }
    const bool longrow = deg >= kPlanThreshold;
    const int slot = block_rank(longrow, wave_sums, &block_base, &b.counters->n_rows);
    if (longrow) {
        if (slot >= b.max_rows)
            atomicExch(&b.counters->overflow, 1);
        else
            b.rows[slot] = make_int4(row, 0, 0, 0);
    }
}

// One wave per long row. A row of deg edges may be cut into P = the largest
// power of two <= deg / 16 pieces (at most the number of bands), so its cut points
// are the boundaries of groups of ceil(n_bands / P) consecutive bands: the lanes
// find where the row's columns cross them (binary search), lane 0 turns the
// crossings into segments (none shorter than kPlanMinSegment), the wave then
// writes the items of every segment: ceil(len / 64) pieces of equal size. Item
// ids of a row are consecutive; a workgroup takes its ids with one atomic.
__global__ __launch_bounds__(kBlock) void plan_items_kernel(BuildBuffers b,
                                                            const int32_t *__restrict__ indptr,
                                                            const int32_t *__restrict__ indices,
                                                            int col_mask) {
    __shared__ int cut[kWavesPerBlock][kPlanMaxBands + 1];
    __shared__ int seg_beg[kWavesPerBlock][kPlanMaxBands + 1];    // [n_seg] = end of the row
    __shared__ int seg_first[kWavesPerBlock][kPlanMaxBands + 1];  // first item of the segment, [n_seg] = total
    __shared__ int n_seg[kWavesPerBlock];
    __shared__ int wave_first[kWavesPerBlock];
    const int lane = lane_id();
    const int wave = threadIdx.x / kWave;
    const int slot = blockIdx.x * kWavesPerBlock + wave;
    const int n_rows = b.counters->overflow ? 0 : min(b.counters->n_rows, b.max_rows);
    const bool active = slot < n_rows;
    int row = 0, beg = 0, end = 0;
    if (active) {
        row = b.rows[slot].x;
        beg = indptr[row];
        end = indptr[row + 1];
    }
    const int deg = end - beg;
    // pieces allowed, bands per group, groups
    int allowed = 1;
    while (allowed * 2 * kPlanMinSegment <= deg && allowed * 2 <= b.n_bands) allowed *= 2;
    if (b.n_bands > 1 && allowed * 2 * kPlanMinSegment <= deg) allowed = b.n_bands;
    const int per_group = (b.n_bands + allowed - 1) / allowed;
    const int n_groups = active ? (b.n_bands + per_group - 1) / per_group : 0;
    for (int k = lane; k <= n_groups; k += kWave) {
        int c = k == 0 ? beg : end;
        if (k > 0 && k < n_groups) {
            const long long bound = ((long long)k * per_group) << b.band_shift;
            int lo = beg, hi = end;  // first edge whose column is >= bound
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if ((long long)(indices[mid] & col_mask) < bound) lo = mid + 1; else hi = mid;
            }
            c = lo;
        }
        cut[wave][k] = c;
    }
    __syncthreads();
    if (active && lane == 0) {
        // columns that are not sorted inside the row give crossings out of order;
        // a running maximum keeps the pieces a partition of the row
        int n = 0, cur = beg, total = 0, reach = beg;
        for (int k = 1; k <= n_groups; k++) {
            reach = min(end, max(reach, cut[wave][k]));
            const bool last = k == n_groups;
            const int len = reach - cur;
            if (last ? len > 0
                     : (len >= kPlanMinSegment && end - reach >= kPlanMinSegment &&
                        n < allowed - 1)) {
                seg_beg[wave][n] = cur;
                seg_first[wave][n] = total;
                total += (len + kPlanChunk - 1) / kPlanChunk;
                cur = reach;
                n++;
            }
        }
        seg_beg[wave][n] = end;
        seg_first[wave][n] = total;
        n_seg[wave] = n;
    }
    if (!active && lane == 0) {
        n_seg[wave] = 0;
        seg_first[wave][0] = 0;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int sum = 0;
        for (int w = 0; w < kWavesPerBlock; w++) {
            wave_first[w] = sum;
            sum += seg_first[w][n_seg[w]];
        }
        const int base = sum > 0 ? atomicAdd(&b.counters->n_items, sum) : 0;
        for (int w = 0; w < kWavesPerBlock; w++) wave_first[w] += base;
    }
    __syncthreads();
    if (!active) return;
    const int n = n_seg[wave];
    const int total = seg_first[wave][n];
    const int first_item = wave_first[wave];
    if (first_item + total > b.max_items) {
        if (lane == 0) atomicExch(&b.counters->overflow, 1);
        return;
    }
    if (lane == 0) b.rows[slot] = make_int4(row, first_item, total, 0);
    int s = 0;  // items of a lane come in ascending order: the segment search resumes
    for (int i = lane; i < total; i += kWave) {
        while (s + 1 < n && seg_first[wave][s + 1] <= i) s++;
        const int sb = seg_beg[wave][s], se = seg_beg[wave][s + 1];
        const int pieces = seg_first[wave][s + 1] - seg_first[wave][s];
        const int size = (se - sb + pieces - 1) / pieces;
        const int ib = sb + (i - seg_first[wave][s]) * size;
        const int ie = min(se, ib + size);
        const int mid_col = indices[(ib + ie) >> 1] & col_mask;
        b.items[first_item + i] = make_int4(ib, ie, slot, row);
        b.keys_in[first_item + i] =
            min((uint32_t)mid_col >> b.key_shift, (1u << kBandBits) - 1u);
    }
}

__global__ __launch_bounds__(kBlock) void plan_records_kernel(BuildBuffers b) {
    const int pos = blockIdx.x * kBlock + threadIdx.x;
    const int n_items = b.counters->overflow ? 0 : min(b.counters->n_items, b.max_items);
    if (pos >= b.max_items) return;
    int4 rec = make_int4(0, 0, 0, 0);
    if (pos < n_items) {
        const int item = b.order[pos];  // stable sort: real items precede the padding
        const int4 it = b.items[item];
        // a row that is a single item is finished by the item kernel itself
        const int single = b.rows[it.z].z == 1 ? (int)0x80000000 : 0;
        rec = make_int4(it.x, it.y, item, it.w | single);
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

constexpr size_t kHeaderBytes = 512;  // counters | at byte 256: {log2 band width, bands}

}  // namespace

size_t plan_bytes(int64_t nnz) {
    return kHeaderBytes + align_up(sizeof(int4) * (size_t)plan_max_rows(nnz), 256) +
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
    w += kHeaderBytes;
    v.max_rows = (int)plan_max_rows(nnz);
    v.max_items = (int)plan_max_items(nnz);
    v.rows = reinterpret_cast<const int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)v.max_rows, 256);
    v.records = reinterpret_cast<const int4 *>(w);
    v.threshold = kPlanThreshold;
    v.info = reinterpret_cast<const int *>(static_cast<const char *>(plan) + 256);
    return v;
}

int plan_build(void *plan, size_t plan_size, const int32_t *indptr, const int32_t *indices,
               int64_t n_rows, int64_t n_src, int64_t nnz, int32_t col_mask, bool with_bands,
               void *workspace, size_t workspace_bytes, hipStream_t stream) {
    YITU_REQUIRE(plan && plan_size >= plan_bytes(nnz), "plan buffer too small: need %zu bytes",
                 plan_bytes(nnz));
    YITU_REQUIRE(workspace && workspace_bytes >= plan_build_workspace_bytes(nnz),
                 "workspace too small: need %zu bytes", plan_build_workspace_bytes(nnz));
    YITU_REQUIRE((reinterpret_cast<uintptr_t>(plan) & 255u) == 0 &&
                     (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "plan and workspace must be 256-byte aligned");
    YITU_REQUIRE(n_rows < INT32_MAX && n_src < INT32_MAX && nnz < INT32_MAX, "size out of range");
    const PlanView v = plan_view(plan, nnz);
    BuildBuffers b{};
    b.counters = const_cast<PlanCounters *>(v.counters);
    b.band_info = reinterpret_cast<int *>(static_cast<char *>(plan) + 256);
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
    w += align_up(b.sort_temp_bytes, 256);
    const int64_t span = std::max<int64_t>(n_src, 1) - 1;  // largest source id
    b.key_shift = 0;
    while ((span >> b.key_shift) >= ((int64_t)1 << kBandBits)) b.key_shift++;
    b.band_shift = kPlanBandShift;
    while ((span >> b.band_shift) + 1 > kPlanMaxBands) b.band_shift++;
    b.n_bands = with_bands ? (int)((span >> b.band_shift) + 1) : 1;

    const int item_grid = (int)ceil_div(b.max_items, kBlock);
    plan_init_kernel<<<std::min(item_grid, 4096), kBlock, 0, stream>>>(b);
    YITU_LAUNCH_CHECK();
    if (n_rows > 0) {
        plan_queue_kernel<<<(int)ceil_div(n_rows, kBlock), kBlock, 0, stream>>>(
            b, indptr, indices, (int)n_rows, (int)n_src, col_mask);
        YITU_LAUNCH_CHECK();
    }
    plan_items_kernel<<<(int)ceil_div(b.max_rows, kWavesPerBlock), kBlock, 0, stream>>>(
        b, indptr, indices, col_mask);
    YITU_LAUNCH_CHECK();
    size_t temp_bytes = b.sort_temp_bytes;
    YITU_HIP(rocprim::radix_sort_pairs(b.sort_temp, temp_bytes, b.keys_in, b.keys_out, b.vals_in,
                                       b.order, (size_t)b.max_items, 0, 16, stream));
    plan_records_kernel<<<item_grid, kBlock, 0, stream>>>(b);
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
    if (plan) {  // also without long rows: the header says whether the graph is local
        view = plan_view(plan, nnz);
        return 0;
    }
    if (!has_items) {
        view = plan_none();
        return 0;
    }
    const size_t pb = plan_bytes(nnz), bw = plan_build_workspace_bytes(nnz);
    YITU_REQUIRE(workspace && workspace_bytes >= pb + bw,
                 "workspace too small for a temporary row plan: need %zu bytes, got %zu", pb + bw,
                 workspace_bytes);
    char *w = static_cast<char *>(workspace);
    int rc = plan_build(w, pb, indptr, indices, n_rows, n_src, nnz, col_mask, false, w + pb, bw,
                        stream);
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
    return plan_build(plan, plan_size, indptr, indices, n_rows, n_src, nnz, col_mask, true,
                      workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}
