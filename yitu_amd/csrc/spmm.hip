// Instantiation table and host-side launch logic of the row-split SpMM.
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "spmm_rows.hpp"

#include <cstdarg>

namespace yitu {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
const char *last_error() { return g_error; }

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(float *p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (; i < n; i += stride) p[i] = 0.0f;
}

int fill_zero(float *p, int64_t n, hipStream_t stream) {
    if (n <= 0) return 0;
    const int grid = (int)std::min<int64_t>(ceil_div(n, kBlock), 8192);
    fill_zero_kernel<<<grid, kBlock, 0, stream>>>(p, n);
    YITU_LAUNCH_CHECK();
    return 0;
}

// A queued row has >= threshold edges and yields ceil(deg / chunk) items, so
// rows <= nnz / threshold and items <= nnz / chunk + rows.
static inline int64_t hub_max_rows(int64_t nnz) { return nnz / kAggThreshold + 1; }
static inline int64_t hub_max_items(int64_t nnz) { return nnz / kAggChunk + hub_max_rows(nnz) + 1; }

static size_t sort_temp_bytes(int64_t n) {
    size_t bytes = 0;
    uint32_t *k = nullptr;
    int32_t *v = nullptr;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, k, k, v, v, (size_t)n, 0, 16);
    return bytes;
}

size_t hub_workspace_bytes(int64_t nnz, int64_t L) {
    const size_t items = (size_t)hub_max_items(nnz);
    size_t b = 256;  // counters
    b += align_up(sizeof(int4) * (size_t)hub_max_rows(nnz), 256);
    b += align_up(sizeof(int4) * items, 256);
    b += 4 * align_up(sizeof(int32_t) * items, 256);  // sort keys / values, in and out
    b += align_up(sizeof(int4) * items, 256);         // band-ordered item records
    b += align_up(sort_temp_bytes((int64_t)items), 256);
    b += align_up(sizeof(float) * items * (size_t)L, 256);
    return b;
}

struct HubSortBuffers {
    uint32_t *keys_in, *keys_out;
    int32_t *vals_in;
    int4 *records;
    void *temp;
    size_t temp_bytes;
};

static int hub_queue_init(HubQueue &q, HubSortBuffers &sb, void *workspace, size_t workspace_bytes,
                          int64_t nnz, int64_t L) {
    YITU_REQUIRE(workspace != nullptr && workspace_bytes >= hub_workspace_bytes(nnz, L),
                 "workspace too small: need %zu bytes, got %zu", hub_workspace_bytes(nnz, L),
                 workspace_bytes);
    YITU_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "workspace must be 256-byte aligned");
    char *w = static_cast<char *>(workspace);
    q.counters = reinterpret_cast<HubCounters *>(w);
    w += 256;
    q.max_rows = (int)hub_max_rows(nnz);
    q.max_items = (int)hub_max_items(nnz);
    q.chunk = kAggChunk;
    q.rows = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)q.max_rows, 256);
    q.items = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)q.max_items, 256);
    const size_t arr = align_up(sizeof(int32_t) * (size_t)q.max_items, 256);
    sb.keys_in = reinterpret_cast<uint32_t *>(w);
    sb.keys_out = reinterpret_cast<uint32_t *>(w + arr);
    sb.vals_in = reinterpret_cast<int32_t *>(w + 2 * arr);
    q.order = reinterpret_cast<int32_t *>(w + 3 * arr);
    w += 4 * arr;
    sb.records = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)q.max_items, 256);
    sb.temp = w;
    sb.temp_bytes = sort_temp_bytes(q.max_items);
    w += align_up(sb.temp_bytes, 256);
    q.partial = reinterpret_cast<float *>(w);
    return 0;
}

// Queue of (row, 512-edge chunk) items without partial rows, for kernels whose
// per-edge results need no cross-chunk reduction (the per-edge dot products).
int hub512_queue_init(HubQueue &q, void *workspace, size_t workspace_bytes, int64_t nnz) {
    const int64_t rows = nnz / kHubThreshold + 1, items = nnz / kHubChunk + rows + 1;
    const size_t need = 256 + align_up(sizeof(int4) * (size_t)rows, 256) +
                        align_up(sizeof(int4) * (size_t)items, 256);
    YITU_REQUIRE(workspace != nullptr && workspace_bytes >= need,
                 "workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
    YITU_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "workspace must be 256-byte aligned");
    char *w = static_cast<char *>(workspace);
    q = HubQueue{};
    q.counters = reinterpret_cast<HubCounters *>(w);
    w += 256;
    q.max_rows = (int)rows;
    q.max_items = (int)items;
    q.chunk = kHubChunk;
    q.rows = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)rows, 256);
    q.items = reinterpret_cast<int4 *>(w);
    return 0;
}

template <int VEC, int G, int KT, int WMODE, typename TIN>
static int launch_variant(const SpmmParams &p, const HubSortBuffers &sb, bool with_hub,
                          hipStream_t stream) {
    const int grid = (int)ceil_div(p.n_rows, kWavesPerBlock * kRowsPerWave);
    if (with_hub) {
        zero_hub_counters_kernel<<<1, kWave, 0, stream>>>(p.hub.counters);
        YITU_LAUNCH_CHECK();
    }
    spmm_rows_kernel<VEC, G, KT, WMODE, TIN><<<grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (with_hub) {
        // order the items by the band of the feature table they read
        int bits = 1;
        while (((int64_t)1 << bits) < p.n_src) bits++;
        spmm_hub_keys_kernel<<<(int)ceil_div(p.hub.max_items, kBlock), kBlock, 0, stream>>>(
            p, sb.keys_in, sb.vals_in, std::max(0, bits - 16));
        YITU_LAUNCH_CHECK();
        size_t temp_bytes = sb.temp_bytes;
        YITU_HIP(rocprim::radix_sort_pairs(sb.temp, temp_bytes, sb.keys_in, sb.keys_out, sb.vals_in,
                                           p.hub.order, (size_t)p.hub.max_items, 0, 16, stream));
        spmm_hub_records_kernel<<<(int)ceil_div(p.hub.max_items, kBlock), kBlock, 0, stream>>>(
            p, sb.records);
        YITU_LAUNCH_CHECK();
        const int hub_grid = (int)std::min<int64_t>(
            ceil_div(p.hub.max_items, kWavesPerBlock * kItemsPerWave), 1 << 16);
        spmm_hub_items_kernel<VEC, G, KT, WMODE, TIN>
            <<<hub_grid, kBlock, 0, stream>>>(p, sb.records);
        YITU_LAUNCH_CHECK();
        const int red_grid = (int)std::min<int64_t>(p.hub.max_rows, 1 << 16);
        constexpr int RV = VEC >= 4 ? 4 : VEC;  // VEC | L whenever this variant is chosen
        if (p.L % RV == 0)
            spmm_hub_reduce_kernel<WMODE, RV><<<red_grid, kBlock, 0, stream>>>(p);
        else
            spmm_hub_reduce_kernel<WMODE, 1><<<red_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int WMODE, typename TIN, int VEC>
static int dispatch_shape(const SpmmParams &p, const HubSortBuffers &sb, bool with_hub,
                          hipStream_t stream) {
    const int lanes = (p.L + VEC - 1) / VEC;
    if constexpr (VEC >= 4) {
        if (lanes <= 16) return launch_variant<VEC, 16, 1, WMODE, TIN>(p, sb, with_hub, stream);
        if (lanes <= 32) return launch_variant<VEC, 32, 1, WMODE, TIN>(p, sb, with_hub, stream);
        if (lanes <= 64) return launch_variant<VEC, 64, 1, WMODE, TIN>(p, sb, with_hub, stream);
        if (lanes <= 128) return launch_variant<VEC, 64, 2, WMODE, TIN>(p, sb, with_hub, stream);
        if constexpr (VEC == 4) return launch_variant<VEC, 64, 4, WMODE, TIN>(p, sb, with_hub, stream);
        return launch_variant<VEC, 64, 2, WMODE, TIN>(p, sb, with_hub, stream);
    } else {
        if (lanes <= 64) return launch_variant<VEC, 64, 1, WMODE, TIN>(p, sb, with_hub, stream);
        return launch_variant<VEC, 64, 4, WMODE, TIN>(p, sb, with_hub, stream);
    }
}

template <int WMODE>
static int dispatch_type(const SpmmParams &p, const HubSortBuffers &sb, bool bf16_in,
                         bool with_hub, hipStream_t stream) {
    // a lane's VEC elements must stay inside one head and one aligned vector
    const int unit = WMODE == W_EDGEHEAD ? p.F : p.L;
    if constexpr (WMODE != W_EDGEHEAD) {
      if (bf16_in) {
        if (unit % 8 == 0 && aligned16(p.feat) && aligned16(p.out))
            return dispatch_shape<WMODE, bf16_t, 8>(p, sb, with_hub, stream);
        return dispatch_shape<WMODE, bf16_t, 1>(p, sb, with_hub, stream);
      }
    }
    if (unit % 4 == 0 && aligned16(p.feat) && aligned16(p.out))
        return dispatch_shape<WMODE, float, 4>(p, sb, with_hub, stream);
    if (unit % 2 == 0 && aligned16(p.feat) && aligned16(p.out))
        return dispatch_shape<WMODE, float, 2>(p, sb, with_hub, stream);
    return dispatch_shape<WMODE, float, 1>(p, sb, with_hub, stream);
}

int launch_spmm(SpmmParams &p, int wmode, bool bf16_in, int64_t nnz, int64_t max_degree_hint,
                void *workspace, size_t workspace_bytes, hipStream_t stream) {
    if (p.n_rows == 0 || p.L == 0) return 0;
    YITU_REQUIRE(nnz < (int64_t)1 << 31 && (int64_t)p.n_rows * p.L < ((int64_t)1 << 40),
                 "problem exceeds the int32 edge-index range");
    // No row can reach the hub threshold when the whole graph (or its widest
    // row, if the caller knows it) is smaller: skip the queue and its kernels.
    bool with_hub = nnz >= kAggThreshold;
    if (max_degree_hint >= 0 && max_degree_hint < kAggThreshold) with_hub = false;
    p.hub_threshold = with_hub ? kAggThreshold : 0x7fffffff;
    HubSortBuffers sb{};
    if (with_hub) {
        int rc = hub_queue_init(p.hub, sb, workspace, workspace_bytes, nnz, p.L);
        if (rc) return rc;
    } else {
        p.hub = HubQueue{};
    }
    switch (wmode) {
        case W_NONE: return dispatch_type<W_NONE>(p, sb, bf16_in, with_hub, stream);
        case W_DEGPROD: return dispatch_type<W_DEGPROD>(p, sb, bf16_in, with_hub, stream);
        case W_EDGEHEAD:
            YITU_REQUIRE(!bf16_in, "edge-weighted SpMM takes fp32 features");
            return dispatch_type<W_EDGEHEAD>(p, sb, false, with_hub, stream);
    }
    set_error("unknown weight mode %d", wmode);
    return -1;
}

}  // namespace yitu
