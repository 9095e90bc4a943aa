// Instantiation table and host-side launch logic of the row-split SpMM.
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

// A hub row has >= kHubThreshold edges and yields ceil(deg / kHubChunk) items,
// so rows <= nnz / threshold and items <= nnz / chunk + rows.
static inline int64_t hub_max_rows(int64_t nnz) { return nnz / kHubThreshold + 1; }
static inline int64_t hub_max_items(int64_t nnz) { return nnz / kHubChunk + hub_max_rows(nnz) + 1; }

size_t hub_workspace_bytes(int64_t nnz, int64_t L) {
    size_t b = 256;  // counters
    b += align_up(sizeof(int4) * (size_t)hub_max_rows(nnz), 256);
    b += align_up(sizeof(int4) * (size_t)hub_max_items(nnz), 256);
    b += align_up(sizeof(float) * (size_t)hub_max_items(nnz) * (size_t)L, 256);
    return b;
}

int hub_queue_init(HubQueue &q, void *workspace, size_t workspace_bytes, int64_t nnz, int64_t L) {
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
    q.rows = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)q.max_rows, 256);
    q.items = reinterpret_cast<int4 *>(w);
    w += align_up(sizeof(int4) * (size_t)q.max_items, 256);
    q.partial = reinterpret_cast<float *>(w);
    return 0;
}

template <int VEC, int G, int KT, int WMODE, typename TIN>
static int launch_variant(const SpmmParams &p, bool with_hub, hipStream_t stream) {
    const int grid = (int)ceil_div(p.n_rows, kWavesPerBlock);
    if (with_hub) {
        zero_hub_counters_kernel<<<1, kWave, 0, stream>>>(p.hub.counters);
        YITU_LAUNCH_CHECK();
    }
    spmm_rows_kernel<VEC, G, KT, WMODE, TIN><<<grid, kBlock, 0, stream>>>(p);
    YITU_LAUNCH_CHECK();
    if (with_hub) {
        const int hub_grid = (int)std::min<int64_t>(p.hub.max_items, 4096);
        spmm_hub_items_kernel<VEC, G, KT, WMODE, TIN><<<hub_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
        const int red_grid = (int)std::min<int64_t>(p.hub.max_rows, 1024);
        spmm_hub_reduce_kernel<WMODE><<<red_grid, kBlock, 0, stream>>>(p);
        YITU_LAUNCH_CHECK();
    }
    return 0;
}

template <int WMODE, typename TIN, int VEC>
static int dispatch_shape(const SpmmParams &p, bool with_hub, hipStream_t stream) {
    const int lanes = (p.L + VEC - 1) / VEC;
    if constexpr (VEC >= 4) {
        if (lanes <= 16) return launch_variant<VEC, 16, 1, WMODE, TIN>(p, with_hub, stream);
        if (lanes <= 32) return launch_variant<VEC, 32, 1, WMODE, TIN>(p, with_hub, stream);
        if (lanes <= 64) return launch_variant<VEC, 64, 1, WMODE, TIN>(p, with_hub, stream);
        if (lanes <= 128) return launch_variant<VEC, 64, 2, WMODE, TIN>(p, with_hub, stream);
        if constexpr (VEC == 4) return launch_variant<VEC, 64, 4, WMODE, TIN>(p, with_hub, stream);
        return launch_variant<VEC, 64, 2, WMODE, TIN>(p, with_hub, stream);
    } else {
        if (lanes <= 64) return launch_variant<VEC, 64, 1, WMODE, TIN>(p, with_hub, stream);
        return launch_variant<VEC, 64, 4, WMODE, TIN>(p, with_hub, stream);
    }
}

template <int WMODE>
static int dispatch_type(const SpmmParams &p, bool bf16_in, bool with_hub, hipStream_t stream) {
    // a lane's VEC elements must stay inside one head and one aligned vector
    const int unit = WMODE == W_EDGEHEAD ? p.F : p.L;
    if constexpr (WMODE != W_EDGEHEAD) {
      if (bf16_in) {
        if (unit % 8 == 0 && aligned16(p.feat) && aligned16(p.out))
            return dispatch_shape<WMODE, bf16_t, 8>(p, with_hub, stream);
        return dispatch_shape<WMODE, bf16_t, 1>(p, with_hub, stream);
      }
    }
    if (unit % 4 == 0 && aligned16(p.feat) && aligned16(p.out))
        return dispatch_shape<WMODE, float, 4>(p, with_hub, stream);
    if (unit % 2 == 0 && aligned16(p.feat) && aligned16(p.out))
        return dispatch_shape<WMODE, float, 2>(p, with_hub, stream);
    return dispatch_shape<WMODE, float, 1>(p, with_hub, stream);
}

int launch_spmm(SpmmParams &p, int wmode, bool bf16_in, int64_t nnz, int64_t max_degree_hint,
                void *workspace, size_t workspace_bytes, hipStream_t stream) {
    if (p.n_rows == 0 || p.L == 0) return 0;
    YITU_REQUIRE(nnz < (int64_t)1 << 31 && (int64_t)p.n_rows * p.L < ((int64_t)1 << 40),
                 "problem exceeds the int32 edge-index range");
    // No row can reach the hub threshold when the whole graph (or its widest
    // row, if the caller knows it) is smaller: skip the queue and its kernels.
    bool with_hub = nnz >= kHubThreshold;
    if (max_degree_hint >= 0 && max_degree_hint < kHubThreshold) with_hub = false;
    p.hub_threshold = with_hub ? kHubThreshold : 0x7fffffff;
    if (with_hub) {
        int rc = hub_queue_init(p.hub, workspace, workspace_bytes, nnz, p.L);
        if (rc) return rc;
    } else {
        p.hub = HubQueue{};
    }
    switch (wmode) {
        case W_NONE: return dispatch_type<W_NONE>(p, bf16_in, with_hub, stream);
        case W_DEGPROD: return dispatch_type<W_DEGPROD>(p, bf16_in, with_hub, stream);
        case W_EDGEHEAD:
            YITU_REQUIRE(!bf16_in, "edge-weighted SpMM takes fp32 features");
            return dispatch_type<W_EDGEHEAD>(p, false, with_hub, stream);
    }
    set_error("unknown weight mode %d", wmode);
    return -1;
}

}  // namespace yitu
