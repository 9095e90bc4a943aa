// Temporal neighbour sampler on the device: YiTu_GNN/YiTu_T/sampler_core.cpp
// (ParallelSampler, :43-359) with the T-CSR resident in HBM, so that a training step
// needs no host sampling and no host-to-device copy of the block. yitu_tsample_recent
// is the `recent = True`, single-snapshot mode in one call; yitu_tsample_advance and
// yitu_tsample_window are the pieces of every mode (cursors or binary search, most
// recent or uniformly drawn neighbours, snapshots of a sliding window), which the
// caller strings together per layer and snapshot as the reference's sample() does.
//
// Semantics are those of the host library (csrc/host/sampler.cpp), which is
// bit-exact against the reference: per node a monotone cursor = the running
// maximum over all queries (n, t) seen so far of "last edge of n with
// ts <= t - 1e-7" (update_ts_ptr, :103-127; a running maximum is order
// independent, so an atomic max per root reproduces the sequential loop); then
// every root emits the edges k = cursor, cursor - 1, ... while
// k > max(first edge of n, cursor - fan) and ts[k] < t - 1e-7 (:295-305), in
// root order (count, exclusive scan, fill: the reference's thread-count
// independent order). Output is the COO block of combine_coo (:153-199).
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_scan.hpp>

#include "../../include/yitu_hip.h"
#include "spmm_rows.hpp"

namespace yitu {

namespace {

__device__ __forceinline__ float query_threshold(float t) { return (t + 0.0f) - 1e-7f; }

__global__ __launch_bounds__(kBlock) void ts_reset_kernel(int32_t *__restrict__ cursor,
                                                          const int32_t *__restrict__ indptr,
                                                          int64_t n_nodes) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n_nodes) cursor[i] = indptr[i];
}

__global__ __launch_bounds__(kBlock) void ts_advance_kernel(
    int32_t *__restrict__ cursor, const int32_t *__restrict__ indptr, const float *__restrict__ ts,
    const int32_t *__restrict__ roots, const float *__restrict__ root_ts, int64_t n_roots,
    int32_t n_nodes, int *__restrict__ bad) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_roots) return;
    const int32_t n = roots[i];
    if (n < 0 || n >= n_nodes) {
        atomicExch(bad, 1);
        return;
    }
    const float thr = query_threshold(root_ts[i]);
    int32_t lo = indptr[n], hi = indptr[n + 1];  // first edge with ts > thr
    const int32_t first = lo;
    while (lo < hi) {
        const int32_t mid = lo + ((hi - lo) >> 1);
        if (ts[mid] <= thr) lo = mid + 1; else hi = mid;
    }
    if (lo - 1 >= first) atomicMax(&cursor[n], lo - 1);
}

__global__ __launch_bounds__(kBlock) void ts_count_kernel(
    int32_t *__restrict__ counts, const int32_t *__restrict__ cursor,
    const int32_t *__restrict__ indptr, const float *__restrict__ ts,
    const int32_t *__restrict__ roots, const float *__restrict__ root_ts, int64_t n_roots,
    int32_t n_nodes, int fan) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_roots) return;
    const int32_t n = roots[i];
    int32_t cnt = 0;
    if (n >= 0 && n < n_nodes) {
        const float thr = query_threshold(root_ts[i]);
        const int32_t first = indptr[n], e = cursor[n];
        for (int32_t k = e; k > max(first, e - fan); k--) cnt += ts[k] < thr ? 1 : 0;
    }
    counts[i] = cnt;
}

struct FillArgs {
    int32_t *row, *col, *eid_out, *nodes_out;
    float *ts_out, *dts_out;
    long long *n_edges_out;
    const int32_t *offsets, *counts, *cursor, *indptr, *indices, *eid, *roots;
    const float *ts, *root_ts;
    const int *bad;
    int64_t n_roots;
    int32_t n_nodes;
    int fan, prop_time;
};

__global__ __launch_bounds__(kBlock) void ts_fill_kernel(FillArgs a) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.n_roots) return;
    if (i == a.n_roots - 1)
        *a.n_edges_out = *a.bad ? -1 : (long long)a.offsets[i] + a.counts[i];
    const int32_t n = a.roots[i];
    const float t = a.root_ts[i];
    a.nodes_out[i] = n;
    a.ts_out[i] = t;
    a.dts_out[i] = 0.0f;
    if (n < 0 || n >= a.n_nodes) return;
    const float thr = query_threshold(t);
    const int32_t first = a.indptr[n], e = a.cursor[n];
    int64_t w = a.offsets[i];
    for (int32_t k = e; k > max(first, e - a.fan); k--) {
        if (a.ts[k] < thr) {
            a.row[w] = (int32_t)i;
            a.col[w] = (int32_t)(a.n_roots + w);
            a.eid_out[w] = a.eid[k];
            a.ts_out[a.n_roots + w] = a.prop_time ? t : a.ts[k];
            a.dts_out[a.n_roots + w] = t - a.ts[k];
            a.nodes_out[a.n_roots + w] = a.indices[k];
            w++;
        }
    }
}

// ---- every mode: windows, draws ---------------------------------------------------

// rand_r of the C library the reference is linked against (glibc stdlib/rand_r.c):
// three steps of x -> 1103515245 x + 12345, of which 11 + 10 + 10 bits are taken.
__device__ __forceinline__ int c_rand_r(unsigned int &seed) {
    unsigned int next = seed;
    next = next * 1103515245u + 12345u;
    int result = (int)((next / 65536u) % 2048u);
    next = next * 1103515245u + 12345u;
    result <<= 10;
    result ^= (int)((next / 65536u) % 1024u);
    next = next * 1103515245u + 12345u;
    result <<= 10;
    result ^= (int)((next / 65536u) % 1024u);
    seed = next;
    return result;
}

// The generator state after `steps` steps from x (powers of one affine map commute, so
// the map is squared along the bits of `steps`).
__device__ __forceinline__ unsigned int lcg_skip(unsigned int x, unsigned long long steps) {
    unsigned int a = 1103515245u, c = 12345u;  // the map of 2^k steps
    unsigned int ra = 1u, rc = 0u;             // the map of the bits seen so far
    while (steps) {
        if (steps & 1ull) {
            ra = a * ra;
            rc = a * rc + c;
        }
        c = a * c + c;
        a = a * a;
        steps >>= 1;
    }
    return ra * x + rc;
}

__global__ __launch_bounds__(kBlock) void ts_advance_offset_kernel(
    int32_t *__restrict__ cursor, const int32_t *__restrict__ indptr, const float *__restrict__ ts,
    const int32_t *__restrict__ roots, const float *__restrict__ root_ts, int64_t n_roots,
    int32_t n_nodes, float offset) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_roots) return;
    const int32_t n = roots[i];
    if (n < 0 || n >= n_nodes) return;  // reported by the sampling call
    const float thr = (root_ts[i] + offset) - 1e-7f;
    int32_t lo = indptr[n], hi = indptr[n + 1];  // first edge with ts > thr
    const int32_t first = lo;
    while (lo < hi) {
        const int32_t mid = lo + ((hi - lo) >> 1);
        if (ts[mid] <= thr) lo = mid + 1; else hi = mid;
    }
    if (lo - 1 >= first) atomicMax(&cursor[n], lo - 1);
}

struct WindowArgs {
    int32_t *row, *col, *eid_out, *nodes_out;
    float *ts_out, *dts_out;
    long long *n_edges_out;
    int32_t *win_lo, *win_hi, *draws, *counts;          // per root
    const int32_t *draw_prefix, *offsets;               // exclusive scans of draws / counts
    const int32_t *lo_cursor, *hi_cursor;               // null: binary search
    const int32_t *indptr, *indices, *eid, *roots;
    const float *ts, *root_ts;
    int *bad;
    int64_t n_roots, chunk;
    int32_t n_nodes;
    int fan, prop_time, recent, windowed;
    float offset, window;
};

// last edge of [b, e) with ts <= t, as an index (b - 1 when none)
__device__ __forceinline__ int32_t last_not_after(const float *ts, int32_t b, int32_t e, float t) {
    while (b < e) {
        const int32_t mid = b + ((e - b) >> 1);
        if (ts[mid] <= t) b = mid + 1; else e = mid;
    }
    return b - 1;
}

// The window [lo, hi] of every root (sampler_core.cpp:224-226 with cursors, :262-279 by
// binary search) and whether the root draws (uniform mode and at least `fan` edges).
__global__ __launch_bounds__(kBlock) void ts_window_kernel(WindowArgs a) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.n_roots) return;
    const int32_t n = a.roots[i];
    int32_t lo = 0, hi = 0, draws = 0;
    if (n < 0 || n >= a.n_nodes) {
        atomicExch(a.bad, 1);
    } else {
        const float t = a.root_ts[i];
        const int32_t b = a.indptr[n], e = a.indptr[n + 1];
        if (a.lo_cursor) {
            lo = a.lo_cursor[n];
            hi = a.hi_cursor[n];
        } else if (!a.windowed) {
            lo = b;
            hi = max(last_not_after(a.ts, b, e, t), lo);
        } else {
            lo = max(last_not_after(a.ts, b, e, (t + a.offset) - a.window), b);
            hi = max(last_not_after(a.ts, b, e, t + a.offset), lo);
        }
        draws = (!a.recent && hi - lo >= a.fan) ? 1 : 0;
    }
    a.win_lo[i] = lo;
    a.win_hi[i] = hi;
    a.draws[i] = draws;
}

// The edges root i keeps, in the reference's order (:295-318): emit(k) per edge.
template <typename Emit>
__device__ __forceinline__ int walk_root(const WindowArgs &a, int64_t i, Emit emit) {
    const int32_t n = a.roots[i];
    if (n < 0 || n >= a.n_nodes) return 0;
    const float thr = (a.root_ts[i] + a.offset) - 1e-7f;
    const int32_t lo = a.win_lo[i], hi = a.win_hi[i];
    int kept = 0;
    if (!a.draws[i]) {
        for (int32_t k = hi; k > max(lo, hi - a.fan); k--)
            if (a.ts[k] < thr) {
                emit(k);
                kept++;
            }
    } else {
        // thread c of the reference owns roots [c chunk, (c + 1) chunk) and the generator
        // seeded with c; every drawing root before this one in the chunk took 3 fan steps
        const int64_t c = i / a.chunk;
        const unsigned long long before = (unsigned long long)(a.draw_prefix[i] - a.draw_prefix[c * a.chunk]);
        unsigned int seed = lcg_skip((unsigned int)c, before * 3ull * (unsigned long long)a.fan);
        for (int j = 0; j < a.fan; j++) {
            const int32_t k = lo + c_rand_r(seed) % (hi - lo + 1);
            if (a.ts[k] < thr) {
                emit(k);
                kept++;
            }
        }
    }
    return kept;
}

__global__ __launch_bounds__(kBlock) void ts_window_count_kernel(WindowArgs a) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.n_roots) return;
    a.counts[i] = walk_root(a, i, [](int32_t) {});
}

__global__ __launch_bounds__(kBlock) void ts_window_fill_kernel(WindowArgs a) {
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= a.n_roots) return;
    if (i == a.n_roots - 1)
        *a.n_edges_out = *a.bad ? -1 : (long long)a.offsets[i] + a.counts[i];
    const float t = a.root_ts[i];
    a.nodes_out[i] = a.roots[i];
    a.ts_out[i] = t;
    a.dts_out[i] = 0.0f;
    int64_t w = a.offsets[i];
    walk_root(a, i, [&](int32_t k) {
        a.row[w] = (int32_t)i;
        a.col[w] = (int32_t)(a.n_roots + w);
        a.eid_out[w] = a.eid[k];
        a.ts_out[a.n_roots + w] = a.prop_time ? t : a.ts[k];
        a.dts_out[a.n_roots + w] = t - a.ts[k];
        a.nodes_out[a.n_roots + w] = a.indices[k];
        w++;
    });
}

size_t scan_bytes(int64_t n) {
    size_t bytes = 0;
    int32_t *p = nullptr;
    (void)rocprim::exclusive_scan(nullptr, bytes, p, p, 0, (size_t)n, rocprim::plus<int32_t>());
    return bytes;
}

}  // namespace

}  // namespace yitu

using namespace yitu;
#define YITU_API extern "C" __attribute__((visibility("default")))

YITU_API int yitu_tsample_reset(int32_t *cursor, const int32_t *indptr, int64_t n_nodes,
                                void *stream) {
    YITU_REQUIRE(n_nodes >= 0 && n_nodes < INT32_MAX, "size out of range");
    if (n_nodes == 0) return 0;
    YITU_REQUIRE(cursor && indptr, "null pointer");
    ts_reset_kernel<<<(int)ceil_div(n_nodes, kBlock), kBlock, 0, static_cast<hipStream_t>(stream)>>>(
        cursor, indptr, n_nodes);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API size_t yitu_tsample_workspace_bytes(int64_t n_roots) {
    const int64_t n = std::max<int64_t>(n_roots, 1);
    return 256 + 2 * align_up(sizeof(int32_t) * (size_t)n, 256) + align_up(scan_bytes(n), 256);
}

YITU_API int yitu_tsample_recent(int32_t *row, int32_t *col, int32_t *eid_out, float *ts_out,
                                 float *dts_out, int32_t *nodes_out, long long *n_edges_out,
                                 int32_t *cursor, const int32_t *indptr, const int32_t *indices,
                                 const int32_t *eid, const float *ts, int64_t n_nodes,
                                 const int32_t *roots, const float *root_ts, int64_t n_roots,
                                 int fan, int prop_time, void *workspace, size_t workspace_bytes,
                                 void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_nodes >= 0 && n_roots >= 0 && fan >= 0, "negative size");
    YITU_REQUIRE(n_nodes < INT32_MAX && n_roots * (int64_t)(fan + 1) < INT32_MAX,
                 "size out of range");
    YITU_REQUIRE(n_edges_out, "null output");
    YITU_REQUIRE(workspace && workspace_bytes >= yitu_tsample_workspace_bytes(n_roots) &&
                     (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "workspace too small or not 256-byte aligned: need %zu bytes",
                 yitu_tsample_workspace_bytes(n_roots));
    int rc = fill_zero(static_cast<float *>(workspace), 64, stream);  // flag, and the count below
    if (rc) return rc;
    if (n_roots == 0) {
        // *n_edges_out = 0: reuse the zeroed words
        YITU_HIP(hipMemcpyAsync(n_edges_out, workspace, sizeof(long long), hipMemcpyDeviceToDevice,
                                stream));
        return 0;
    }
    YITU_REQUIRE(row && col && eid_out && ts_out && dts_out && nodes_out && cursor && indptr &&
                     roots && root_ts,
                 "null pointer");
    char *w = static_cast<char *>(workspace);
    int *bad = reinterpret_cast<int *>(w);
    w += 256;
    const size_t arr = align_up(sizeof(int32_t) * (size_t)n_roots, 256);
    int32_t *counts = reinterpret_cast<int32_t *>(w);
    int32_t *offsets = reinterpret_cast<int32_t *>(w + arr);
    void *temp = w + 2 * arr;
    const int grid = (int)ceil_div(n_roots, kBlock);
    ts_advance_kernel<<<grid, kBlock, 0, stream>>>(cursor, indptr, ts, roots, root_ts, n_roots,
                                                   (int32_t)n_nodes, bad);
    YITU_LAUNCH_CHECK();
    ts_count_kernel<<<grid, kBlock, 0, stream>>>(counts, cursor, indptr, ts, roots, root_ts,
                                                 n_roots, (int32_t)n_nodes, fan);
    YITU_LAUNCH_CHECK();
    size_t bytes = scan_bytes(n_roots);
    YITU_HIP(rocprim::exclusive_scan(temp, bytes, counts, offsets, 0, (size_t)n_roots,
                                     rocprim::plus<int32_t>(), stream));
    FillArgs a{};
    a.row = row;
    a.col = col;
    a.eid_out = eid_out;
    a.nodes_out = nodes_out;
    a.ts_out = ts_out;
    a.dts_out = dts_out;
    a.n_edges_out = n_edges_out;
    a.offsets = offsets;
    a.counts = counts;
    a.cursor = cursor;
    a.indptr = indptr;
    a.indices = indices;
    a.eid = eid;
    a.roots = roots;
    a.ts = ts;
    a.root_ts = root_ts;
    a.bad = bad;
    a.n_roots = n_roots;
    a.n_nodes = (int32_t)n_nodes;
    a.fan = fan;
    a.prop_time = prop_time;
    ts_fill_kernel<<<grid, kBlock, 0, stream>>>(a);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API int yitu_tsample_advance(int32_t *cursor, const int32_t *indptr, const float *ts,
                                  int64_t n_nodes, const int32_t *roots, const float *root_ts,
                                  int64_t n_roots, float offset, void *stream) {
    YITU_REQUIRE(n_nodes >= 0 && n_roots >= 0, "negative size");
    YITU_REQUIRE(n_nodes < INT32_MAX && n_roots < INT32_MAX, "size out of range");
    if (n_roots == 0) return 0;
    YITU_REQUIRE(cursor && indptr && roots && root_ts, "null pointer");
    ts_advance_offset_kernel<<<(int)ceil_div(n_roots, kBlock), kBlock, 0,
                               static_cast<hipStream_t>(stream)>>>(
        cursor, indptr, ts, roots, root_ts, n_roots, (int32_t)n_nodes, offset);
    YITU_LAUNCH_CHECK();
    return 0;
}

YITU_API size_t yitu_tsample_window_workspace_bytes(int64_t n_roots) {
    const int64_t n = std::max<int64_t>(n_roots, 1);
    return 256 + 6 * align_up(sizeof(int32_t) * (size_t)n, 256) + align_up(scan_bytes(n), 256);
}

YITU_API int yitu_tsample_window(int32_t *row, int32_t *col, int32_t *eid_out, float *ts_out,
                                 float *dts_out, int32_t *nodes_out, long long *n_edges_out,
                                 const int32_t *lo_cursor, const int32_t *hi_cursor,
                                 const int32_t *indptr, const int32_t *indices, const int32_t *eid,
                                 const float *ts, int64_t n_nodes, const int32_t *roots,
                                 const float *root_ts, int64_t n_roots, int fan, int prop_time,
                                 int recent, int windowed, float offset, float window,
                                 int64_t chunk, void *workspace, size_t workspace_bytes,
                                 void *stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    YITU_REQUIRE(n_nodes >= 0 && n_roots >= 0 && fan >= 0, "negative size");
    YITU_REQUIRE(n_nodes < INT32_MAX && n_roots * (int64_t)(fan + 1) < INT32_MAX,
                 "size out of range");
    YITU_REQUIRE(n_edges_out, "null output");
    YITU_REQUIRE((lo_cursor == nullptr) == (hi_cursor == nullptr),
                 "give both window cursors or neither");
    YITU_REQUIRE(recent || chunk > 0, "uniform draws need the roots per nominal thread");
    YITU_REQUIRE(workspace && workspace_bytes >= yitu_tsample_window_workspace_bytes(n_roots) &&
                     (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                 "workspace too small or not 256-byte aligned: need %zu bytes",
                 yitu_tsample_window_workspace_bytes(n_roots));
    int rc = fill_zero(static_cast<float *>(workspace), 64, stream);  // flag, and the count below
    if (rc) return rc;
    if (n_roots == 0) {
        YITU_HIP(hipMemcpyAsync(n_edges_out, workspace, sizeof(long long), hipMemcpyDeviceToDevice,
                                stream));
        return 0;
    }
    YITU_REQUIRE(row && col && eid_out && ts_out && dts_out && nodes_out && indptr && roots &&
                     root_ts,
                 "null pointer");
    char *w = static_cast<char *>(workspace);
    WindowArgs a{};
    a.bad = reinterpret_cast<int *>(w);
    w += 256;
    const size_t arr = align_up(sizeof(int32_t) * (size_t)n_roots, 256);
    a.win_lo = reinterpret_cast<int32_t *>(w);
    a.win_hi = reinterpret_cast<int32_t *>(w + arr);
    a.draws = reinterpret_cast<int32_t *>(w + 2 * arr);
    int32_t *draw_prefix = reinterpret_cast<int32_t *>(w + 3 * arr);
    a.counts = reinterpret_cast<int32_t *>(w + 4 * arr);
    int32_t *offsets = reinterpret_cast<int32_t *>(w + 5 * arr);
    void *temp = w + 6 * arr;
    a.draw_prefix = draw_prefix;
    a.offsets = offsets;
    a.row = row;
    a.col = col;
    a.eid_out = eid_out;
    a.nodes_out = nodes_out;
    a.ts_out = ts_out;
    a.dts_out = dts_out;
    a.n_edges_out = n_edges_out;
    a.lo_cursor = lo_cursor;
    a.hi_cursor = hi_cursor;
    a.indptr = indptr;
    a.indices = indices;
    a.eid = eid;
    a.roots = roots;
    a.ts = ts;
    a.root_ts = root_ts;
    a.n_roots = n_roots;
    a.chunk = std::max<int64_t>(chunk, 1);
    a.n_nodes = (int32_t)n_nodes;
    a.fan = fan;
    a.prop_time = prop_time;
    a.recent = recent;
    a.windowed = windowed;
    a.offset = offset;
    a.window = window;
    const int grid = (int)ceil_div(n_roots, kBlock);
    ts_window_kernel<<<grid, kBlock, 0, stream>>>(a);
    YITU_LAUNCH_CHECK();
    size_t bytes = scan_bytes(n_roots);
    if (!recent) {
        YITU_HIP(rocprim::exclusive_scan(temp, bytes, a.draws, draw_prefix, 0, (size_t)n_roots,
                                         rocprim::plus<int32_t>(), stream));
    }
    ts_window_count_kernel<<<grid, kBlock, 0, stream>>>(a);
    YITU_LAUNCH_CHECK();
    bytes = scan_bytes(n_roots);
    YITU_HIP(rocprim::exclusive_scan(temp, bytes, a.counts, offsets, 0, (size_t)n_roots,
                                     rocprim::plus<int32_t>(), stream));
    ts_window_fill_kernel<<<grid, kBlock, 0, stream>>>(a);
    YITU_LAUNCH_CHECK();
    return 0;
}
