// Most-recent-neighbour temporal sampler over a T-CSR (per-node edge lists sorted
// by timestamp), the `recent = True`, single-snapshot mode of
// YiTu_GNN/YiTu_T/sampler_core.cpp (ParallelSampler, :43-359).
//
// Per root (n, t) the sampler keeps a monotone cursor into n's edge list that is
// advanced to the last edge with ts <= t - 1e-7 (update_ts_ptr, :103-127), then
// emits the edges k = cursor, cursor-1, ... while k > max(first edge of n,
// cursor - k_neigh) and ts[k] < t - 1e-7 (:295-305): at most k_neigh edges, the
// node's first edge is never emitted, and roots that repeat a node share the
// cursor (so the one with the smaller t may get fewer edges). Output is the COO
// block of combine_coo (:153-199): row = root slot, col = n_roots + running
// index, nodes = [roots..., neighbours...].
//
// The cursor update for a batch is order independent (it is a running maximum),
// so it runs first, sequentially and in amortised O(1) per root; the emission is
// parallel over roots with a count / prefix-sum / fill scheme, which gives the
// reference's thread-count-independent ordering by construction.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include <omp.h>

#include "../../../include/yitu_host.h"

namespace {

struct Block {
    std::vector<int32_t> row, col, eid, nodes;
    std::vector<float> ts, dts;
    int64_t dim_in = 0, dim_out = 0;
};

}  // namespace

struct yitu_sampler {
    std::vector<int32_t> indptr, indices, eid;
    std::vector<float> ts;
    std::vector<int32_t> cursor;  // per node: last edge with ts <= (latest query time - 1e-7)
    std::vector<int32_t> fanout;
    int num_layers = 1;
    int num_threads = 1;
    bool prop_time = false;
    std::vector<Block> blocks;
    char err[256] = "";
};

namespace {

void sample_layer(yitu_sampler *s, const int32_t *roots, const float *root_ts, int64_t n_roots,
                  int fan, Block &out) {
    // 1. advance the cursors (sampler_core.cpp:103-127 with slc = 1, offset = 0)
    for (int64_t i = 0; i < n_roots; i++) {
        const int32_t n = roots[i];
        const float thr = (root_ts[i] + 0.0f) - 1e-7f;
        const int32_t end = s->indptr[n + 1];
        const int32_t c0 = s->cursor[n];
        for (int32_t j = c0; j < end; j++) {
            if (s->ts[j] > thr) {
                if (j != c0) s->cursor[n] = j - 1;
                break;
            }
            if (j == end - 1) s->cursor[n] = j;
        }
    }
    // 2. count, prefix, fill
    std::vector<int64_t> offs((size_t)n_roots + 1, 0);
#pragma omp parallel for schedule(static) num_threads(s->num_threads)
    for (int64_t i = 0; i < n_roots; i++) {
        const int32_t n = roots[i];
        const float thr = (root_ts[i] + 0.0f) - 1e-7f;
        const int32_t first = s->indptr[n], e = s->cursor[n];
        int64_t cnt = 0;
        for (int32_t k = e; k > std::max(first, e - fan); k--) cnt += s->ts[k] < thr;
        offs[(size_t)i + 1] = cnt;
    }
    for (int64_t i = 0; i < n_roots; i++) offs[(size_t)i + 1] += offs[(size_t)i];
    const int64_t m = offs[(size_t)n_roots];
    out.row.resize((size_t)m);
    out.col.resize((size_t)m);
    out.eid.resize((size_t)m);
    out.ts.resize((size_t)(m + n_roots));
    out.dts.assign((size_t)(m + n_roots), 0.0f);
    out.nodes.resize((size_t)(m + n_roots));
    std::copy(roots, roots + n_roots, out.nodes.begin());
    std::copy(root_ts, root_ts + n_roots, out.ts.begin());
#pragma omp parallel for schedule(static) num_threads(s->num_threads)
    for (int64_t i = 0; i < n_roots; i++) {
        const int32_t n = roots[i];
        const float t = root_ts[i];
        const float thr = (t + 0.0f) - 1e-7f;
        const int32_t first = s->indptr[n], e = s->cursor[n];
        int64_t w = offs[(size_t)i];
        for (int32_t k = e; k > std::max(first, e - fan); k--) {
            if (s->ts[k] < thr) {
                out.row[(size_t)w] = (int32_t)i;
                out.col[(size_t)w] = (int32_t)(n_roots + w);
                out.eid[(size_t)w] = s->eid[k];
                out.ts[(size_t)(n_roots + w)] = s->prop_time ? t : s->ts[k];
                out.dts[(size_t)(n_roots + w)] = t - s->ts[k];
                out.nodes[(size_t)(n_roots + w)] = s->indices[k];
                w++;
            }
        }
    }
    out.dim_in = m + n_roots;
    out.dim_out = n_roots;
}

}  // namespace

#define YITU_HOST_API extern "C" __attribute__((visibility("default")))

YITU_HOST_API yitu_sampler *yitu_sampler_create(const int32_t *indptr, const int32_t *indices,
                                                const int32_t *eid, const float *ts,
                                                int64_t n_nodes, int64_t n_edges, int num_threads,
                                                int num_layers, const int32_t *num_neighbors,
                                                int prop_time) {
    if (!indptr || n_nodes < 0 || n_edges < 0 || num_layers < 1 || !num_neighbors) return nullptr;
    if (n_edges > 0 && (!indices || !eid || !ts)) return nullptr;
    if (indptr[0] != 0 || indptr[n_nodes] != n_edges) return nullptr;
    for (int64_t v = 0; v < n_nodes; v++)
        if (indptr[v + 1] < indptr[v]) return nullptr;
    yitu_sampler *s = new yitu_sampler;
    s->indptr.assign(indptr, indptr + n_nodes + 1);
    s->indices.assign(indices, indices + n_edges);
    s->eid.assign(eid, eid + n_edges);
    s->ts.assign(ts, ts + n_edges);
    s->fanout.assign(num_neighbors, num_neighbors + num_layers);
    s->num_layers = num_layers;
    s->num_threads = std::max(1, num_threads);
    s->prop_time = prop_time != 0;
    s->cursor.assign(indptr, indptr + n_nodes);
    return s;
}

YITU_HOST_API void yitu_sampler_destroy(yitu_sampler *s) { delete s; }

YITU_HOST_API int yitu_sampler_reset(yitu_sampler *s) {
    if (!s) return -1;
    std::copy(s->indptr.begin(), s->indptr.end() - 1, s->cursor.begin());
    return 0;
}

YITU_HOST_API int yitu_sampler_sample(yitu_sampler *s, const int32_t *root_nodes,
                                      const float *root_ts, int64_t n_roots) {
    if (!s || n_roots < 0 || (n_roots > 0 && (!root_nodes || !root_ts))) return -1;
    const int64_t n_nodes = (int64_t)s->indptr.size() - 1;
    for (int64_t i = 0; i < n_roots; i++) {
        if (root_nodes[i] < 0 || root_nodes[i] >= n_nodes) {
            snprintf(s->err, sizeof(s->err), "root %lld: node id %d out of range",
                     (long long)i, root_nodes[i]);
            return -1;
        }
    }
    s->blocks.assign((size_t)s->num_layers, Block{});
    const int32_t *nodes = root_nodes;
    const float *ts = root_ts;
    int64_t n = n_roots;
    for (int l = 0; l < s->num_layers; l++) {
        sample_layer(s, nodes, ts, n, s->fanout[(size_t)l], s->blocks[(size_t)l]);
        // the next layer expands every node of this block (roots and neighbours)
        nodes = s->blocks[(size_t)l].nodes.data();
        ts = s->blocks[(size_t)l].ts.data();
        n = (int64_t)s->blocks[(size_t)l].nodes.size();
    }
    return 0;
}

YITU_HOST_API int64_t yitu_sampler_num_blocks(const yitu_sampler *s) {
    return s ? (int64_t)s->blocks.size() : -1;
}

YITU_HOST_API int yitu_sampler_block_sizes(const yitu_sampler *s, int block, int64_t *n_edges,
                                           int64_t *dim_in, int64_t *dim_out) {
    if (!s || block < 0 || (size_t)block >= s->blocks.size()) return -1;
    const Block &b = s->blocks[(size_t)block];
    if (n_edges) *n_edges = (int64_t)b.row.size();
    if (dim_in) *dim_in = b.dim_in;
    if (dim_out) *dim_out = b.dim_out;
    return 0;
}

YITU_HOST_API int yitu_sampler_block_copy(const yitu_sampler *s, int block, int32_t *row,
                                          int32_t *col, int32_t *eid, float *ts, float *dts,
                                          int32_t *nodes) {
    if (!s || block < 0 || (size_t)block >= s->blocks.size()) return -1;
    const Block &b = s->blocks[(size_t)block];
    if (row) std::copy(b.row.begin(), b.row.end(), row);
    if (col) std::copy(b.col.begin(), b.col.end(), col);
    if (eid) std::copy(b.eid.begin(), b.eid.end(), eid);
    if (ts) std::copy(b.ts.begin(), b.ts.end(), ts);
    if (dts) std::copy(b.dts.begin(), b.dts.end(), dts);
    if (nodes) std::copy(b.nodes.begin(), b.nodes.end(), nodes);
    return 0;
}

YITU_HOST_API const char *yitu_sampler_last_error(const yitu_sampler *s) { return s ? s->err : ""; }
