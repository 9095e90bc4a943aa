// Temporal neighbour sampler over a T-CSR (per-node edge lists sorted by timestamp):
// YiTu_GNN/YiTu_T/sampler_core.cpp (ParallelSampler, :43-359) in all its modes.
//
// Most-recent mode (recent = true). Per root (n, t) the sampler keeps a monotone
// cursor into n's edge list that is advanced to the last edge with ts <= t - 1e-7
// (update_ts_ptr, :103-127), then emits the edges k = cursor, cursor-1, ... while
// k > max(first edge of n, cursor - k_neigh) and ts[k] < t - 1e-7 (:295-305): at most
// k_neigh edges, the node's first edge is never emitted, and roots that repeat a
// node share the cursor (so the one with the smaller t may get fewer edges).
//
// Uniform mode (recent = false). The same window [s, e] of a root; when it holds at
// least k_neigh edges, k_neigh draws picked = s + rand_r(&seed) % (e - s + 1) are made
// and the ones older than the root kept (:306-318), duplicates included. The
// reference's threads each own a seed that starts at the thread id and a static chunk
// of ceil(n_roots / threads) consecutive roots (:238-253), so the draws are a function
// of the NOMINAL thread count; they are reproduced here by giving every such chunk its
// own generator, whatever number of threads really runs. rand_r is the C library's
// (glibc stdlib/rand_r.c: three steps of x -> 1103515245 x + 12345, of which 11 + 10 +
// 10 bits are taken).
//
// Layers after the first do not use cursors unless recent or prop_time ask for them
// (:344-356): the window end is found by binary search (:262-268), and the roots of
// layer l are the nodes of layer l-1's block. With num_history > 1 a layer yields one
// block per snapshot i, whose window is [t - (i+1) w, t - i w] (cursors :224-226, or the
// two searches :271-279); blocks are stored as the reference stores them, snapshot i of
// a layer at position (blocks so far) - 1 - i.
//
// Output of one (layer, snapshot) is the COO block of combine_coo (:153-199): row = root
// slot, col = n_roots + running index, nodes = [roots..., neighbours...], in root order,
// which is what the reference's per-thread pieces give when concatenated by thread id.
// Cursor updates of a batch are order independent (running maxima) and run first.
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
    // ts_ptr[k] per node, k = 0 .. num_history: cursor k marks the last edge with
    // ts <= (latest query time - (num_history - k) * window - 1e-7); [0] never moves
    // without a window. All start at the node's first edge.
    std::vector<std::vector<int32_t>> ts_ptr;
    std::vector<int32_t> fanout;
    int num_layers = 1;
    int num_threads = 1;  // the NOMINAL thread count: chunking of the roots, generator seeds
    bool prop_time = false;
    bool recent = true;
    int num_history = 1;
    float window = 0.0f;
    std::vector<Block> blocks;
    char err[256] = "";
};

namespace {

// rand_r of the C library the reference is linked against (glibc stdlib/rand_r.c)
inline int c_rand_r(unsigned int *seed) {
    unsigned int next = *seed;
    next = next * 1103515245u + 12345u;
    int result = (int)((next / 65536u) % 2048u);
    next = next * 1103515245u + 12345u;
    result <<= 10;
    result ^= (int)((next / 65536u) % 1024u);
    next = next * 1103515245u + 12345u;
    result <<= 10;
    result ^= (int)((next / 65536u) % 1024u);
    *seed = next;
    return result;
}

// update_ts_ptr (sampler_core.cpp:103-127): cursor `slc` of every root's node moves to the
// last edge with ts <= t + offset - 1e-7; never backwards.
void advance_cursors(yitu_sampler *s, int slc, const int32_t *roots, const float *root_ts,
                     int64_t n_roots, float offset) {
    std::vector<int32_t> &cur = s->ts_ptr[(size_t)slc];
    for (int64_t i = 0; i < n_roots; i++) {
        const int32_t n = roots[i];
        const float thr = root_ts[i] + offset - 1e-7f;
        const int32_t end = s->indptr[n + 1];
        const int32_t c0 = cur[n];
        for (int32_t j = c0; j < end; j++) {
            if (s->ts[j] > thr) {
                if (j != c0) cur[n] = j - 1;
                break;
            }
            if (j == end - 1) cur[n] = j;
        }
    }
}

struct Piece {  // what one chunk of roots emits
    std::vector<int32_t> row, eid, nodes;
    std::vector<float> ts, dts;
};

// One snapshot of one layer (the body of the loop at sampler_core.cpp:216-333).
void sample_snapshot(yitu_sampler *s, const int32_t *roots, const float *root_ts, int64_t n_roots,
                     int fan, bool use_ptr, int snapshot, Block &out) {
    const float offset = -(float)snapshot * s->window;
    const int H = s->num_history;
    const int T = s->num_threads;
    const int64_t chunk = n_roots > 0 ? (int64_t)std::ceil((float)n_roots / (float)T) : 1;
    const int64_t n_chunks = n_roots > 0 ? (n_roots + chunk - 1) / chunk : 0;
    std::vector<Piece> pieces((size_t)n_chunks);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t c = 0; c < n_chunks; c++) {
        Piece &p = pieces[(size_t)c];
        unsigned int seed = (unsigned int)c;  // chunk c is thread c's (schedule(static, chunk))
        const int64_t hi = std::min(n_roots, (c + 1) * chunk);
        for (int64_t j = c * chunk; j < hi; j++) {
            const int32_t n = roots[j];
            const float t = root_ts[j];
            int32_t lo_e, hi_e;
            const float *tb = s->ts.data() + s->indptr[n], *te = s->ts.data() + s->indptr[n + 1];
            if (use_ptr) {
                lo_e = s->ts_ptr[(size_t)(H - 1 - snapshot)][n];
                hi_e = s->ts_ptr[(size_t)(H - snapshot)][n];
            } else if (H == 1) {
                lo_e = s->indptr[n];
                hi_e = std::max((int32_t)(std::upper_bound(tb, te, t) - s->ts.data()) - 1, lo_e);
            } else {
                lo_e = std::max((int32_t)(std::upper_bound(tb, te, t + offset - s->window) -
                                          s->ts.data()) - 1, s->indptr[n]);
                hi_e = std::max((int32_t)(std::upper_bound(tb, te, t + offset) - s->ts.data()) - 1,
                                lo_e);
            }
            const float thr = t + offset - 1e-7f;
            auto emit = [&](int32_t k) {
                p.row.push_back((int32_t)j);
                p.eid.push_back(s->eid[k]);
                p.ts.push_back(s->prop_time ? t : s->ts[k]);
                p.dts.push_back(t - s->ts[k]);
                p.nodes.push_back(s->indices[k]);
            };
            if (s->recent || hi_e - lo_e < fan) {
                for (int32_t k = hi_e; k > std::max(lo_e, hi_e - fan); k--)
                    if (s->ts[k] < thr) emit(k);
            } else {
                for (int i = 0; i < fan; i++) {
                    const int32_t k = lo_e + c_rand_r(&seed) % (hi_e - lo_e + 1);
                    if (s->ts[k] < thr) emit(k);
                }
            }
        }
    }
    std::vector<int64_t> offs((size_t)n_chunks + 1, 0);
    for (int64_t c = 0; c < n_chunks; c++)
        offs[(size_t)c + 1] = offs[(size_t)c] + (int64_t)pieces[(size_t)c].row.size();
    const int64_t m = offs[(size_t)n_chunks];
    out.row.resize((size_t)m);
    out.col.resize((size_t)m);
    out.eid.resize((size_t)m);
    out.ts.resize((size_t)(m + n_roots));
    out.dts.assign((size_t)(m + n_roots), 0.0f);
    out.nodes.resize((size_t)(m + n_roots));
    std::copy(roots, roots + n_roots, out.nodes.begin());
    std::copy(root_ts, root_ts + n_roots, out.ts.begin());
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t c = 0; c < n_chunks; c++) {
        const Piece &p = pieces[(size_t)c];
        const int64_t w = offs[(size_t)c];
        for (size_t i = 0; i < p.row.size(); i++) {
            out.row[(size_t)w + i] = p.row[i];
            out.col[(size_t)w + i] = (int32_t)(n_roots + w + (int64_t)i);
            out.eid[(size_t)w + i] = p.eid[i];
            out.ts[(size_t)(n_roots + w) + i] = p.ts[i];
            out.dts[(size_t)(n_roots + w) + i] = p.dts[i];
            out.nodes[(size_t)(n_roots + w) + i] = p.nodes[i];
        }
    }
    out.dim_in = m + n_roots;
    out.dim_out = n_roots;
}

}  // namespace

#define YITU_HOST_API extern "C" __attribute__((visibility("default")))

YITU_HOST_API yitu_sampler *yitu_sampler_create_modes(
    const int32_t *indptr, const int32_t *indices, const int32_t *eid, const float *ts,
    int64_t n_nodes, int64_t n_edges, int num_threads, int num_layers, const int32_t *num_neighbors,
    int recent, int prop_time, int num_history, float window_duration) {
    if (!indptr || n_nodes < 0 || n_edges < 0 || num_layers < 1 || !num_neighbors) return nullptr;
    if (num_history < 1) return nullptr;
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
    s->recent = recent != 0;
    s->num_history = num_history;
    s->window = window_duration;
    s->ts_ptr.assign((size_t)num_history + 1, std::vector<int32_t>(indptr, indptr + n_nodes));
    return s;
}

YITU_HOST_API yitu_sampler *yitu_sampler_create(const int32_t *indptr, const int32_t *indices,
                                                const int32_t *eid, const float *ts,
                                                int64_t n_nodes, int64_t n_edges, int num_threads,
                                                int num_layers, const int32_t *num_neighbors,
                                                int prop_time) {
    return yitu_sampler_create_modes(indptr, indices, eid, ts, n_nodes, n_edges, num_threads,
                                     num_layers, num_neighbors, 1, prop_time, 1, 0.0f);
}

YITU_HOST_API void yitu_sampler_destroy(yitu_sampler *s) { delete s; }

YITU_HOST_API int yitu_sampler_reset(yitu_sampler *s) {
    if (!s) return -1;
    for (auto &cur : s->ts_ptr) std::copy(s->indptr.begin(), s->indptr.end() - 1, cur.begin());
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
    // sample() of the reference (sampler_core.cpp:337-359)
    const int H = s->num_history;
    s->blocks.clear();
    bool first_layer = true;
    for (int l = 0; l < s->num_layers; l++) {
        s->blocks.resize(s->blocks.size() + (size_t)H);
        bool use_ptr = false;
        if (first_layer || (s->prop_time && H == 1) || s->recent) {
            first_layer = false;
            use_ptr = true;
        }
        const int fan = s->fanout[(size_t)l];
        const bool from_root = l == 0;
        const size_t n_blocks = s->blocks.size();
        if (use_ptr) {
            // The reference advances cursor H from the layer's roots; for layers after the
            // first it reads them through a pointer it never set (:204-213). Here they are
            // the nodes of the previous layer's first snapshot.
            const Block *prev = from_root ? nullptr : &s->blocks[n_blocks - 1 - (size_t)H];
            advance_cursors(s, H, from_root ? root_nodes : prev->nodes.data(),
                            from_root ? root_ts : prev->ts.data(),
                            from_root ? n_roots : (int64_t)prev->nodes.size(), 0.0f);
        }
        for (int i = 0; i < H; i++) {
            const Block *prev = from_root ? nullptr : &s->blocks[n_blocks - 1 - (size_t)i - (size_t)H];
            const int32_t *nodes = from_root ? root_nodes : prev->nodes.data();
            const float *ts = from_root ? root_ts : prev->ts.data();
            const int64_t n = from_root ? n_roots : (int64_t)prev->nodes.size();
            const float offset = -(float)i * s->window;
            if (use_ptr && std::fabs(s->window) > 1e-7f)
                advance_cursors(s, H - 1 - i, nodes, ts, n, offset - s->window);
            sample_snapshot(s, nodes, ts, n, fan, use_ptr, i, s->blocks[n_blocks - 1 - (size_t)i]);
        }
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
