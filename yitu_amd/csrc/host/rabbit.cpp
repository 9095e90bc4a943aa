// Rabbit-Order vertex relabelling (community-based, locality-improving) on the
// host: the graph preparation step behind YiTu_GNN.rabbit.reorder
// (ccsrc/reorder/reorder.cpp:235-290, algorithm in ccsrc/reorder/rabbit_order.hpp).
//
// Pipeline:
//   1. symmetrise the edge list, drop self loops, merge duplicates with summed
//      unit weights (reorder.cpp:31-97)                       [parallel, counting sort]
//   2. visit vertices in ascending degree; each visited vertex gathers the edges
//      of its community, re-targets them to community roots, and merges into the
//      neighbour with the best modularity gain w_vu - str_v str_u / W, if any is
//      positive (rabbit_order.hpp:393-526, 554-621)            [sequential]
//   3. number the vertices by a depth-first walk of each top-level community's
//      merge dendrogram; communities are laid out in the order in which they
//      became top-level (rabbit_order.hpp:623-673)
//
// Step 2 exists twice. On one thread it is a function of the graph alone (the
// reproducible order, the default). With several threads it follows the
// reference's protocol (rabbit_order.hpp:393-526, 554-621): threads take the
// degree-sorted vertices in turn; a vertex is locked by swapping its strength for
// -1, merged into its best neighbour with one compare-and-swap on that
// neighbour's (strength, last child) word, and put on the thread's retry list
// when the neighbour is locked or the swap loses a race. Which vertex wins such
// a race depends on timing, so the permutation differs from run to run, as the
// reference's does; every outcome is a valid merge dendrogram. Edge weights are
// counts held in float (exact below 2^24), so the order in which duplicates are
// summed does not change any comparison.
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <new>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <utility>
#include <vector>

#include <omp.h>

#include "../../../include/yitu_host.h"

namespace {

using vint = uint32_t;
constexpr vint kNone = 0xffffffffu;

struct Edge {
    vint to;
    float w;
};

thread_local char g_err[256] = "";

// Symmetric weighted adjacency in CSR form: row v = distinct neighbours of v
// (ascending id) with the number of input edges between them in either direction.
// Storage that is not cleared when it is made: the arrays of the adjacency are written in
// full by the threads that fill them, and clearing 400 MB from one thread first (which is
// what a vector does) took longer than everything else in the build.
template <typename T>
struct RawArray {
    T *p = nullptr;
    explicit RawArray(size_t n) : p(static_cast<T *>(std::malloc(std::max<size_t>(n, 1) * sizeof(T)))) {
        if (!p) throw std::bad_alloc();
    }
    RawArray() = default;
    RawArray(RawArray &&o) noexcept : p(o.p) { o.p = nullptr; }
    RawArray &operator=(RawArray &&o) noexcept {
        std::swap(p, o.p);
        return *this;
    }
    RawArray(const RawArray &) = delete;
    RawArray &operator=(const RawArray &) = delete;
    ~RawArray() { std::free(p); }
    T *data() const { return p; }
    T &operator[](size_t i) const { return p[i]; }
};

struct Adjacency {
    std::vector<int64_t> ptr;
    RawArray<Edge> edges;
};

Adjacency build_adjacency(const int32_t *src, const int32_t *dst, int64_t m, vint n) {
    // counting sort by end point. Every thread reads the whole edge list and keeps the end
    // points that fall into its own range of vertices: no counter is shared, where atomic
    // adds from all threads met on the few vertices that hold most edges of a power-law
    // graph (and took most of the reorder's time). The rows are sorted afterwards, so the
    // order of arrival does not matter.
    std::vector<int64_t> count(n + 1, 0);
    const int n_threads = omp_get_max_threads();
#pragma omp parallel num_threads(n_threads)
    {
        const int tid = omp_get_thread_num(), nt = omp_get_num_threads();
        const vint lo = (vint)((uint64_t)n * tid / nt), hi = (vint)((uint64_t)n * (tid + 1) / nt);
        for (int64_t i = 0; i < m; i++) {
            const vint s = (vint)src[i], d = (vint)dst[i];
            if (s == d) continue;
            if (s >= lo && s < hi) count[s + 1]++;
            if (d >= lo && d < hi) count[d + 1]++;
        }
    }
    for (vint v = 0; v < n; v++) count[v + 1] += count[v];
    RawArray<vint> raw((size_t)count[n]);
    {
        std::vector<int64_t> fill(count.begin(), count.end() - 1);
        // ranges of about equal numbers of end points this time (the low ids of a
        // power-law graph hold far more than their share)
        std::vector<vint> cut(n_threads + 1, n);
        cut[0] = 0;
        for (int t = 1; t < n_threads; t++) {
            const int64_t want = count[n] / n_threads * t;
            cut[t] = (vint)(std::lower_bound(count.begin(), count.end(), want) - count.begin());
            if (cut[t] > n) cut[t] = n;
        }
#pragma omp parallel num_threads(n_threads)
        {
            const int tid = omp_get_thread_num(), nt = omp_get_num_threads();
            // (fewer threads than asked for: the last one takes the rest)
            const vint lo = cut[tid], hi = tid + 1 == nt ? n : cut[tid + 1];
            for (int64_t i = 0; i < m; i++) {
                const vint s = (vint)src[i], d = (vint)dst[i];
                if (s == d) continue;
                if (s >= lo && s < hi) raw[(size_t)fill[s]++] = d;
                if (d >= lo && d < hi) raw[(size_t)fill[d]++] = s;
            }
        }
    }
    // sort each row, count distinct targets
    std::vector<int64_t> uniq(n + 1, 0);
#pragma omp parallel for schedule(dynamic, 1024)
    for (int64_t v = 0; v < (int64_t)n; v++) {
        vint *b = raw.data() + count[v], *e = raw.data() + count[v + 1];
        std::sort(b, e);
        int64_t u = 0;
        for (vint *p = b; p != e; ++p) u += (p == b || p[0] != p[-1]);
        uniq[v + 1] = u;
    }
    for (vint v = 0; v < n; v++) uniq[v + 1] += uniq[v];
    Adjacency adj;
    adj.edges = RawArray<Edge>((size_t)uniq[n]);
#pragma omp parallel for schedule(dynamic, 1024)
    for (int64_t v = 0; v < (int64_t)n; v++) {
        const vint *b = raw.data() + count[v], *e = raw.data() + count[v + 1];
        Edge *out = adj.edges.data() + uniq[v];
        for (const vint *p = b; p != e;) {
            const vint t = *p;
            float w = 0.0f;
            while (p != e && *p == t) {
                w += 1.0f;
                ++p;
            }
            *out++ = Edge{t, w};
        }
    }
    adj.ptr = std::move(uniq);
    return adj;
}

struct Dendrogram {
    vint n = 0;
    std::vector<vint> com;      // community pointer (root: com[v] == v)
    std::vector<vint> child;    // last vertex merged into v
    std::vector<vint> sibling;  // previous vertex merged into the same parent
    std::vector<float> str;     // community strength; -1 once v has been merged away
    std::vector<vint> tops;     // top-level vertices in the order they were fixed
    std::vector<std::vector<Edge>> es;  // current (aggregated) edge list of each vertex
    double total = 0.0;
};

inline vint find_root(Dendrogram &g, vint v) {
    vint c = v;
    while (g.com[c] != c) c = g.com[c];
    if (v != c && g.com[v] != c) g.com[v] = c;  // one-step shortcut for the next lookup
    return c;
}

// sort by target and add up the weights of equal targets, in place
inline size_t combine(Edge *b, Edge *e) {
    if (b == e) return 0;
    std::sort(b, e, [](const Edge &x, const Edge &y) { return x.to < y.to; });
    Edge *o = b;
    for (Edge *p = b + 1; p != e; ++p) {
        if (p->to == o->to)
            o->w += p->w;
        else
            *++o = *p;
    }
    return (size_t)(o - b) + 1;
}

// Edges of v's whole community, re-targeted to current roots, self loops removed,
// duplicates merged: becomes v's own edge list.
void gather_community_edges(Dendrogram &g, vint v, std::vector<Edge> &buf,
                            std::vector<vint> &united_child) {
    buf.clear();
    size_t combined = 0;
    auto push = [&](vint u) {
        for (const Edge &e : g.es[u]) {
            const vint c = find_root(g, e.to);
            if (c != v) buf.push_back(Edge{c, e.w});
        }
        if (buf.size() - combined >= 2048) {  // keep the working set small
            combined += combine(buf.data() + combined, buf.data() + buf.size());
            buf.resize(combined);
        }
    };
    push(v);
    while (united_child[v] != g.child[v]) {
        const vint c = g.child[v];
        for (vint w = c; w != kNone && w != united_child[v]; w = g.sibling[w]) push(w);
        united_child[v] = c;
    }
    buf.resize(combine(buf.data(), buf.data() + buf.size()));
    g.es[v].assign(buf.begin(), buf.end());
}

Dendrogram aggregate(const Adjacency &adj, vint n) {
    Dendrogram g;
    g.n = n;
    g.com.resize(n);
    g.child.assign(n, kNone);
    g.sibling.assign(n, kNone);
    g.str.resize(n);
    g.es.resize(n);
    std::iota(g.com.begin(), g.com.end(), 0u);
    double total = 0.0;
#pragma omp parallel for reduction(+ : total) schedule(static)
    for (int64_t v = 0; v < (int64_t)n; v++) {
        const Edge *b = adj.edges.data() + adj.ptr[v], *e = adj.edges.data() + adj.ptr[v + 1];
        float s = 0.0f;
        for (const Edge *p = b; p != e; ++p) s += p->w;
        g.es[v].assign(b, e);
        g.str[v] = s;
        total += s;
    }
    g.total = total;

    // ascending (unweighted) degree; ties fall where std::sort leaves them, the
    // comparator looks at the degree only (rabbit_order.hpp:531-541)
    std::vector<std::pair<vint, vint>> order(n);
    for (vint v = 0; v < n; v++) order[v] = {v, (vint)g.es[v].size()};
    std::sort(order.begin(), order.end(),
              [](const std::pair<vint, vint> &x, const std::pair<vint, vint> &y) {
                  return x.second < y.second;
              });

    std::vector<Edge> buf;
    buf.reserve((size_t)std::min<int64_t>((int64_t)n * 2, (int64_t)1 << 24));
    std::vector<vint> united_child(n, kNone);
    for (vint i = 0; i < n; i++) {
        const vint v = order[i].first;
        gather_community_edges(g, v, buf, united_child);
        const float vstr = g.str[v];
        // neighbour with the largest positive modularity gain; first one wins ties
        double best_gain = 0.0;
        vint best = v;
        for (const Edge &e : g.es[v]) {
            const double d = (double)e.w - (double)vstr * (double)g.str[e.to] / g.total;
            if (best_gain < d) {
                best_gain = d;
                best = e.to;
            }
        }
        if (best == v) {
            g.tops.push_back(v);
        } else {
            g.str[best] += vstr;
            g.sibling[v] = g.child[best];
            g.child[best] = v;
            g.com[v] = best;
            g.str[v] = -1.0f;
        }
    }
    return g;
}

// ---- parallel aggregation ---------------------------------------------------------
// (strength, last merged child) of a vertex in one 64-bit word, so that a merge is
// one compare-and-swap; strength < 0 = locked by the thread that is merging it away
// (or merged for good).
struct Atom {
    float str;
    vint child;
};
inline uint64_t pack(Atom a) {
    uint32_t s;
    std::memcpy(&s, &a.str, 4);
    return (uint64_t)a.child << 32 | s;
}
inline Atom unpack(uint64_t x) {
    Atom a;
    const uint32_t s = (uint32_t)x;
    std::memcpy(&a.str, &s, 4);
    a.child = (vint)(x >> 32);
    return a;
}

struct SharedGraph {
    vint n = 0;
    std::vector<std::atomic<uint64_t>> atom;
    std::vector<vint> com;           // read and shortened by every thread (relaxed)
    std::vector<vint> sibling;
    std::vector<vint> united_child;  // touched only by the thread that merges the vertex
    std::vector<std::vector<Edge>> es;
    double total = 0.0;
    explicit SharedGraph(vint n_) : n(n_), atom(n_), com(n_), sibling(n_, kNone),
                                    united_child(n_, kNone), es(n_) {}
};

inline vint load_com(const SharedGraph &g, vint v) {
    return __atomic_load_n(&g.com[v], __ATOMIC_RELAXED);
}

inline vint shared_root(SharedGraph &g, vint v) {
    vint c = v;
    for (vint next = load_com(g, c); next != c; next = load_com(g, c)) c = next;
    if (v != c && load_com(g, v) != c) __atomic_store_n(&g.com[v], c, __ATOMIC_RELAXED);
    return c;
}

// like gather_community_edges, on the shared structure; other threads may append
// children to v meanwhile, the caller checks for that after locking v
void unite_shared(SharedGraph &g, vint v, std::vector<Edge> &buf) {
    buf.clear();
    size_t combined = 0;
    auto push = [&](vint u) {
        for (const Edge &e : g.es[u]) {
            const vint c = shared_root(g, e.to);
            if (c != v) buf.push_back(Edge{c, e.w});
        }
        if (buf.size() - combined >= 2048) {
            combined += combine(buf.data() + combined, buf.data() + buf.size());
            buf.resize(combined);
        }
    };
    push(v);
    for (vint c = unpack(g.atom[v].load()).child; g.united_child[v] != c;
         c = unpack(g.atom[v].load()).child) {
        // the vertices on the sibling list are merged for good: nobody modifies them
        for (vint w = c; w != kNone && w != g.united_child[v]; w = g.sibling[w]) push(w);
        g.united_child[v] = c;
    }
    buf.resize(combine(buf.data(), buf.data() + buf.size()));
    g.es[v].assign(buf.begin(), buf.end());
}

// v itself: top-level for good; kNone: lost a race, try again later; else: merged into it
vint merge_shared(SharedGraph &g, vint v, std::vector<Edge> &buf) {
    unite_shared(g, v, buf);
    // lock v: strength -> -1, child kept
    uint64_t cur = g.atom[v].load();
    while (!g.atom[v].compare_exchange_weak(cur, pack(Atom{-1.0f, unpack(cur).child}))) {
    }
    const float vstr = unpack(cur).str;
    if (unpack(g.atom[v].load()).child != g.united_child[v]) unite_shared(g, v, buf);
    auto unlock = [&] {
        uint64_t x = g.atom[v].load();
        while (!g.atom[v].compare_exchange_weak(x, pack(Atom{vstr, unpack(x).child}))) {
        }
    };
    double best_gain = 0.0;
    vint best = v;
    for (const Edge &e : g.es[v]) {
        const double d =
            (double)e.w - (double)vstr * (double)unpack(g.atom[e.to].load()).str / g.total;
        if (best_gain < d) {
            best_gain = d;
            best = e.to;
        }
    }
    if (best == v) {
        unlock();
        return v;
    }
    uint64_t target = g.atom[best].load();
    const Atom ta = unpack(target);
    if (ta.str < 0.0f) {  // the neighbour is being merged itself
        unlock();
        return kNone;
    }
    g.sibling[v] = ta.child;  // visible to whoever sees v as best's child
    if (!g.atom[best].compare_exchange_strong(target, pack(Atom{ta.str + vstr, v}))) {
        g.sibling[v] = kNone;
        unlock();
        return kNone;
    }
    __atomic_store_n(&g.com[v], best, __ATOMIC_RELAXED);
    return best;
}

Dendrogram aggregate_parallel(const Adjacency &adj, vint n, int n_threads) {
    SharedGraph g(n);
    double total = 0.0;
#pragma omp parallel for reduction(+ : total) schedule(static) num_threads(n_threads)
    for (int64_t v = 0; v < (int64_t)n; v++) {
        const Edge *b = adj.edges.data() + adj.ptr[v], *e = adj.edges.data() + adj.ptr[v + 1];
        float s = 0.0f;
        for (const Edge *p = b; p != e; ++p) s += p->w;
        g.es[v].assign(b, e);
        g.com[v] = (vint)v;
        g.atom[v].store(pack(Atom{s, kNone}));
        total += s;
    }
    g.total = total;
    std::vector<std::pair<vint, vint>> order(n);
    for (vint v = 0; v < n; v++) order[v] = {v, (vint)g.es[v].size()};
    std::stable_sort(order.begin(), order.end(),
                     [](const std::pair<vint, vint> &x, const std::pair<vint, vint> &y) {
                         return x.second < y.second;
                     });
    std::vector<std::vector<vint>> tops_of(n_threads);
#pragma omp parallel num_threads(n_threads)
    {
        const int tid = omp_get_thread_num();
        std::vector<vint> tops, pending, still;
        std::vector<Edge> buf;
        buf.reserve(1 << 16);
        auto attempt = [&](vint v) {
            const vint u = merge_shared(g, v, buf);
            if (u == v) tops.push_back(v);
            return u != kNone;
        };
#pragma omp for schedule(static, 1)
        for (int64_t i = 0; i < (int64_t)n; i++) {
            if (!pending.empty()) {
                still.clear();
                for (const vint w : pending)
                    if (!attempt(w)) still.push_back(w);
                pending.swap(still);
            }
            const vint v = order[(size_t)i].first;
            if (!attempt(v)) pending.push_back(v);
        }
        // (implicit barrier) what is still pending is merged one thread at a time:
        // nothing is locked any more, so every attempt succeeds
#pragma omp critical
        {
            for (const vint w : pending)
                while (!attempt(w)) {
                }
            tops_of[tid] = std::move(tops);
        }
    }
    Dendrogram d;
    d.n = n;
    d.child.resize(n);
    d.sibling = std::move(g.sibling);
    for (vint v = 0; v < n; v++) d.child[v] = unpack(g.atom[v].load()).child;
    for (auto &t : tops_of) d.tops.insert(d.tops.end(), t.begin(), t.end());
    d.total = total;
    return d;
}

// new id of every vertex: depth-first over each top-level community's merge tree
std::vector<vint> permutation(const Dendrogram &g) {
    std::vector<vint> perm(g.n, kNone);
    std::vector<vint> stack;
    vint next = 0;
    auto push_chain = [&](vint v) {  // v, its last child, that one's last child, ...
        for (; v != kNone; v = g.child[v]) stack.push_back(v);
    };
    for (const vint top : g.tops) {
        push_chain(top);
        while (!stack.empty()) {
            const vint v = stack.back();
            stack.pop_back();
            perm[v] = next++;
            if (g.sibling[v] != kNone) push_chain(g.sibling[v]);
        }
    }
    return perm;
}

}  // namespace

extern "C" __attribute__((visibility("default"))) const char *yitu_host_last_error(void) {
    return g_err;
}

extern "C" __attribute__((visibility("default"))) int yitu_rabbit_reorder_threads(
    int32_t *out_edge_index, int32_t *perm_out, int64_t perm_capacity, int64_t *n_vertices,
    const int32_t *in_edge_index, int64_t n_edges, int n_threads) {
    if (n_edges < 0 || (n_edges > 0 && !in_edge_index)) {
        snprintf(g_err, sizeof(g_err), "bad edge list");
        return -1;
    }
    const int32_t *src = in_edge_index, *dst = in_edge_index + n_edges;
    int64_t n64 = 0;
    for (int64_t i = 0; i < n_edges; i++) {
        if (src[i] < 0 || dst[i] < 0) {
            snprintf(g_err, sizeof(g_err), "negative vertex id at edge %lld", (long long)i);
            return -1;
        }
        n64 = std::max<int64_t>(n64, (int64_t)std::max(src[i], dst[i]) + 1);
    }
    if (n_vertices) *n_vertices = n64;
    const vint n = (vint)n64;
    if (perm_out && perm_capacity < n64) {
        snprintf(g_err, sizeof(g_err), "perm buffer holds %lld ids, graph has %lld vertices",
                 (long long)perm_capacity, (long long)n64);
        return -1;
    }
    if (n == 0) return 0;
    const Adjacency adj = build_adjacency(src, dst, n_edges, n);
    if (n_threads <= 0) n_threads = omp_get_max_threads();
    const Dendrogram g = n_threads == 1 ? aggregate(adj, n) : aggregate_parallel(adj, n, n_threads);
    const std::vector<vint> perm = permutation(g);
    for (vint v = 0; v < n; v++) {
        if (perm[v] == kNone) {
            snprintf(g_err, sizeof(g_err), "internal error: vertex %u not numbered", v);
            return -2;
        }
    }
    if (perm_out)
        for (vint v = 0; v < n; v++) perm_out[v] = (int32_t)perm[v];
    if (out_edge_index) {
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n_edges; i++) {
            out_edge_index[i] = (int32_t)perm[(vint)src[i]];
            out_edge_index[n_edges + i] = (int32_t)perm[(vint)dst[i]];
        }
    }
    return 0;
}

extern "C" __attribute__((visibility("default"))) int yitu_rabbit_reorder(
    int32_t *out_edge_index, int32_t *perm_out, int64_t perm_capacity, int64_t *n_vertices,
    const int32_t *in_edge_index, int64_t n_edges) {
    return yitu_rabbit_reorder_threads(out_edge_index, perm_out, perm_capacity, n_vertices,
                                       in_edge_index, n_edges, 1);
}
