// Row plan of a CSR: the long rows (>= 64 edges) cut into items of at most 64
// edges, listed in ascending order of the source id in the middle of each item.
//
// Kernels that gather one feature row per edge (SpMM, the per-edge dot, the GAT
// aggregate) process the items in this order, one wave per item: at any moment
// the waves read one narrow band of the feature table, whose hot rows stay in
// L2. On a power-law graph the same gathers in CSR order run at about half the
// speed. Short rows are not in the plan; a wave of the row kernels walks 4 of
// them in a row.
//
// Bands: the source ids are cut into bands of 2^17 consecutive ids (wider when
// that would give more than 64 bands) and a long row is cut where its (sorted)
// columns cross band boundaries, so that most items gather from one band and
// the items of a band, which the sort puts side by side, share their sources.
// A row of deg edges is cut into at most deg / 16 pieces, none shorter than 16
// edges: rows too short for one piece per band are cut at the boundaries of
// groups of 2, 4, ... bands. With items that straddle the whole id space, the
// band that the chip reads at one moment is polluted by the far ends of every
// item; with the cuts it is not. Measured on a 2^21-node R-MAT graph (fp32,
// F = 128, 3.08 ms per call without cuts): bands of 2^12 .. 2^19 ids give 2.78,
// 2.79, 2.78, 2.76, 2.69, 2.71 ms: a band is far wider than what an L2 holds
// (8 k rows of 512 bytes) at any of these widths, so narrow bands only add
// partial rows. A plan built without bands (the temporary plan of a call that
// was given none) makes no such cuts.
//
// The plan depends on the graph only. It is the counterpart of the reference's
// neighbour-group partition (build_part, ccsrc/kernel/YiTu_GNN.cpp:203-245):
// built once per graph, reused by every call; entry points also accept no plan
// and then build a temporary one in their workspace.
#pragma once
#include "common.hpp"

namespace yitu {

constexpr int kPlanChunk = 64;      // edges per item = one edge window of a wave
constexpr int kPlanThreshold = 64;  // rows with at least this many edges are planned
constexpr int kPlanBandShift = 17;  // log2 of the narrowest source band
constexpr int kPlanMaxBands = 64;   // bands get wider beyond 2^23 sources
constexpr int kPlanMinSegment = 16; // a row of deg edges is cut into at most deg / 16 pieces,
                                    // none shorter than this

struct PlanCounters {
    int n_items;
    int n_rows;
    int overflow;  // capacity exceeded while building: the plan is unusable, item kernels do nothing
    int pad;
};

// Device view handed to kernels by value.
struct PlanView {
    const PlanCounters *counters;
    const int4 *rows;     // {row, first item id, number of items, 0}; item ids of a row are consecutive
    const int4 *records;  // band order: {first edge, end edge, item id, row | (single-item row) << 31}
    int max_rows;
    int max_items;
    int threshold;  // rows with >= threshold edges are left to the item kernels
    const int *info;  // header words behind the counters (kPlanInfo*), or null
};

// Header words: {log2 of the band width, number of bands, local edges, sampled edges}.
// The builder samples edges of the short rows; an edge is local when its source lies
// near the row's own relative position in the id space. A graph three quarters of
// whose sampled edges are local (community structure with ids to match, as planted
// or as a reorder leaves them) has its short rows walked XCD by XCD. Measured on two
// graphs of 2^21 vertices and 62 M edges, fp32 rows of 128 floats: planted
// communities of 512 (97 % local) 4.43 ms round robin, 2.69 ms XCD by XCD (16 rows
// per wave; 2.07 ms with 4); an R-MAT graph after the Rabbit-Order reorder (51 %
// local: its rows of one or two edges sit next to their source, its hot sources are
// everybody's) 2.70 and 2.94 ms.
constexpr int kPlanInfoLocal = 2;
constexpr int kPlanInfoSampled = 3;

__device__ __forceinline__ bool plan_says_local(const PlanView &v) {
    return v.info && 4ll * v.info[kPlanInfoLocal] > 3ll * v.info[kPlanInfoSampled];
}

inline int64_t plan_max_rows(int64_t nnz) { return nnz / kPlanThreshold + 1; }
// A row of deg >= 64 edges gives at most deg / 64 + min(bands, deg / 16) items.
inline int64_t plan_max_items(int64_t nnz) {
    return nnz / kPlanChunk + nnz / kPlanMinSegment + plan_max_rows(nnz) + 1;
}

size_t plan_bytes(int64_t nnz);
size_t plan_build_workspace_bytes(int64_t nnz);
// Builds into `plan` (plan_bytes(nnz) of device memory, 256-byte aligned).
// with_bands = false cuts no row at band boundaries.
int plan_build(void *plan, size_t plan_size, const int32_t *indptr, const int32_t *indices,
               int64_t n_rows, int64_t n_src, int64_t nnz, int32_t col_mask, bool with_bands,
               void *workspace, size_t workspace_bytes, hipStream_t stream);
PlanView plan_view(const void *plan, int64_t nnz);
// A view that plans nothing (every row is handled by the row kernels).
inline PlanView plan_none() {
    PlanView v{};
    v.threshold = 0x7fffffff;
    return v;
}

// Resolves the plan of one call: the caller's, or a temporary one built at the
// start of `workspace`; `*rest` / `*rest_bytes` receive what is left of the
// workspace. With no long row possible (few edges, or a max-degree hint below
// the threshold) nothing is built.
int plan_resolve(PlanView &view, bool &has_items, const void *plan, const int32_t *indptr,
                 const int32_t *indices, int64_t n_rows, int64_t n_src, int64_t nnz,
                 int32_t col_mask, int64_t max_degree_hint, void *workspace,
                 size_t workspace_bytes, void **rest, size_t *rest_bytes, hipStream_t stream);
// Workspace a call needs on top of its own buffers when it is given no plan.
size_t plan_temp_bytes(int64_t nnz);

}  // namespace yitu
