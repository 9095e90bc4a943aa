// Row plan of a CSR: the long rows (>= 64 edges) cut into items of at most 64
// edges, listed in ascending order of the source id in the middle of each item.
//
// Kernels that gather one feature row per edge (SpMM, the per-edge dot, the GAT
// aggregate) process the items in this order, one wave per item: at any moment
// the waves read one narrow band of the feature table, whose hot rows stay in
// L2. On a power-law graph the same gathers in CSR order run at about half the
// speed. Short rows are not in the plan; a wave of the row kernels walks 16 of
// them in a row.
//
// Slabs: the source ids are cut into 4 contiguous ranges and a long row is cut
// where its (sorted) columns cross a range boundary (at most deg / 16 pieces,
// none shorter than 16 edges), so most items gather from one range only. With
// items that straddle the whole id space, the band that the chip reads at one
// moment is polluted by the far ends of every item; with the cuts it is not
// (measured on a 2^21-node R-MAT graph: 3 to 7 % less time for the fp32 SpMM;
// 8 and 16 ranges cut the rows into smaller items and cost the bf16 path more
// than they gain).
// Boundaries are placed so that the ranges have equal sums of popularity^0.75
// over their sources: a hot source is fetched into L2 once and then hit, so its
// cost grows more slowly than its edge count, and equal-cost ranges keep the
// pieces of a row from being either tiny or huge. A plan built without slabs
// (the temporary plan of a call that was given none) makes no such cuts.
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
constexpr int kPlanSlabs = 4;       // source ranges at whose boundaries long rows are cut
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
};

inline int64_t plan_max_rows(int64_t nnz) { return nnz / kPlanThreshold + 1; }
// A row of deg >= 64 edges gives at most deg / 64 + min(4, deg / 16) items.
inline int64_t plan_max_items(int64_t nnz) {
    return nnz / kPlanChunk + nnz / kPlanMinSegment + plan_max_rows(nnz) + 1;
}

size_t plan_bytes(int64_t nnz);
size_t plan_build_workspace_bytes(int64_t nnz);
// Builds into `plan` (plan_bytes(nnz) of device memory, 256-byte aligned).
// with_slabs = false skips the popularity pass and puts every item in slab 0.
int plan_build(void *plan, size_t plan_size, const int32_t *indptr, const int32_t *indices,
               int64_t n_rows, int64_t n_src, int64_t nnz, int32_t col_mask, bool with_slabs,
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
