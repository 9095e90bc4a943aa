/*
 * C ABI of libyitu_host.so: the host-side (CPU, OpenMP) graph preparation steps
 * of YiTu's sparse message-passing path. All pointers are host memory.
 * Return value: 0 on success, non-zero on rejected arguments.
 */
#ifndef YITU_HOST_H
#define YITU_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *yitu_host_last_error(void);

/*
 * Rabbit-Order relabelling: replaces YiTu_GNN.rabbit.reorder
 * (ccsrc/reorder/reorder.cpp:235-290, binding :293-295).
 * in_edge_index is int32 [2, n_edges] (sources then destinations); the number
 * of vertices is max id + 1 and is returned through n_vertices.
 *   out_edge_index [2, n_edges] (may be NULL): every edge with both ends renamed,
 *       same edge order -- what the reference returns;
 *   perm_out [perm_capacity] (may be NULL): new id of old vertex v -- the
 *       permutation itself, which the reference computes but does not expose.
 * Reproducible: the aggregation runs on one thread (the reference's result
 * depends on its thread count and on CAS timing, rabbit_order.hpp:509-516).
 */
int yitu_rabbit_reorder(int32_t *out_edge_index, int32_t *perm_out, int64_t perm_capacity,
                        int64_t *n_vertices, const int32_t *in_edge_index, int64_t n_edges);

/*
 * The same with the community aggregation on n_threads threads (<= 0: all the
 * OpenMP runtime offers; 1: the reproducible order above), by the reference's
 * protocol (rabbit_order.hpp:393-526, 554-621: lock by strength swap, merge by one
 * compare-and-swap, per-thread retry list). Like the reference's, the result then
 * depends on timing: a valid Rabbit-Order permutation, not the same one twice.
 */
int yitu_rabbit_reorder_threads(int32_t *out_edge_index, int32_t *perm_out,
                                int64_t perm_capacity, int64_t *n_vertices,
                                const int32_t *in_edge_index, int64_t n_edges, int n_threads);

/*
 * Temporal neighbour sampler: replaces sampler_core.ParallelSampler
 * (YiTu_GNN/YiTu_T/sampler_core.cpp:43-359, binding :374-402).
 * T-CSR inputs: indptr [n_nodes+1], indices / eid [n_edges] int32, ts [n_edges]
 * float32 ascending inside every node. num_neighbors [num_layers] is the fan-out
 * per layer. yitu_sampler_create is the most-recent mode (recent = True,
 * num_history = 1, window_duration = 0); yitu_sampler_create_modes takes the
 * reference constructor's remaining arguments: recent = 0 draws num_neighbors
 * edges uniformly from a root's window with the C library's rand_r, one generator
 * per chunk of ceil(n_roots / num_threads) roots seeded with the chunk's index, as
 * the reference's threads do (:238-253, 306-318), so the draws depend on the
 * NOMINAL num_threads only; num_history > 1 yields one block per snapshot and
 * layer, of windows window_duration wide (:216-226, 271-279), in the reference's
 * block order. A layer after the first that uses cursors (recent or prop_time)
 * advances them from the nodes of the previous layer's block (the reference reads
 * an uninitialised pointer there, sampler_core.cpp:204-213).
 */
typedef struct yitu_sampler yitu_sampler;
yitu_sampler *yitu_sampler_create(const int32_t *indptr, const int32_t *indices, const int32_t *eid,
                                  const float *ts, int64_t n_nodes, int64_t n_edges,
                                  int num_threads, int num_layers, const int32_t *num_neighbors,
                                  int prop_time);
yitu_sampler *yitu_sampler_create_modes(const int32_t *indptr, const int32_t *indices,
                                        const int32_t *eid, const float *ts, int64_t n_nodes,
                                        int64_t n_edges, int num_threads, int num_layers,
                                        const int32_t *num_neighbors, int recent, int prop_time,
                                        int num_history, float window_duration);
void yitu_sampler_destroy(yitu_sampler *s);
int yitu_sampler_reset(yitu_sampler *s);
int yitu_sampler_sample(yitu_sampler *s, const int32_t *root_nodes, const float *root_ts,
                        int64_t n_roots);
int64_t yitu_sampler_num_blocks(const yitu_sampler *s);
int yitu_sampler_block_sizes(const yitu_sampler *s, int block, int64_t *n_edges, int64_t *dim_in,
                             int64_t *dim_out);
/* row, col, eid: [n_edges]; ts, dts, nodes: [dim_in]. Any pointer may be NULL. */
int yitu_sampler_block_copy(const yitu_sampler *s, int block, int32_t *row, int32_t *col,
                            int32_t *eid, float *ts, float *dts, int32_t *nodes);
const char *yitu_sampler_last_error(const yitu_sampler *s);

#ifdef __cplusplus
}
#endif
#endif /* YITU_HOST_H */
