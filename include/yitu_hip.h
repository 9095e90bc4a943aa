/*
 * C ABI of libyitu_hip.so: hand-written gfx950 (MI355X) kernels for YiTu's
 * sparse message-passing path. Plain pointers and sizes only; every pointer
 * named "device" below is HIP device memory on the current device, `stream` is
 * a hipStream_t passed as void* (NULL = the default stream) and launches are
 * asynchronous on it. Nothing here allocates device memory: kernels that need
 * scratch take a caller-provided workspace whose size is given by the matching
 * *_workspace_bytes function (256-byte aligned; contents need not be cleared).
 *
 * Return value: 0 on success, < 0 for rejected arguments, > 0 a hipError_t.
 * yitu_last_error() returns the message of the calling thread's last failure.
 *
 * Each entry point names the reference interface it replaces (paths relative
 * to the CGCL-codes/YiTu checkout).
 */
#ifndef YITU_HIP_H
#define YITU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *yitu_last_error(void);
int yitu_abi_version(void);

/* Plain device-to-device streaming copy of n_bytes (multiple of 16): the known-
 * size kernel used to calibrate HBM traffic counters and to measure achievable
 * copy bandwidth. No reference counterpart. */
int yitu_stream_copy(void *dst_device, const void *src_device, int64_t n_bytes, void *stream);

/* ------------------------------------------------------------------------- */
/* Row plan (per graph, built once)                                            */
/* ------------------------------------------------------------------------- */

/*
 * The counterpart of the reference's neighbour-group partition build_part
 * (ccsrc/kernel/YiTu_GNN.cpp:203-245), which its callers compute once per graph
 * and pass to every op as part_pointers / part2Node: rows with >= 64 edges are
 * cut where their columns cross the boundaries of source bands (2^17 ids) and
 * into items of at most 64 edges, listed in ascending order of the source id in
 * the middle of each item. The gather kernels (aggregation, SpMM, per-edge dot, GAT
 * aggregate) run one wave per item in that order, which keeps the hot rows of
 * the feature table in L2. The plan depends on (indptr, indices) only.
 * Every op that takes `plan_device` also accepts NULL and then builds a
 * temporary plan in its workspace on each call.
 * col_mask selects the column bits of indices (0xffffff for packed graph_ext
 * indices, 0x7fffffff for plain ones).
 */
size_t yitu_plan_bytes(int64_t nnz);
size_t yitu_plan_workspace_bytes(int64_t nnz);
int yitu_plan_build(void *plan_device, size_t plan_bytes, const int32_t *indptr_device,
                    const int32_t *indices_device, int64_t n_rows, int64_t n_src, int64_t nnz,
                    int32_t col_mask, void *workspace_device, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------- */
/* Module 1: YiTu_GNN.YiTu_GNN_kernel  (ccsrc/kernel/YiTu_GNN.cpp:247-258)     */
/* ------------------------------------------------------------------------- */

/* Scratch for the aggregation / SpMM kernels: partial sums of the rows with
 * >= 64 edges, plus a temporary row plan when the call is given none
 * (with_plan = 0). row_len = floats per feature row. */
size_t yitu_spmm_workspace_bytes(int64_t nnz, int64_t row_len, int with_plan);

/*
 * CSR neighbour aggregation, the kernel inside
 *   SAG          (YiTu_GNN.cpp:71-92;  YiTu_GNN_kernel.cu:104-257): degrees = NULL, alpha = 1
 *   forward      (YiTu_GNN.cpp:94-117; cu:320-415)  on X.W:   degrees = s,    alpha = 1
 *   backward     (YiTu_GNN.cpp:119-145; cu:478-556) on dY:    degrees = s,    alpha = 1
 *   forward_gin  (YiTu_GNN.cpp:150-172; cu:621-694) on X:     degrees = NULL, alpha = epsilon
 *   backward_gin (YiTu_GNN.cpp:177-201; cu:754-823) on dY.W^T: degrees = NULL, alpha = epsilon
 *
 *   out[r, :] = alpha * s[r] * sum_{e in row r} s[col[e]] * x[col[e], :]      (s = 1 if NULL)
 *
 * x is fp32 [n_src, dim], or bf16 (raw 16-bit patterns) when x_is_bf16 != 0;
 * accumulation and out [n_rows, dim] are fp32. Every row of out is written
 * (empty rows get zeros), without atomics: results are bitwise reproducible.
 * The neighbour-group arguments of the reference (part_pointers, part2Node,
 * partSize, dimWorker, warpPerBlock) are replaced by the row plan (or nothing).
 * max_degree: widest row if known, else -1.
 * edge_scale_device: NULL, or the per-edge column scales s[col[e]] of this graph
 * and this degrees array, written once by yitu_edge_scale: the kernels then read
 * them in edge order instead of one random 4-byte read of s per edge. On a large
 * graph those reads cost more than their bytes: the lines of s (32 sources each)
 * are all warm and push the feature rows out of L2 (2^21 nodes, F = 128 fp32:
 * 3.08 ms per call without, 2.69 ms with). Ignored when degrees is NULL.
 */
int yitu_agg_csr(float *out_device, const void *x_device, int x_is_bf16,
                 const int32_t *row_pointers_device, const int32_t *column_index_device,
                 const float *degrees_device, int64_t n_rows, int64_t n_src, int64_t nnz,
                 int64_t dim, float alpha, int64_t max_degree, const void *plan_device,
                 const float *edge_scale_device, void *workspace_device, size_t workspace_bytes,
                 void *stream);

/*
 * yitu_agg_csr for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same result as
 * yitu_agg_csr given no plan and no edge scales, but its scratch (the temporary
 * row plan and the partial rows of long rows) is a static device array of
 * yitu_agg_csr_noalloc_max_bytes() = 32 MiB inside the library instead of a
 * caller's workspace. No counterpart in the reference. It calls no hipMalloc /
 * hipFree or any allocating routine; problems whose
 * yitu_spmm_workspace_bytes(nnz, dim, 0) exceeds the array are rejected (< 0),
 * except that a graph which cannot hold a row of 64 edges (nnz < 64, or a stated
 * 0 <= max_degree < 64) uses no scratch and is accepted at any size.
 * All calls on one GPU share that GPU's array: calls that overlap in time on
 * one GPU (different streams or threads) race and must be serialised by the caller.
 * yitu_agg_csr_noalloc_init() looks up the array's address on the current device
 * (hipGetSymbolAddress, once per device); the first call on a device does the same,
 * so a caller that captures a stream calls init, or the function once, beforehand.
 */
size_t yitu_agg_csr_noalloc_max_bytes(void);
int yitu_agg_csr_noalloc_init(void);
int yitu_agg_csr_noalloc(float *out_device, const void *x_device, int x_is_bf16,
                         const int32_t *row_pointers_device, const int32_t *column_index_device,
                         const float *degrees_device, int64_t n_rows, int64_t n_src, int64_t nnz,
                         int64_t dim, float alpha, int64_t max_degree, void *stream);

/* edge_scale[e] = degrees[column_index[e]] for the nnz edges of a CSR: per-graph
 * preparation for yitu_agg_csr, like the row plan (the reference's callers hold
 * `degrees` per graph, data/dataset.py:131-136, and pass it to every call). */
int yitu_edge_scale(float *edge_scale_device, const int32_t *column_index_device,
                    const float *degrees_device, int64_t nnz, int64_t n_src, void *stream);

/* ------------------------------------------------------------------------- */
/* Module 2: graph_ext  (YiTu_GNN/YiTu_H/src/entry.cpp:184-193)                */
/* ------------------------------------------------------------------------- */

/*
 * spmm_forward (entry.cpp:80-90; spmm_cuda.cu:4-21,44-62):
 *   out[r,h,k] = sum_{i in row r} values[i,h] * features[indices[i] & 0xffffff, h, k]
 * values [nnz,H], features [n_src,H,F], out [n_dst,H,F], all fp32.
 * Workspace: yitu_spmm_workspace_bytes(nnz, H*F, plan != NULL).
 */
int yitu_spmm_forward(float *out_device, const float *values_device, const int32_t *indptr_device,
                      const int32_t *indices_device, const float *features_device, int64_t n_dst,
                      int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_features,
                      int64_t max_degree, const void *plan_device, void *workspace_device,
                      size_t workspace_bytes, void *stream);

/*
 * The same product with bf16 feature rows (fp32 edge values, fp32 accumulate,
 * fp32 out): the reference's op is fp32 only (spmm_cuda.cu:44-62); this is the
 * aggregation step of a bf16 pipeline whose dense transforms write bf16 rows
 * (yitu_gemm_bf16).
 */
int yitu_spmm_forward_bf16(float *out_device, const float *values_device,
                           const int32_t *indptr_device, const int32_t *indices_device,
                           const void *features_bf16_device, int64_t n_dst, int64_t n_src,
                           int64_t nnz, int64_t n_heads, int64_t n_features, int64_t max_degree,
                           const void *plan_device, void *workspace_device, size_t workspace_bytes,
                           void *stream);

/*
 * The same with bf16 rows out as well (fp32 sums, one rounding to nearest even per
 * output): the gradient rows of a bf16 pipeline, which the next bf16 product reads
 * without a conversion pass. n_features must be a multiple of 8 and both row buffers
 * 16-byte aligned.
 */
int yitu_spmm_forward_bf16_rows(void *out_bf16_device, const float *values_device,
                                const int32_t *indptr_device, const int32_t *indices_device,
                                const void *features_bf16_device, int64_t n_dst, int64_t n_src,
                                int64_t nnz, int64_t n_heads, int64_t n_features,
                                int64_t max_degree, const void *plan_device,
                                void *workspace_device, size_t workspace_bytes, void *stream);

/*
 * spmm_backward (entry.cpp:92-104; spmm_cuda.cu:24-42,64-86):
 *   grad_a[i,h]   = sum_k grad_out[row_i,h,k] * features[col_i,h,k]
 *   grad_x[c,h,k] = sum_{i: col_i = c} grad_out[row_i,h,k] * values[i,h]
 * Either output may be NULL to skip it (values may then be NULL for grad_a
 * alone, which is the plain per-edge dot product of a destination row with a
 * source row). grad_x is computed as a gather over
 * the transposed structure (t_* from yitu_csr_transpose, required when grad_x
 * is requested) instead of the reference's 2*E*H*F float atomics; both outputs
 * are fully written and bitwise reproducible. max_degree / max_degree_t: widest
 * row of the CSR / of its transpose if known, else -1. plan_device /
 * plan_t_device: row plans of (indptr, indices) and of (t_indptr, t_rows), or NULL.
 * Workspace: yitu_spmm_workspace_bytes(nnz, H*F, both plans given).
 */
int yitu_spmm_backward(float *grad_a_device, float *grad_x_device, const float *values_device,
                       const int32_t *indptr_device, const int32_t *indices_device,
                       const float *features_device, const float *grad_out_device,
                       const int32_t *t_indptr_device, const int32_t *t_rows_device,
                       const int32_t *t_perm_device, int64_t n_dst, int64_t n_src, int64_t nnz,
                       int64_t n_heads, int64_t n_features, int64_t max_degree,
                       int64_t max_degree_t, const void *plan_device, const void *plan_t_device,
                       void *workspace_device, size_t workspace_bytes, void *stream);

/*
 * sddmm_forward (entry.cpp:106-116; sddmm_cuda.cu:5-33,69-89):
 *   attn[i,h] = softmax over {i' in row r with the same bid} of
 *               leaky_relu(query[bid,r,h] + key[col,h], 0.2),
 *   bid = indices[i] >> 24, col = indices[i] & 0xffffff.
 * query [n_bid,n_dst,H], key [n_src,H], attn [nnz,H] (every entry is written).
 * The softmax subtracts the running maximum; the reference does not
 * (sddmm_cuda.cu:15-21) and overflows for logits above ~88.
 * plan_device: row plan of the CSR (yitu_plan_build with col_mask 0xffffff), or NULL.
 */
size_t yitu_sddmm_workspace_bytes(int64_t n_dst, int64_t nnz, int64_t n_heads, int64_t n_bid,
                                  int with_plan);
int yitu_sddmm_forward(float *attn_device, const int32_t *indptr_device,
                       const int32_t *indices_device, const float *query_device,
                       const float *key_device, int64_t n_dst, int64_t n_src, int64_t nnz,
                       int64_t n_heads, int64_t n_bid, int64_t max_degree, const void *plan_device,
                       void *workspace_device, size_t workspace_bytes, void *stream);

/*
 * sddmm_backward (entry.cpp:118-134; sddmm_cuda.cu:36-67,91-118):
 *   gv[i,h] = attn (grad_out - sum_j attn_j grad_out_j) * (x < 0 ? 0.2 : 1)
 *   grad_query[bid,r,h] = sum_i gv ;  grad_key[col,h] = sum_{i: col_i = col} gv
 * grad_query and grad_key are fully written. Two forms of the grad_key sum:
 *   t_indptr == NULL: float atomics (as the reference; order not reproducible);
 *   t_indptr, t_perm from yitu_csr_transpose and grad_edge_device [nnz,H]
 *   scratch: gv is stored per edge and summed by a gather over the transposed
 *   structure (bitwise reproducible).
 * max_degree / max_degree_t: widest row of the CSR / of its transpose, or -1.
 * plan_device / plan_t_device: row plans of the CSR and of the transposed structure
 * (gather form only), or NULL.
 */
int yitu_sddmm_backward(float *grad_query_device, float *grad_key_device, float *grad_edge_device,
                        const int32_t *indptr_device, const int32_t *indices_device,
                        const float *query_device, const float *key_device,
                        const float *attn_device, const float *grad_out_device,
                        const int32_t *t_indptr_device, const int32_t *t_perm_device,
                        int64_t n_dst, int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_bid,
                        int64_t max_degree, int64_t max_degree_t, const void *plan_device,
                        const void *plan_t_device, void *workspace_device, size_t workspace_bytes,
                        void *stream);

/* ------------------------------------------------------------------------- */
/* Fused GAT attention (composition of the two ops above in one pass)          */
/* ------------------------------------------------------------------------- */

/*
 * No single reference entry point: the reference lowers a GAT layer to
 * sddmm_forward followed by spmm_forward (xgnn_h/executor.py:22-40,
 * test/common/model.py:96-106). This computes the same composition
 *   attn = sddmm_forward(indptr, indices, query[None], key)     (n_bid = 1)
 *   out  = spmm_forward(attn, indptr, indices, features)
 * reading each destination row once. attn_device [nnz,H] receives the
 * probabilities for the backward pass; it may be NULL when the shape takes the
 * fused kernel (n_features % 4 == 0, n_heads <= 64, 16-byte aligned pointers).
 * row_stats_device [n_dst,H,2] (optional, fused kernel only) receives each row's
 * softmax (max, 1 / sum): with it the backward recomputes a probability from
 * query, key and these two numbers instead of reading attn, so attn need not be
 * stored at all. With attn_device NULL the rows of 64 edges and more are summed
 * from per-piece sums taken against each piece's own maximum: out then differs
 * from the attn_device != NULL result in the last bits (same tolerance against
 * the reference), and is reproducible from call to call like every other result.
 */
size_t yitu_gat_workspace_bytes(int64_t n_dst, int64_t nnz, int64_t n_heads, int64_t n_features,
                                int with_plans);
int yitu_gat_forward(float *out_device, float *attn_device, float *row_stats_device,
                     const int32_t *indptr_device, const int32_t *indices_device,
                     const float *query_device, const float *key_device,
                     const float *features_device, int64_t n_dst, int64_t n_src, int64_t nnz,
                     int64_t n_heads, int64_t n_features, int64_t max_degree,
                     const void *plan_device, void *workspace_device, size_t workspace_bytes,
                     void *stream);

/*
 * Backward of the composition (spmm_backward then sddmm_backward,
 * xgnn_h/sparse.py:22-35,67-81) in one call, given grad_out [n_dst,H,F]:
 * grad_query [n_dst,H], grad_key [n_src,H], grad_features [n_src,H,F], all
 * fully written, no atomics. The two scratch buffers are [nnz,H] floats.
 * attn_device may be NULL when row_stats_device (the forward's statistics) and
 * out_device are given and the shape is a one-pass shape.
 * out_device: the forward's output [n_dst,H,F], or NULL. With it (and rows of
 * 256 floats) the softmax row sums come from <grad_out[row], out[row]> and one
 * pass over the by-source edges finishes every gradient; the workspace must
 * then be given whatever the degrees (yitu_gat_workspace_bytes).
 * grad_out_is_head_mean: nonzero when the caller's result was the mean of out over
 * the heads (test/common/model.py:106) and grad_out_device is its gradient
 * g [n_dst,F], standing for grad_out[r,h,:] = g[r,:] / H. The pass then gathers
 * F floats per edge instead of H*F. One-pass shapes only (rows of 256 floats, or
 * 512 / 1024 with out_device, head width a power of two in 32..256).
 */
int yitu_gat_backward(float *grad_query_device, float *grad_key_device,
                      float *grad_features_device, float *grad_attn_scratch_device,
                      float *grad_edge_scratch_device, const int32_t *indptr_device,
                      const int32_t *indices_device, const float *query_device,
                      const float *key_device, const float *features_device,
                      const float *attn_device, const float *row_stats_device,
                      const float *out_device, const float *grad_out_device,
                      const int32_t *t_indptr_device,
                      const int32_t *t_rows_device,
                      const int32_t *t_perm_device, int64_t n_dst, int64_t n_src, int64_t nnz,
                      int64_t n_heads, int64_t n_features, int64_t max_degree,
                      int64_t max_degree_t, const void *plan_device, const void *plan_t_device,
                      int grad_out_is_head_mean, void *workspace_device, size_t workspace_bytes,
                      void *stream);

/*
 * Per-head projections of a GAT layer stated with attention vectors:
 *   out_a[n,h] = <vec_a[h,:], x[n,h,:]>   (and out_b with vec_b; vec_b / out_b may be NULL)
 * x [n,H,F], vec_* [H,F], out_* [n,H], fp32. The reference's example layer makes
 * query and key with dense H*F -> H Linears (test/common/model.py:70-71); the
 * per-head vectors are their block-diagonal, bias-free case. n_features must be
 * 4 * a power of two (4..256) and H*F at most 1024.
 * Backward: grad_x[n,h,:] (+)= grad_a[n,h] vec_a[h,:] + grad_b[n,h] vec_b[h,:]
 * (accumulate != 0 adds to what grad_x holds: the gradient that reached x through
 * the attention itself), grad_vec_a[h,:] = sum_n grad_a[n,h] x[n,h,:]. The sums over
 * n are taken per wave and then in wave order (reproducible).
 */
int yitu_head_dot(float *out_a_device, float *out_b_device, const float *x_device,
                  const float *vec_a_device, const float *vec_b_device, int64_t n, int64_t n_heads,
                  int64_t n_features, void *stream);
size_t yitu_head_dot_workspace_bytes(int64_t n, int64_t n_heads, int64_t n_features);
int yitu_head_dot_backward(float *grad_x_device, int accumulate, float *grad_vec_a_device,
                           float *grad_vec_b_device, const float *x_device,
                           const float *vec_a_device, const float *vec_b_device,
                           const float *grad_a_device, const float *grad_b_device, int64_t n,
                           int64_t n_heads, int64_t n_features, void *workspace_device,
                           size_t workspace_bytes, void *stream);

/*
 * Linear layers with a handful of outputs per row: y[n,J] = x[n,K] . w[J,K]^T + bias[J]
 * (bias may be NULL). The dense query / key projections of the reference's GATLayer
 * (nn.Linear(H*F, H), test/common/model.py:70-71) are this shape; stack the weights
 * of the two to make both with one read of x. K a multiple of 4 up to 1024, J up to 16
 * with J * tiles <= 16 (tiles = 1, 2, 4 for K up to 256, 512, 1024).
 * Backward: grad_x (+)= grad_y . w (accumulate != 0 adds to what grad_x holds),
 * grad_w [J,K], grad_bias [J] (may be NULL), summed in a fixed order.
 */
int yitu_skinny_linear(float *y_device, const float *x_device, const float *w_device,
                       const float *bias_device, int64_t n, int64_t in_features,
                       int64_t out_features, void *stream);
size_t yitu_skinny_linear_workspace_bytes(int64_t n, int64_t in_features, int64_t out_features);
int yitu_skinny_linear_backward(float *grad_x_device, int accumulate, float *grad_w_device,
                                float *grad_bias_device, const float *x_device,
                                const float *w_device, const float *grad_y_device, int64_t n,
                                int64_t in_features, int64_t out_features, void *workspace_device,
                                size_t workspace_bytes, void *stream);

/*
 * out[j] = sum_r x[r,j] for a row-major [n_rows, n_cols] fp32 matrix: the bias
 * gradient of a Linear layer, in two stages with a fixed order of additions and no
 * cleared accumulator, so the call can be recorded into a HIP graph and replayed.
 */
size_t yitu_column_sum_workspace_bytes(int64_t n_rows, int64_t n_cols);
/* The same for a list of short matrices x_i [n_rows_i, n_cols] (row stride ld floats) in one
 * launch per 32 of them: out_i[j] = sum_r x_i[r, j], rows added by a fixed number of threads
 * in a fixed order. The bias gradients of the per-relation Linears of a small heterogeneous
 * graph (test/common/model.py:137-171 over :25-29); meant for matrices of up to a few thousand
 * rows, longer ones take yitu_column_sum. out, x, n_rows are HOST arrays. */
int yitu_column_sum_typed(float *const *out_device_ptrs, const float *const *x_device_ptrs,
                          const int64_t *n_rows, int64_t n_problems, int64_t n_cols, int64_t ld,
                          void *stream);
int yitu_column_sum(float *out_device, const float *x_device, int64_t n_rows, int64_t n_cols,
                    void *workspace_device, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------- */
/* Dense products on the matrix cores (fp32 MFMA)                              */
/* ------------------------------------------------------------------------- */

/*
 * C[m,n] (+)= op(A)[m,k] . op(B)[k,n], row-major, fp32. trans_a: A is stored
 * [k,m]; trans_b: B is stored [n,k]. Replaces the torch::mm (cuBLAS SGEMM)
 * calls around the aggregation kernels: X.W (YiTu_GNN_kernel.cu:276,606),
 * G.W^T and X^T.G (cu:471-472,715-716). Products with few output tiles and a long
 * inner dimension (X^T.G) are split along k over the chip; the slabs go to the
 * workspace (yitu_sgemm_workspace_bytes; NULL = no split) and are summed in a
 * fixed order. With k = 64, 128 or 256, at least 49,152 rows, at least 192 columns in
 * the last block of 256 and no transposed A, the product runs with the weight held in
 * registers; a weight stored [k,n] is first
 * copied as [n,k] into the workspace when that is large enough.
 */
/* n_problems: how many products a typed call brings (1 for a single product). */
size_t yitu_sgemm_workspace_bytes(int64_t m, int64_t n, int64_t k, int64_t n_problems);
int yitu_sgemm(float *c_device, const float *a_device, const float *b_device, int64_t m, int64_t n,
               int64_t k, int trans_a, int trans_b, int64_t lda, int64_t ldb, int64_t ldc,
               int accumulate, void *workspace_device, size_t workspace_bytes, void *stream);

/*
 * y[m,n] = x[m,k] . w^T + bias, w stored [n,k] like nn.Linear.weight, bias [n] or NULL:
 * the forward of the Linear layers of the models (test/common/model.py:25-29, 86-88).
 * On the many-rows kernel (see yitu_sgemm) the bias is added before the rows are stored;
 * otherwise by a pass of its own. Workspace as for yitu_sgemm(m, n, k).
 */
int yitu_linear_forward(float *y_device, const float *x_device, const float *w_device,
                        const float *bias_device, int64_t m, int64_t n, int64_t k,
                        void *workspace_device, size_t workspace_bytes, void *stream);

/*
 * The same for the Linear layers of several node or edge types at once (the
 * per-relation loop of HeteroGraphConv, test/common/model.py:137-171, over layers
 * of model.py:25-29): y_i[m_i,n] = x_i[m_i,k] . w_i^T + bias_i for i < n_problems, up to
 * 32 layers per launch. y, x, w, bias, m are HOST arrays (of device pointers and sizes); the
 * bias table or single entries of it may be NULL. All y_i are contiguous (row stride n).
 * Workspace: yitu_sgemm_workspace_bytes(max m_i, n, k, n_problems).
 */
int yitu_linear_forward_typed(float *const *y, const float *const *x, const float *const *w,
                              const float *const *bias, const int64_t *m, int64_t n_problems,
                              int64_t n, int64_t k, void *workspace_device,
                              size_t workspace_bytes, void *stream);

/*
 * Typed products in one launch per 32 problems: C_i[m_i,n] (+)= op(A_i)[m_i,k_i] .
 * op(B_i)[k_i,n] for i < n_problems, with shared n, transposes and leading
 * dimensions. c, a, b, m, k are HOST arrays (of device pointers and sizes).
 * Replaces the loop of per-relation / per-type Linear layers of the
 * heterogeneous models (test/common/model.py:137-171 over :7-30, one cuBLAS SGEMM each and
 * its two gradient products): the row tiles of all node types fill the chip
 * together instead of one short launch after another. Workspace for the split
 * products (X_t^T . G_t): yitu_sgemm_workspace_bytes(max m_i, n, max k_i,
 * n_problems); the same workspace serves every group of 32.
 */
int yitu_sgemm_typed(float *const *c_device_ptrs, const float *const *a_device_ptrs,
                     const float *const *b_device_ptrs, const int64_t *m, const int64_t *k,
                     int64_t n_problems, int64_t n, int trans_a, int trans_b, int64_t lda,
                     int64_t ldb, int64_t ldc, int accumulate, void *workspace_device,
                     size_t workspace_bytes, void *stream);

/*
 * hfused_forward (entry.cpp:136-155; hfused_cuda.cu:5-45,96-137): the SpMM of
 * graph A and the SDDMM + LeakyReLU + edge softmax of graph B (same number of
 * rows, same head count) in ONE launch: the first workgroups of the grid run the
 * SpMM row kernel on A, the others the SDDMM row kernel on B. That holds when
 * both longest rows are known (max_degree_* >= 0) and below the long-row
 * thresholds (A: 64 edges, B: 512), n_heads <= 16, n_features a multiple of 4
 * and n_heads * n_features <= 1024; any other case runs yitu_spmm_forward and
 * then yitu_sddmm_forward. spmm_out [n_rows,H,F], attn [nnz_b,H]; query
 * [n_bid,n_rows,H], key [n_src_b,H]. Workspace (used by the two-op case only):
 * yitu_hfused_forward_workspace_bytes.
 */
size_t yitu_hfused_forward_workspace_bytes(int64_t n_rows, int64_t nnz_a, int64_t row_len,
                                           int64_t nnz_b, int64_t n_heads, int64_t n_bid);
int yitu_hfused_forward(float *spmm_out_device, float *attn_device, const float *spmm_values_device,
                        const int32_t *spmm_indptr_device, const int32_t *spmm_indices_device,
                        const float *spmm_features_device, const int32_t *sddmm_indptr_device,
                        const int32_t *sddmm_indices_device, const float *sddmm_query_device,
                        const float *sddmm_key_device, int64_t n_rows, int64_t n_src_a,
                        int64_t nnz_a, int64_t n_heads, int64_t n_features, int64_t n_src_b,
                        int64_t nnz_b, int64_t n_bid, int64_t max_degree_a, int64_t max_degree_b,
                        void *workspace_device, size_t workspace_bytes, void *stream);

/*
 * hfused_backward (entry.cpp:157-182; hfused_cuda.cu:47-94, unreachable in the
 * reference: sparse.py:109-110, and indexing heads by the wrong thread
 * coordinate, :59,186): the backward of both ops in TWO launches shared by the
 * two graphs. First the per-row passes (per-edge dot products of A -> grad_values
 * [nnz_a,H]; softmax backward of B -> grad_query [n_bid,n_rows,H] and the per-edge
 * logit gradient grad_edge [nnz_b,H], a scratch output), then the two by-source
 * gathers (grad_features [n_src_a,H,F] over A's by-source structure; grad_key
 * [n_src_b,H] = sums of grad_edge over B's). No atomics. That holds when all four
 * longest rows (A, A by source, B, B by source) are known and below the long-row
 * thresholds (64; B by destination: 512), n_heads <= 16, n_features a multiple of
 * 4, n_heads * n_features <= 1024; any other case runs yitu_spmm_backward and
 * yitu_sddmm_backward. Both by-source structures come from yitu_csr_transpose.
 */
size_t yitu_hfused_backward_workspace_bytes(int64_t n_rows, int64_t n_src_a, int64_t nnz_a,
                                            int64_t row_len, int64_t n_src_b, int64_t nnz_b,
                                            int64_t n_heads, int64_t n_bid);
int yitu_hfused_backward(float *grad_values_device, float *grad_features_device,
                         float *grad_query_device, float *grad_key_device, float *grad_edge_device,
                         const float *spmm_values_device, const int32_t *spmm_indptr_device,
                         const int32_t *spmm_indices_device, const float *spmm_features_device,
                         const float *spmm_grad_device, const int32_t *spmm_t_indptr_device,
                         const int32_t *spmm_t_rows_device, const int32_t *spmm_t_perm_device,
                         const int32_t *sddmm_indptr_device, const int32_t *sddmm_indices_device,
                         const float *sddmm_query_device, const float *sddmm_key_device,
                         const float *sddmm_attn_device, const float *sddmm_grad_device,
                         const int32_t *sddmm_t_indptr_device, const int32_t *sddmm_t_perm_device,
                         int64_t n_rows, int64_t n_src_a, int64_t nnz_a, int64_t n_heads,
                         int64_t n_features, int64_t n_src_b, int64_t nnz_b, int64_t n_bid,
                         int64_t max_degree_a, int64_t max_degree_a_t, int64_t max_degree_b,
                         int64_t max_degree_b_t, void *workspace_device, size_t workspace_bytes,
                         void *stream);

/*
 * b2gemm (entry.cpp:56-64; fc_cuda.cu:4-75): y_a = x . w_a^T, y_b = x . w_b^T
 * as one grouped launch. x [n,k], w_* [m,k], y_* [n,m], contiguous.
 */
int yitu_b2gemm(float *y_a_device, float *y_b_device, const float *x_device,
                const float *w_a_device, const float *w_b_device, int64_t n, int64_t k, int64_t m,
                void *stream);

/*
 * b2gemm_backward (entry.cpp:66-78; fc_cuda.cu:77-215):
 * dw_* [m,k] = grad_*^T . x ; dx [n,k] = grad_a . w_a + grad_b . w_b.
 * Workspace: yitu_sgemm_workspace_bytes(m, k, n, 2).
 */
int yitu_b2gemm_backward(float *dx_device, float *dw_a_device, float *dw_b_device,
                         const float *x_device, const float *w_a_device, const float *w_b_device,
                         const float *grad_a_device, const float *grad_b_device, int64_t n,
                         int64_t k, int64_t m, void *workspace_device, size_t workspace_bytes,
                         void *stream);

/*
 * C[m,n] = A[m,k] . op(B) with bf16 operands and fp32 accumulation on the matrix
 * cores; C is fp32 or bf16 (round to nearest even). A is row-major [m, lda];
 * trans_b: B is stored [n, ldb] (the layout of a Linear weight), else [k, ldb]
 * (it is then transposed into the workspace, yitu_gemm_bf16_workspace_bytes).
 * k and the leading dimensions of the K-contiguous operands must be multiples
 * of 8. The bf16 form of the per-type / per-relation feature transform of the
 * heterogeneous layers (fc_cuda.cu:4-75 and the nn.Linear calls of
 * YiTu_H/test/common/model.py:25-29, 86-88, which the reference runs in fp32).
 */
size_t yitu_gemm_bf16_workspace_bytes(int64_t n, int64_t k, int trans_b);
int yitu_gemm_bf16(void *c_device, int c_is_bf16, const void *a_bf16_device,
                   const void *b_bf16_device, int64_t m, int64_t n, int64_t k, int trans_b,
                   int64_t lda, int64_t ldb, int64_t ldc, void *workspace_device,
                   size_t workspace_bytes, void *stream);

/*
 * The same product for a list of operand pairs of one width, one launch per 8 pairs: C_i[m_i,n] = A_i[m_i,k] . op(B_i), shared n, k, trans_b and leading
 * dimensions; c, a, b are HOST arrays of device pointers, m a HOST array of row
 * counts. The bf16 form of yitu_sgemm_typed's forward and input-gradient products
 * (the loop of per-type / per-relation Linear layers, test/common/model.py:137-171
 * over :7-30). With k = 64, 128 or 256 and at least 4,096 rows in all, the row tiles
 * of every pair share one grid whose workgroups keep the pair's weight in registers;
 * other shapes run as one yitu_gemm_bf16 per pair.
 * Workspace: yitu_gemm_bf16_typed_workspace_bytes(n_problems, n, k, trans_b).
 */
size_t yitu_gemm_bf16_typed_workspace_bytes(int64_t n_problems, int64_t n, int64_t k, int trans_b);
int yitu_gemm_bf16_typed(void *const *c_device_ptrs, int c_is_bf16,
                         const void *const *a_bf16_device_ptrs,
                         const void *const *b_bf16_device_ptrs, const int64_t *m,
                         int64_t n_problems, int64_t n, int64_t k, int trans_b, int64_t lda,
                         int64_t ldb, int64_t ldc, void *workspace_device, size_t workspace_bytes,
                         void *stream);

/*
 * C[ki, no] (+)= A^T . B with bf16 operands A [m, lda], B [m, ldb] (row-major,
 * summed over their m rows) and fp32 accumulation on the matrix cores; C fp32
 * [ki, ldc]. The weight gradient dW = X^T . dY of a bf16 layer (fc_cuda.cu:77-215,
 * which the reference computes in fp32). ki, no and the leading dimensions must be
 * multiples of 8. The rows are split over the chip and the partial products are
 * added in a fixed order (bitwise reproducible); accumulate != 0 adds to C.
 * Workspace: yitu_gemm_bf16_tn_workspace_bytes(m, ki, no).
 */
size_t yitu_gemm_bf16_tn_workspace_bytes(int64_t m, int64_t ki, int64_t no);
int yitu_gemm_bf16_tn(float *c_device, const void *a_bf16_device, const void *b_bf16_device,
                      int64_t m, int64_t ki, int64_t no, int64_t lda, int64_t ldb, int64_t ldc,
                      int accumulate, void *workspace_device, size_t workspace_bytes, void *stream);

/*
 * The same for a list of operand pairs of one shape [m_i, ki], [m_i, no] (the weight
 * gradients of the per-type / per-relation Linear layers, test/common/model.py:137-171
 * over :7-30, backward), one launch pair per 8 problems: the row chunks of every pair
 * share one grid. c, a, b are HOST arrays of device pointers, m a HOST array of row
 * counts; a pair without rows writes zeros (or leaves C_i as it is with accumulate).
 * Workspace: yitu_gemm_bf16_tn_typed_workspace_bytes(m, n_problems, ki, no).
 */
size_t yitu_gemm_bf16_tn_typed_workspace_bytes(const int64_t *m, int64_t n_problems, int64_t ki,
                                               int64_t no);
int yitu_gemm_bf16_tn_typed(float *const *c_device_ptrs, const void *const *a_bf16_device_ptrs,
                            const void *const *b_bf16_device_ptrs, const int64_t *m,
                            int64_t n_problems, int64_t ki, int64_t no, int64_t lda, int64_t ldb,
                            int64_t ldc, int accumulate, void *workspace_device,
                            size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------- */
/* Temporal neighbour attention                                                */
/* ------------------------------------------------------------------------- */

/*
 * TransfomerAttentionLayer.forward, non-combined branches
 * (YiTu_GNN/YiTu_T/layers.py:75-142): for a sampled block of n_dst roots whose
 * n_edges neighbour edges are grouped by root (indptr [n_dst+1]), with node
 * features h [n_dst + n_edges, dim_node] (roots first, one row per edge after
 * them), edge features f [n_edges, dim_edge] and time deltas dt [n_edges],
 *   Q = w_q [h_root | cos(time_b)] + b_q
 *   K, V = w_{k,v} [h_edge | f | cos(time_w dt + time_b)] + b_{k,v}      (layers.py:6-17, 109-125)
 *   agg[r] = sum_e softmax_r(LeakyReLU_0.2(<Q[r], K[e]>_head)) V[e]      (layers.py:126-135)
 *   out = LayerNorm(ReLU(w_out [agg | h_root] + b_out))                  (layers.py:136-142)
 * The three products run on yitu_sgemm / yitu_sgemm_typed between these calls;
 * every matrix they touch has rows of ld = yitu_tattn_row_length(...) floats
 * whose last column carries the ones (inputs) or the bias (weights), so the
 * products add the biases and their transposed forms return the bias gradients.
 *
 * yitu_tattn_prepare fills, in one launch: x_kv [n_edges, ld], x_q [n_dst, ld],
 * columns dim_out.. of x_r [n_dst, ld] (h_root, ones), w_kv [2 dim_out, ld]
 * (w_k above w_v), w_q2 [2 dim_out, ld] (w_q, then zero rows: its product has the
 * width of the K|V product and shares its launch), w_r [dim_out, ld]. Weights are
 * row-major [out, in] like nn.Linear.weight. Needs dim_node + dim_time > 0.
 * Then: kv [n_edges, 2 dim_out] = x_kv . w_kv^T, q2 [n_dst, 2 dim_out] = x_q . w_q2^T.
 *
 * yitu_tattn_forward: attn [n_edges, n_heads] and x_r[:, 0..dim_out) = agg (zero
 * for a root without edges), one wave per root. Then pre [n_dst, dim_out] =
 * x_r . w_r^T and yitu_relu_layernorm_forward.
 *
 * Backward: yitu_relu_layernorm_backward (d_pre with a row stride, partial sums
 * of the affine gradients: [yitu_tattn_partial_rows(n_rows), 2 n_cols], gamma's
 * then beta's), dx_r = d_pre . w_r, yitu_tattn_backward (dq2 [n_dst, 2 dim_out]
 * columns 0..dim_out-1, dkv [n_edges, 2 dim_out]; scratch [n_edges, n_heads, 2]),
 * dx_kv = dkv . w_kv, dx_q = dq2 . w_q2, the weight gradients as transposed
 * products, yitu_tattn_finalize (grad_h [n_dst + n_edges, dim_node], grad_f, either
 * may be NULL; partial sums of the time encoder's gradients
 * [yitu_tattn_partial_rows(n_dst + n_edges), 2 dim_time], frequency then phase) and
 * yitu_partial_sums (column sums of two partial tables, rows added in ascending
 * order). No atomics: bitwise reproducible. Limits: dim_out, dim_time <= 256,
 * n_heads <= 8 and a divisor of dim_out.
 */
int64_t yitu_tattn_row_length(int64_t dim_node, int64_t dim_edge, int64_t dim_time,
                              int64_t dim_out);
int64_t yitu_tattn_partial_rows(int64_t n_rows);
int yitu_tattn_prepare(float *x_kv_device, float *x_q_device, float *x_r_device,
                       float *w_kv_device, float *w_q2_device, float *w_r_device,
                       const float *h_device, const float *f_device, const float *dt_device,
                       const float *time_w_device, const float *time_b_device,
                       const float *w_q_device, const float *b_q_device, const float *w_k_device,
                       const float *b_k_device, const float *w_v_device, const float *b_v_device,
                       const float *w_out_device, const float *b_out_device, int64_t n_dst,
                       int64_t n_edges, int64_t dim_node, int64_t dim_edge, int64_t dim_time,
                       int64_t dim_out, int64_t ld, void *stream);
int yitu_tattn_forward(float *x_r_device, float *attn_device, const float *q2_device,
                       const float *kv_device, const int32_t *indptr_device, int64_t n_dst,
                       int64_t n_edges, int64_t dim_out, int64_t n_heads, int64_t ld, void *stream);
int yitu_tattn_backward(float *dq2_device, float *dkv_device, float *scratch_device,
                        const float *dx_r_device, const float *q2_device, const float *kv_device,
                        const float *attn_device, const int32_t *indptr_device, int64_t n_dst,
                        int64_t n_edges, int64_t dim_out, int64_t n_heads, int64_t ld,
                        void *stream);
int yitu_relu_layernorm_forward(float *out_device, const float *pre_device,
                                const float *gamma_device, const float *beta_device,
                                int64_t n_rows, int64_t n_cols, float eps, void *stream);
int yitu_relu_layernorm_backward(float *d_pre_device, float *partial_device,
                                 const float *grad_out_device, const float *pre_device,
                                 const float *gamma_device, int64_t n_rows, int64_t n_cols,
                                 int64_t d_pre_row_stride, float eps, void *stream);
int yitu_tattn_finalize(float *grad_h_device, float *grad_f_device, float *partial_device,
                        const float *dx_kv_device, const float *dx_q_device,
                        const float *dx_r_device, const float *dt_device,
                        const float *time_w_device, const float *time_b_device, int64_t n_dst,
                        int64_t n_edges, int64_t dim_node, int64_t dim_edge, int64_t dim_time,
                        int64_t dim_out, int64_t ld, void *stream);
int yitu_partial_sums(float *out_a_device, const float *partial_a_device, int64_t rows_a,
                      int64_t cols_a, float *out_b_device, const float *partial_b_device,
                      int64_t rows_b, int64_t cols_b, void *stream);
/*
 * The last launch of the layer's backward: both column sums (grad_ln [2 dim_out] =
 * gamma's, beta's; grad_time [2 dim_time] = frequency, phase) and the parameter
 * gradients out of the bias-augmented rows of dw_kv [2 dim_out, ld], dw_q, dw_r
 * [dim_out, ld] into one contiguous tensor per parameter (shapes of the
 * nn.Linear weights / biases of layers.py:63-68).
 */
int yitu_tattn_collect(float *grad_ln_device, float *grad_time_device, float *grad_w_q_device,
                       float *grad_b_q_device, float *grad_w_k_device, float *grad_b_k_device,
                       float *grad_w_v_device, float *grad_b_v_device, float *grad_w_out_device,
                       float *grad_b_out_device, const float *partial_ln_device, int64_t rows_ln,
                       const float *partial_time_device, int64_t rows_time,
                       const float *dw_kv_device, const float *dw_q_device,
                       const float *dw_r_device, int64_t dim_node, int64_t dim_edge,
                       int64_t dim_time, int64_t dim_out, int64_t ld, void *stream);

/* ------------------------------------------------------------------------- */
/* Temporal most-recent-neighbour sampling on the device                       */
/* ------------------------------------------------------------------------- */

/*
 * One layer of sampler_core.ParallelSampler.sample in its recent = True mode
 * (YiTu_GNN/YiTu_T/sampler_core.cpp:103-127, 153-199, 295-305) with the T-CSR
 * (indptr [n_nodes+1], indices / eid [E] int32, ts [E] float32 ascending per
 * node) and the per-node cursors [n_nodes] in device memory. cursor is state:
 * yitu_tsample_reset sets it to indptr[0..n_nodes) (ParallelSampler.reset),
 * every call advances it. Outputs (device): row, col, eid_out with room for
 * n_roots * fan entries; ts_out, dts_out, nodes_out with room for
 * n_roots * (fan + 1); *n_edges_out (device int64) = number of sampled edges,
 * or -1 if a root id is out of range. Same bits as yitu_sampler_sample of the
 * host library.
 */
int yitu_tsample_reset(int32_t *cursor_device, const int32_t *indptr_device, int64_t n_nodes,
                       void *stream);
size_t yitu_tsample_workspace_bytes(int64_t n_roots);
int yitu_tsample_recent(int32_t *row_device, int32_t *col_device, int32_t *eid_out_device,
                        float *ts_out_device, float *dts_out_device, int32_t *nodes_out_device,
                        long long *n_edges_device, int32_t *cursor_device,
                        const int32_t *indptr_device, const int32_t *indices_device,
                        const int32_t *eid_device, const float *ts_device, int64_t n_nodes,
                        const int32_t *roots_device, const float *root_ts_device, int64_t n_roots,
                        int fan, int prop_time, void *workspace_device, size_t workspace_bytes,
                        void *stream);

/*
 * The other modes of ParallelSampler (sampler_core.cpp:201-359), as the two pieces its
 * sample() strings together per layer and snapshot.
 * yitu_tsample_advance: update_ts_ptr (:103-127) for one cursor array [n_nodes]: the
 * cursor of every root's node moves to the last edge with ts <= t + offset - 1e-7,
 * never backwards.
 * yitu_tsample_window: one snapshot of one layer (:216-333). The window [lo, hi] of a
 * root is read from two cursor arrays, or, with both null, found by binary search:
 * [first edge, last edge with ts <= t] (windowed = 0), or [last edge with ts <= t +
 * offset - window, last edge with ts <= t + offset] (windowed = 1: num_history > 1).
 * recent = 1 keeps the `fan` most recent edges of the window; recent = 0 makes `fan`
 * draws lo + rand_r() % (hi - lo + 1) when the window holds at least `fan` edges
 * (:306-318), from the generators of the reference's threads: thread c owns the roots
 * [c chunk, (c + 1) chunk), chunk = ceil(n_roots / threads), and rand_r state c (the C
 * library's rand_r, restated in the kernel; a root's state is reached by skipping
 * ahead, so the result does not depend on how the device schedules the roots). Edges
 * not older than t + offset - 1e-7 are dropped either way. Outputs as
 * yitu_tsample_recent's. Same bits as the host library in every mode.
 */
int yitu_tsample_advance(int32_t *cursor_device, const int32_t *indptr_device,
                         const float *ts_device, int64_t n_nodes, const int32_t *roots_device,
                         const float *root_ts_device, int64_t n_roots, float offset, void *stream);
size_t yitu_tsample_window_workspace_bytes(int64_t n_roots);
int yitu_tsample_window(int32_t *row_device, int32_t *col_device, int32_t *eid_out_device,
                        float *ts_out_device, float *dts_out_device, int32_t *nodes_out_device,
                        long long *n_edges_device, const int32_t *lo_cursor_device,
                        const int32_t *hi_cursor_device, const int32_t *indptr_device,
                        const int32_t *indices_device, const int32_t *eid_device,
                        const float *ts_device, int64_t n_nodes, const int32_t *roots_device,
                        const float *root_ts_device, int64_t n_roots, int fan, int prop_time,
                        int recent, int windowed, float offset, float window, int64_t chunk,
                        void *workspace_device, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------- */
/* Graph preparation                                                           */
/* ------------------------------------------------------------------------- */

/*
 * Edge list -> canonical CSR on the device: rows ascending, columns ascending
 * inside a row, duplicate edges merged, int32 -- the form the reference gets
 * from scipy's coo_matrix(...).tocsr() (YiTu_GNN/data/dataset.py:116-129).
 * indices_device must hold n_edges entries; the number of distinct edges is
 * written to *nnz_device (a device int64; -1 if an id is out of range).
 * Workspace 256-byte aligned.
 */
size_t yitu_coo_to_csr_workspace_bytes(int64_t n_edges, int64_t n_rows);
int yitu_coo_to_csr(int32_t *indptr_device, int32_t *indices_device, long long *nnz_device,
                    const int32_t *rows_device, const int32_t *cols_device, int64_t n_edges,
                    int64_t n_rows, int64_t n_cols, void *workspace_device, size_t workspace_bytes,
                    void *stream);

/*
 * build_part on the device (ccsrc/kernel/YiTu_GNN.cpp:203-245, which walks the rows on
 * the host): neighbour group p covers edges [part_ptr[p], part_ptr[p+1]) of row
 * part2node[p], at most part_size of them; row r has ceil(deg_r / part_size) groups.
 * Same integers as the reference's arrays, including part_ptr[n_parts], which is the
 * number of edges only when the last row has edges and 0 otherwise (cpp:240-241).
 * part_ptr has room for capacity + 1 entries, part2node for capacity;
 * capacity >= nnz / part_size + n_rows always suffices. *n_parts (device int64) receives
 * the number of groups; entries beyond the capacity are not written.
 */
size_t yitu_build_part_workspace_bytes(int64_t n_rows);
int yitu_build_part(int32_t *part_ptr_device, int32_t *part2node_device,
                    long long *n_parts_device, const int32_t *indptr_device, int64_t n_rows,
                    int64_t part_size, int64_t capacity, void *workspace_device,
                    size_t workspace_bytes, void *stream);

/*
 * By-source (transposed) view of a CSR, built once per graph on the device.
 * The reference has no such step: its backward kernels scatter with atomics
 * (spmm_cuda.cu:33-38, sddmm_cuda.cu:59-63); this turns those scatters into
 * gathers. For the stable order of a canonical CSR:
 *   t_indptr [n_cols+1]: edges of source c are t_indptr[c] .. t_indptr[c+1]-1
 *   t_rows   [nnz]     : destination row of each of them (ascending per source)
 *   t_perm   [nnz]     : its position in the original indices/values arrays
 * col_mask selects the column bits of indices (0xffffff for packed graph_ext
 * indices, 0x7fffffff for plain ones).
 */
size_t yitu_csr_transpose_workspace_bytes(int64_t nnz, int64_t n_cols);
int yitu_csr_transpose(int32_t *t_indptr_device, int32_t *t_rows_device, int32_t *t_perm_device,
                       const int32_t *indptr_device, const int32_t *indices_device, int64_t n_rows,
                       int64_t n_cols, int64_t nnz, int32_t col_mask, void *workspace_device,
                       size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* YITU_HIP_H */
