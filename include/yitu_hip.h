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

/* ------------------------------------------------------------------------- */
/* Module 1: YiTu_GNN.YiTu_GNN_kernel  (ccsrc/kernel/YiTu_GNN.cpp:247-258)     */
/* ------------------------------------------------------------------------- */

/* Scratch for the aggregation / SpMM kernels: queue and partial sums of rows
 * with >= 512 edges. row_len = floats per feature row. */
size_t yitu_spmm_workspace_bytes(int64_t nnz, int64_t row_len);

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
 * partSize, dimWorker, warpPerBlock) have no counterpart: the row split is
 * done on the device per call. max_degree: widest row if known, else -1.
 */
int yitu_agg_csr(float *out_device, const void *x_device, int x_is_bf16,
                 const int32_t *row_pointers_device, const int32_t *column_index_device,
                 const float *degrees_device, int64_t n_rows, int64_t n_src, int64_t nnz,
                 int64_t dim, float alpha, int64_t max_degree, void *workspace_device,
                 size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------- */
/* Module 2: graph_ext  (YiTu_GNN/YiTu_H/src/entry.cpp:184-193)                */
/* ------------------------------------------------------------------------- */

/*
 * spmm_forward (entry.cpp:80-90; spmm_cuda.cu:4-21,44-62):
 *   out[r,h,k] = sum_{i in row r} values[i,h] * features[indices[i] & 0xffffff, h, k]
 * values [nnz,H], features [n_src,H,F], out [n_dst,H,F], all fp32.
 * Workspace: yitu_spmm_workspace_bytes(nnz, H*F).
 */
int yitu_spmm_forward(float *out_device, const float *values_device, const int32_t *indptr_device,
                      const int32_t *indices_device, const float *features_device, int64_t n_dst,
                      int64_t n_src, int64_t nnz, int64_t n_heads, int64_t n_features,
                      int64_t max_degree, void *workspace_device, size_t workspace_bytes,
                      void *stream);

#ifdef __cplusplus
}
#endif
#endif /* YITU_HIP_H */
