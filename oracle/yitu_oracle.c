/*
 * CPU restatement of YiTu's sparse message-passing arithmetic.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker that the HIP kernels are
 * compared against and the timed "cpu_baseline" of the benchmark; nothing in
 * the shipped package may call into it. Paths cited below are relative to the
 * reference checkout.
 *
 * Two flavours exist for every aggregation:
 *   *_f32  follows the reference's float arithmetic and loop order (one float
 *          partial per neighbour group, groups added in ascending order);
 *   *_f64  accumulates in double and rounds once, the referee used for
 *          tolerance checks because the reference's own result depends on the
 *          nondeterministic order of its atomic adds.
 * Functions with the suffix _omp are the row-parallel float builds used only
 * for timing.
 *
 * Pinning (see tests/test_oracle_*.py): every function here is checked against
 * an independent formulation -- scipy.sparse CSR @ dense, dense torch matmul /
 * softmax with autograd for the gradients (the method of the reference's own
 * YiTu_GNN/YiTu_H/test/test_kernel.py), closed forms for build_part and
 * brute-force Python loops for stitch_csr.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* A1: neighbour-group partition. ccsrc/kernel/YiTu_GNN.cpp:203-245           */
/* ------------------------------------------------------------------------- */

/* number of groups: sum over rows of ceil(deg / partSize) (YiTu_GNN.cpp:211-219) */
ORC_EXPORT int64_t orc_build_part_count(int part_size, const int32_t *indptr, int64_t n_rows)
{
    int64_t n_parts = 0;
    for (int64_t i = 0; i < n_rows; i++) {
        int32_t deg = indptr[i + 1] - indptr[i];
        n_parts += deg / part_size + (deg % part_size != 0);
    }
    return n_parts;
}

/*
 * part_ptr has n_parts + 1 slots and must be zero-filled by the caller exactly
 * as torch::zeros does in the reference (YiTu_GNN.cpp:222); the sentinel slot
 * is only written when the last row ends a group (YiTu_GNN.cpp:240-241), so for
 * a graph whose last row is empty it keeps the zero.
 */
ORC_EXPORT void orc_build_part(int part_size, const int32_t *indptr, int64_t n_rows,
                               int32_t *part_ptr, int32_t *part2node)
{
    int64_t p = 0;
    for (int64_t i = 0; i < n_rows; i++) {
        int32_t beg = indptr[i], end = indptr[i + 1];
        int32_t deg = end - beg;
        int32_t cnt = deg / part_size + (deg % part_size != 0);
        for (int32_t g = 0; g < cnt; g++) {
            int32_t pb = beg + g * part_size;
            int32_t pe = pb + part_size < end ? pb + part_size : end;
            part_ptr[p] = pb;
            part2node[p++] = (int32_t)i;
            if (i == n_rows - 1 && pe == end)
                part_ptr[p] = pe;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* A2/A3/A4/A5/A6: module-1 aggregation. ccsrc/kernel/YiTu_GNN_kernel.cu      */
/* ------------------------------------------------------------------------- */

/*
 * Group-ordered float aggregation, the arithmetic of
 *   spmm_forward_cuda_kernel   (cu:320-415)  mode 0: w = fmaf(s_r, s_j, 0)
 *   SAG_cuda_kernel            (cu:180-257)  mode 1: w = 1
 *   spmm_forward_cuda_kernel_gin (cu:621-694) mode 2: w = 1, group sum * eps
 * One float partial per neighbour group (cu:380-405), then added to the output
 * row (cu:408-413); the atomic order is fixed here to ascending group index.
 * The end of group p is part_ptr[p + 1] as in the kernel (cu:352).
 */
ORC_EXPORT void orc_group_agg_f32(float *out, const float *in, const int32_t *col,
                                  const float *deg, const int32_t *part_ptr,
                                  const int32_t *part2node, int64_t n_parts,
                                  int64_t n_rows, int64_t dim, int mode, float eps)
{
    float *partial = (float *)malloc(sizeof(float) * (size_t)dim);
    memset(out, 0, sizeof(float) * (size_t)(n_rows * dim));
    for (int64_t p = 0; p < n_parts; p++) {
        int32_t r = part2node[p];
        int32_t pb = part_ptr[p], pe = part_ptr[p + 1];
        float sr = mode == 0 ? deg[r] : 1.0f;
        for (int64_t d = 0; d < dim; d++) partial[d] = 0.0f;
        for (int32_t e = pb; e < pe; e++) {
            int32_t j = col[e];
            if (mode == 0) {
                float w = fmaf(sr, deg[j], 0.0f);
                for (int64_t d = 0; d < dim; d++)
                    partial[d] += fmaf(w, in[(int64_t)j * dim + d], 0.0f);
            } else {
                for (int64_t d = 0; d < dim; d++)
                    partial[d] += in[(int64_t)j * dim + d];
            }
        }
        float *o = out + (int64_t)r * dim;
        if (mode == 2)
            for (int64_t d = 0; d < dim; d++) o[d] += eps * partial[d];
        else
            for (int64_t d = 0; d < dim; d++) o[d] += partial[d];
    }
    free(partial);
}

/*
 * Row-wise double-accumulate referee of the same three closed forms:
 *   mode 0: out[r] = sum_j (s_r * s_j) * in[j]        (cu:386,402)
 *   mode 1: out[r] = sum_j in[j]                       (cu:247)
 *   mode 2: out[r] = eps * sum_j in[j]                 (cu:691)
 * The edge weight s_r*s_j is still formed in float, as the kernel does.
 */
ORC_EXPORT void orc_row_agg_f64(float *out, const float *in, const int32_t *indptr,
                                const int32_t *col, const float *deg, int64_t n_rows,
                                int64_t dim, int mode, float eps)
{
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)dim);
#pragma omp for schedule(dynamic, 256)
        for (int64_t r = 0; r < n_rows; r++) {
            for (int64_t d = 0; d < dim; d++) acc[d] = 0.0;
            float sr = mode == 0 ? deg[r] : 1.0f;
            for (int32_t e = indptr[r]; e < indptr[r + 1]; e++) {
                int32_t j = col[e];
                double w = mode == 0 ? (double)(sr * deg[j]) : 1.0;
                const float *x = in + (int64_t)j * dim;
                for (int64_t d = 0; d < dim; d++) acc[d] += w * (double)x[d];
            }
            float *o = out + r * dim;
            if (mode == 2)
                for (int64_t d = 0; d < dim; d++) o[d] = (float)((double)eps * acc[d]);
            else
                for (int64_t d = 0; d < dim; d++) o[d] = (float)acc[d];
        }
        free(acc);
    }
}

/* Same closed forms, float accumulation, row-parallel: the timed CPU baseline. */
ORC_EXPORT void orc_row_agg_f32_omp(float *out, const float *in, const int32_t *indptr,
                                    const int32_t *col, const float *deg, int64_t n_rows,
                                    int64_t dim, int mode, float eps)
{
#pragma omp parallel for schedule(dynamic, 256)
    for (int64_t r = 0; r < n_rows; r++) {
        float *o = out + r * dim;
        for (int64_t d = 0; d < dim; d++) o[d] = 0.0f;
        float sr = mode == 0 ? deg[r] : 1.0f;
        for (int32_t e = indptr[r]; e < indptr[r + 1]; e++) {
            int32_t j = col[e];
            float w = mode == 0 ? sr * deg[j] : 1.0f;
            const float *x = in + (int64_t)j * dim;
#pragma omp simd
            for (int64_t d = 0; d < dim; d++) o[d] += w * x[d];
        }
        if (mode == 2)
            for (int64_t d = 0; d < dim; d++) o[d] *= eps;
    }
}

/* bf16 (upper 16 bits of an IEEE float) input, float accumulate, row-parallel. */
ORC_EXPORT void orc_row_agg_bf16_f64(float *out, const uint16_t *in, const int32_t *indptr,
                                     const int32_t *col, const float *deg, int64_t n_rows,
                                     int64_t dim, int mode, float eps)
{
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)dim);
#pragma omp for schedule(dynamic, 256)
        for (int64_t r = 0; r < n_rows; r++) {
            for (int64_t d = 0; d < dim; d++) acc[d] = 0.0;
            float sr = mode == 0 ? deg[r] : 1.0f;
            for (int32_t e = indptr[r]; e < indptr[r + 1]; e++) {
                int32_t j = col[e];
                double w = mode == 0 ? (double)(sr * deg[j]) : 1.0;
                const uint16_t *x = in + (int64_t)j * dim;
                for (int64_t d = 0; d < dim; d++) {
                    uint32_t bits = (uint32_t)x[d] << 16;
                    float f;
                    memcpy(&f, &bits, 4);
                    acc[d] += w * (double)f;
                }
            }
            float *o = out + r * dim;
            double s = mode == 2 ? (double)eps : 1.0;
            for (int64_t d = 0; d < dim; d++) o[d] = (float)(s * acc[d]);
        }
        free(acc);
    }
}

/* ------------------------------------------------------------------------- */
/* B1/B2: multi-head edge-weighted SpMM. YiTu_GNN/YiTu_H/src/spmm_cuda.cu     */
/* ------------------------------------------------------------------------- */

#define COL_MASK 0xffffff

/* out[r,h,k] = sum_i values[i,h] * feat[col_i,h,k]   (spmm_cuda.cu:8-19) */
ORC_EXPORT void orc_mh_spmm_fwd(float *out, const float *values, const int32_t *indptr,
                                const int32_t *indices, const float *feat, int64_t n_dst,
                                int64_t n_heads, int64_t n_feat, int use_f64)
{
    int64_t L = n_heads * n_feat;
#pragma omp parallel
    {
        double *acc = (double *)malloc(sizeof(double) * (size_t)L);
#pragma omp for schedule(dynamic, 64)
        for (int64_t r = 0; r < n_dst; r++) {
            for (int64_t t = 0; t < L; t++) acc[t] = 0.0;
            for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
                int64_t c = indices[i] & COL_MASK;
                for (int64_t h = 0; h < n_heads; h++) {
                    float v = values[(int64_t)i * n_heads + h];
                    const float *x = feat + c * L + h * n_feat;
                    double *a = acc + h * n_feat;
                    if (use_f64)
                        for (int64_t k = 0; k < n_feat; k++) a[k] += (double)v * (double)x[k];
                    else /* serial float accumulate in edge order, as each thread does */
                        for (int64_t k = 0; k < n_feat; k++) a[k] = (double)((float)a[k] + v * x[k]);
                }
            }
            for (int64_t t = 0; t < L; t++) out[r * L + t] = (float)acc[t];
        }
        free(acc);
    }
}

/*
 * grad_a[i,h] = sum_k g[r,h,k] * feat[col_i,h,k]
 * grad_x[c,h,k] = sum_{i: col_i = c} g[row_i,h,k] * values[i,h]   (spmm_cuda.cu:28-40)
 * Accumulated in double (the reference uses float atomics in arbitrary order).
 */
ORC_EXPORT void orc_mh_spmm_bwd(float *grad_a, float *grad_x, const float *values,
                                const int32_t *indptr, const int32_t *indices,
                                const float *feat, const float *grad_out, int64_t n_dst,
                                int64_t n_src, int64_t n_heads, int64_t n_feat)
{
    int64_t L = n_heads * n_feat;
    double *gx = (double *)calloc((size_t)(n_src * L), sizeof(double));
    for (int64_t r = 0; r < n_dst; r++) {
        const float *g = grad_out + r * L;
        for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
            int64_t c = indices[i] & COL_MASK;
            for (int64_t h = 0; h < n_heads; h++) {
                double dot = 0.0;
                float v = values[(int64_t)i * n_heads + h];
                for (int64_t k = 0; k < n_feat; k++) {
                    dot += (double)g[h * n_feat + k] * (double)feat[c * L + h * n_feat + k];
                    gx[c * L + h * n_feat + k] += (double)g[h * n_feat + k] * (double)v;
                }
                grad_a[(int64_t)i * n_heads + h] = (float)dot;
            }
        }
    }
    for (int64_t t = 0; t < n_src * L; t++) grad_x[t] = (float)gx[t];
    free(gx);
}

/*
 * By-source view of a CSR (stable counting sort on the column): t_indptr [n_src + 1],
 * t_rows[j] = destination row and t_perm[j] = CSR position of the j-th by-source edge.
 * Per-graph preparation of the timed _omp gradients below, which must not race on a
 * source's row the way the reference's atomics do (spmm_cuda.cu:33-38).
 */
ORC_EXPORT void orc_csr_transpose(int32_t *t_indptr, int32_t *t_rows, int32_t *t_perm,
                                  const int32_t *indptr, const int32_t *indices, int64_t n_dst,
                                  int64_t n_src)
{
    for (int64_t c = 0; c <= n_src; c++) t_indptr[c] = 0;
    for (int64_t i = 0; i < indptr[n_dst]; i++) t_indptr[(indices[i] & COL_MASK) + 1]++;
    for (int64_t c = 0; c < n_src; c++) t_indptr[c + 1] += t_indptr[c];
    int32_t *cursor = (int32_t *)malloc(sizeof(int32_t) * (size_t)(n_src + 1));
    memcpy(cursor, t_indptr, sizeof(int32_t) * (size_t)(n_src + 1));
    for (int64_t r = 0; r < n_dst; r++)
        for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
            int32_t j = cursor[indices[i] & COL_MASK]++;
            t_rows[j] = (int32_t)r;
            t_perm[j] = i;
        }
    free(cursor);
}

/*
 * orc_mh_spmm_bwd in float on all cores, for timing only: grad_a row-parallel, grad_x
 * source-parallel over the by-source view (each source's row has one writer, edges
 * added in ascending destination order). Either output may be NULL.
 */
ORC_EXPORT void orc_mh_spmm_bwd_omp(float *grad_a, float *grad_x, const float *values,
                                    const int32_t *indptr, const int32_t *indices,
                                    const float *feat, const float *grad_out,
                                    const int32_t *t_indptr, const int32_t *t_rows,
                                    const int32_t *t_perm, int64_t n_dst, int64_t n_src,
                                    int64_t n_heads, int64_t n_feat)
{
    int64_t L = n_heads * n_feat;
    if (grad_a) {
#pragma omp parallel for schedule(dynamic, 64)
        for (int64_t r = 0; r < n_dst; r++) {
            const float *g = grad_out + r * L;
            for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
                const float *x = feat + (int64_t)(indices[i] & COL_MASK) * L;
                for (int64_t h = 0; h < n_heads; h++) {
                    float dot = 0.0f;
                    for (int64_t k = 0; k < n_feat; k++) dot += g[h * n_feat + k] * x[h * n_feat + k];
                    grad_a[(int64_t)i * n_heads + h] = dot;
                }
            }
        }
    }
    if (grad_x) {
#pragma omp parallel for schedule(dynamic, 64)
        for (int64_t c = 0; c < n_src; c++) {
            float *o = grad_x + c * L;
            for (int64_t t = 0; t < L; t++) o[t] = 0.0f;
            for (int32_t j = t_indptr[c]; j < t_indptr[c + 1]; j++) {
                const float *g = grad_out + (int64_t)t_rows[j] * L;
                const float *v = values + (int64_t)t_perm[j] * n_heads;
                for (int64_t h = 0; h < n_heads; h++)
                    for (int64_t k = 0; k < n_feat; k++) o[h * n_feat + k] += v[h] * g[h * n_feat + k];
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* B3/B4: SDDMM(u_add_v) + LeakyReLU(0.2) + edge softmax.                     */
/* YiTu_GNN/YiTu_H/src/sddmm_cuda.cu, ops.cuh                                 */
/* ------------------------------------------------------------------------- */

static inline float leaky_relu_f(float x, float slope) /* ops.cuh:1-3 */
{
    return fmaxf(0.0f, x) + slope * fminf(0.0f, x);
}

/*
 * attn[i,h] = c_i / sum_{i' in row r, bid' = bid} c_i',
 * c_i = expf(leaky_relu(q[bid,r,h] + k[col,h], 0.2)); no max shift, float sums
 * in edge order, multiplication by the float reciprocal (sddmm_cuda.cu:10-31).
 * attn must be zero-filled by the caller (sddmm_cuda.cu:82).
 */
ORC_EXPORT void orc_sddmm_fwd(float *attn, const int32_t *indptr, const int32_t *indices,
                              const float *query, const float *key, int64_t n_dst,
                              int64_t n_heads)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_dst; r++) {
        for (int64_t h = 0; h < n_heads; h++) {
            float exp_sum[16] = {0.0f};
            for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
                int32_t bid = (int32_t)((uint32_t)indices[i] >> 24);
                int64_t c = indices[i] & COL_MASK;
                float x = query[(int64_t)bid * n_dst * n_heads + r * n_heads + h] +
                          key[c * n_heads + h];
                float coeff = expf(leaky_relu_f(x, 0.2f));
                attn[(int64_t)i * n_heads + h] = coeff;
                exp_sum[bid] += coeff;
            }
            for (int b = 0; b < 16; b++) exp_sum[b] = 1.0f / exp_sum[b];
            for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
                int32_t bid = (int32_t)((uint32_t)indices[i] >> 24);
                attn[(int64_t)i * n_heads + h] *= exp_sum[bid];
            }
        }
    }
}

/*
 * S_bid = -sum_j attn_j g_j ; gs_i = attn_i (S_bid + g_i);
 * gv = gs_i * (x < 0 ? 0.2 : 1); grad_q[bid,r,h] += gv; grad_k[col,h] += gv
 * (sddmm_cuda.cu:42-65, ops.cuh:5-10). Sums in double.
 */
ORC_EXPORT void orc_sddmm_bwd(float *grad_q, float *grad_k, const int32_t *indptr,
                              const int32_t *indices, const float *query, const float *key,
                              const float *attn, const float *grad_out, int64_t n_dst,
                              int64_t n_src, int64_t n_heads, int64_t n_bid)
{
    double *gq = (double *)calloc((size_t)(n_bid * n_dst * n_heads), sizeof(double));
    double *gk = (double *)calloc((size_t)(n_src * n_heads), sizeof(double));
    for (int64_t r = 0; r < n_dst; r++) {
        for (int64_t h = 0; h < n_heads; h++) {
            double cache[16] = {0.0};
            for (int32_t j = indptr[r]; j < indptr[r + 1]; j++) {
                int32_t bid = (int32_t)((uint32_t)indices[j] >> 24);
                cache[bid] -= (double)attn[(int64_t)j * n_heads + h] *
                              (double)grad_out[(int64_t)j * n_heads + h];
            }
            for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
                int32_t bid = (int32_t)((uint32_t)indices[i] >> 24);
                int64_t c = indices[i] & COL_MASK;
                double gs = (double)attn[(int64_t)i * n_heads + h] *
                            (cache[bid] + (double)grad_out[(int64_t)i * n_heads + h]);
                float x = query[(int64_t)bid * n_dst * n_heads + r * n_heads + h] +
                          key[c * n_heads + h];
                double gv = gs * (x < 0.0f ? 0.2 : 1.0);
                gq[(int64_t)bid * n_dst * n_heads + r * n_heads + h] += gv;
                gk[c * n_heads + h] += gv;
            }
        }
    }
    for (int64_t t = 0; t < n_bid * n_dst * n_heads; t++) grad_q[t] = (float)gq[t];
    for (int64_t t = 0; t < n_src * n_heads; t++) grad_k[t] = (float)gk[t];
    free(gq);
    free(gk);
}

/*
 * orc_sddmm_bwd in float on all cores, for timing only: a row-parallel pass writes the
 * per-edge logit gradient gv into edge_grad [nnz, H] (caller's scratch) and sums grad_q,
 * a source-parallel pass sums grad_k over the by-source view.
 */
ORC_EXPORT void orc_sddmm_bwd_omp(float *grad_q, float *grad_k, float *edge_grad,
                                  const int32_t *indptr, const int32_t *indices,
                                  const float *query, const float *key, const float *attn,
                                  const float *grad_out, const int32_t *t_indptr,
                                  const int32_t *t_perm, int64_t n_dst, int64_t n_src,
                                  int64_t n_heads, int64_t n_bid)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t r = 0; r < n_dst; r++) {
        for (int64_t h = 0; h < n_heads; h++) {
            float cache[16] = {0.0f}, gq[16] = {0.0f};
            for (int32_t j = indptr[r]; j < indptr[r + 1]; j++) {
                int32_t bid = (int32_t)((uint32_t)indices[j] >> 24);
                cache[bid] -= attn[(int64_t)j * n_heads + h] * grad_out[(int64_t)j * n_heads + h];
            }
            for (int32_t i = indptr[r]; i < indptr[r + 1]; i++) {
                int32_t bid = (int32_t)((uint32_t)indices[i] >> 24);
                int64_t c = indices[i] & COL_MASK;
                float gs = attn[(int64_t)i * n_heads + h] *
                           (cache[bid] + grad_out[(int64_t)i * n_heads + h]);
                float x = query[(int64_t)bid * n_dst * n_heads + r * n_heads + h] +
                          key[c * n_heads + h];
                float gv = gs * (x < 0.0f ? 0.2f : 1.0f);
                edge_grad[(int64_t)i * n_heads + h] = gv;
                gq[bid] += gv;
            }
            for (int64_t b = 0; b < n_bid; b++)
                grad_q[b * n_dst * n_heads + r * n_heads + h] = gq[b];
        }
    }
#pragma omp parallel for schedule(dynamic, 256)
    for (int64_t c = 0; c < n_src; c++)
        for (int64_t h = 0; h < n_heads; h++) {
            float acc = 0.0f;
            for (int32_t j = t_indptr[c]; j < t_indptr[c + 1]; j++)
                acc += edge_grad[(int64_t)t_perm[j] * n_heads + h];
            grad_k[c * n_heads + h] = acc;
        }
}

/* ------------------------------------------------------------------------- */
/* B10: stitch_csr. YiTu_GNN/YiTu_H/xgnn_h/block.py:36-67                      */
/* ------------------------------------------------------------------------- */

/*
 * Row-wise concatenation of n_blk CSR blocks with equal row counts: block b's
 * columns are shifted by the source-node counts of blocks 0..b-1 and tagged
 * (b << 24) + col  (block.py:46-55). Returns -1 if a shifted column exceeds
 * 2^24 (the reference asserts col <= 2**24, block.py:53) or n_blk > 16.
 */
ORC_EXPORT int orc_stitch_csr(int n_blk, int64_t n_rows, const int32_t *const *indptrs,
                              const int32_t *const *indicess, const int64_t *n_srcs,
                              int32_t *new_indptr, int32_t *new_indices)
{
    if (n_blk > 16) return -1;
    int64_t w = 0;
    for (int64_t r = 0; r < n_rows; r++) {
        int64_t cursor = 0;
        new_indptr[r] = (int32_t)w;
        for (int b = 0; b < n_blk; b++) {
            for (int32_t i = indptrs[b][r]; i < indptrs[b][r + 1]; i++) {
                int64_t c = cursor + indicess[b][i];
                if (c > (1 << 24)) return -1;
                new_indices[w++] = (int32_t)(((int64_t)b << 24) + c);
            }
            cursor += n_srcs[b];
        }
    }
    new_indptr[n_rows] = (int32_t)w;
    return 0;
}

/* ------------------------------------------------------------------------- */
/* B7/B8: two-way bundled GEMM. YiTu_GNN/YiTu_H/src/fc_cuda.cu                */
/* ------------------------------------------------------------------------- */

/*
 * c[n,m] (+)= op(a) . op(b) in float on all cores, for timing only (the reference calls
 * cuBLAS, fc_cuda.cu:61-69, 131, 178; torch::mm in YiTu_GNN_kernel.cu:276, 471-472).
 * Row-major operands; ta / tb say whether a is stored [k,n] / b is stored [m,k]. Rows of
 * c are dealt to the threads, the inner loops run over contiguous memory where the
 * layout allows it, so that the compiler vectorises them.
 */
ORC_EXPORT void orc_gemm_f32_omp(float *c, const float *a, const float *b, int64_t n, int64_t m,
                                 int64_t k, int ta, int tb)
{
    if (!ta) {
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n; i++) {
            float *ci = c + i * m;
            for (int64_t j = 0; j < m; j++) ci[j] = 0.0f;
            if (!tb) {
                for (int64_t t = 0; t < k; t++) {
                    const float av = a[i * k + t];
                    const float *bt = b + t * m;
                    for (int64_t j = 0; j < m; j++) ci[j] += av * bt[j];
                }
            } else {
                for (int64_t j = 0; j < m; j++) {
                    const float *bj = b + j * k;
                    float acc = 0.0f;
                    for (int64_t t = 0; t < k; t++) acc += a[i * k + t] * bj[t];
                    ci[j] = acc;
                }
            }
        }
        return;
    }
    /* a stored [k, n]: c = a^T . b, a sum over the k rows; threads own output rows in blocks
       and walk k together so that every row of a and b is streamed once per block */
#pragma omp parallel for schedule(static)
    for (int64_t i0 = 0; i0 < n; i0 += 8) {
        int64_t i1 = i0 + 8 < n ? i0 + 8 : n;
        for (int64_t i = i0; i < i1; i++)
            for (int64_t j = 0; j < m; j++) c[i * m + j] = 0.0f;
        for (int64_t t = 0; t < k; t++) {
            const float *bt = tb ? NULL : b + t * m;
            for (int64_t i = i0; i < i1; i++) {
                const float av = a[t * n + i];
                float *ci = c + i * m;
                if (bt)
                    for (int64_t j = 0; j < m; j++) ci[j] += av * bt[j];
                else
                    for (int64_t j = 0; j < m; j++) ci[j] += av * b[j * k + t];
            }
        }
    }
}

/* y[n,m] = x[n,k] . w[m,k]^T, double accumulate (fc_cuda.cu:61-69, batch member) */
ORC_EXPORT void orc_gemm_nt_f64(float *y, const float *x, const float *w, int64_t n, int64_t m,
                                int64_t k)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++)
        for (int64_t j = 0; j < m; j++) {
            double acc = 0.0;
            for (int64_t t = 0; t < k; t++) acc += (double)x[i * k + t] * (double)w[j * k + t];
            y[i * m + j] = (float)acc;
        }
}
