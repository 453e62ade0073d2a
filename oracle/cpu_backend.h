/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle for the DeepJ HIP backend.
 * Nothing in the shipped library links or loads this code.
 *
 * Plain-C restatement of the reference's eager CPU backend
 *   src/main/java/io/github/kirstenali/deepj/tensor/cpu/CpuBackend.java
 * on flat row-major fp32 arrays (element (r,c) at data[r*cols+c], as in
 * src/main/java/io/github/kirstenali/deepj/tensor/Tensor.java:9-11).
 * Loop order, accumulation type and the "f64 transcendental, then cast to
 * fp32" convention (CpuBackend.java:24-28) are kept; Java's Math.exp/log/
 * tanh/pow are evaluated with the C library's double routines, which may
 * differ from a JVM in the last f64 bit (parity unpinned for that bit only).
 *
 * Row loops run like DeepJExecutor.forRange
 *   src/main/java/io/github/kirstenali/deepj/concurrent/DeepJExecutor.java:80-148
 * (contiguous chunks of ceil(n/chunks) rows on min(threads,n) workers); the
 * worker count is set with ref_set_threads and never changes results.
 */
#ifndef DEEPJ_ORACLE_CPU_BACKEND_H
#define DEEPJ_ORACLE_CPU_BACKEND_H

#include <stdint.h>
#include "jrandom.h"

#ifdef __cplusplus
extern "C" {
#endif

void ref_set_threads(int n);          /* DeepJExecutor.setNumThreads */
int  ref_get_threads(void);
int  ref_default_threads(void);       /* availableProcessors() - 1, at least 1 */
/* When non-zero, matmul with few rows splits its COLUMNS over the workers.
 * Each output element is still the same sequential k-sum, so results are
 * bit-identical; only used to generate fixtures faster, never for timing. */
void ref_set_column_parallel(int on);

/* factories (CpuBackend.java:138-161) */
void ref_random(float *out, int64_t n, jrandom *rnd);           /* (float)(g*0.1) */
void ref_causal_mask(float *out, int size);

/* core binary (CpuBackend.java:168-193) */
void ref_matmul(const float *a, const float *b, float *out, int m, int n, int k);
void ref_add(const float *a, const float *b, float *out, int rows, int cols);
void ref_subtract(const float *a, const float *b, float *out, int rows, int cols);
void ref_multiply(const float *a, const float *b, float *out, int rows, int cols);
void ref_divide(const float *a, const float *b, float *out, int rows, int cols);

/* broadcasts (CpuBackend.java:199-206) */
void ref_add_row_vector(const float *a, const float *rv, float *out, int rows, int cols);
void ref_multiply_broadcast_rows(const float *a, const float *rv, float *out, int rows, int cols);
void ref_add_broadcast_cols(const float *a, const float *cv, float *out, int rows, int cols);
void ref_subtract_broadcast_cols(const float *a, const float *cv, float *out, int rows, int cols);
void ref_multiply_broadcast_cols(const float *a, const float *cv, float *out, int rows, int cols);
void ref_divide_broadcast_cols(const float *a, const float *cv, float *out, int rows, int cols);

/* scalar (CpuBackend.java:212-214) */
void ref_multiply_scalar(const float *a, float s, float *out, int rows, int cols);
void ref_add_scalar(const float *a, float s, float *out, int rows, int cols);
void ref_divide_scalar(const float *a, float s, float *out, int rows, int cols);

/* reductions (CpuBackend.java:220-294) */
void  ref_sum_rows(const float *a, float *out, int rows, int cols);          /* -> [1 x cols] */
void  ref_sum_along_rows(const float *a, float *out, int rows, int cols);    /* -> [rows x 1] */
void  ref_mean_along_rows(const float *a, float *out, int rows, int cols);
void  ref_variance_along_rows(const float *a, float *out, int rows, int cols);
void  ref_max_along_rows(const float *a, float *out, int rows, int cols);
float ref_sum(const float *a, int64_t n);
float ref_sum_abs(const float *a, int64_t n);

/* unary (CpuBackend.java:300-324) */
void ref_transpose(const float *a, float *out, int rows, int cols);
void ref_clamp(const float *a, float lo, float hi, float *out, int rows, int cols);
void ref_sqrt(const float *a, float *out, int rows, int cols);
void ref_pow(const float *a, float e, float *out, int rows, int cols);
void ref_neg(const float *a, float *out, int rows, int cols);
void ref_exp(const float *a, float *out, int rows, int cols);
void ref_log(const float *a, float *out, int rows, int cols);
void ref_tanh(const float *a, float *out, int rows, int cols);
void ref_sigmoid(const float *a, float *out, int rows, int cols);
void ref_relu(const float *a, float *out, int rows, int cols);
void ref_gelu(const float *a, float *out, int rows, int cols);
void ref_relu_backward(const float *x, const float *g, float *out, int rows, int cols);
void ref_gelu_backward(const float *x, const float *g, float *out, int rows, int cols);

/* softmax / cross entropy (CpuBackend.java:360-464) */
void  ref_softmax_rows(const float *logits, float *out, int rows, int cols);
void  ref_softmax_backward(const float *g, const float *s, float *out, int rows, int cols);
float ref_cross_entropy_loss(const float *logits, const int32_t *targets, int rows, int cols);
void  ref_cross_entropy_gradient(const float *logits, const int32_t *targets, float *out, int rows, int cols);

/* fused training ops (CpuBackend.java:466-516, 542-549) */
void ref_adamw_update(float *w, const float *g, float *mt, float *vt, int64_t n,
                      float lr, float beta1, float beta2, float eps,
                      float weight_decay, float bc1, float bc2);
void ref_layer_norm_backward(const float *dxhat, const float *xhat, const float *std,
                             float *out, int rows, int dim);
void ref_scatter_add_rows(float *target, const int32_t *indices, int n_idx,
                          const float *grad, int cols);
void ref_slice_rows(const float *t, const int32_t *idx, int n_idx, int cols, float *out);

#ifdef __cplusplus
}
#endif
#endif
