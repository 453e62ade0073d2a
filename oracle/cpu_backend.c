/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle (see cpu_backend.h for what this
 * restates and how it is pinned).  Build with -ffp-contract=off: Java never
 * fuses a multiply with an add.
 */
#include "cpu_backend.h"

#include <math.h>
#include <omp.h>
#include <string.h>
#include <unistd.h>

static int g_threads = 1;
static int g_colpar = 0;

int ref_default_threads(void) {
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    return n > 1 ? (int)(n - 1) : 1;       /* DeepJExecutor.java:22-24 */
}
void ref_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int  ref_get_threads(void) { return g_threads; }
void ref_set_column_parallel(int on) { g_colpar = on; }

/* DeepJExecutor.forRange: chunks = min(threads, n), chunk = ceil(n/chunks),
 * worker t takes rows [t*chunk, min(n, (t+1)*chunk)).  DeepJExecutor.java:93-98,125-131 */
#define FOR_RANGE(r, n, ...)                                                     \
    do {                                                                         \
        int n__ = (n);                                                           \
        if (n__ <= 0) break;                                                     \
        if (g_threads <= 1) {                                                    \
            for (int r = 0; r < n__; r++) { __VA_ARGS__; }                              \
        } else {                                                                 \
            int chunks__ = g_threads < n__ ? g_threads : n__;                    \
            int chunk__ = (n__ + chunks__ - 1) / chunks__;                       \
            _Pragma("omp parallel for schedule(static, 1) num_threads(chunks__)") \
            for (int t__ = 0; t__ < chunks__; t__++) {                           \
                int s__ = t__ * chunk__;                                         \
                int e__ = s__ + chunk__ < n__ ? s__ + chunk__ : n__;             \
                for (int r = s__; r < e__; r++) { __VA_ARGS__; }                        \
            }                                                                    \
        }                                                                        \
    } while (0)

/* CpuBackend.java:24-28 */
static inline float f_sqrt(float x) { return (float)sqrt((double)x); }
static inline float f_pow(float x, float e) { return (float)pow((double)x, (double)e); }
static inline float f_exp(float x) { return (float)exp((double)x); }
static inline float f_log(float x) { return (float)log((double)x); }
static inline float f_tanh(float x) { return (float)tanh((double)x); }

/* ── factories ──────────────────────────────────────────────────────── */

void ref_random(float *out, int64_t n, jrandom *rnd) {
    for (int64_t i = 0; i < n; i++) out[i] = (float)(jr_next_gaussian(rnd) * 0.1);
}

void ref_causal_mask(float *out, int size) {
    for (int r = 0; r < size; r++)
        for (int c = 0; c < size; c++) out[(int64_t)r * size + c] = (c > r) ? -1e9f : 0.0f;
}

/* ── matmul: ikj order, fp32 accumulate in the output row ───────────── */

void ref_matmul(const float *a, const float *b, float *out, int m, int n, int k) {
    memset(out, 0, (size_t)m * n * sizeof(float));
    if (g_colpar && g_threads > 1 && m < g_threads) {
        /* Same arithmetic per element (sequential k for every (r,c)); columns split
         * over workers instead of rows.  Bit-identical to the loop below. */
        int chunks = g_threads < n ? g_threads : n;
        int chunk = (n + chunks - 1) / chunks;
        #pragma omp parallel for schedule(static, 1) num_threads(chunks)
        for (int t = 0; t < chunks; t++) {
            int c0 = t * chunk, c1 = c0 + chunk < n ? c0 + chunk : n;
            for (int r = 0; r < m; r++) {
                const float *arow = a + (int64_t)r * k;
                float *orow = out + (int64_t)r * n;
                for (int kk = 0; kk < k; kk++) {
                    float av = arow[kk];
                    const float *brow = b + (int64_t)kk * n;
                    for (int c = c0; c < c1; c++) orow[c] += av * brow[c];
                }
            }
        }
        return;
    }
    FOR_RANGE(r, m, {
        const float *arow = a + (int64_t)r * k;
        float *orow = out + (int64_t)r * n;
        for (int kk = 0; kk < k; kk++) {
            float av = arow[kk];
            const float *brow = b + (int64_t)kk * n;
            for (int c = 0; c < n; c++) orow[c] += av * brow[c];
        }
    });
}

#define BINARY(NAME, EXPR)                                                           \
    void NAME(const float *a, const float *b, float *out, int rows, int cols) {      \
        FOR_RANGE(r, rows, {                                                         \
            int64_t base = (int64_t)r * cols;                                        \
            for (int c = 0; c < cols; c++) {                                         \
                float x = a[base + c], y = b[base + c]; out[base + c] = (EXPR);      \
            }                                                                        \
        });                                                                          \
    }
BINARY(ref_add, x + y)
BINARY(ref_subtract, x - y)
BINARY(ref_multiply, x * y)
BINARY(ref_divide, x / y)
BINARY(ref_relu_backward, x > 0.0f ? y : 0.0f)

#define ROW_BCAST(NAME, EXPR)                                                        \
    void NAME(const float *a, const float *rv, float *out, int rows, int cols) {     \
        FOR_RANGE(r, rows, {                                                         \
            int64_t base = (int64_t)r * cols;                                        \
            for (int c = 0; c < cols; c++) {                                         \
                float x = a[base + c], y = rv[c]; out[base + c] = (EXPR);            \
            }                                                                        \
        });                                                                          \
    }
ROW_BCAST(ref_add_row_vector, x + y)
ROW_BCAST(ref_multiply_broadcast_rows, x * y)

#define COL_BCAST(NAME, EXPR)                                                        \
    void NAME(const float *a, const float *cv, float *out, int rows, int cols) {     \
        FOR_RANGE(r, rows, {                                                         \
            int64_t base = (int64_t)r * cols;                                        \
            float y = cv[r];                                                         \
            for (int c = 0; c < cols; c++) { float x = a[base + c]; out[base + c] = (EXPR); } \
        });                                                                          \
    }
COL_BCAST(ref_add_broadcast_cols, x + y)
COL_BCAST(ref_subtract_broadcast_cols, x - y)
COL_BCAST(ref_multiply_broadcast_cols, x * y)
COL_BCAST(ref_divide_broadcast_cols, x / y)

#define SCALAR(NAME, EXPR)                                                           \
    void NAME(const float *a, float s, float *out, int rows, int cols) {             \
        FOR_RANGE(r, rows, {                                                         \
            int64_t base = (int64_t)r * cols;                                        \
            for (int c = 0; c < cols; c++) { float x = a[base + c]; out[base + c] = (EXPR); } \
        });                                                                          \
    }
SCALAR(ref_multiply_scalar, x * s)
SCALAR(ref_add_scalar, x + s)
SCALAR(ref_divide_scalar, x / s)
SCALAR(ref_pow, f_pow(x, s))

/* ── reductions ─────────────────────────────────────────────────────── */

static inline float row_sum(const float *d, int64_t base, int cols) {
    float s = 0.0f;
    for (int c = 0; c < cols; c++) s += d[base + c];
    return s;
}
static inline float row_max(const float *d, int64_t base, int cols) {
    float m = -INFINITY;
    for (int c = 0; c < cols; c++) if (d[base + c] > m) m = d[base + c];
    return m;
}

void ref_sum_rows(const float *a, float *out, int rows, int cols) {
    memset(out, 0, (size_t)cols * sizeof(float));
    for (int r = 0; r < rows; r++) {
        int64_t base = (int64_t)r * cols;
        for (int c = 0; c < cols; c++) out[c] += a[base + c];
    }
}

void ref_sum_along_rows(const float *a, float *out, int rows, int cols) {
    FOR_RANGE(r, rows, { out[r] = row_sum(a, (int64_t)r * cols, cols); });
}

void ref_mean_along_rows(const float *a, float *out, int rows, int cols) {
    float inv = 1.0f / cols;
    FOR_RANGE(r, rows, { out[r] = row_sum(a, (int64_t)r * cols, cols) * inv; });
}

void ref_variance_along_rows(const float *a, float *out, int rows, int cols) {
    float inv = 1.0f / cols;
    FOR_RANGE(r, rows, {
        int64_t base = (int64_t)r * cols;
        float mean = row_sum(a, base, cols) * inv;
        float acc = 0.0f;
        for (int c = 0; c < cols; c++) { float d = a[base + c] - mean; acc += d * d; }
        out[r] = acc * inv;
    });
}

void ref_max_along_rows(const float *a, float *out, int rows, int cols) {
    FOR_RANGE(r, rows, { out[r] = row_max(a, (int64_t)r * cols, cols); });
}

float ref_sum(const float *a, int64_t n) {
    float s = 0.0f;
    for (int64_t i = 0; i < n; i++) s += a[i];
    return s;
}

float ref_sum_abs(const float *a, int64_t n) {
    float s = 0.0f;
    for (int64_t i = 0; i < n; i++) s += fabsf(a[i]);
    return s;
}

/* ── unary ──────────────────────────────────────────────────────────── */

void ref_transpose(const float *a, float *out, int rows, int cols) {
    FOR_RANGE(r, rows, {
        int64_t base = (int64_t)r * cols;
        for (int c = 0; c < cols; c++) out[(int64_t)c * rows + r] = a[base + c];
    });
}

void ref_clamp(const float *a, float lo, float hi, float *out, int rows, int cols) {
    FOR_RANGE(r, rows, {
        int64_t base = (int64_t)r * cols;
        for (int c = 0; c < cols; c++) {
            float x = a[base + c];
            float mx = x > lo ? x : lo;        /* Math.max(min, x) */
            if (x != x) mx = x;                /* Math.max propagates NaN */
            float mn = mx < hi ? mx : hi;      /* Math.min(max, .) */
            if (mx != mx) mn = mx;
            out[base + c] = mn;
        }
    });
}

static inline float gelu_scalar(float x) {
    float c = f_sqrt(2.0f / (float)M_PI);
    float x3 = x * x * x;
    float t = c * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + f_tanh(t));
}
static inline float gelu_deriv_scalar(float x) {
    float c = f_sqrt(2.0f / (float)M_PI);
    float x2 = x * x;
    float x3 = x2 * x;
    float t = c * (x + 0.044715f * x3);
    float th = f_tanh(t);
    float sech2 = 1.0f - th * th;
    float dtdx = c * (1.0f + 3.0f * 0.044715f * x2);
    return 0.5f * (1.0f + th) + 0.5f * x * sech2 * dtdx;
}

#define UNARY(NAME, EXPR)                                                            \
    void NAME(const float *a, float *out, int rows, int cols) {                      \
        FOR_RANGE(r, rows, {                                                         \
            int64_t base = (int64_t)r * cols;                                        \
            for (int c = 0; c < cols; c++) { float x = a[base + c]; out[base + c] = (EXPR); } \
        });                                                                          \
    }
UNARY(ref_sqrt, f_sqrt(x))
UNARY(ref_neg, -x)
UNARY(ref_exp, f_exp(x))
UNARY(ref_log, f_log(x))
UNARY(ref_tanh, f_tanh(x))
UNARY(ref_sigmoid, 1.0f / (1.0f + f_exp(-x)))
UNARY(ref_relu, (x > 0.0f ? x : (x != x ? x : 0.0f)))   /* Math.max(0f, x) */
UNARY(ref_gelu, gelu_scalar(x))

void ref_gelu_backward(const float *x, const float *g, float *out, int rows, int cols) {
    FOR_RANGE(r, rows, {
        int64_t base = (int64_t)r * cols;
        for (int c = 0; c < cols; c++) out[base + c] = g[base + c] * gelu_deriv_scalar(x[base + c]);
    });
}

/* ── softmax / cross entropy ────────────────────────────────────────── */

static inline float row_sum_exp_shifted(const float *d, int64_t base, int cols, float mx) {
    float s = 0.0f;
    for (int c = 0; c < cols; c++) s += f_exp(d[base + c] - mx);
    return s;
}

/* rowWriteSoftmax, CpuBackend.java:392-397: exp written first, the sum is a
 * second evaluation of the same exps, then an in-place divide. */
static void row_write_softmax(const float *logits, float *out, int64_t base, int cols) {
    float mx = row_max(logits, base, cols);
    for (int c = 0; c < cols; c++) out[base + c] = f_exp(logits[base + c] - mx);
    float se = row_sum_exp_shifted(logits, base, cols, mx);
    for (int c = 0; c < cols; c++) out[base + c] /= se;
}

void ref_softmax_rows(const float *logits, float *out, int rows, int cols) {
    FOR_RANGE(r, rows, { row_write_softmax(logits, out, (int64_t)r * cols, cols); });
}

void ref_softmax_backward(const float *g, const float *s, float *out, int rows, int cols) {
    FOR_RANGE(r, rows, {
        int64_t base = (int64_t)r * cols;
        float dot = 0.0f;
        for (int c = 0; c < cols; c++) dot += g[base + c] * s[base + c];
        for (int c = 0; c < cols; c++) out[base + c] = s[base + c] * (g[base + c] - dot);
    });
}

float ref_cross_entropy_loss(const float *logits, const int32_t *targets, int rows, int cols) {
    float loss = 0.0f;
    for (int i = 0; i < rows; i++) {
        int64_t base = (int64_t)i * cols;
        float mx = row_max(logits, base, cols);
        float se = row_sum_exp_shifted(logits, base, cols, mx);
        loss += f_log(se) + mx - logits[base + targets[i]];
    }
    return loss / rows;
}

void ref_cross_entropy_gradient(const float *logits, const int32_t *targets, float *out, int rows, int cols) {
    for (int i = 0; i < rows; i++) {
        int64_t base = (int64_t)i * cols;
        row_write_softmax(logits, out, base, cols);
        out[base + targets[i]] -= 1.0f;
    }
    float s = (float)rows;                     /* divideScalarInPlace(grad, logits.rows) */
    for (int64_t i = 0; i < (int64_t)rows * cols; i++) out[i] = out[i] / s;
}

/* ── fused training ops ─────────────────────────────────────────────── */

void ref_adamw_update(float *w, const float *g, float *mt, float *vt, int64_t n,
                      float lr, float beta1, float beta2, float eps,
                      float weight_decay, float bc1, float bc2) {
    for (int64_t i = 0; i < n; i++) {
        float grad = g[i];
        float m_new = beta1 * mt[i] + (1.0f - beta1) * grad;
        float v_new = beta2 * vt[i] + (1.0f - beta2) * (grad * grad);
        mt[i] = m_new;
        vt[i] = v_new;
        float m_hat = m_new / bc1;
        float v_hat = v_new / bc2;
        float update = (lr * m_hat) / (f_sqrt(v_hat) + eps);
        if (weight_decay != 0.0f) update += lr * weight_decay * w[i];
        w[i] -= update;
    }
}

void ref_layer_norm_backward(const float *dxhat, const float *xhat, const float *std,
                             float *out, int rows, int dim) {
    FOR_RANGE(r, rows, {
        int64_t base = (int64_t)r * dim;
        float inv_std = 1.0f / std[r];
        float sum_d = 0.0f;
        float sum_dx = 0.0f;
        for (int c = 0; c < dim; c++) {
            float d = dxhat[base + c];
            sum_d += d;
            sum_dx += d * xhat[base + c];
        }
        for (int c = 0; c < dim; c++) {
            float d = dxhat[base + c];
            float xh = xhat[base + c];
            out[base + c] = inv_std * (d - sum_d / dim - xh * (sum_dx / dim));
        }
    });
}

void ref_scatter_add_rows(float *target, const int32_t *indices, int n_idx,
                          const float *grad, int cols) {
    for (int i = 0; i < n_idx; i++) {
        int64_t tb = (int64_t)indices[i] * cols;
        int64_t gb = (int64_t)i * cols;
        for (int c = 0; c < cols; c++) target[tb + c] += grad[gb + c];
    }
}

void ref_slice_rows(const float *t, const int32_t *idx, int n_idx, int cols, float *out) {
    for (int i = 0; i < n_idx; i++)
        memcpy(out + (int64_t)i * cols, t + (int64_t)idx[i] * cols, (size_t)cols * sizeof(float));
}
