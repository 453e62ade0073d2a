/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle (see model_ref.h for the reference
 * files each function restates).  Build with -ffp-contract=off.
 */
#include "model_ref.h"

#include <math.h>
#include <omp.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static float *falloc(int64_t n) {
    float *p = (float *)calloc((size_t)(n > 0 ? n : 1), sizeof(float));
    if (!p) { fprintf(stderr, "oracle: out of memory (%lld floats)\n", (long long)n); abort(); }
    return p;
}

/* ── layers ─────────────────────────────────────────────────────────── */

/* Linear.java:31-36: x.matmul(W).addRowVector(b) */
void ref_linear(const float *x, const float *w, const float *b, float *out, int rows, int d_in, int d_out) {
    float *y = falloc((int64_t)rows * d_out);
    ref_matmul(x, w, y, rows, d_out, d_in);
    ref_add_row_vector(y, b, out, rows, d_out);
    free(y);
}

/* RMSNorm1D.java:46-57: six backend ops in this order. */
void ref_rmsnorm(const float *x, const float *gamma, float *out, int rows, int dim) {
    int64_t n = (int64_t)rows * dim;
    float *sq = falloc(n), *mean = falloc(rows), *rms = falloc(rows), *xhat = falloc(n);
    ref_multiply(x, x, sq, rows, dim);
    ref_mean_along_rows(sq, mean, rows, dim);
    ref_add_scalar(mean, REF_RMS_EPS, rms, rows, 1);
    ref_sqrt(rms, rms, rows, 1);
    ref_divide_broadcast_cols(x, rms, xhat, rows, dim);
    ref_multiply_broadcast_rows(xhat, gamma, out, rows, dim);
    free(sq); free(mean); free(rms); free(xhat);
}

/* LayerNorm1D.java:34-66: mean = meanAlongRows, var = varianceAlongRows (population), std = sqrt(var + EPS),
 * xHat = (x - mean) / std, out = xHat * gamma + beta; EPS = 1e-5f (LayerNorm1D.java:15). */
void ref_layernorm(const float *x, const float *gamma, const float *beta, float *out, int rows, int dim) {
    int64_t n = (int64_t)rows * dim;
    float *mean = falloc(rows), *var = falloc(rows), *std = falloc(rows), *c = falloc(n), *xhat = falloc(n), *sc = falloc(n);
    ref_mean_along_rows(x, mean, rows, dim);
    ref_variance_along_rows(x, var, rows, dim);
    ref_add_scalar(var, 1e-5f, std, rows, 1);
    ref_sqrt(std, std, rows, 1);
    ref_subtract_broadcast_cols(x, mean, c, rows, dim);
    ref_divide_broadcast_cols(c, std, xhat, rows, dim);
    ref_multiply_broadcast_rows(xhat, gamma, sc, rows, dim);
    ref_add_row_vector(sc, beta, out, rows, dim);
    free(mean); free(var); free(std); free(c); free(xhat); free(sc);
}

/* FNN.java:57-73 with one hidden layer and GELU: Linear -> GELU -> Linear */
static void gpt_fnn(const float *x, const float *w1, const float *b1, const float *w2, const float *b2,
                    float *out, int rows, int d, int dff) {
    float *z = falloc((int64_t)rows * dff), *hh = falloc((int64_t)rows * dff);
    ref_linear(x, w1, b1, z, rows, d, dff);
    ref_gelu(z, hh, rows, dff);
    ref_linear(hh, w2, b2, out, rows, dff, d);
    free(z); free(hh);
}

/* SiLU.java:20-24: input.multiply(input.sigmoidActivation()) */
void ref_silu(const float *x, float *out, int rows, int cols) {
    float *s = falloc((int64_t)rows * cols);
    ref_sigmoid(x, s, rows, cols);
    ref_multiply(x, s, out, rows, cols);
    free(s);
}

/* SwiGLULayer.java:63-70 */
void ref_swiglu(const float *x, const float *wg, const float *bg, const float *wu, const float *bu,
                const float *wd, const float *bd, float *out, int rows, int d, int dff) {
    int64_t n = (int64_t)rows * dff;
    float *gate = falloc(n), *up = falloc(n), *sg = falloc(n), *fused = falloc(n);
    ref_linear(x, wg, bg, gate, rows, d, dff);
    ref_linear(x, wu, bu, up, rows, d, dff);
    ref_silu(gate, sg, rows, dff);
    ref_multiply(sg, up, fused, rows, dff);
    ref_linear(fused, wd, bd, out, rows, dff, d);
    free(gate); free(up); free(sg); free(fused);
}

/* RotaryEmbedding.java:63-70 */
void ref_rope_tables(int head_dim, int max_seq, float *cos_t, float *sin_t) {
    int half = head_dim / 2;
    for (int pos = 0; pos < max_seq; pos++) {
        for (int i = 0; i < half; i++) {
            float expo = (2.0f * (float)i) / (float)head_dim;
            float theta = (float)((double)pos / pow((double)10000.0f, (double)expo));
            cos_t[(int64_t)pos * half + i] = (float)cos((double)theta);
            sin_t[(int64_t)pos * half + i] = (float)sin((double)theta);
        }
    }
}

/* RotaryEmbedding.java:81-89,112-122 */
void ref_rope_apply(const float *t, float *out, int seq, int n_heads, int head_dim,
                    const float *cos_t, const float *sin_t, int pos0) {
    int half = head_dim / 2;
    for (int h = 0; h < n_heads; h++) {
        for (int p = 0; p < seq; p++) {
            int64_t base = ((int64_t)h * seq + p) * head_dim;
            const float *ct = cos_t + (int64_t)(pos0 + p) * half;
            const float *st = sin_t + (int64_t)(pos0 + p) * half;
            for (int i = 0; i < half; i++) {
                float c = ct[i], s = st[i];
                float x0 = t[base + 2 * i], x1 = t[base + 2 * i + 1];
                out[base + 2 * i]     = x0 * c - x1 * s;
                out[base + 2 * i + 1] = x0 * s + x1 * c;
            }
        }
    }
}

/* HeadOps.java:33-46 */
void ref_split_heads(const float *t, float *out, int seq, int n_heads, int head_dim) {
    int d = n_heads * head_dim;
    for (int i = 0; i < seq; i++)
        for (int h = 0; h < n_heads; h++)
            memcpy(out + ((int64_t)h * seq + i) * head_dim, t + (int64_t)i * d + h * head_dim,
                   (size_t)head_dim * sizeof(float));
}

/* HeadOps.java:52-64 */
void ref_merge_heads(const float *t, float *out, int seq, int n_heads, int head_dim) {
    int d = n_heads * head_dim;
    for (int i = 0; i < seq; i++)
        for (int h = 0; h < n_heads; h++)
            memcpy(out + (int64_t)i * d + h * head_dim, t + ((int64_t)h * seq + i) * head_dim,
                   (size_t)head_dim * sizeof(float));
}

/* HeadOps.java:90-140 with Softmax.java:16-19 between mask and values:
 * per head s = (q . k^T) * scale; s + mask; softmax over [H*S x S]; y = p . v */
void ref_attention_heads(const float *qh, const float *kh, const float *vh, float *outh,
                         int seq, int n_heads, int head_dim, int causal) {
    float scale = (float)(1.0 / sqrt((double)head_dim));   /* MultiHeadSelfAttention.java:45 */
    int64_t ss = (int64_t)seq * seq;
    float *scores = falloc((int64_t)n_heads * ss);
    float *kt = falloc((int64_t)head_dim * seq);
    float *mask = NULL;
    if (causal) { mask = falloc(ss); ref_causal_mask(mask, seq); }
    for (int h = 0; h < n_heads; h++) {
        const float *q = qh + (int64_t)h * seq * head_dim;
        const float *k = kh + (int64_t)h * seq * head_dim;
        float *s = scores + (int64_t)h * ss;
        ref_transpose(k, kt, seq, head_dim);
        ref_matmul(q, kt, s, seq, seq, head_dim);
        ref_multiply_scalar(s, scale, s, seq, seq);
        if (causal) ref_add(s, mask, s, seq, seq);
    }
    float *prob = falloc((int64_t)n_heads * ss);
    ref_softmax_rows(scores, prob, n_heads * seq, seq);
    for (int h = 0; h < n_heads; h++)
        ref_matmul(prob + (int64_t)h * ss, vh + (int64_t)h * seq * head_dim,
                   outh + (int64_t)h * seq * head_dim, seq, head_dim, seq);
    free(scores); free(kt); free(prob); free(mask);
}

static void attention_from_qkv(const float *q, const float *k, const float *v, float *merged,
                               int seq, int d, int n_heads,
                               const float *cos_t, const float *sin_t, int causal) {
    int hd = d / n_heads;
    int64_t n = (int64_t)seq * d;
    float *qh = falloc(n), *kh = falloc(n), *vh = falloc(n), *oh = falloc(n);
    ref_split_heads(q, qh, seq, n_heads, hd);
    ref_split_heads(k, kh, seq, n_heads, hd);
    ref_split_heads(v, vh, seq, n_heads, hd);
    if (cos_t) {
        float *qr = falloc(n), *kr = falloc(n);
        ref_rope_apply(qh, qr, seq, n_heads, hd, cos_t, sin_t, 0);
        ref_rope_apply(kh, kr, seq, n_heads, hd, cos_t, sin_t, 0);
        free(qh); free(kh); qh = qr; kh = kr;
    }
    ref_attention_heads(qh, kh, vh, oh, seq, n_heads, hd, causal);
    ref_merge_heads(oh, merged, seq, n_heads, hd);
    free(qh); free(kh); free(vh); free(oh);
}

/* MultiHeadSelfAttention.java:60-86 */
void ref_mhsa_forward(const float *x, const float *wq, const float *wk, const float *wv, const float *wo,
                      float *out, int seq, int d, int n_heads,
                      const float *cos_t, const float *sin_t, int causal) {
    int64_t n = (int64_t)seq * d;
    float *q = falloc(n), *k = falloc(n), *v = falloc(n), *merged = falloc(n);
    ref_matmul(x, wq, q, seq, d, d);
    ref_matmul(x, wk, k, seq, d, d);
    ref_matmul(x, wv, v, seq, d, d);
    attention_from_qkv(q, k, v, merged, seq, d, n_heads, cos_t, sin_t, causal);
    ref_matmul(merged, wo, out, seq, d, d);
    free(q); free(k); free(v); free(merged);
}

/* MultiHeadLatentAttention.java:92-123 */
void ref_mla_forward(const float *x, const float *wdq, const float *wuq, const float *wdkv,
                     const float *wuk, const float *wuv, const float *wo, float *out,
                     int seq, int d, int n_heads, int q_rank, int kv_rank,
                     const float *cos_t, const float *sin_t) {
    int64_t n = (int64_t)seq * d;
    float *cq = falloc((int64_t)seq * q_rank), *ckv = falloc((int64_t)seq * kv_rank);
    float *q = falloc(n), *k = falloc(n), *v = falloc(n), *merged = falloc(n);
    ref_matmul(x, wdq, cq, seq, q_rank, d);
    ref_matmul(cq, wuq, q, seq, d, q_rank);
    ref_matmul(x, wdkv, ckv, seq, kv_rank, d);
    ref_matmul(ckv, wuk, k, seq, d, kv_rank);
    ref_matmul(ckv, wuv, v, seq, d, kv_rank);
    attention_from_qkv(q, k, v, merged, seq, d, n_heads, cos_t, sin_t, 1);
    ref_matmul(merged, wo, out, seq, d, d);
    free(cq); free(ckv); free(q); free(k); free(v); free(merged);
}

/* ── Q8 ─────────────────────────────────────────────────────────────── */

int ref_q8_padded_k(int k) { return (k + REF_Q8_GROUP - 1) / REF_Q8_GROUP * REF_Q8_GROUP; }

void ref_q8_quantize(const float *w, int k, int n, int8_t *q, float *scales) {
    int kp = ref_q8_padded_k(k);
    int groups = kp / REF_Q8_GROUP;
    #pragma omp parallel for schedule(static)
    for (int col = 0; col < n; col++) {
        for (int g = 0; g < groups; g++) {
            int k0 = g * REF_Q8_GROUP;
            int k1 = k0 + REF_Q8_GROUP < k ? k0 + REF_Q8_GROUP : k;
            float amax = 0.0f;
            for (int kk = k0; kk < k1; kk++) {
                float a = fabsf(w[(int64_t)kk * n + col]);
                if (a > amax) amax = a;
            }
            float scale = amax / 127.0f;
            scales[(int64_t)col * groups + g] = scale;
            for (int kk = k0; kk < k0 + REF_Q8_GROUP; kk++) {
                int8_t v = 0;
                if (kk < k && scale != 0.0f) {
                    float r = rintf(w[(int64_t)kk * n + col] / scale);   /* round half to even */
                    if (r > 127.0f) r = 127.0f;
                    if (r < -127.0f) r = -127.0f;
                    v = (int8_t)r;
                }
                q[(int64_t)col * kp + kk] = v;
            }
        }
    }
}

void ref_q8_dequantize(const int8_t *q, const float *scales, int k, int n, float *w_out) {
    int kp = ref_q8_padded_k(k);
    int groups = kp / REF_Q8_GROUP;
    #pragma omp parallel for schedule(static)
    for (int col = 0; col < n; col++)
        for (int kk = 0; kk < k; kk++)
            w_out[(int64_t)kk * n + col] =
                (float)q[(int64_t)col * kp + kk] * scales[(int64_t)col * groups + kk / REF_Q8_GROUP];
}

static void q8_roundtrip(float *w, int k, int n) {
    int kp = ref_q8_padded_k(k);
    int8_t *q = (int8_t *)malloc((size_t)n * kp);
    float *s = falloc((int64_t)n * (kp / REF_Q8_GROUP));
    ref_q8_quantize(w, k, n, q, s);
    ref_q8_dequantize(q, s, k, n, w);
    free(q); free(s);
}

/* ── models ─────────────────────────────────────────────────────────── */

/* Timing-only switch: fill weights with a cheap counter hash (uniform, variance of N(0,1)*0.1)
 * instead of the java.util.Random Gaussian stream, which is sequential and takes minutes for a
 * full-size model.  Such a model has the memory footprint and arithmetic of the real one but NOT
 * its values: it is for measuring the CPU path's speed only, never for parity. */
static int g_fast_fill = 0;
void ref_set_fast_fill(int on) { g_fast_fill = on; }

static float *rand_tensor(int rows, int cols, jrandom *r) {
    int64_t n = (int64_t)rows * cols;
    float *t = falloc(n);
    if (g_fast_fill) {
        uint64_t salt = (uint64_t)jr_next_int(r);
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < n; i++) {
            uint64_t z = (uint64_t)i * 0x9E3779B97F4A7C15ull + salt;
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
            z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
            z ^= z >> 31;
            t[i] = ((float)(z >> 40) * (1.0f / 16777216.0f) - 0.5f) * 0.34641016f;   /* sqrt(12) * 0.1 */
        }
        return t;
    }
    ref_random(t, n, r);
    return t;
}
static float *ones(int n) {
    float *t = falloc(n);
    for (int i = 0; i < n; i++) t[i] = 1.0f;
    return t;
}

ref_model *ref_model_create(const ref_config *cfg, int64_t seed) {
    ref_model *m = (ref_model *)calloc(1, sizeof(ref_model));
    m->cfg = *cfg;
    int d = cfg->d, dff = cfg->dff, hd = d / cfg->heads;
    jrandom emb_r, stack_r, head_r;
    jr_init(&emb_r, seed);          /* LlamaModel.java:29 / DeepSeekModel.java:31 */
    jr_init(&stack_r, seed);        /* builder .seed(seed): its own Random(seed) */
    jr_init(&head_r, seed + 1);     /* LlamaModel.java:39 */
    m->emb = rand_tensor(cfg->vocab, d, &emb_r);
    m->layer = (ref_layer *)calloc((size_t)cfg->layers, sizeof(ref_layer));
    for (int l = 0; l < cfg->layers; l++) {
        ref_layer *L = &m->layer[l];
        L->g1 = ones(d); L->g2 = ones(d);
        if (cfg->kind == 2) {       /* GPTTransformerBlock.java:45-50: ln1, ln2, attention, then the FNN's two Linears */
            L->be1 = falloc(d); L->be2 = falloc(d);
            L->wq = rand_tensor(d, d, &stack_r);
            L->wk = rand_tensor(d, d, &stack_r);
            L->wv = rand_tensor(d, d, &stack_r);
            L->wo = rand_tensor(d, d, &stack_r);
            L->wg = rand_tensor(d, dff, &stack_r);  L->bg = falloc(dff);
            L->wd = rand_tensor(dff, d, &stack_r);  L->bd = falloc(d);
            continue;
        }
        if (cfg->kind == 0) {       /* MultiHeadSelfAttention.java:47-50 */
            L->wq = rand_tensor(d, d, &stack_r);
            L->wk = rand_tensor(d, d, &stack_r);
            L->wv = rand_tensor(d, d, &stack_r);
            L->wo = rand_tensor(d, d, &stack_r);
        } else {                    /* MultiHeadLatentAttention.java:81-86 */
            L->wdq  = rand_tensor(d, cfg->q_rank, &stack_r);
            L->wuq  = rand_tensor(cfg->q_rank, d, &stack_r);
            L->wdkv = rand_tensor(d, cfg->kv_rank, &stack_r);
            L->wuk  = rand_tensor(cfg->kv_rank, d, &stack_r);
            L->wuv  = rand_tensor(cfg->kv_rank, d, &stack_r);
            L->wo   = rand_tensor(d, d, &stack_r);
        }
        /* SwiGLULayer.java:56-58, Linear.java:26-27 (bias zeros, no RNG draw) */
        L->wg = rand_tensor(d, dff, &stack_r);  L->bg = falloc(dff);
        L->wu = rand_tensor(d, dff, &stack_r);  L->bu = falloc(dff);
        L->wd = rand_tensor(dff, d, &stack_r);  L->bd = falloc(d);
    }
    m->gf = ones(d);
    m->wlm = rand_tensor(d, cfg->vocab, &head_r);
    m->blm = falloc(cfg->vocab);
    m->cos_t = falloc((int64_t)cfg->max_seq * (hd / 2));
    m->sin_t = falloc((int64_t)cfg->max_seq * (hd / 2));
    ref_rope_tables(hd, cfg->max_seq, m->cos_t, m->sin_t);
    if (cfg->kind == 2) {
        /* GPTModel.java:27-45: final LayerNorm, positional table from Random(seed + 2); no rotary embedding:
         * the incremental path keeps its rotation code and gets the identity (cos 1, sin 0: x*1 - y*0 == x). */
        jrandom pos_r; jr_init(&pos_r, seed + 2);
        m->bf = falloc(d);
        m->pos = rand_tensor(cfg->max_seq, d, &pos_r);
        for (int64_t i = 0; i < (int64_t)cfg->max_seq * (hd / 2); i++) { m->cos_t[i] = 1.0f; m->sin_t[i] = 0.0f; }
        float f = cfg->init_scale;
        if (f != 1.0f) {            /* applyInitScale: every parameter, gains and biases included */
            #define SCALE(p, n) do { for (int64_t i_ = 0; i_ < (int64_t)(n); i_++) (p)[i_] *= f; } while (0)
            SCALE(m->emb, (int64_t)cfg->vocab * d); SCALE(m->pos, (int64_t)cfg->max_seq * d);
            for (int l = 0; l < cfg->layers; l++) {
                ref_layer *L = &m->layer[l];
                SCALE(L->g1, d); SCALE(L->be1, d); SCALE(L->g2, d); SCALE(L->be2, d);
                SCALE(L->wq, (int64_t)d * d); SCALE(L->wk, (int64_t)d * d); SCALE(L->wv, (int64_t)d * d); SCALE(L->wo, (int64_t)d * d);
                SCALE(L->wg, (int64_t)d * dff); SCALE(L->bg, dff); SCALE(L->wd, (int64_t)dff * d); SCALE(L->bd, d);
            }
            SCALE(m->gf, d); SCALE(m->bf, d); SCALE(m->wlm, (int64_t)d * cfg->vocab); SCALE(m->blm, cfg->vocab);
            #undef SCALE
        }
    }
    return m;
}

void ref_model_free(ref_model *m) {
    if (!m) return;
    for (int l = 0; l < m->cfg.layers; l++) {
        ref_layer *L = &m->layer[l];
        free(L->g1); free(L->g2); free(L->wq); free(L->wk); free(L->wv); free(L->wo);
        free(L->wdq); free(L->wuq); free(L->wdkv); free(L->wuk); free(L->wuv);
        free(L->wg); free(L->bg); free(L->wu); free(L->bu); free(L->wd); free(L->bd);
        free(L->be1); free(L->be2);
    }
    free(m->bf); free(m->pos);
    free(m->layer); free(m->emb); free(m->gf); free(m->wlm); free(m->blm);
    free(m->cos_t); free(m->sin_t); free(m->kcache); free(m->vcache);
    free(m);
}

void ref_model_q8_roundtrip(ref_model *m) {
    const ref_config *c = &m->cfg;
    for (int l = 0; l < c->layers; l++) {
        ref_layer *L = &m->layer[l];
        if (c->kind == 2) {
            q8_roundtrip(L->wq, c->d, c->d); q8_roundtrip(L->wk, c->d, c->d);
            q8_roundtrip(L->wv, c->d, c->d); q8_roundtrip(L->wo, c->d, c->d);
            q8_roundtrip(L->wg, c->d, c->dff); q8_roundtrip(L->wd, c->dff, c->d);
            continue;
        }
        if (c->kind == 0) {
            q8_roundtrip(L->wq, c->d, c->d); q8_roundtrip(L->wk, c->d, c->d);
            q8_roundtrip(L->wv, c->d, c->d);
        } else {
            q8_roundtrip(L->wdq, c->d, c->q_rank);  q8_roundtrip(L->wuq, c->q_rank, c->d);
            q8_roundtrip(L->wdkv, c->d, c->kv_rank);
            q8_roundtrip(L->wuk, c->kv_rank, c->d); q8_roundtrip(L->wuv, c->kv_rank, c->d);
        }
        q8_roundtrip(L->wo, c->d, c->d);
        q8_roundtrip(L->wg, c->d, c->dff); q8_roundtrip(L->wu, c->d, c->dff);
        q8_roundtrip(L->wd, c->dff, c->d);
    }
    q8_roundtrip(m->wlm, c->d, c->vocab);
}

float *ref_model_weight(ref_model *m, const char *name, int *rows, int *cols) {
    const ref_config *c = &m->cfg;
    int r = 0, k = 0; float *p = NULL;
    if (!strcmp(name, "emb")) { p = m->emb; r = c->vocab; k = c->d; }
    else if (!strcmp(name, "gf")) { p = m->gf; r = 1; k = c->d; }
    else if (!strcmp(name, "bf") && m->bf) { p = m->bf; r = 1; k = c->d; }
    else if (!strcmp(name, "pos") && m->pos) { p = m->pos; r = c->max_seq; k = c->d; }
    else if (!strcmp(name, "wlm")) { p = m->wlm; r = c->d; k = c->vocab; }
    else if (!strcmp(name, "blm")) { p = m->blm; r = 1; k = c->vocab; }
    else if (name[0] == 'L') {
        int l = atoi(name + 1);
        const char *dot = strchr(name, '.');
        if (!dot || l < 0 || l >= c->layers) return NULL;
        const char *w = dot + 1;
        ref_layer *L = &m->layer[l];
        if (!strcmp(w, "be1")) { p = L->be1; r = 1; k = c->d; }
        else if (!strcmp(w, "be2")) { p = L->be2; r = 1; k = c->d; }
        else if (!strcmp(w, "g1")) { p = L->g1; r = 1; k = c->d; }
        else if (!strcmp(w, "g2")) { p = L->g2; r = 1; k = c->d; }
        else if (!strcmp(w, "wq")) { p = L->wq; r = c->d; k = c->d; }
        else if (!strcmp(w, "wk")) { p = L->wk; r = c->d; k = c->d; }
        else if (!strcmp(w, "wv")) { p = L->wv; r = c->d; k = c->d; }
        else if (!strcmp(w, "wo")) { p = L->wo; r = c->d; k = c->d; }
        else if (!strcmp(w, "wdq")) { p = L->wdq; r = c->d; k = c->q_rank; }
        else if (!strcmp(w, "wuq")) { p = L->wuq; r = c->q_rank; k = c->d; }
        else if (!strcmp(w, "wdkv")) { p = L->wdkv; r = c->d; k = c->kv_rank; }
        else if (!strcmp(w, "wuk")) { p = L->wuk; r = c->kv_rank; k = c->d; }
        else if (!strcmp(w, "wuv")) { p = L->wuv; r = c->kv_rank; k = c->d; }
        else if (!strcmp(w, "wg")) { p = L->wg; r = c->d; k = c->dff; }
        else if (!strcmp(w, "bg")) { p = L->bg; r = 1; k = c->dff; }
        else if (!strcmp(w, "wu")) { p = L->wu; r = c->d; k = c->dff; }
        else if (!strcmp(w, "bu")) { p = L->bu; r = 1; k = c->dff; }
        else if (!strcmp(w, "wd")) { p = L->wd; r = c->dff; k = c->d; }
        else if (!strcmp(w, "bd")) { p = L->bd; r = 1; k = c->d; }
    }
    if (p && rows) *rows = r;
    if (p && cols) *cols = k;
    return p;
}

/* Embedding.java:28-34 */
static int embed(const ref_model *m, const int32_t *ids, int n, float *x) {
    for (int i = 0; i < n; i++)
        if (ids[i] < 0 || ids[i] >= m->cfg.vocab) return -1;    /* "Token id out of range" */
    ref_slice_rows(m->emb, ids, n, m->cfg.d, x);
    return 0;
}

/* GPTModel.java:52-54: token rows plus position rows 0..n-1 (PositionalEmbedding slices the first n rows);
 * pos0 is the position of the first row for the incremental path. */
static void add_positions(const ref_model *m, float *x, int n, int pos0) {
    int d = m->cfg.d;
    float *t = falloc((int64_t)n * d);
    ref_add(x, m->pos + (int64_t)pos0 * d, t, n, d);
    memcpy(x, t, (size_t)n * d * sizeof(float));
    free(t);
}

/* DecoderOnlyModel.java:58-64 with GPT blocks (GPTTransformerBlock.java:65-73) */
static void gpt_forward(ref_model *m, float *x, float *h, float *a, float *x2, int n, float *logits) {
    const ref_config *c = &m->cfg;
    int d = c->d;
    add_positions(m, x, n, 0);
    for (int l = 0; l < c->layers; l++) {
        const ref_layer *L = &m->layer[l];
        ref_layernorm(x, L->g1, L->be1, h, n, d);
        ref_mhsa_forward(h, L->wq, L->wk, L->wv, L->wo, a, n, d, c->heads, NULL, NULL, 1);
        ref_add(x, a, x2, n, d);
        ref_layernorm(x2, L->g2, L->be2, h, n, d);
        gpt_fnn(h, L->wg, L->bg, L->wd, L->bd, a, n, d, c->dff);
        ref_add(x2, a, x, n, d);
    }
    ref_layernorm(x, m->gf, m->bf, h, n, d);
    ref_linear(h, m->wlm, m->blm, logits, n, d, c->vocab);
}

/* LlamaTransformerBlock.java:50-53 / DeepSeekTransformerBlock.java:54-57, the first n_layers blocks in order */
static void run_blocks(ref_model *m, float *x, float *h, float *a, float *x2, int n, int n_layers) {
    const ref_config *c = &m->cfg;
    int d = c->d;
    for (int l = 0; l < n_layers; l++) {
        const ref_layer *L = &m->layer[l];
        ref_rmsnorm(x, L->g1, h, n, d);
        if (c->kind == 0)
            ref_mhsa_forward(h, L->wq, L->wk, L->wv, L->wo, a, n, d, c->heads, m->cos_t, m->sin_t, 1);
        else
            ref_mla_forward(h, L->wdq, L->wuq, L->wdkv, L->wuk, L->wuv, L->wo, a, n, d, c->heads,
                            c->q_rank, c->kv_rank, m->cos_t, m->sin_t);
        ref_add(x, a, x2, n, d);
        ref_rmsnorm(x2, L->g2, h, n, d);
        ref_swiglu(h, L->wg, L->bg, L->wu, L->bu, L->wd, L->bd, a, n, d, c->dff);
        ref_add(x2, a, x, n, d);
    }
}

/* DecoderOnlyModel.java:58-64 with Llama/DeepSeek blocks */
int ref_model_forward(ref_model *m, const int32_t *ids, int n, float *logits) {
    const ref_config *c = &m->cfg;
    int d = c->d;
    int64_t nd = (int64_t)n * d;
    float *x = falloc(nd), *h = falloc(nd), *a = falloc(nd), *x2 = falloc(nd);
    if (embed(m, ids, n, x) != 0) { free(x); free(h); free(a); free(x2); return -1; }
    if (c->kind == 2) {
        if (n > c->max_seq) { free(x); free(h); free(a); free(x2); return -2; }   /* PositionalEmbedding.java: seqLen > maxSeqLen throws */
        gpt_forward(m, x, h, a, x2, n, logits);
        free(x); free(h); free(a); free(x2);
        return 0;
    }
    run_blocks(m, x, h, a, x2, n, c->layers);
    ref_rmsnorm(x, m->gf, h, n, d);
    ref_linear(h, m->wlm, m->blm, logits, n, d, c->vocab);
    free(x); free(h); free(a); free(x2);
    return 0;
}

/* The block stack's state after its first n_layers blocks (TransformerStack.java:28-35 stopped early), [n x d]:
 * the input the next block sees.  Llama / DeepSeek only.  Test infrastructure: lets a test feed one block of a deep
 * model the exact input the CPU path gives it. */
int ref_model_hidden(ref_model *m, const int32_t *ids, int n, int n_layers, float *x_out) {
    const ref_config *c = &m->cfg;
    int d = c->d;
    int64_t nd = (int64_t)n * d;
    if (c->kind == 2 || n_layers < 0 || n_layers > c->layers) return -3;
    float *x = falloc(nd), *h = falloc(nd), *a = falloc(nd), *x2 = falloc(nd);
    if (embed(m, ids, n, x) != 0) { free(x); free(h); free(a); free(x2); return -1; }
    run_blocks(m, x, h, a, x2, n, n_layers);
    memcpy(x_out, x, (size_t)nd * sizeof(float));
    free(x); free(h); free(a); free(x2);
    return 0;
}

void ref_model_reset_cache(ref_model *m) { m->cached = 0; }

/* Incremental attention for the new rows [p0, p0+n) of one layer.  Every
 * output element is produced by the same sequence of fp32 operations as the
 * literal path (sequential dot over head_dim, scale, row max / exp / sum /
 * divide, values accumulated over ascending key index); masked keys there add
 * exact zeros, so dropping them changes nothing. */
static void cached_attention(ref_model *m, int l, const float *q, const float *k, const float *v,
                             float *merged, int n) {
    const ref_config *c = &m->cfg;
    int d = c->d, H = c->heads, hd = d / H, half = hd / 2, p0 = m->cached;
    float scale = (float)(1.0 / sqrt((double)hd));
    float *kc = m->kcache + (int64_t)l * c->max_seq * d;
    float *vc = m->vcache + (int64_t)l * c->max_seq * d;
    float *qr = falloc((int64_t)n * d);
    for (int i = 0; i < n; i++) {
        const float *ct = m->cos_t + (int64_t)(p0 + i) * half;
        const float *st = m->sin_t + (int64_t)(p0 + i) * half;
        for (int h = 0; h < H; h++) {
            for (int j = 0; j < half; j++) {
                int64_t e = (int64_t)i * d + h * hd + 2 * j;
                float cs = ct[j], sn = st[j];
                float q0 = q[e], q1 = q[e + 1], k0 = k[e], k1 = k[e + 1];
                qr[e] = q0 * cs - q1 * sn;  qr[e + 1] = q0 * sn + q1 * cs;
                int64_t ce = (int64_t)(p0 + i) * d + h * hd + 2 * j;
                kc[ce] = k0 * cs - k1 * sn; kc[ce + 1] = k0 * sn + k1 * cs;
            }
        }
        memcpy(vc + (int64_t)(p0 + i) * d, v + (int64_t)i * d, (size_t)d * sizeof(float));
    }
    int threads = ref_get_threads();
    #pragma omp parallel for schedule(static) num_threads(threads) collapse(2)
    for (int h = 0; h < H; h++) {
        for (int i = 0; i < n; i++) {
            int p = p0 + i;                      /* keys 0..p */
            float *s = (float *)malloc((size_t)(p + 1) * sizeof(float));
            const float *qv = qr + (int64_t)i * d + h * hd;
            float mx = -INFINITY;
            for (int cidx = 0; cidx <= p; cidx++) {
                const float *kv = kc + (int64_t)cidx * d + h * hd;
                float acc = 0.0f;
                for (int j = 0; j < hd; j++) acc += qv[j] * kv[j];
                acc = acc * scale;
                acc = acc + 0.0f;                /* mask entry for c <= r */
                s[cidx] = acc;
                if (acc > mx) mx = acc;
            }
            float se = 0.0f;
            for (int cidx = 0; cidx <= p; cidx++) se += (float)exp((double)(s[cidx] - mx));
            for (int cidx = 0; cidx <= p; cidx++) s[cidx] = (float)exp((double)(s[cidx] - mx)) / se;
            float *o = merged + (int64_t)i * d + h * hd;
            for (int j = 0; j < hd; j++) o[j] = 0.0f;
            for (int cidx = 0; cidx <= p; cidx++) {
                float a = s[cidx];
                const float *vv = vc + (int64_t)cidx * d + h * hd;
                for (int j = 0; j < hd; j++) o[j] += a * vv[j];
            }
            free(s);
        }
    }
    free(qr);
}

int ref_model_forward_cached(ref_model *m, const int32_t *ids, int n, float *logits, int last_only) {
    const ref_config *c = &m->cfg;
    int d = c->d;
    if (m->cached + n > c->max_seq) return -2;
    if (!m->kcache) {
        m->kcache = falloc((int64_t)c->layers * c->max_seq * d);
        m->vcache = falloc((int64_t)c->layers * c->max_seq * d);
    }
    int64_t nd = (int64_t)n * d;
    float *x = falloc(nd), *h = falloc(nd), *a = falloc(nd), *x2 = falloc(nd);
    float *q = falloc(nd), *k = falloc(nd), *v = falloc(nd), *mg = falloc(nd);
    int rc = embed(m, ids, n, x);
    if (rc == 0) {
        int gpt = c->kind == 2;
        if (gpt) add_positions(m, x, n, m->cached);
        for (int l = 0; l < c->layers; l++) {
            const ref_layer *L = &m->layer[l];
            if (gpt) ref_layernorm(x, L->g1, L->be1, h, n, d);
            else ref_rmsnorm(x, L->g1, h, n, d);
            if (c->kind != 1) {
                ref_matmul(h, L->wq, q, n, d, d);
                ref_matmul(h, L->wk, k, n, d, d);
                ref_matmul(h, L->wv, v, n, d, d);
            } else {
                float *cq = falloc((int64_t)n * c->q_rank), *ckv = falloc((int64_t)n * c->kv_rank);
                ref_matmul(h, L->wdq, cq, n, c->q_rank, d);
                ref_matmul(cq, L->wuq, q, n, d, c->q_rank);
                ref_matmul(h, L->wdkv, ckv, n, c->kv_rank, d);
                ref_matmul(ckv, L->wuk, k, n, d, c->kv_rank);
                ref_matmul(ckv, L->wuv, v, n, d, c->kv_rank);
                free(cq); free(ckv);
            }
            cached_attention(m, l, q, k, v, mg, n);
            ref_matmul(mg, L->wo, a, n, d, d);
            ref_add(x, a, x2, n, d);
            if (gpt) {
                ref_layernorm(x2, L->g2, L->be2, h, n, d);
                gpt_fnn(h, L->wg, L->bg, L->wd, L->bd, a, n, d, c->dff);
            } else {
                ref_rmsnorm(x2, L->g2, h, n, d);
                ref_swiglu(h, L->wg, L->bg, L->wu, L->bu, L->wd, L->bd, a, n, d, c->dff);
            }
            ref_add(x2, a, x, n, d);
        }
        m->cached += n;
        int rows = last_only ? 1 : n;
        const float *xr = last_only ? x + (int64_t)(n - 1) * d : x;
        if (gpt) ref_layernorm(xr, m->gf, m->bf, h, rows, d);
        else ref_rmsnorm(xr, m->gf, h, rows, d);
        ref_linear(h, m->wlm, m->blm, logits, rows, d, c->vocab);
    }
    free(x); free(h); free(a); free(x2); free(q); free(k); free(v); free(mg);
    return rc;
}

/* ── TextGenerator ──────────────────────────────────────────────────── */

/* Float.compare(x, y): -0.0 < 0.0, NaN greater than everything and equal to itself. */
static int java_float_compare(float x, float y) {
    if (x < y) return -1;
    if (x > y) return 1;
    int32_t bx, by;
    memcpy(&bx, &x, 4); memcpy(&by, &y, 4);
    if (x != x) bx = 0x7fc00000;     /* floatToIntBits canonicalises NaN */
    if (y != y) by = 0x7fc00000;
    return bx == by ? 0 : (bx < by ? -1 : 1);
}

/* Stable merge sort of indices by descending logit: Arrays.sort(Integer[], cmp) is a
 * stable sort, comparator (i, j) -> Float.compare(a[j], a[i]).  TextGenerator.java:163-170 */
static void argsort_desc(const float *a, int n, int32_t *idx) {
    int32_t *tmp = (int32_t *)malloc((size_t)n * sizeof(int32_t));
    for (int i = 0; i < n; i++) idx[i] = i;
    for (int w = 1; w < n; w *= 2) {
        for (int lo = 0; lo < n; lo += 2 * w) {
            int mid = lo + w < n ? lo + w : n, hi = lo + 2 * w < n ? lo + 2 * w : n;
            int i = lo, j = mid, o = lo;
            while (i < mid && j < hi) {
                /* take right only if it sorts strictly before left */
                if (java_float_compare(a[idx[i]], a[idx[j]]) < 0) tmp[o++] = idx[j++];
                else tmp[o++] = idx[i++];
            }
            while (i < mid) tmp[o++] = idx[i++];
            while (j < hi) tmp[o++] = idx[j++];
        }
        memcpy(idx, tmp, (size_t)n * sizeof(int32_t));
    }
    free(tmp);
}

int32_t ref_sample_from_logits(const float *logits, int vocab, float temperature, int top_k, jrandom *rnd) {
    int32_t *order = (int32_t *)malloc((size_t)vocab * sizeof(int32_t));
    argsort_desc(logits, vocab, order);
    int k = (top_k == 0) ? vocab : (top_k < vocab ? top_k : vocab);
    float mx = -INFINITY;
    for (int i = 0; i < k; i++) { float v = logits[order[i]] / temperature; if (v > mx) mx = v; }
    float *probs = falloc(k);
    float sum = 0.0f;
    for (int i = 0; i < k; i++) {
        float p = (float)exp((double)(logits[order[i]] / temperature - mx));
        probs[i] = p; sum += p;
    }
    for (int i = 0; i < k; i++) probs[i] /= sum;
    float r = jr_next_float(rnd);
    float cum = 0.0f;
    int32_t pick = order[k - 1];
    for (int i = 0; i < k; i++) { cum += probs[i]; if (r <= cum) { pick = order[i]; break; } }
    free(order); free(probs);
    return pick;
}

int ref_generate(ref_model *m, const int32_t *prompt, int n_prompt, int max_new,
                 float temperature, int top_k, int64_t seed, int use_cache,
                 int32_t *out_ids, float *last_logits) {
    if (max_new < 0 || !(temperature > 0.0f) || top_k < 0) return -3;   /* validateArgs */
    const ref_config *c = &m->cfg;
    jrandom rnd; jr_init(&rnd, seed);
    memcpy(out_ids, prompt, (size_t)n_prompt * sizeof(int32_t));
    int len = n_prompt;
    float *row = falloc(c->vocab);
    if (use_cache) {
        if (n_prompt + max_new > c->max_seq || n_prompt < 1) { free(row); return -2; }
        ref_model_reset_cache(m);
    }
    for (int t = 0; t < max_new; t++) {
        int rc;
        if (use_cache) {
            if (t == 0) rc = ref_model_forward_cached(m, out_ids, len, row, 1);
            else rc = ref_model_forward_cached(m, out_ids + len - 1, 1, row, 1);
        } else {
            int ctx = len <= c->max_seq ? len : c->max_seq;          /* last(ids, maxSeqLen) */
            float *logits = falloc((int64_t)ctx * c->vocab);
            rc = ref_model_forward(m, out_ids + len - ctx, ctx, logits);
            memcpy(row, logits + (int64_t)(ctx - 1) * c->vocab, (size_t)c->vocab * sizeof(float));
            free(logits);
        }
        if (rc != 0) { free(row); return rc; }
        if (last_logits) memcpy(last_logits + (int64_t)t * c->vocab, row, (size_t)c->vocab * sizeof(float));
        out_ids[len++] = ref_sample_from_logits(row, c->vocab, temperature, top_k, &rnd);
    }
    free(row);
    return 0;
}
