/*
 * TEST INFRASTRUCTURE ONLY - CPU oracle for the DeepJ HIP backend.
 * Nothing in the shipped library links or loads this code.
 *
 * Restatement of the reference's inference layers and models on top of
 * cpu_backend.c (paths below are under src/main/java/io/github/kirstenali/deepj/):
 *   layers/Linear.java:31-36                         ref_linear
 *   layers/transformer/norm/RMSNorm1D.java:30,46-57   ref_rmsnorm
 *   activations/SiLU.java:20-24                       ref_silu
 *   layers/transformer/SwiGLULayer.java:63-70         ref_swiglu
 *   transformer/embeddings/RotaryEmbedding.java:52-71,81-122   ref_rope_tables / ref_rope_apply
 *   layers/transformer/attention/HeadOps.java:33-140  split/merge/scores/mask/values
 *   layers/transformer/attention/MultiHeadSelfAttention.java:60-86 (+ RoPEMultiHeadSelfAttention.java:55-58)
 *   layers/transformer/attention/MultiHeadLatentAttention.java:92-123
 *   layers/transformer/blocks/LlamaTransformerBlock.java:50-53, DeepSeekTransformerBlock.java:54-57
 *   transformer/TransformerStack.java:28-35, models/DecoderOnlyModel.java:58-64
 *   models/llama/LlamaModel.java:27-42, models/deepseek/DeepSeekModel.java:29-46 (seeded init order)
 *   layers/transformer/norm/LayerNorm1D.java:34-66       ref_layernorm
 *   layers/FNN.java:57-73 + activations/GELU.java:15-18   the GPT feed-forward (Linear, GELU, Linear)
 *   transformer/embeddings/PositionalEmbedding.java:26-33, models/gpt/GPTModel.java:27-81,
 *   layers/transformer/blocks/GPTTransformerBlock.java:52-73   GPT model: learned positions, init order, initScale
 *   models/TextGenerator.java:66-181 (sliding window, stable argsort, top-k, temperature, categorical draw)
 *
 * The reference's tests hold no forward known answers for LayerNorm1D, FNN or GPTModel (gradient checks and
 * shapes only): those functions are pinned by closed forms and fp64 brute force (tests/test_oracle_invariants.py),
 * plus GPTModelTest's parameter count and init-scale ratio.
 *
 * The Q8 weight format and the incremental (KV-cached) forward have no
 * counterpart in the reference: parity unpinned by the reference.  They are
 * pinned here instead by (a) the round-trip bound |w - dq(q(w))| <= scale/2,
 * (b) exactness on representable inputs, and (c) the cached forward being
 * bit-identical to the last rows of the literal full-context forward.
 */
#ifndef DEEPJ_ORACLE_MODEL_REF_H
#define DEEPJ_ORACLE_MODEL_REF_H

#include <stdint.h>
#include "cpu_backend.h"

#ifdef __cplusplus
extern "C" {
#endif

#define REF_RMS_EPS 1e-6f       /* RMSNorm1D.java:30 */
#define REF_Q8_GROUP 32

/* ── layers ─────────────────────────────────────────────────────────── */
void ref_linear(const float *x, const float *w, const float *b, float *out, int rows, int d_in, int d_out);
void ref_rmsnorm(const float *x, const float *gamma, float *out, int rows, int dim);
void ref_silu(const float *x, float *out, int rows, int cols);
void ref_swiglu(const float *x, const float *wg, const float *bg, const float *wu, const float *bu,
                const float *wd, const float *bd, float *out, int rows, int d, int dff);
void ref_rope_tables(int head_dim, int max_seq, float *cos_t, float *sin_t);   /* [max_seq x head_dim/2] */
/* t is split-head [n_heads*seq x head_dim]; row h*seq+i gets position pos0+i. */
void ref_rope_apply(const float *t, float *out, int seq, int n_heads, int head_dim,
                    const float *cos_t, const float *sin_t, int pos0);
void ref_split_heads(const float *t, float *out, int seq, int n_heads, int head_dim);
void ref_merge_heads(const float *t, float *out, int seq, int n_heads, int head_dim);
/* Literal causal attention on split-head q,k,v -> split-head out. */
void ref_attention_heads(const float *qh, const float *kh, const float *vh, float *outh,
                         int seq, int n_heads, int head_dim, int causal);
void ref_mhsa_forward(const float *x, const float *wq, const float *wk, const float *wv, const float *wo,
                      float *out, int seq, int d, int n_heads,
                      const float *cos_t, const float *sin_t /* NULL = no RoPE */, int causal);
void ref_mla_forward(const float *x, const float *wdq, const float *wuq, const float *wdkv,
                     const float *wuk, const float *wuv, const float *wo, float *out,
                     int seq, int d, int n_heads, int q_rank, int kv_rank,
                     const float *cos_t, const float *sin_t);

/* LayerNorm1D.java:34-66: (x - mean) / sqrt(var + 1e-5) * gamma + beta, population variance */
void ref_layernorm(const float *x, const float *gamma, const float *beta, float *out, int rows, int dim);

/* ── Q8 (this build's format; see header comment) ───────────────────── */
/* w is [K x N] row-major fp32 (the reference's weight orientation, Linear.java:13).
 * q is [N x Kp] int8 with Kp = K rounded up to 32 (zero padded), scales [N x Kp/32]. */
int  ref_q8_padded_k(int k);
void ref_q8_quantize(const float *w, int k, int n, int8_t *q, float *scales);
void ref_q8_dequantize(const int8_t *q, const float *scales, int k, int n, float *w_out /* [K x N] */);

/* ── models ─────────────────────────────────────────────────────────── */
typedef struct {
    int kind;          /* 0 = Llama, 1 = DeepSeek (MLA), 2 = GPT (LayerNorm, GELU FNN, learned positions) */
    int vocab, max_seq, d, heads, layers, dff;
    int q_rank, kv_rank;   /* DeepSeek only */
    float init_scale;      /* GPT only: every parameter is multiplied by it after init (GPTModel.java:76-81) */
} ref_config;

typedef struct {
    float *g1, *g2;
    float *wq, *wk, *wv, *wo;                 /* Llama */
    float *wdq, *wuq, *wdkv, *wuk, *wuv;      /* DeepSeek (wo shared above) */
    float *wg, *bg, *wu, *bu, *wd, *bd;       /* GPT: wg,bg = first FNN linear, wd,bd = second; wu,bu unused */
    float *be1, *be2;                         /* GPT: LayerNorm betas (g1, g2 are the gammas) */
} ref_layer;

typedef struct {
    ref_config cfg;
    float *emb;            /* [vocab x d] */
    ref_layer *layer;
    float *gf;             /* final norm gain */
    float *bf;             /* GPT: final LayerNorm beta */
    float *pos;            /* GPT: positional embedding [max_seq x d] */
    float *wlm, *blm;      /* [d x vocab], [vocab] */
    float *cos_t, *sin_t;  /* [max_seq x hd/2] */
    /* incremental state (not in the reference) */
    float *kcache, *vcache;   /* [layers][max_seq][d], K stored after RoPE */
    int cached;               /* rows in the cache */
} ref_model;

ref_model *ref_model_create(const ref_config *cfg, int64_t seed);
/* timing-only: later ref_model_create calls fill weights with a cheap hash instead of java.util.Random */
void       ref_set_fast_fill(int on);
void       ref_model_free(ref_model *m);
/* Replace every matmul weight (attention/MLA projections, SwiGLU, LM head) by
 * dequant(quant(W)); embedding, gains and biases stay fp32. */
void       ref_model_q8_roundtrip(ref_model *m);
/* Pointer to a named weight: "emb","gf","wlm","blm", or "L<i>.<name>". NULL if unknown. */
float     *ref_model_weight(ref_model *m, const char *name, int *rows, int *cols);

/* DecoderOnlyModel.forward: logits [n x vocab] for the whole context. Returns 0, or -1 on a bad id. */
int ref_model_forward(ref_model *m, const int32_t *ids, int n, float *logits);
/* x after the first n_layers blocks, [n x d] (Llama / DeepSeek); -1 bad token id, -3 bad layer count or GPT */
int ref_model_hidden(ref_model *m, const int32_t *ids, int n, int n_layers, float *x_out);
/* Incremental: appends n rows after the m->cached rows already seen; logits [n x vocab]
 * (or only the last row when last_only != 0: logits [1 x vocab]). */
void ref_model_reset_cache(ref_model *m);
int  ref_model_forward_cached(ref_model *m, const int32_t *ids, int n, float *logits, int last_only);

/* TextGenerator.sampleFromLogits */
int32_t ref_sample_from_logits(const float *logits, int vocab, float temperature, int top_k, jrandom *rnd);
/* TextGenerator.generate on token ids; out_ids holds n_prompt + max_new ids.
 * use_cache != 0 uses the incremental forward (requires n_prompt+max_new <= max_seq).
 * If last_logits != NULL it receives the [max_new x vocab] last-row logits of each step. */
int ref_generate(ref_model *m, const int32_t *prompt, int n_prompt, int max_new,
                 float temperature, int top_k, int64_t seed, int use_cache,
                 int32_t *out_ids, float *last_logits);

#ifdef __cplusplus
}
#endif
#endif
