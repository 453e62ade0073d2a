// Native decode driver: the caller on the host side of the C ABI.  It plays the part of
// the reference's LlamaModel / DeepSeekModel / GPTModel + TextGenerator
//   (src/main/java/io/github/kirstenali/deepj/models/{DecoderOnlyModel,TextGenerator}.java,
//    models/llama/LlamaModel.java, models/deepseek/DeepSeekModel.java, models/gpt/GPTModel.java)
// for inference, but instead of re-running the whole context for every token
// (TextGenerator.java:91-100) it keeps a KV cache in HBM, records ONE fused command
// stream per token and replays it as a HIP graph.  Position, current token and the
// generated ids live in device memory, so a run of N tokens needs no host round trip.
//
// Everything here goes through the public deepj_hip_* functions only: buffers are named
// by int ids, work is submitted as int32 command streams - the same boundary a Java
// HipBackend uses - so a Java facade can emit the identical streams.
//
// Weight names: "emb", "gf", "wlm", "blm" and per layer "L<i>.<w>" with w in
//   g1 g2 wq wk wv wo           (Llama;  MultiHeadSelfAttention.java:47-50)
//   g1 g2 wdq wuq wdkv wuk wuv wo (DeepSeek; MultiHeadLatentAttention.java:81-86)
//     kept as two Q8 matrices: the down-projections stacked by output row, [Wdq | pad | Wdkv], and the
//     up-projections as one block matrix that maps [cQ | pad | cKV] to [Q | K | V] (zero blocks elsewhere),
//     so MLA costs two projections and then shares the Llama attention path and its rotated K/V cache
//   wg bg wu bu wd bd           (SwiGLULayer.java:56-58)
// GPT (GPTTransformerBlock.java:52-57): g1 be1 g2 be2 (LayerNorm gamma/beta), wq wk wv wo, and the FNN's two
//   Linears as wg bg (dModel -> dFF) and wd bd (dFF -> dModel); model level adds "pos" and "bf".
// Matrices are given in the reference's orientation, fp32 [dIn x dOut] row-major.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../../include/deepj_hip.h"

extern "C" {
void *deepj_host_random_create(int64_t seed);
void deepj_host_random_destroy(void *h);
void deepj_host_random_fill(void *h, float *out, int64_t n, double scale, int32_t threads);
float deepj_host_random_next_float(void *h);
}

namespace {

struct Config {
    int32_t kind;       // 0 Llama, 1 DeepSeek (MLA), 2 GPT; DeepSeek with the latent KV cache arrives as kind 3 and
                        // is kept here as kind 1 with `latent` set
    int32_t vocab, max_seq, d, heads, layers, dff, q_rank, kv_rank;
    bool latent = false;
};

struct Error : std::runtime_error { using std::runtime_error::runtime_error; };

constexpr int kGraphUnroll = 4;     // tokens per replay of the unrolled decode graph

void hip(int rc) {
    if (rc != 0) throw Error(deepj_hip_last_error());
}

struct Layer {
    int32_t g1 = -1, g2 = -1, be1 = -1, be2 = -1;     // be*: LayerNorm betas (GPT)
    int32_t wqkv = -1, wo = -1;                       // Llama: fused [3d x d]
    int32_t wdown = -1, wup = -1;                     // MLA: stacked down-projections, block up-projection
    int32_t wdq = -1, wuq = -1, wdkv = -1, wukv = -1; // MLA with the latent cache: Wdq, Wuq, Wdkv, and [Wuk | Wuv] by output row
    int32_t wgu = -1, bg = -1, bu = -1, wd = -1, bd = -1;
};

struct Acts {          // activation buffers for S rows
    int32_t rows = 0;
    int32_t x = -1, x2 = -1, qkv = -1, q = -1, att = -1, ff = -1, ids = -1;
    int32_t cq = -1;                                                 // MLA: [cQ | pad | cKV] rows (latent cache: cQ rows)
    int32_t ckv = -1;                                                // MLA with the latent cache: cKV rows
};

struct Runner {
    Config cfg{};
    int32_t next_id = 0;
    std::map<std::string, bool> have;
    std::vector<Layer> layers;
    int32_t emb = -1, gf = -1, wlm = -1, blm = -1;
    int32_t pos_table = -1, bf = -1;                       // GPT: learned positions, final LayerNorm beta
    int32_t cos_t = -1, sin_t = -1, kc = -1, vc = -1;
    int32_t state = -1, tokens = -1, scratch = -1, logits = -1, last_x = -1;
    int32_t records = -1;                                  // decode attention records (merged by the Wo matvec)
    int32_t latent = -1, kv_all = -1;                      // latent cache [L][maxSeq][kvRank]; re-expanded [maxSeq][K | V] of one layer
    std::vector<int32_t> prepared;                         // the weights in the many-row GEMM's layout (first long prompt)
    bool prepared_done = false;
    int64_t prepared_budget = -1;                          // bytes such copies may take in all; -1: no limit
    int64_t prepared_bytes = 0;
    Acts dec, pre;
    int32_t graph = 0, graph_unrolled = 0;                 // one token per replay / kGraphUnroll tokens per replay
    bool finalized = false;
    int32_t pos = 0;          // host mirror of state[0]
    int32_t generated = 0;    // host mirror of state[2]
    std::string error;

    int hd() const { return cfg.d / cfg.heads; }
    // MLA: width of [cQ | pad | cKV]; cKV starts at a multiple of 32 so that the Q8 groups of Wuk and Wuv
    // (32 consecutive inputs) are the ones each matrix would get on its own
    int q_rank_padded() const { return (cfg.q_rank + 31) / 32 * 32; }
    int latent_width() const { return q_rank_padded() + cfg.kv_rank; }

    int32_t alloc(int64_t floats) {
        if (floats > 0x7fffffffLL) throw Error("buffer too large for an int32 float count");
        int32_t id = next_id++;
        int32_t sz = (int32_t)floats;
        hip(deepj_hip_alloc_buffers(&id, &sz, 1));
        return id;
    }
    void release(int32_t &id) {
        if (id >= 0) { hip(deepj_hip_release(&id, 1)); id = -1; }
    }
    int32_t upload_new(const float *data, int64_t n) {
        int32_t id = alloc(n);
        hip(deepj_hip_upload(id, data, n));
        return id;
    }
    void run(const std::vector<int32_t> &s) { hip(deepj_hip_flush_ops(s.data(), (int32_t)s.size())); }
};

using Stream = std::vector<int32_t>;
template <class... A> void emit(Stream &s, A... words) { (s.push_back((int32_t)words), ...); }

void q8_linear(Stream &s, int32_t x, int32_t w, int32_t out, int m, int k, int n, int flags, int32_t gamma = -1,
               int32_t bias = -1, int32_t bias2 = -1, int32_t residual = -1) {
    emit(s, DJ_OP_Q8_LINEAR, x, w, out, m, k, n, flags, gamma, bias, bias2, residual);
}

// ── weights ────────────────────────────────────────────────────────────────

void quantize_into(Runner &r, int32_t &dst, const float *data, int k, int n, int row_off, int row_step, int total) {
    if (dst < 0) dst = r.alloc(deepj_hip_q8_floats(k, total));
    int32_t tmp = r.upload_new(data, (int64_t)k * n);
    Stream s;
    emit(s, DJ_OP_Q8_QUANTIZE, tmp, dst, k, n, row_off, row_step, total);
    r.run(s);
    r.release(tmp);
}

void expect_shape(const std::string &name, int rows, int cols, int er, int ec) {
    if (rows != er || cols != ec)
        throw Error("weight " + name + ": expected " + std::to_string(er) + "x" + std::to_string(ec) + " but got " +
                    std::to_string(rows) + "x" + std::to_string(cols));
}

void set_weight(Runner &r, const std::string &name, const float *data, int rows, int cols) {
    const Config &c = r.cfg;
    const int d = c.d;
    if (r.finalized) throw Error("set_weight after finalize");
    if (name == "emb") { expect_shape(name, rows, cols, c.vocab, d); r.emb = r.upload_new(data, (int64_t)rows * cols); }
    else if (name == "gf") { expect_shape(name, rows, cols, 1, d); r.gf = r.upload_new(data, d); }
    else if (c.kind == 2 && name == "bf") { expect_shape(name, rows, cols, 1, d); r.bf = r.upload_new(data, d); }
    else if (c.kind == 2 && name == "pos") { expect_shape(name, rows, cols, c.max_seq, d); r.pos_table = r.upload_new(data, (int64_t)rows * cols); }
    else if (name == "blm") { expect_shape(name, rows, cols, 1, c.vocab); r.blm = r.upload_new(data, c.vocab); }
    else if (name == "wlm") { expect_shape(name, rows, cols, d, c.vocab); quantize_into(r, r.wlm, data, d, c.vocab, 0, 1, c.vocab); }
    else if (name.size() > 2 && name[0] == 'L') {
        size_t dot = name.find('.');
        if (dot == std::string::npos) throw Error("unknown weight " + name);
        int l = std::atoi(name.substr(1, dot - 1).c_str());
        if (l < 0 || l >= c.layers) throw Error("weight " + name + ": no such layer");
        Layer &L = r.layers[l];
        std::string w = name.substr(dot + 1);
        if (w == "g1") { expect_shape(name, rows, cols, 1, d); L.g1 = r.upload_new(data, d); }
        else if (w == "g2") { expect_shape(name, rows, cols, 1, d); L.g2 = r.upload_new(data, d); }
        else if (c.kind == 2 && w == "be1") { expect_shape(name, rows, cols, 1, d); L.be1 = r.upload_new(data, d); }
        else if (c.kind == 2 && w == "be2") { expect_shape(name, rows, cols, 1, d); L.be2 = r.upload_new(data, d); }
        else if (c.kind == 2 && w == "wg") { expect_shape(name, rows, cols, d, c.dff); quantize_into(r, L.wgu, data, d, c.dff, 0, 1, c.dff); }
        else if (c.kind == 2 && (w == "wu" || w == "bu")) throw Error("unknown weight " + name);
        else if (w == "bg") { expect_shape(name, rows, cols, 1, c.dff); L.bg = r.upload_new(data, c.dff); }
        else if (w == "bu") { expect_shape(name, rows, cols, 1, c.dff); L.bu = r.upload_new(data, c.dff); }
        else if (w == "bd") { expect_shape(name, rows, cols, 1, d); L.bd = r.upload_new(data, d); }
        else if (w == "wg") { expect_shape(name, rows, cols, d, c.dff); quantize_into(r, L.wgu, data, d, c.dff, 0, 2, 2 * c.dff); }
        else if (w == "wu") { expect_shape(name, rows, cols, d, c.dff); quantize_into(r, L.wgu, data, d, c.dff, 1, 2, 2 * c.dff); }
        else if (w == "wd") { expect_shape(name, rows, cols, c.dff, d); quantize_into(r, L.wd, data, c.dff, d, 0, 1, d); }
        else if (w == "wo") { expect_shape(name, rows, cols, d, d); quantize_into(r, L.wo, data, d, d, 0, 1, d); }
        else if (c.kind != 1 && (w == "wq" || w == "wk" || w == "wv")) {
            expect_shape(name, rows, cols, d, d);
            int part = w == "wq" ? 0 : (w == "wk" ? 1 : 2);
            quantize_into(r, L.wqkv, data, d, d, part * d, 1, 3 * d);
        }
        else if (c.latent && w == "wdq") { expect_shape(name, rows, cols, d, c.q_rank); quantize_into(r, L.wdq, data, d, c.q_rank, 0, 1, c.q_rank); }
        else if (c.latent && w == "wuq") { expect_shape(name, rows, cols, c.q_rank, d); quantize_into(r, L.wuq, data, c.q_rank, d, 0, 1, d); }
        else if (c.latent && w == "wdkv") { expect_shape(name, rows, cols, d, c.kv_rank); quantize_into(r, L.wdkv, data, d, c.kv_rank, 0, 1, c.kv_rank); }
        else if (c.latent && (w == "wuk" || w == "wuv")) {
            // Q8 rows [0, d) = the columns of Wuk, [d, 2d) = those of Wuv: one product re-expands a latent row to [K | V]
            expect_shape(name, rows, cols, c.kv_rank, d);
            quantize_into(r, L.wukv, data, c.kv_rank, d, w == "wuk" ? 0 : d, 1, 2 * d);
        }
        else if (c.kind == 1 && (w == "wdq" || w == "wdkv")) {
            // output rows [0, qRank) = Wdq, [qRankPadded, +kvRank) = Wdkv; the pad rows stay zero (the buffer is
            // zero-filled when it is created) and so produce zeros
            const bool q = w == "wdq";
            expect_shape(name, rows, cols, d, q ? c.q_rank : c.kv_rank);
            if (L.wdown < 0) {
                L.wdown = r.alloc(deepj_hip_q8_floats(d, r.latent_width()));
                Stream z; emit(z, DJ_OP_FILL, L.wdown, 0, deepj_hip_q8_floats(d, r.latent_width())); r.run(z);
            }
            quantize_into(r, L.wdown, data, d, cols, q ? 0 : r.q_rank_padded(), 1, r.latent_width());
        }
        else if (c.kind == 1 && (w == "wuq" || w == "wuk" || w == "wuv")) {
            // block matrix over the inputs [cQ | pad | cKV]: the matrix is widened with zero rows to the full
            // input width on the host, then its columns become Q8 rows [0,d) / [d,2d) / [2d,3d)
            const bool q = w == "wuq";
            const int in = q ? c.q_rank : c.kv_rank, k2 = r.latent_width(), off = q ? 0 : r.q_rank_padded();
            expect_shape(name, rows, cols, in, d);
            std::vector<float> wide((size_t)k2 * d, 0.0f);
            std::memcpy(wide.data() + (size_t)off * d, data, (size_t)in * d * sizeof(float));
            if (L.wup < 0) L.wup = r.alloc(deepj_hip_q8_floats(k2, 3 * d));
            quantize_into(r, L.wup, wide.data(), k2, d, (q ? 0 : (w == "wuk" ? 1 : 2)) * d, 1, 3 * d);
        }
        else throw Error("unknown weight " + name);
    } else throw Error("unknown weight " + name);
    r.have[name] = true;
}

std::vector<std::string> weight_names(const Config &c) {
    std::vector<std::string> names{"emb"};
    if (c.kind == 2) {
        names.push_back("pos");
        for (int l = 0; l < c.layers; l++) {
            std::string p = "L" + std::to_string(l) + ".";
            for (const char *w : {"g1", "be1", "g2", "be2", "wq", "wk", "wv", "wo", "wg", "bg", "wd", "bd"}) names.push_back(p + w);
        }
        names.insert(names.end(), {"gf", "bf", "wlm", "blm"});
        return names;
    }
    for (int l = 0; l < c.layers; l++) {
        std::string p = "L" + std::to_string(l) + ".";
        for (const char *w : {"g1", "g2"}) names.push_back(p + w);
        if (c.kind == 0) for (const char *w : {"wq", "wk", "wv", "wo"}) names.push_back(p + w);
        else for (const char *w : {"wdq", "wuq", "wdkv", "wuk", "wuv", "wo"}) names.push_back(p + w);
        for (const char *w : {"wg", "bg", "wu", "bu", "wd", "bd"}) names.push_back(p + w);
    }
    names.insert(names.end(), {"gf", "wlm", "blm"});
    return names;
}

// new LlamaModel(cfg, seed) / new DeepSeekModel(cfg, seed): same RNG wiring and draw order
// (LlamaModel.java:27-42, LlamaTransformerBuilder.java:45-55, DeepSeekTransformerBuilder.java:56-68).
// GPT: new GPTModel(cfg, seed) - Random(seed) for the token table, a second Random(seed) shared by the
// blocks, Random(seed + 1) for the head, Random(seed + 2) for the positions, then every parameter times
// initScale (GPTModel.java:27-46,76-81; GPTTransformerBlock.java:52-57; FNN draws its Linears in order).
void init_seeded(Runner &r, int64_t seed, int threads, float init_scale) {
    const Config &c = r.cfg;
    const int d = c.d;
    std::vector<float> buf;
    auto draw = [&](void *rng, const std::string &name, int rows, int cols) {
        buf.resize((size_t)rows * cols);
        deepj_host_random_fill(rng, buf.data(), (int64_t)rows * cols, 0.1, threads);
        if (init_scale != 1.0f) for (float &v : buf) v *= init_scale;
        set_weight(r, name, buf.data(), rows, cols);
    };
    auto constant = [&](const std::string &name, int cols, float v) {
        buf.assign((size_t)cols, init_scale != 1.0f ? v * init_scale : v);
        set_weight(r, name, buf.data(), 1, cols);
    };
    void *emb_rng = deepj_host_random_create(seed);
    void *stack_rng = deepj_host_random_create(seed);
    void *head_rng = deepj_host_random_create(seed + 1);
    void *pos_rng = deepj_host_random_create(seed + 2);
    try {
        draw(emb_rng, "emb", c.vocab, d);
        if (c.kind == 2) draw(pos_rng, "pos", c.max_seq, d);
        for (int l = 0; l < c.layers; l++) {
            std::string p = "L" + std::to_string(l) + ".";
            constant(p + "g1", d, 1.0f);
            constant(p + "g2", d, 1.0f);
            if (c.kind == 2) {
                constant(p + "be1", d, 0.0f);
                constant(p + "be2", d, 0.0f);
                for (const char *w : {"wq", "wk", "wv", "wo"}) draw(stack_rng, p + w, d, d);
                draw(stack_rng, p + "wg", d, c.dff);  constant(p + "bg", c.dff, 0.0f);
                draw(stack_rng, p + "wd", c.dff, d);  constant(p + "bd", d, 0.0f);
                continue;
            }
            if (c.kind == 0) {
                for (const char *w : {"wq", "wk", "wv", "wo"}) draw(stack_rng, p + w, d, d);
            } else {
                draw(stack_rng, p + "wdq", d, c.q_rank);
                draw(stack_rng, p + "wuq", c.q_rank, d);
                draw(stack_rng, p + "wdkv", d, c.kv_rank);
                draw(stack_rng, p + "wuk", c.kv_rank, d);
                draw(stack_rng, p + "wuv", c.kv_rank, d);
                draw(stack_rng, p + "wo", d, d);
            }
            draw(stack_rng, p + "wg", d, c.dff);  constant(p + "bg", c.dff, 0.0f);
            draw(stack_rng, p + "wu", d, c.dff);  constant(p + "bu", c.dff, 0.0f);
            draw(stack_rng, p + "wd", c.dff, d);  constant(p + "bd", d, 0.0f);
        }
        constant("gf", d, 1.0f);
        if (c.kind == 2) constant("bf", d, 0.0f);
        draw(head_rng, "wlm", d, c.vocab);
        constant("blm", c.vocab, 0.0f);
    } catch (...) {
        deepj_host_random_destroy(emb_rng); deepj_host_random_destroy(stack_rng); deepj_host_random_destroy(head_rng);
        deepj_host_random_destroy(pos_rng);
        throw;
    }
    deepj_host_random_destroy(emb_rng); deepj_host_random_destroy(stack_rng); deepj_host_random_destroy(head_rng);
    deepj_host_random_destroy(pos_rng);
}

// ── buffers ────────────────────────────────────────────────────────────────

// Buffers for `rows` rows (they only ever grow: every op takes its row count explicitly).
void alloc_acts(Runner &r, Acts &a, int rows) {
    const Config &c = r.cfg;
    if (a.rows >= rows) return;
    for (int32_t *id : {&a.x, &a.x2, &a.qkv, &a.q, &a.att, &a.ff, &a.ids, &a.cq, &a.ckv}) r.release(*id);
    int64_t S = rows, d = c.d;
    a.x = r.alloc(S * d); a.x2 = r.alloc(S * d); a.q = r.alloc(S * d); a.att = r.alloc(S * d);
    a.ff = r.alloc(S * c.dff); a.ids = r.alloc(std::max<int64_t>(S, 4));
    a.qkv = r.alloc(S * 3 * d);
    if (c.latent) { a.cq = r.alloc(S * c.q_rank); a.ckv = r.alloc(S * c.kv_rank); }
    else if (c.kind == 1) a.cq = r.alloc(S * r.latent_width());
    a.rows = rows;
}

void warm_up(Runner &r);

void finalize(Runner &r) {
    const Config &c = r.cfg;
    if (r.finalized) return;
    for (const auto &n : weight_names(c))
        if (!r.have.count(n)) throw Error("weight " + n + " was never set");
    const int hd = r.hd(), half = hd / 2;
    // RotaryEmbedding.java:63-70
    std::vector<float> ct((size_t)c.max_seq * half), st((size_t)c.max_seq * half);
    for (int pos = 0; pos < c.max_seq; pos++)
        for (int i = 0; i < half; i++) {
            float expo = (2.0f * (float)i) / (float)hd;
            float theta = (float)((double)pos / std::pow((double)10000.0f, (double)expo));
            // GPT attends without rotation (MultiHeadSelfAttention.java:60-86): the identity tables turn the
            // rotation inside the attention kernels into x * 1 - y * 0 = x.
            ct[(size_t)pos * half + i] = c.kind == 2 ? 1.0f : (float)std::cos((double)theta);
            st[(size_t)pos * half + i] = c.kind == 2 ? 0.0f : (float)std::sin((double)theta);
        }
    r.cos_t = r.upload_new(ct.data(), (int64_t)ct.size());
    r.sin_t = r.upload_new(st.data(), (int64_t)st.size());
    int64_t per_layer = (int64_t)c.max_seq * c.d;
    // K (after RoPE) and V of every position, per layer [H][maxSeq][hd].  DeepSeek too: its latent rows could
    // be cached instead (kvRank floats per token rather than 2*dModel), but the reference rotates K after the
    // up-projection (MultiHeadLatentAttention.java:108-112), so the up-projection cannot be folded into the query
    // and every step would have to re-expand and re-rotate all cached positions.
    if (c.latent) {
        // The latent cache (MultiHeadLatentAttention.java:98-106 computes K and V from cKV = x.Wdkv): kvRank floats per
        // token and layer instead of 2 * dModel.  Every step re-expands the layer's cached rows to [K | V] and rotates
        // K (the reference rotates K after the up-projection, :108-112), into ONE buffer all layers take turns with.
        r.latent = r.alloc((int64_t)c.layers * c.max_seq * c.kv_rank);
        r.kv_all = r.alloc((int64_t)c.max_seq * 2 * c.d);
    } else {
        r.kc = r.alloc(per_layer * c.layers);
        r.vc = r.alloc(per_layer * c.layers);
    }
    r.state = r.alloc(4);
    r.tokens = r.alloc(c.max_seq);
    r.logits = r.alloc(c.vocab);
    r.last_x = r.alloc(c.d);
    int ns = std::max(1, std::min(16, 512 / c.heads));
    // attention scratch: the split records of one row (decode paths) or of a short prompt whose key rounds are shared
    int64_t sf = (int64_t)c.heads * ns * (hd + 4);
    for (int rows = 2; rows <= 32; rows++) sf = std::max(sf, deepj_hip_attention_scratch_floats(rows, c.heads, hd, c.max_seq));
    r.scratch = r.alloc(sf);
    r.records = r.alloc((int64_t)c.heads * deepj_hip_attn_record_splits() * (hd + 4));
    Stream s;
    emit(s, DJ_OP_FILL, r.state, 0, 4);
    r.run(s);
    alloc_acts(r, r.dec, 1);
    // the prompt-sized buffers for the longest prompt the cache can take, so that no request pays for allocation
    alloc_acts(r, r.pre, c.max_seq);
    r.finalized = true;
    warm_up(r);
}

// ── command streams ────────────────────────────────────────────────────────

// One transformer block on S rows held in a.x; result back in a.x.
void block_stream(Runner &r, Stream &s, Acts &a, int l, int S) {
    const Config &c = r.cfg;
    const Layer &L = r.layers[l];
    const int d = c.d, H = c.heads, hd = r.hd();
    bool wo_done = false, rope_fused = false;
    // a prompt's q | k | v projection takes RoPE and the cache append as its epilogue where the library has that kernel
    auto fuse_rope = [&](int k_in) { return !c.latent && !(S == 1 && &a == &r.dec) && S > 1 && deepj_hip_q8_linear_rope_ok(S, k_in, d) != 0; };
    // x2 = x + Wo . attention(RoPE(split(norm1(x) . [Wq|Wk|Wv])))      LlamaTransformerBlock.java:51
    // GPT: LayerNorm instead of RMSNorm and no rotation                  GPTTransformerBlock.java:66-68
    // DeepSeek: [Q|K|V] = ([cQ|cKV] = norm1(x).[Wdq|Wdkv]) . blockdiag(Wuq, [Wuk|Wuv])   MultiHeadLatentAttention.java:92-123
    if (c.latent) {
        // cQ = norm1(x).Wdq, Q = cQ.Wuq, cKV = norm1(x).Wdkv appended to the layer's latent rows; then, for ALL
        // cached positions, [K | V] = cKV.[Wuk | Wuv] (the row count lives on the device), RoPE on the K halves and
        // on Q, attention over the token-major rows (MultiHeadLatentAttention.java:92-123).
        const int qr = c.q_rank, kvr = c.kv_rank;
        const int64_t lat_off = (int64_t)l * c.max_seq * kvr;
        q8_linear(s, a.x, L.wdq, a.cq, S, d, qr, DJ_LIN_RMSNORM, L.g1);
        q8_linear(s, a.cq, L.wuq, a.qkv, S, qr, d, 0);
        q8_linear(s, a.x, L.wdkv, a.ckv, S, d, kvr, DJ_LIN_RMSNORM, L.g1);
        emit(s, DJ_OP_APPEND_ROWS, a.ckv, r.latent, r.state, S, kvr, c.max_seq, lat_off);
        emit(s, DJ_OP_Q8_LINEAR_DYN, r.latent, L.wukv, r.kv_all, c.max_seq, kvr, 2 * d, r.state, S, lat_off);
        emit(s, DJ_OP_ROPE_ROWS, r.kv_all, r.kv_all, r.state, r.cos_t, r.sin_t, c.max_seq, H, hd, c.max_seq, 1, 2 * d, S);
        emit(s, DJ_OP_ROPE_ROWS, a.qkv, a.q, r.state, r.cos_t, r.sin_t, S, H, hd, c.max_seq, 0, 0, -1);
        emit(s, DJ_OP_ATTENTION_KV, a.q, r.kv_all, r.kv_all, a.att, r.state, r.scratch, S, H, hd, c.max_seq, 0, 2 * d, d);
        q8_linear(s, a.att, L.wo, a.x2, S, d, d, DJ_LIN_RESIDUAL, -1, -1, -1, a.x);
        wo_done = true;
    } else if (c.kind == 1) {
        const int k2 = r.latent_width();
        q8_linear(s, a.x, L.wdown, a.cq, S, d, k2, DJ_LIN_RMSNORM, L.g1);
        if (!(rope_fused = fuse_rope(k2))) q8_linear(s, a.cq, L.wup, a.qkv, S, k2, 3 * d, 0);
        else emit(s, DJ_OP_Q8_LINEAR_ROPE, a.cq, L.wup, a.q, S, k2, d, 0, -1, -1, -1, r.kc, r.vc, r.state, r.cos_t, r.sin_t, H, hd, c.max_seq, l);
    } else if (c.kind == 2) {
        if (!(rope_fused = fuse_rope(d))) q8_linear(s, a.x, L.wqkv, a.qkv, S, d, 3 * d, DJ_LIN_LAYERNORM, L.g1, -1, L.be1);
        else emit(s, DJ_OP_Q8_LINEAR_ROPE, a.x, L.wqkv, a.q, S, d, d, DJ_LIN_LAYERNORM, L.g1, -1, L.be1, r.kc, r.vc, r.state, r.cos_t, r.sin_t, H, hd, c.max_seq, l);
    } else {
        if (!(rope_fused = fuse_rope(d))) q8_linear(s, a.x, L.wqkv, a.qkv, S, d, 3 * d, DJ_LIN_RMSNORM, L.g1);
        else emit(s, DJ_OP_Q8_LINEAR_ROPE, a.x, L.wqkv, a.q, S, d, d, DJ_LIN_RMSNORM, L.g1, -1, -1, r.kc, r.vc, r.state, r.cos_t, r.sin_t, H, hd, c.max_seq, l);
    }
    if (c.latent) {
        // attention and Wo were emitted above
    } else if (S == 1 && &a == &r.dec) {
        // the key splits' records go straight to the Wo matvec, whose prologue merges them
        emit(s, DJ_OP_ATTN_DECODE_RECORDS, a.qkv, r.kc, r.vc, r.records, r.state, r.cos_t, r.sin_t, H, hd, c.max_seq, l);
        emit(s, DJ_OP_Q8_LINEAR, r.records, L.wo, a.x2, 1, d, d, DJ_LIN_RESIDUAL | DJ_LIN_ATTN_MERGE, hd, -1, -1, a.x);
        wo_done = true;
    } else {
        if (!rope_fused) emit(s, DJ_OP_ROPE_KV_STORE, a.qkv, a.q, r.kc, r.vc, r.state, r.cos_t, r.sin_t, S, H, hd, c.max_seq, l);
        emit(s, DJ_OP_ATTENTION, a.q, r.kc, r.vc, a.att, r.state, r.scratch, S, H, hd, c.max_seq, l);
    }
    if (!wo_done) q8_linear(s, a.att, L.wo, a.x2, S, d, d, DJ_LIN_RESIDUAL, -1, -1, -1, a.x);
    if (c.kind == 2) {
        // x = x2 + W2 . GELU(W1 . ln2(x2) + b1) + b2                        GPTTransformerBlock.java:70-72, FNN.java:57-73
        q8_linear(s, a.x2, L.wgu, a.ff, S, d, c.dff, DJ_LIN_LAYERNORM | DJ_LIN_BIAS | DJ_LIN_GELU, L.g2, L.bg, L.be2);
        q8_linear(s, a.ff, L.wd, a.x, S, c.dff, d, DJ_LIN_BIAS | DJ_LIN_RESIDUAL, -1, L.bd, -1, a.x2);
        return;
    }
    // x = x2 + down(SiLU(gate(norm2(x2))) * up(norm2(x2)))                  LlamaTransformerBlock.java:52
    q8_linear(s, a.x2, L.wgu, a.ff, S, d, c.dff, DJ_LIN_RMSNORM | DJ_LIN_BIAS | DJ_LIN_SWIGLU, L.g2, L.bg, L.bu);
    q8_linear(s, a.ff, L.wd, a.x, S, c.dff, d, DJ_LIN_BIAS | DJ_LIN_RESIDUAL, -1, L.bd, -1, a.x2);
}

// logits = lmHead(normF(x)) on `rows` rows                                   DecoderOnlyModel.java:62-63
void head_rows(Runner &r, Stream &s, int32_t x, int32_t out, int rows) {
    const Config &c = r.cfg;
    if (c.kind == 2) q8_linear(s, x, r.wlm, out, rows, c.d, c.vocab, DJ_LIN_LAYERNORM | DJ_LIN_BIAS, r.gf, r.blm, r.bf);
    else q8_linear(s, x, r.wlm, out, rows, c.d, c.vocab, DJ_LIN_RMSNORM | DJ_LIN_BIAS, r.gf, r.blm);
}
void head_stream(Runner &r, Stream &s, int32_t x_row) { head_rows(r, s, x_row, r.logits, 1); }

// GPT: the token rows in x (first one at position state[0]) get their learned position rows added
// (GPTModel.java:52-54).
void positions(Runner &r, Stream &s, int32_t x, int rows) {
    const Config &c = r.cfg;
    if (c.kind == 2) emit(s, DJ_OP_ADD_POSITIONS, x, r.pos_table, r.state, rows, c.d, c.max_seq);
}

Stream decode_stream(Runner &r, bool sample_on_device) {
    const Config &c = r.cfg;
    Stream s;
    // Greedy on the device: the previous step (or the prefill) already left the embedding of
    // the token to process in dec.x.  Host sampling: gather it from state[1] first.
    if (!sample_on_device) {
        emit(s, DJ_OP_EMBED_GATHER, r.emb, r.state, r.dec.x, 1, c.d, c.vocab, 1);
        positions(r, s, r.dec.x, 1);
    }
    for (int l = 0; l < c.layers; l++) block_stream(r, s, r.dec, l, 1);
    head_stream(r, s, r.dec.x);
    if (sample_on_device) {
        emit(s, DJ_OP_DECODE_NEXT, r.logits, r.state, r.tokens, c.max_seq, r.emb, r.dec.x, c.vocab, c.d, 1);
        positions(r, s, r.dec.x, 1);        // state[0] is already the position of the token just chosen
    }
    return s;
}

// A prompt of some length runs its projections on the GEMM that loads fp16 weights straight into LDS.  The first such
// prompt writes the weights once in that layout (about 2 bytes per weight more, kept until the runner goes) instead of every
// call converting them into the workspace - layer by layer while the byte budget lasts; the layers past it convert on
// every call (same results, 40 us or so per layer and prompt slower).  (finalize()'s warm-up pass runs long prompts
// when maxSeqLen allows them, so with the warm-up on the copies exist from the start.)
void ensure_prepared(Runner &r, int n) {
    if (r.prepared_done || n < 64) return;      // (with the copies in place the GEMM takes prompts from 16 rows on where its plan says so)
    r.prepared_done = true;
    const Config &c = r.cfg;
    const int d = c.d;
    Stream s;
    bool room = true;
    auto prepare = [&](int32_t w, int k, int rows) {
        int32_t tile_rows = 0;      // would the longest prompt reach the fp16 GEMM with a copy in place?
        deepj_hip_q8_gemm_tile_prepared(c.max_seq, k, rows, &tile_rows, nullptr, nullptr);
        if (!room || w < 0 || !tile_rows) return;
        const int64_t floats = deepj_hip_q8_prepared_floats(k, rows);
        if (r.prepared_budget >= 0 && r.prepared_bytes + 4 * floats > r.prepared_budget) { room = false; return; }
        int32_t p = r.alloc(floats);
        r.prepared.push_back(p);
        r.prepared_bytes += 4 * floats;
        emit(s, DJ_OP_Q8_PREPARE, w, p, k, rows);
    };
    for (const Layer &L : r.layers) {
        prepare(L.wqkv, d, 3 * d);
        prepare(L.wo, d, d);
        prepare(L.wgu, d, c.kind == 2 ? c.dff : 2 * c.dff);
        prepare(L.wd, c.dff, d);
    }
    if (!s.empty()) r.run(s);
}

void release_prepared(Runner &r) {
    for (int32_t &id : r.prepared) r.release(id);
    r.prepared.clear();
    r.prepared_bytes = 0;
    r.prepared_done = false;
}

void check_ids(const Config &c, const int32_t *ids, int n) {
    for (int i = 0; i < n; i++)
        if (ids[i] < 0 || ids[i] >= c.vocab) throw Error("Token id out of range: " + std::to_string(ids[i]));   // Embedding.java:30-32
}

// The command stream that takes the n token ids in r.pre.ids through the model at the current position.
Stream prompt_stream(Runner &r, int n, bool choose) {
    const Config &c = r.cfg;
    alloc_acts(r, r.pre, n);
    ensure_prepared(r, n);
    Stream s;
    emit(s, DJ_OP_EMBED_GATHER, r.emb, r.pre.ids, r.pre.x, n, c.d, c.vocab, 0);
    positions(r, s, r.pre.x, n);
    for (int l = 0; l < c.layers; l++) block_stream(r, s, r.pre, l, n);
    emit(s, DJ_OP_COPY, r.pre.x, r.last_x, c.d, (int64_t)(n - 1) * c.d, 0);
    head_stream(r, s, r.last_x);
    if (choose) {
        emit(s, DJ_OP_DECODE_NEXT, r.logits, r.state, r.tokens, c.max_seq, r.emb, r.dec.x, c.vocab, c.d, n);
        if (r.pos + n < c.max_seq) positions(r, s, r.dec.x, 1);     // a full cache takes no further token
    }
    return s;
}

// Runs the prompt rows through the model, filling the cache.  Leaves the last row's
// logits in r.logits; with choose != 0 also picks the next token greedily on the device.
void prefill(Runner &r, const int32_t *ids, int n, float *all_logits, bool choose) {
    const Config &c = r.cfg;
    if (!r.finalized) finalize(r);
    if (n <= 0) throw Error("prefill: empty prompt");
    check_ids(c, ids, n);
    if (r.pos + n > c.max_seq)
        throw Error("context of " + std::to_string(r.pos + n) + " tokens exceeds maxSeqLen " + std::to_string(c.max_seq));
    Stream s = prompt_stream(r, n, choose);
    hip(deepj_hip_upload(r.pre.ids, reinterpret_cast<const float *>(ids), n));   // (prompt_stream sized r.pre for n rows)
    r.run(s);
    if (all_logits) {
        // DecoderOnlyModel.forward returns logits for every row; only parity tests ask for them.
        int32_t full = r.alloc((int64_t)n * c.vocab);
        Stream t;
        head_rows(r, t, r.pre.x, full, n);
        r.run(t);
        hip(deepj_hip_download(full, all_logits, (int64_t)n * c.vocab));
        r.release(full);
    }
    if (choose) { r.pos += n; r.generated += 1; }
    else {
        // advance the position without choosing a token
        int32_t st[4] = {r.pos + n, 0, r.generated, 0};
        hip(deepj_hip_upload(r.state, reinterpret_cast<const float *>(st), 4));
        r.pos += n;
    }
}

void reset(Runner &r) {
    if (!r.finalized) finalize(r);
    int32_t st[4] = {0, 0, 0, 0};
    hip(deepj_hip_upload(r.state, reinterpret_cast<const float *>(st), 4));
    r.pos = 0;
    r.generated = 0;
}

// The runtime builds a kernel's function object on its first launch (a few hundred microseconds each), and the
// decode graphs are captured on first use.  One pass over prompts of the lengths that select the different GEMM and
// attention variants, and a few graph-replayed tokens, move those costs from the first request to finalize();
// the sequence state is cleared afterwards (the cache rows written here are never read: every row is rewritten
// before the position counter reaches it).
void decode_greedy(Runner &r, int steps, int mode);
void warm_up(Runner &r) {
    const Config &c = r.cfg;
    const char *env = getenv("DEEPJ_HIP_WARMUP");           // "0": skip (profiling runs that want only the request's launches)
    if (env && env[0] == '0') return;
    std::vector<int32_t> ids((size_t)std::min(c.max_seq, 2048), 0);
    for (int n : {2048, 1024, 512, 256, 128, 64, 32, 16, 4}) {
        if (n > (int)ids.size()) continue;
        reset(r);
        prefill(r, ids.data(), n, nullptr, true);
    }
    reset(r);
    const int steps = kGraphUnroll + 1;
    if (c.max_seq >= steps + 2) {
        prefill(r, ids.data(), 1, nullptr, true);
        decode_greedy(r, steps, 1);
    }
    reset(r);
}

// Greedy steps on the device: each consumes state[1] at position state[0] and appends the argmax.
// mode 0: the per-token stream, eagerly; 1: the same stream as a replayed HIP graph.
void decode_greedy(Runner &r, int steps, int mode) {
    const Config &c = r.cfg;
    if (steps <= 0) return;
    if (r.pos + steps > c.max_seq)
        throw Error("context of " + std::to_string(r.pos + steps) + " tokens exceeds maxSeqLen " + std::to_string(c.max_seq));
    const bool use_graph = mode == 1;
    if (use_graph) {
        // A replay costs a few microseconds of its own on top of its kernels: long runs go through a graph
        // that holds kGraphUnroll consecutive tokens, the remainder through the one-token graph.
        const int runs = steps / kGraphUnroll, rest = steps % kGraphUnroll;
        if (runs > 0) {
            if (!r.graph_unrolled) {
                Stream one = decode_stream(r, true), s;
                for (int i = 0; i < kGraphUnroll; i++) s.insert(s.end(), one.begin(), one.end());
                hip(deepj_hip_graph_capture(s.data(), (int32_t)s.size(), &r.graph_unrolled));
            }
            hip(deepj_hip_graph_launch(r.graph_unrolled, runs));
        }
        if (rest > 0) {
            if (!r.graph) {
                Stream s = decode_stream(r, true);
                hip(deepj_hip_graph_capture(s.data(), (int32_t)s.size(), &r.graph));
            }
            hip(deepj_hip_graph_launch(r.graph, rest));
        }
    } else {
        Stream s = decode_stream(r, true);
        for (int i = 0; i < steps; i++) r.run(s);
    }
    r.pos += steps;
    r.generated += steps;
}

// One token through the single-row path with the token chosen by the caller: logits of the
// new position end up in r.logits.  (Incremental decode with sampling done elsewhere.)
void step_token(Runner &r, int32_t token) {
    const Config &c = r.cfg;
    if (!r.finalized) finalize(r);
    check_ids(c, &token, 1);
    if (r.pos + 1 > c.max_seq)
        throw Error("context of " + std::to_string(r.pos + 1) + " tokens exceeds maxSeqLen " + std::to_string(c.max_seq));
    int32_t st[4] = {r.pos, token, r.generated, 0};
    hip(deepj_hip_upload(r.state, reinterpret_cast<const float *>(st), 4));
    Stream fwd = decode_stream(r, false);
    r.run(fwd);
    r.pos += 1;
    st[0] = r.pos;
    hip(deepj_hip_upload(r.state, reinterpret_cast<const float *>(st), 4));
}

// ── TextGenerator.sampleFromLogits on the host (temperature / top-k > 1) ────

int java_float_compare(float x, float y) {
    if (x < y) return -1;
    if (x > y) return 1;
    int32_t bx, by;
    std::memcpy(&bx, &x, 4); std::memcpy(&by, &y, 4);
    if (x != x) bx = 0x7fc00000;
    if (y != y) by = 0x7fc00000;
    return bx == by ? 0 : (bx < by ? -1 : 1);
}

int32_t sample_from_logits(const std::vector<float> &logits, float temperature, int top_k, void *rng) {
    int n = (int)logits.size();
    std::vector<int32_t> order(n);
    for (int i = 0; i < n; i++) order[i] = i;
    // stable sort, descending (TextGenerator.java:163-170)
    std::stable_sort(order.begin(), order.end(),
                     [&](int32_t i, int32_t j) { return java_float_compare(logits[j], logits[i]) < 0; });
    int k = top_k == 0 ? n : std::min(top_k, n);
    float mx = -INFINITY;
    for (int i = 0; i < k; i++) mx = std::max(mx, logits[order[i]] / temperature);
    std::vector<float> probs(k);
    float sum = 0.0f;
    for (int i = 0; i < k; i++) {
        float p = (float)std::exp((double)(logits[order[i]] / temperature - mx));
        probs[i] = p;
        sum += p;
    }
    for (float &p : probs) p /= sum;
    float u = deepj_host_random_next_float(rng), cum = 0.0f;
    for (int i = 0; i < k; i++) {
        cum += probs[i];
        if (u <= cum) return order[i];
    }
    return order[k - 1];
}

// TextGenerator.generate on token ids (TextGenerator.java:66-87).  out holds n_prompt + max_new ids.
//
// Token t is drawn from the logits of the last row of forward(last(ids, maxSeqLen)) (TextGenerator.java:91-100,
// 172-175).  While the whole sequence fits the window its rows keep their positions, so the KV cache serves them;
// once it is longer the window slides by one per token and every row's position changes, so each further token is
// a fresh forward of the maxSeqLen-row window - what the reference does for every token.
void generate(Runner &r, const int32_t *prompt, int n_prompt, int max_new, float temperature, int top_k,
              int64_t seed, int32_t *out, int mode) {
    const Config &c = r.cfg;
    if (max_new < 0) throw Error("maxNewTokens must be >= 0");
    if (!(temperature > 0.0f)) throw Error("temperature must be > 0");
    if (top_k < 0) throw Error("topK must be >= 0");
    if (n_prompt <= 0 && max_new > 0) throw Error("prefill: empty prompt");
    check_ids(c, prompt, n_prompt);
    std::memcpy(out, prompt, (size_t)n_prompt * sizeof(int32_t));
    if (max_new == 0) return;
    // tokens 0 .. cached-1 see a context that fits the window (n_prompt + t <= maxSeqLen)
    const int cached = n_prompt > c.max_seq ? 0 : std::min(max_new, c.max_seq - n_prompt + 1);
    const bool greedy = top_k == 1;       // argmax needs no random draw to pick, and greedy output is seed independent
    void *rng = greedy ? nullptr : deepj_host_random_create(seed);
    try {
        std::vector<float> logits(greedy ? 0 : (size_t)c.vocab);
        auto sample = [&](int t) {
            hip(deepj_hip_download(r.logits, logits.data(), c.vocab));
            out[n_prompt + t] = sample_from_logits(logits, temperature, top_k, rng);
        };
        reset(r);
        if (cached > 0 && greedy) {
            prefill(r, prompt, n_prompt, nullptr, true);
            decode_greedy(r, cached - 1, mode);
            hip(deepj_hip_download(r.tokens, reinterpret_cast<float *>(out + n_prompt), cached));
        } else if (cached > 0) {
            Stream fwd = decode_stream(r, false);
            prefill(r, prompt, n_prompt, nullptr, false);
            for (int t = 0; t < cached; t++) {
                if (t > 0) {
                    r.run(fwd);          // consumes the token in state[1] at position state[0]
                    r.pos += 1;
                }
                sample(t);
                int32_t st[4] = {r.pos, out[n_prompt + t], t + 1, 0};
                hip(deepj_hip_upload(r.state, reinterpret_cast<const float *>(st), 4));
                r.generated = t + 1;
            }
        }
        for (int t = cached; t < max_new; t++) {
            reset(r);
            prefill(r, out + n_prompt + t - c.max_seq, c.max_seq, nullptr, greedy);
            if (greedy) hip(deepj_hip_download(r.tokens, reinterpret_cast<float *>(out + n_prompt + t), 1));
            else sample(t);
        }
    } catch (...) {
        if (rng) deepj_host_random_destroy(rng);
        throw;
    }
    if (rng) deepj_host_random_destroy(rng);
}

template <class F> int guarded(Runner *r, F &&f) {
    try {
        f();
        if (r) r->error.clear();
        return 0;
    } catch (const std::exception &ex) {
        if (r) r->error = ex.what();
        return 1;
    }
}

}  // namespace

extern "C" {

// cfg: {kind, vocab, maxSeq, dModel, nHeads, nLayers, dFF, qRank, kvRank}; id_base: first buffer id this
// runner may use (pick a range the ComputeGraph never reaches, e.g. 1 << 29).
void *deepj_runner_create(const int32_t cfg[9], int32_t id_base) {
    Config c{cfg[0], cfg[1], cfg[2], cfg[3], cfg[4], cfg[5], cfg[6], cfg[7], cfg[8]};
    if (c.kind == 3) { c.kind = 1; c.latent = true; }      // DeepSeek with the latent KV cache
    // TransformerConfig.validateCommon (models/TransformerConfig.java:19-31) + DeepSeekConfig.java:31-35
    if (c.vocab <= 0 || c.max_seq <= 0 || c.d <= 0 || c.heads <= 0 || c.layers <= 0 || c.dff <= 0) return nullptr;
    if (c.d % c.heads != 0) return nullptr;
    if (c.kind == 1 && (c.q_rank <= 0 || c.kv_rank <= 0)) return nullptr;
    if (c.kind < 0 || c.kind > 2) return nullptr;
    int hd = c.d / c.heads;
    if (hd != 32 && hd != 64 && hd != 128) return nullptr;
    auto *r = new Runner;
    r->cfg = c;
    r->next_id = id_base;
    r->layers.resize((size_t)c.layers);
    return r;
}

void deepj_runner_destroy(void *h) {
    auto *r = static_cast<Runner *>(h);
    if (!r) return;
    if (r->graph) deepj_hip_graph_destroy(r->graph);
    if (r->graph_unrolled) deepj_hip_graph_destroy(r->graph_unrolled);
    deepj_hip_synchronize();
    // every id in [id_base, next_id) that is still live belongs to this runner
    std::vector<int32_t> ids;
    auto add = [&](int32_t id) { if (id >= 0) ids.push_back(id); };
    for (auto &L : r->layers)
        for (int32_t id : {L.g1, L.g2, L.be1, L.be2, L.wqkv, L.wo, L.wdown, L.wup, L.wdq, L.wuq, L.wdkv, L.wukv, L.wgu, L.bg,
                           L.bu, L.wd, L.bd})
            add(id);
    for (int32_t id : {r->emb, r->gf, r->wlm, r->blm, r->cos_t, r->sin_t, r->kc, r->vc, r->state,
                       r->tokens, r->scratch, r->records, r->logits, r->last_x,
                       r->pos_table, r->bf, r->latent, r->kv_all})
        add(id);
    for (Acts *a : {&r->dec, &r->pre})
        for (int32_t id : {a->x, a->x2, a->qkv, a->q, a->att, a->ff, a->ids, a->cq, a->ckv}) add(id);
    for (int32_t id : r->prepared) add(id);
    if (!ids.empty()) deepj_hip_release(ids.data(), (int32_t)ids.size());
    delete r;
}

const char *deepj_runner_last_error(void *h) { return h ? static_cast<Runner *>(h)->error.c_str() : "null runner"; }

int deepj_runner_set_weight(void *h, const char *name, const float *data, int32_t rows, int32_t cols) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] { set_weight(*r, name, data, rows, cols); });
}

int deepj_runner_init_seeded(void *h, int64_t seed, int32_t threads) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        if (r->cfg.kind == 2) throw Error("a GPT model is seeded through deepj_runner_init_seeded_gpt (it needs initScale)");
        init_seeded(*r, seed, threads, 1.0f);
    });
}

int deepj_runner_init_seeded_gpt(void *h, int64_t seed, float init_scale, int32_t threads) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        if (r->cfg.kind != 2) throw Error("deepj_runner_init_seeded_gpt: not a GPT model");
        if (!std::isfinite(init_scale) || init_scale <= 0.0f) throw Error("initScale must be finite and > 0");   // GPTConfig.java:22-23
        init_seeded(*r, seed, threads, init_scale);
    });
}

// Bytes the runner may spend on fp16 copies of its weights for the many-row (prompt) GEMM: -1 no limit (every layer:
// + 2 bytes per weight), 0 none (every call converts into the workspace), otherwise layers in order while the budget
// lasts.  Copies held under an earlier budget are released; the next long prompt prepares anew.  Results do not
// depend on it.
int deepj_runner_set_prepared_budget(void *h, int64_t bytes) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        if (bytes < -1) throw Error("prepared-weight budget must be -1 (no limit) or a byte count");
        release_prepared(*r);
        r->prepared_budget = bytes;
    });
}

int64_t deepj_runner_prepared_bytes(void *h) { return h ? static_cast<Runner *>(h)->prepared_bytes : 0; }

int deepj_runner_finalize(void *h) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] { finalize(*r); });
}

int deepj_runner_reset(void *h) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] { reset(*r); });
}

// all_logits: null, or room for n*vocab floats (logits of every prompt row, as DecoderOnlyModel.forward returns)
int deepj_runner_prefill(void *h, const int32_t *ids, int32_t n, float *all_logits, int32_t choose_next) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] { prefill(*r, ids, n, all_logits, choose_next != 0); });
}

int deepj_runner_decode(void *h, int32_t steps, int32_t mode) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        if (mode < 0 || mode > 1) throw Error("decode: mode must be 0 (eager) or 1 (graph)");
        decode_greedy(*r, steps, mode);
    });
}

int deepj_runner_step(void *h, int32_t token) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] { step_token(*r, token); });
}

int deepj_runner_last_logits(void *h, float *out) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        hip(deepj_hip_download(r->logits, out, r->cfg.vocab));
    });
}

// tokens generated so far in this sequence (device order); returns the count through *n
int deepj_runner_tokens(void *h, int32_t *out, int32_t capacity, int32_t *n) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        int32_t count = std::min(r->generated, capacity);
        if (count > 0) hip(deepj_hip_download(r->tokens, reinterpret_cast<float *>(out), count));
        else hip(deepj_hip_synchronize());
        if (n) *n = count;
    });
}

int deepj_runner_generate(void *h, const int32_t *prompt, int32_t n_prompt, int32_t max_new, float temperature,
                          int32_t top_k, int64_t seed, int32_t mode, int32_t *out) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        if (mode < 0 || mode > 1) throw Error("generate: mode must be 0 (eager) or 1 (graph)");
        generate(*r, prompt, n_prompt, max_new, temperature, top_k, seed, out, mode);
    });
}

// The command stream of an n-token prompt at the current position, over the ids of the last prefill of that length
// (for inspection and timing by the caller; running it advances nothing on the host side).
int deepj_runner_prefill_stream(void *h, int32_t n, int32_t *out, int32_t capacity, int32_t *len) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        if (!r->finalized) finalize(*r);
        if (n <= 0 || r->pos + n > r->cfg.max_seq) throw Error("prefill_stream: row count outside the context window");
        Stream s = prompt_stream(*r, n, false);
        if (len) *len = (int32_t)s.size();
        if (out && capacity >= (int32_t)s.size()) std::memcpy(out, s.data(), s.size() * sizeof(int32_t));
    });
}

// The per-token command stream (for inspection, timing and graph capture by the caller).
int deepj_runner_decode_stream(void *h, int32_t *out, int32_t capacity, int32_t *len) {
    auto *r = static_cast<Runner *>(h);
    return guarded(r, [&] {
        if (!r->finalized) finalize(*r);
        Stream s = decode_stream(*r, true);
        if (len) *len = (int32_t)s.size();
        if (out && capacity >= (int32_t)s.size()) std::memcpy(out, s.data(), s.size() * sizeof(int32_t));
    });
}

}  // extern "C"
