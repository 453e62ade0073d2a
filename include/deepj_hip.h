/*
 * deepj_hip.h - C ABI of libdeepj_hip.so, the MI355X (gfx950) device runtime
 * behind DeepJ's GpuRuntime boundary.
 *
 * Every function returns 0 on success and a non-zero code on failure; the
 * message is then available from deepj_hip_last_error().  Nothing throws
 * across this boundary.  A single caller thread is assumed, as in the
 * reference (its ComputeGraph and native pool are unsynchronised globals:
 * src/main/java/io/github/kirstenali/deepj/tensor/ComputeGraph.java:67-78,
 * native/deepj_metal_jni.mm:63,1358).
 *
 * Paths cited below are relative to the reference tree:
 *   J/ = src/main/java/io/github/kirstenali/deepj/
 */
#ifndef DEEPJ_HIP_H
#define DEEPJ_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ── the five GpuRuntime calls (J/tensor/GpuRuntime.java:9-28) ─────────────
 * These are what HipNative's five `static native` methods bind, one to one,
 * the way J/tensor/metal/MetalNative.java:41-57 binds the Metal library. */

/* GpuRuntime.allocBuffers (native/deepj_metal_jni.mm:1480-1505).
 * sizes are in floats.  Allocating an id that already exists is a no-op. */
int deepj_hip_alloc_buffers(const int32_t *ids, const int32_t *sizes_in_floats, int32_t count);

/* GpuRuntime.uploadBuffer (deepj_metal_jni.mm:1509-1521).  Copies n floats
 * (the Java array length) into the buffer; src is only borrowed for the
 * call.  Unknown id: error "Buffer not found for upload". */
int deepj_hip_upload(int32_t id, const float *src, int64_t n);

/* GpuRuntime.downloadBuffer (deepj_metal_jni.mm:1525-1537).  Waits for all
 * work queued so far, then copies n floats out.  This is the only call that
 * synchronises with the device.  Unknown id: "Buffer not found for download". */
int deepj_hip_download(int32_t id, float *dst, int64_t n);

/* GpuRuntime.releaseBuffers (deepj_metal_jni.mm:1541-1549).  Unknown ids are
 * ignored.  Memory returns to the size-class cache, not to the driver. */
int deepj_hip_release(const int32_t *ids, int32_t count);

/* GpuRuntime.flushOps (deepj_metal_jni.mm:1554-2140).  Executes the int32
 * command stream recorded by ComputeGraph (opcodes 1..42 exactly as encoded
 * by J/tensor/ComputeGraph.java:260-518) plus the fused inference opcodes
 * listed below.  The whole stream is validated first (opcode, stride, buffer
 * ids, sizes); on error nothing is launched.  An unknown opcode N fails with
 * "Unknown op code in graph: N" (deepj_metal_jni.mm:2120-2121).  The call
 * only enqueues work: results are observable through deepj_hip_download. */
int deepj_hip_flush_ops(const int32_t *cmd, int32_t len);

/* deepj_hip_flush_ops for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same streams and
 * the same kernels and bits as deepj_hip_flush_ops, with ONE exception: a Q8_LINEAR of more than one row always
 * runs as a single launch of the bf16 GEMM here, where flush_ops - with a workspace sized by the shape - takes
 * the fp16 GEMM (256 rows and more - 16 and more with prepared weights - and enough tiles) or lets several workgroups
 * share a tile's K (few tiles, long K); both meet the per-op tolerance against the CPU backend, their bits differ.  The
 * device scratch the kernels need - the workspace that Q8_LINEAR with a norm
 * prologue and M > 1 writes its normalised rows to, and the arrival counters of the split decode attention
 * (ATTENTION / ATTENTION_KV with S = 1, ATTN_DECODE) - is a fixed array inside the library's code object instead
 * of memory the runtime allocates and grows.  The call never calls hipMalloc or hipFree: it fails when the
 * runtime is not initialised yet (deepj_hip_init allocates), when the stream needs more than
 * DEEPJ_HIP_NOALLOC_WORKSPACE_FLOATS floats of workspace (M * K of the largest such Q8_LINEAR).
 * Every buffer the stream names must already exist.  All calls on a GPU share the one array,
 * which keeps the previous call's contents (the counters are cleared by a kernel at the start of each call);
 * calls that overlap on one GPU would race - the single-caller rule above already excludes that. */
#define DEEPJ_HIP_NOALLOC_WORKSPACE_FLOATS (2 << 20)
int deepj_hip_flush_ops_noalloc(const int32_t *cmd, int32_t len);

/* Message of the last failure on this thread ("" if none). */
const char *deepj_hip_last_error(void);

/* ── runtime control (no counterpart in the reference: Metal's context is
 * created lazily, deepj_metal_jni.mm:909-984) ──────────────────────────── */
int deepj_hip_init(int32_t device);        /* optional; first use initialises device 0 */
int deepj_hip_synchronize(void);
int deepj_hip_shutdown(void);              /* frees every buffer and the cache */
int deepj_hip_trim(void);                  /* returns cached (released) memory to the driver */
/* out[0]=live buffers, out[1]=live bytes, out[2]=cached bytes, out[3]=driver allocations so far */
int deepj_hip_pool_stats(int64_t out[4]);
/* The HIP stream all work is queued on, as a hipStream_t, for callers that time with HIP events. */
void *deepj_hip_stream(void);

/* Times `iters` back-to-back executions of a validated stream with HIP events
 * recorded on the library's stream; *ms_total receives the elapsed time. */
int deepj_hip_time_ops(const int32_t *cmd, int32_t len, int32_t iters, float *ms_total);

/* Runs a validated stream `iters` times in order with a start and a stop event attached to every kernel dispatch
 * of every op: us_per_op[i] receives the mean over the passes of the summed begin-to-end times of op i's
 * dispatches on the device, in microseconds - the durations a kernel trace reports, helpers of the op included
 * (-1 for an op that launched nothing).  us_longest (optional, same length): the op's longest single dispatch, its
 * main kernel; dispatches (optional): how many the op made.  *n_ops = ops in the stream; fails when capacity is
 * smaller. */
int deepj_hip_profile_ops(const int32_t *cmd, int32_t len, int32_t iters, float *us_per_op, int32_t capacity,
                          int32_t *n_ops, float *us_longest, int32_t *dispatches);
/* Measurement aid, no counterpart in the reference: the shader clock while a stream runs.  A one-wavefront kernel on a
 * second stream writes `samples` pairs (shader clock counter, 100 MHz wall clock) into pairs[2 * samples], sleeping
 * sleep_reps x 127 x 64 clocks between two samples, while `cmd` runs `iters` times on the library's stream;
 * window[0..1] are the wall clock before and after those runs.  Clock over an interval = counter difference / wall
 * difference x 100 MHz.  The sampler ends by itself; the call returns when both streams are idle. */
int deepj_hip_clock_probe(const int32_t *cmd, int32_t len, int32_t iters, int32_t samples, int32_t sleep_reps,
                          uint64_t *pairs, uint64_t *window);

/* Captures a command stream into a HIP graph (no allocation may be pending:
 * every buffer it names must exist) and replays it.  Used for the per-token
 * decode stream, whose position and token live in device memory.  A graph replays raw addresses: graph_launch fails,
 * launching nothing, once a buffer the stream names was released or reallocated, the workspace it used was replaced, or
 * Q8 weights it read through a prepared copy (DJ_OP_Q8_PREPARE) were written again - capture the stream again then. */
int deepj_hip_graph_capture(const int32_t *cmd, int32_t len, int32_t *handle);
int deepj_hip_graph_launch(int32_t handle, int32_t times);
int deepj_hip_graph_destroy(int32_t handle);

/* ── opcodes ──────────────────────────────────────────────────────────── */
/* 1..42: J/tensor/ComputeGraph.java:19-60 (same numbers, same encodings). */
enum {
    DJ_OP_ADD = 1, DJ_OP_SUBTRACT = 2, DJ_OP_MULTIPLY = 3, DJ_OP_DIVIDE = 4, DJ_OP_MATMUL = 5,
    DJ_OP_MULTIPLY_SCALAR = 6, DJ_OP_SQRT = 7, DJ_OP_NEG = 8, DJ_OP_EXP = 9, DJ_OP_LOG = 10,
    DJ_OP_TANH = 11, DJ_OP_SIGMOID = 12, DJ_OP_RELU = 13, DJ_OP_RELU_BACKWARD = 14, DJ_OP_GELU = 15,
    DJ_OP_GELU_BACKWARD = 16, DJ_OP_SOFTMAX_ROWS = 17, DJ_OP_SOFTMAX_BACKWARD = 18,
    DJ_OP_LAYERNORM_BACKWARD = 19, DJ_OP_ADAMW_UPDATE = 20, DJ_OP_ADD_SCALAR = 21,
    DJ_OP_DIVIDE_SCALAR = 22, DJ_OP_TRANSPOSE = 23, DJ_OP_ADD_ROW_VECTOR = 24,
    DJ_OP_ADD_BROADCAST_COLS = 25, DJ_OP_SUBTRACT_BROADCAST_COLS = 26, DJ_OP_DIVIDE_BROADCAST_COLS = 27,
    DJ_OP_MULTIPLY_BROADCAST_ROWS = 28, DJ_OP_SUM_ROWS = 29, DJ_OP_MEAN_ALONG_ROWS = 30,
    DJ_OP_VARIANCE_ALONG_ROWS = 31, DJ_OP_MULTIPLY_BROADCAST_COLS = 32, DJ_OP_SUM_ALONG_ROWS = 33,
    DJ_OP_MAX_ALONG_ROWS = 34, DJ_OP_CLAMP = 35, DJ_OP_POW = 36, DJ_OP_SCATTER_ADD_ROWS = 37,
    DJ_OP_SUM_ABS = 38, DJ_OP_CROSS_ENTROPY_LOSS = 39, DJ_OP_CROSS_ENTROPY_GRADIENT = 40,
    DJ_OP_SUM_SCALAR = 41, DJ_OP_SCATTER_ADD_ROWS_ATOMIC = 42,

    /* Fused inference opcodes.  The reference has none of these: it composes
     * them from primitives in Java (J/layers/transformer/norm/RMSNorm1D.java:46-57,
     * J/layers/transformer/SwiGLULayer.java:63-70, J/transformer/embeddings/
     * RotaryEmbedding.java:81-122, J/layers/transformer/attention/HeadOps.java:33-140).
     * Encodings (all words int32; "buf" = buffer id, -1 = absent):
     *
     * Q8_QUANTIZE   [op, src, dst, K, N, rowOff, rowStep, totalRows]
     *     src fp32 [K x N] (Linear weight orientation, J/layers/Linear.java:13);
     *     column n becomes Q8 row rowOff + n*rowStep of dst, which holds
     *     totalRows rows of Kp = roundup(K,32) int8 plus one fp32 scale per
     *     32-group.  dst must hold deepj_hip_q8_floats(K, totalRows) floats.
     * Q8_DEQUANTIZE [op, src, dst, K, N, rowOff, rowStep, totalRows]   inverse view, dst fp32 [K x N]
     * Q8_LINEAR     [op, x, w, out, M, K, N, flags, gamma, bias, bias2, residual]
     *     out[M x N] = f(x[M x K]) . W  (+ bias) (+ residual)
     *     flags bit0: RMSNorm prologue, f(x) = gamma * x / sqrt(mean(x^2)+1e-6)
     *           bit1: add bias[N]          bit2: add residual[M x N]
     *           bit3: SwiGLU: w has 2N rows (gate n at row 2n, up n at 2n+1),
     *                 out = SiLU(gate + bias) * (up + bias2)
     *           bit4: LayerNorm prologue, f(x) = (x - mean) / sqrt(var + 1e-5) * gamma + beta with the beta
     *                 buffer in the bias2 word (J/layers/transformer/norm/LayerNorm1D.java:34-66)
     *           bit5: GELU (tanh form) on x.W + bias, before the residual (J/activations/GELU.java:15-18)
     *           bit6: ATTN_MERGE prologue (M = 1): x is the records buffer ATTN_DECODE_RECORDS wrote, the gamma
     *                 word holds the head dim, K = H * hd; f(x) = the merged attention row
     *           bit3 excludes bits 2, 4, 5 and 6; bit0 excludes bit4; bit6 excludes bits 0, 4 and 5
     * RMSNORM       [op, x, gamma, out, rows, cols]
     * SILU_MUL      [op, gate, up, out, n]            out = gate*sigmoid(gate)*up
     * EMBED_GATHER  [op, table, ids, out, nIds, d, vocab, idsOff]  ids are int32 words
     * ROPE_KV_STORE [op, qkv, qOut, kCache, vCache, state, cosT, sinT, S, H, hd, maxSeq, layer]
     *     qkv [S x 3d]; rows sit at positions state[0]..state[0]+S-1
     * ATTENTION     [op, q, kCache, vCache, out, state, scratch, S, H, hd, maxSeq, layer]
     *     scratch (deepj_hip_attention_scratch_floats(S, H, hd, maxSeq) floats, no initialisation) is used by one
     *     row, whose keys are split over workgroups, and by 2 to 32 rows, whose key tiles are dealt to several
     *     workgroups per head (a short continuation of a long cached prefix would otherwise leave most of the chip idle)
     * ARGMAX_ROWS   [op, logits, out, rows, cols]      out int32 words, ties -> lowest index
     * DECODE_ADVANCE[op, state, token, tokens, capacity, nPos]
     *     state (int32 words): [0] positions held in the cache, [1] current token, [2] tokens generated;
     *     tokens[state[2]++] = token[0]; state[1] = token[0]; state[0] += nPos
     * COPY          [op, src, dst, n, srcOff, dstOff]
     * FILL          [op, dst, bits, n]
     * ROPE_ROWS     [op, x, out, state, cosT, sinT, rows, H, hd, maxSeq, posFromRow, rowStride, liveExtra]
     *     token-major rows rowStride floats apart (0 = H*hd); posFromRow: row i sits at position i, else at
     *     state[0]+i; liveExtra >= 0: only rows below state[0]+liveExtra are touched (-1 = all rows)
     * ATTENTION_KV  [op, q, k, v, out, state, scratch, S, H, hd, maxSeq, 0, tokStride, vOff]
     *     k, v token-major rows tokStride floats apart (0 = H*hd); values start vOff floats into buffer v
     * DECODE_NEXT   [op, logits, state, tokens, capacity, table, x, vocab, d, nPos]
     *     argmax + DECODE_ADVANCE + EMBED_GATHER of the chosen token into x, one launch
     * ATTN_DECODE   [op, qkv, kCache, vCache, out, state, scratch, cosT, sinT, H, hd, maxSeq, layer]
     *     ROPE_KV_STORE + ATTENTION for one new row (S = 1) in two launches
     * APPEND_ROWS   [op, src, dst, state, rows, rowFloats, maxRows, dstOff]
     *     dst[dstOff + (state[0]+i)*rowFloats ...] = src row i: append to a cache whose fill level is state[0]
     * Q8_LINEAR_DYN [op, x, w, out, Mmax, K, N, state, extraRows, xOff]
     *     Q8_LINEAR (no prologue/epilogue) on rows [0, min(Mmax, state[0]+extraRows)) of x + xOff: the row count
     *     lives on the device, so the op can sit in a replayed graph while a cache grows
     * ATTN_DECODE_RECORDS [op, qkv, kCache, vCache, records, state, cosT, sinT, H, hd, maxSeq, layer]
     *     ATTN_DECODE that stops before the merge of its key splits: records holds
     *     H * deepj_hip_attn_record_splits() * (hd + 4) floats, per (head, split) {max, sum, -, -, o[hd]} with the
     *     maximum in base-2 units (score * log2 e); a Q8_LINEAR with the ATTN_MERGE prologue consumes them.
     *     (Merging across workgroups inside one kernel costs three dependent trips to memory; across the
     *     kernel boundary it is free.)
     * LAYERNORM     [op, x, gamma, beta, out, rows, cols]      J/layers/transformer/norm/LayerNorm1D.java:34-66
     * ADD_POSITIONS [op, x, table, state, rows, d, maxSeq]
     *     x[i, :] += table[state[0] + i, :]: the learned positional rows of J/models/gpt/GPTModel.java:52-54 for
     *     rows that sit at positions state[0].. of the sequence
     * STREAM_READ   [op, src, sink, n]    measurement floor: reads n floats of src with 128-bit loads and keeps nothing
     * NOP           [op, grid]            measurement floor: an empty kernel of `grid` workgroups of 256 threads
     * Q8_PREPARE    [op, weight, prepared, K, rows]
     *     Writes the Q8 weight [rows x K] into `prepared` (deepj_hip_q8_prepared_floats(K, rows) floats, a buffer of
     *     its own) as fp16 rows plus scales transposed to [group][row], the layout the many-row GEMM loads straight
     *     into LDS, and lets `prepared` stand for `weight` in later Q8_LINEARs with M > 1 (they otherwise convert the
     *     weights into the workspace on every call).  The association ends when either buffer is released, uploaded
     *     to, or the destination of Q8_QUANTIZE / COPY / FILL - the ways Q8 data gets into a buffer; an op that writes
     *     floats over a Q8 weight (which no longer is one then) does not end it.  A graph captured before that keeps the
     *     copy it was captured with.  Results are the same with and without it.
     * Q8_LINEAR_ROPE [op, x, weight, qOut, M, K, d, flags, gamma, bias, beta, kCache, vCache, state, cos, sin, H, hd, maxSeq, layer]
     *     The fused q | k | v projection of a prompt (weight rows 3 d = 3 H hd, flags RMSNORM / LAYERNORM / BIAS as in
     *     Q8_LINEAR) with ROPE_KV_STORE as its epilogue: row r is the token at position state[0] + r; its queries go
     *     rotated to qOut [M x d], its keys rotated and its values as they are into the caches of `layer` - one launch
     *     and one pass over the [M x 3 d] product less than Q8_LINEAR followed by ROPE_KV_STORE, same results to the
     *     last bit or two of the rotation.  Only for shapes the fp16 GEMM takes with an unshared K
     *     (deepj_hip_q8_linear_rope_ok(M, K, d) != 0) and not through deepj_hip_flush_ops_noalloc; refused otherwise.
     */
    DJ_OP_Q8_QUANTIZE = 64, DJ_OP_Q8_DEQUANTIZE = 65, DJ_OP_Q8_LINEAR = 66, DJ_OP_RMSNORM = 67,
    DJ_OP_SILU_MUL = 68, DJ_OP_EMBED_GATHER = 69, DJ_OP_ROPE_KV_STORE = 70, DJ_OP_ATTENTION = 71,
    DJ_OP_ARGMAX_ROWS = 72, DJ_OP_DECODE_ADVANCE = 73, DJ_OP_COPY = 74, DJ_OP_FILL = 75,
    DJ_OP_ROPE_ROWS = 76, DJ_OP_ATTENTION_KV = 77, DJ_OP_DECODE_NEXT = 78, DJ_OP_ATTN_DECODE = 79,
    DJ_OP_APPEND_ROWS = 80, DJ_OP_Q8_LINEAR_DYN = 81, /* 82 unused */ DJ_OP_LAYERNORM = 83,
    DJ_OP_ADD_POSITIONS = 84, DJ_OP_ATTN_DECODE_RECORDS = 85, DJ_OP_STREAM_READ = 86, DJ_OP_NOP = 87, DJ_OP_Q8_PREPARE = 88,
    DJ_OP_Q8_LINEAR_ROPE = 89
};

enum { DJ_LIN_RMSNORM = 1, DJ_LIN_BIAS = 2, DJ_LIN_RESIDUAL = 4, DJ_LIN_SWIGLU = 8, DJ_LIN_LAYERNORM = 16,
       DJ_LIN_GELU = 32, DJ_LIN_ATTN_MERGE = 64 };

/* Key splits per head of ATTN_DECODE_RECORDS: its records buffer holds H * splits * (hd + 4) floats. */
int32_t deepj_hip_attn_record_splits(void);

/* Floats the scratch buffer of ATTENTION / ATTENTION_KV must hold for S query rows (0: none needed). */
int64_t deepj_hip_attention_scratch_floats(int32_t S, int32_t H, int32_t hd, int32_t max_seq);

/* Floats a Q8 weight buffer with `rows` output rows over K inputs must hold. */
int64_t deepj_hip_q8_floats(int32_t k, int32_t rows);

/* Floats of the buffer Q8_PREPARE fills for such a weight (about 2 bytes per weight), and which kernel a Q8_LINEAR of m
 * rows over it runs on when its workspace may grow: the fp16 direct-load GEMM with 128 or 64 rows per workgroup tile
 * (returns 128 or 64), or the bf16 kernels / the matvec (returns 0).
 * No counterpart in the reference, whose weights are fp32 (J/layers/Linear.java:9-24). */
int64_t deepj_hip_q8_prepared_floats(int32_t k, int32_t rows);
int32_t deepj_hip_q8_gemm_path(int32_t m, int32_t k, int32_t rows);
/* 1 when Q8_LINEAR_ROPE takes a projection of M rows over K inputs to 3 d outputs, 0 when the caller has to record
 * Q8_LINEAR and ROPE_KV_STORE instead */
int32_t deepj_hip_q8_linear_rope_ok(int32_t m, int32_t k, int32_t d);
/* the same with the tile's columns (256 or 192) and the number of workgroups that share a tile's K (1: none) */
void deepj_hip_q8_gemm_tile(int32_t m, int32_t k, int32_t rows, int32_t *tile_rows, int32_t *tile_cols, int32_t *k_shares);
/* the same for a weight that Q8_PREPARE has written in the fp16 GEMM's layout: from 16 rows on instead of 256 (64-row tiles,
 * K shared so that as many workgroups as possible stream weights) */
void deepj_hip_q8_gemm_tile_prepared(int32_t m, int32_t k, int32_t rows, int32_t *tile_rows, int32_t *tile_cols, int32_t *k_shares);
/* Host arithmetic only (no GPU call): the last byte + 1 that the fp16 GEMM's direct global -> LDS loads reach in its three
 * operand buffers {activation planes, fp16 weights, transposed scales} for a tile of tile_rows x tile_cols (128 or 64 rows
 * by 256 or 192 columns; tile_rows 0: the tile the library would choose), and the bytes those buffers hold.  Returns 1
 * when every load stays inside, 0 when one does not (a launch then fails instead of running), -1 when the shape is not
 * one of these kernels'.  Every launch runs the same check. */
int32_t deepj_hip_q8_gemm_f16_extents(int32_t m, int32_t k, int32_t rows, int32_t tile_rows, int32_t tile_cols, int64_t *reach3, int64_t *size3);

/* ── host side: java.util.Random twin ─────────────────────────────────────
 * Tensor.random(rows, cols, Random) of the reference (J/tensor/cpu/CpuBackend.java:148-152)
 * reproduced bit for bit (JDK-specified LCG + polar nextGaussian with StrictMath.log),
 * multi-threaded for large tensors. */
void   *deepj_host_random_create(int64_t seed);
void    deepj_host_random_destroy(void *rng);
void    deepj_host_random_fill(void *rng, float *out, int64_t n, double scale, int32_t threads);
double  deepj_host_random_next_gaussian(void *rng);
int32_t deepj_host_random_next_int(void *rng, int32_t bound);   /* bound <= 0: nextInt() */
float   deepj_host_random_next_float(void *rng);

/* ── host side: decode driver ─────────────────────────────────────────────
 * The inference caller above the five GpuRuntime calls: LlamaModel / DeepSeekModel +
 * TextGenerator of the reference (J/models/DecoderOnlyModel.java:58-64,
 * J/models/TextGenerator.java:66-181) with a device-resident KV cache, Q8 weights and one
 * fused command stream per token replayed as a HIP graph.  It uses only the functions
 * above.  cfg = {kind (0 Llama, 1 DeepSeek, 2 GPT, 3 DeepSeek with the latent KV cache), vocab, maxSeq, dModel,
 * nHeads, nLayers, dFF, qRank, kvRank}; id_base = first buffer id the runner may use.  Kind 1 caches the rotated
 * K and V of every position (2 * dModel floats per token and layer) like the Llama path; kind 3 caches the MLA
 * latent rows cKV = norm(x).Wdkv (kvRank floats per token and layer, J/layers/transformer/attention/
 * MultiHeadLatentAttention.java:98-106) and re-expands and re-rotates them every step - less memory, more work.  Weight names: "emb",
 * "gf", "wlm", "blm", "L<i>.g1|g2|wq|wk|wv|wo|wdq|wuq|wdkv|wuk|wuv|wg|bg|wu|bu|wd|bd";
 * GPT (J/models/gpt/GPTModel.java:27-45, J/layers/transformer/blocks/GPTTransformerBlock.java:52-73) adds
 * "pos" [maxSeq x dModel], "bf" and "L<i>.be1|be2" (LayerNorm betas; g1, g2, gf are the gammas), names its
 * FNN's two Linears wg,bg (dModel -> dFF) and wd,bd (dFF -> dModel) and has no wu,bu.
 * Matrices in the reference's [dIn x dOut] fp32 orientation. */
void       *deepj_runner_create(const int32_t cfg[9], int32_t id_base);   /* NULL: invalid config */
void        deepj_runner_destroy(void *runner);
const char *deepj_runner_last_error(void *runner);
int deepj_runner_set_weight(void *runner, const char *name, const float *data, int32_t rows, int32_t cols);
int deepj_runner_init_seeded(void *runner, int64_t seed, int32_t threads);  /* new LlamaModel(cfg, seed) */
/* new GPTModel(cfg, seed) with GPTConfig.initScale = init_scale (J/models/gpt/GPTModel.java:27-46,76-81) */
int deepj_runner_init_seeded_gpt(void *runner, int64_t seed, float init_scale, int32_t threads);
/* Bytes a runner may spend on fp16 copies of its weights for the many-row (prompt) GEMM, which reads them in that
 * form: -1 (default) no limit - a copy of every layer, written at the first prompt of 64 rows or more (+ 2 bytes
 * per weight); 0 none - every call converts into the workspace; otherwise layers in order while the budget lasts.
 * Prompts of 256 rows and more give the same bits whatever the budget; shorter ones take the fp16 GEMM only where a
 * copy exists (the bf16 kernels otherwise: same tolerance, other last bits).  deepj_runner_prepared_bytes: what the copies take now. */
int deepj_runner_set_prepared_budget(void *runner, int64_t bytes);
int64_t deepj_runner_prepared_bytes(void *runner);
int deepj_runner_finalize(void *runner);
int deepj_runner_reset(void *runner);
int deepj_runner_prefill(void *runner, const int32_t *ids, int32_t n, float *all_logits, int32_t choose_next);
/* Greedy decode of `steps` tokens on the device.  mode 0: the per-token stream, launched eagerly; 1: the same
 * stream replayed as a HIP graph. */
int deepj_runner_decode(void *runner, int32_t steps, int32_t mode);
int deepj_runner_step(void *runner, int32_t token);     /* one caller-chosen token through the S=1 path */
int deepj_runner_last_logits(void *runner, float *out);
int deepj_runner_tokens(void *runner, int32_t *out, int32_t capacity, int32_t *n);
int deepj_runner_generate(void *runner, const int32_t *prompt, int32_t n_prompt, int32_t max_new,
                          float temperature, int32_t top_k, int64_t seed, int32_t mode, int32_t *out);
int deepj_runner_decode_stream(void *runner, int32_t *out, int32_t capacity, int32_t *len);
/* the command stream of an n-token prompt at the current position (over the ids the last prefill uploaded) */
int deepj_runner_prefill_stream(void *runner, int32_t n, int32_t *out, int32_t capacity, int32_t *len);

#ifdef __cplusplus
}
#endif
#endif /* DEEPJ_HIP_H */
