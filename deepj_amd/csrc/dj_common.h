// Shared declarations of the device runtime: buffer records, error plumbing and
// the launcher prototypes each kernel file exports to the stream interpreter.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "../../include/deepj_hip.h"
#include "gemm_epilogue.h"

namespace dj {

constexpr int kQ8Group = 32;          // weights per fp32 scale, along the input (K) axis
constexpr float kRmsEps = 1e-6f;      // RMSNorm1D.java:30 in the reference
constexpr float kLayerNormEps = 1e-5f;  // LayerNorm1D.java:15

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

[[noreturn]] inline void fail(const std::string &msg) { throw Error(msg); }

inline void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) fail(std::string(what) + ": " + hipGetErrorString(e));
}
#define DJ_HIP(expr) ::dj::hip_check((expr), #expr)

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }
inline int q8_padded_k(int k) { return (int)round_up(k, kQ8Group); }
// Q8 weight buffer: [rows x Kp] int8, padded to 256 B, then [rows x Kp/32] fp32 scales.
inline int64_t q8_scale_offset_bytes(int k, int rows) { return round_up((int64_t)rows * q8_padded_k(k), 256); }
inline int64_t q8_bytes(int k, int rows) {
    return q8_scale_offset_bytes(k, rows) + (int64_t)rows * (q8_padded_k(k) / kQ8Group) * 4;
}

// Per-kernel timing for deepj_hip_profile_ops: while `armed`, every kernel that goes through launch_kernel() is
// launched with a start and a stop event of its own attached to that one dispatch (its begin and end time stamps on
// the device, the quantity a kernel trace reports), up to kMaxTimedLaunches per op; every other launch is an
// ordinary one.
constexpr int kMaxTimedLaunches = 6;
struct LaunchTiming {
    hipEvent_t *pairs = nullptr;     // 2 * kMaxTimedLaunches events of the op being run: start, stop, start, stop ...
    int used = 0;                    // dispatches of the op that carried events so far
    bool armed = false;
};
extern LaunchTiming g_launch_timing;

template <typename... Params, typename... Args>
inline void launch_kernel(void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds, hipStream_t s, Args... args) {
    if (g_launch_timing.armed && g_launch_timing.used < kMaxTimedLaunches) {
        hipEvent_t *pair = g_launch_timing.pairs + 2 * g_launch_timing.used++;
        hipExtLaunchKernelGGL(kernel, grid, block, lds, s, pair[0], pair[1], 0, static_cast<Params>(args)...);
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds, s, static_cast<Params>(args)...);
    }
}

// ── launchers (each validates nothing: the interpreter has already checked
//    ids, sizes and shapes on the host before any of these is called) ──────

// kernels_elementwise.hip
void launch_binary(hipStream_t s, int op, const float *a, const float *b, float *out, int64_t n);
void launch_unary(hipStream_t s, int op, const float *a, float *out, int64_t n);
void launch_scalar(hipStream_t s, int op, const float *a, float *out, float s0, float s1, int64_t n);
void launch_broadcast(hipStream_t s, int op, const float *a, const float *v, float *out, int rows, int cols);
void launch_transpose(hipStream_t s, const float *a, float *out, int rows, int cols);
void launch_adamw(hipStream_t s, float *w, const float *g, float *mt, float *vt, int64_t n, float lr,
                  float beta1, float beta2, float eps, float wd, float bc1, float bc2);
void launch_scatter_add(hipStream_t s, float *target, const float *idx, const float *grad, int target_rows,
                        int cols, int n_idx);
void launch_fill(hipStream_t s, uint32_t *dst, uint32_t bits, int64_t n);
void launch_copy(hipStream_t s, const float *src, float *dst, int64_t n);
// measurement floors: a pure streaming read of n floats (nothing kept), and an empty kernel of `grid` workgroups
void launch_stream_read(hipStream_t s, const float *src, float *sink, int64_t n);
void launch_nop(hipStream_t s, int grid);
void launch_clock_probe(hipStream_t s, unsigned long long *out, int samples, int sleep_reps);
void launch_wall_stamp(hipStream_t s, unsigned long long *out);
void launch_silu_mul(hipStream_t s, const float *gate, const float *up, float *out, int64_t n);
void launch_append_rows(hipStream_t s, const float *src, float *dst, const int32_t *state, int rows, int row_floats,
                        int max_rows);
void launch_embed_gather(hipStream_t s, const float *table, const int32_t *ids, float *out, int n_ids, int d,
                         int vocab);
void launch_decode_advance(hipStream_t s, int32_t *state, const int32_t *token, int32_t *tokens, int capacity,
                           int n_positions);

// kernels_reduce.hip
void launch_row_reduce(hipStream_t s, int op, const float *a, float *out, int rows, int cols);
void launch_sum_rows(hipStream_t s, const float *a, float *out, int rows, int cols);
void launch_sum_scalar(hipStream_t s, const float *a, float *out, int64_t n);
void launch_softmax_rows(hipStream_t s, const float *a, float *out, int rows, int cols);
void launch_softmax_backward(hipStream_t s, const float *g, const float *sm, float *out, int rows, int cols);
void launch_layernorm_backward(hipStream_t s, const float *dxhat, const float *xhat, const float *stdv,
                               float *out, int rows, int cols);
void launch_cross_entropy(hipStream_t s, bool gradient, const float *logits, const float *targets, float *out,
                          int rows, int cols);
void launch_rmsnorm(hipStream_t s, const float *x, const float *gamma, float *out, int rows, int cols);
void launch_layernorm(hipStream_t s, const float *x, const float *gamma, const float *beta, float *out, int rows,
                      int cols);
void launch_add_positions(hipStream_t s, float *x, const float *table, const int32_t *state, int rows, int d,
                          int max_seq);
void launch_argmax_rows(hipStream_t s, const float *a, int32_t *out, int rows, int cols);

// kernels_matmul.hip
void launch_matmul_f32(hipStream_t s, const float *a, const float *b, float *out, int m, int n, int k);

// kernels_q8.hip
// Two consecutive fp16 GEMMs of a stream, the second normalising (RMSNorm) and multiplying the first one's output: when
// the first shares its tiles' K among workgroups, the kernel that adds their partial products also writes the second
// one's activations in its layout, and the second skips its own split.
struct GemmChain {
    const float *next_gamma = nullptr;   // to the first launch: the gain the next GEMM normalises this output with
    bool left_planes = false;            // from the first launch: it left the next GEMM's activations in the workspace
    bool planes_ready = false;           // to the second launch: they are there
};

struct Q8Linear {
    const float *x; const int8_t *wq; const float *scales; float *out;
    int m, k, n, flags;
    const float *gamma, *bias, *bias2, *residual;
    const float *beta = nullptr;      // LayerNorm prologue only
    int rec_hd = 0;                   // ATTN_MERGE prologue only: head width of the records in x
    const int32_t *m_dev = nullptr;   // GEMM path only: live row count = min(m, m_dev[0] + m_extra)
    int m_extra = 0;
    const float *prepared = nullptr;  // the weights in the fp16 GEMM's layout (launch_q8_prepare), or null: converted per call
    GemmChain *chain = nullptr;       // fp16 GEMM only
    RopeStore rope;                   // fp16 GEMM only: out = nullptr, the q | k | v row goes through RoPE to q and the caches
    bool small_workspace_only = false; // the caller's workspace cannot grow: stay on the kernels that need M * K floats at most
};
void launch_q8_quantize(hipStream_t s, const float *w, int8_t *q, float *scales, int k, int n, int row_off,
                        int row_step);
void launch_q8_dequantize(hipStream_t s, const int8_t *q, const float *scales, float *w, int k, int n,
                          int row_off, int row_step);
void launch_q8_linear(hipStream_t s, const Q8Linear &p, float *workspace, int64_t workspace_floats);
int64_t q8_linear_workspace_floats(int m, int k, int n, int flags);
// The size at which launch_q8_linear takes its fastest path (>= the one above); callers that may grow their workspace
// offer this much, callers that may not offer what they have.
int64_t q8_linear_preferred_workspace_floats(int m, int k, int n, int flags, bool prepared);

// kernels_gemm_f16.hip: the many-row Q8 GEMM on fp16 matrix cores (two-piece activations, direct loads to LDS)
bool q8_gemm_f16_shape_ok(int m, int n_rows, int k, bool prepared = false);   // prepared: the weights are in these kernels' layout already (fewer than 256 rows take them only then)
int q8_gemm_f16_tile_rows(int m, int n_rows, int k, bool prepared = false);   // 128 or 64 rows per workgroup tile, 0: not for these kernels
void q8_gemm_f16_tile(int m, int n_rows, int k, int *tile_rows, int *tile_cols, int *k_shares, bool prepared = false);
// bytes the direct loads of a launch with this tile reach in {planes, fp16 weights, transposed scales} and bytes those
// hold; false when any load would pass its buffer
bool q8_gemm_f16_extents(int m, int n_rows, int k, int tile_rows, int tile_cols, int64_t reach[3], int64_t size[3]);
void q8_gemm_f16_configure();   // once per device, before the first launch
int64_t q8_gemm_f16_workspace_floats(int m, int n_rows, int k, bool prepared);
// floats of the weights in that kernel's layout: fp16 [rows up to a multiple of 256][Kp + 64], then the scales as
// [Kp / 32][rows up to a multiple of 256]
int64_t q8_prepared_floats(int k, int n_rows);
void launch_q8_prepare(hipStream_t s, const int8_t *wq, const float *scales, float *prepared, int k, int n_rows);
// gamma (and beta): the rows are RMS- (Layer-) normalised on their way into the kernel's layout
void launch_q8_gemm_f16(hipStream_t s, const float *x, const float *gamma, const float *beta, const int8_t *wq, const float *scales,
                        const float *prepared, float *out, int m, int k, int n_rows, const float *bias, const float *bias2,
                        const float *residual, int interleaved_bias, int gelu, int swiglu, float *workspace, int64_t workspace_floats,
                        const RopeStore *rope = nullptr, GemmChain *chain = nullptr);
bool q8_gemm_f16_rope_ok(int m, int d, int k);

// kernels_attn.hip
struct AttnArgs {
    const float *q;        // [S x H*hd], already rotated
    const float *k, *v;    // key/value base for this layer
    int64_t k_tok_stride, k_head_stride;   // in floats
    float *out;            // [S x H*hd]
    const int32_t *state;  // state[0] = number of positions before this chunk
    float *scratch; int64_t scratch_floats;
    unsigned *counters;    // S = 1: kAttnCounterHeads zeroed words owned by the runtime (split arrival counters)
    int s, h, hd, max_seq;
};
constexpr int kAttnCounterHeads = 1024;
void launch_rope_kv_store(hipStream_t s, const float *qkv, float *q_out, float *k_cache, float *v_cache,
                          const int32_t *state, const float *cos_t, const float *sin_t, int S, int H, int hd,
                          int max_seq);
void launch_rope_rows(hipStream_t s, const float *x, float *out, const int32_t *state, const float *cos_t,
                      const float *sin_t, int rows, int H, int hd, int max_seq, int pos_from_row, int row_stride,
                      int live_extra);
void launch_attention(hipStream_t s, const AttnArgs &a);
void launch_attn_decode(hipStream_t s, const float *qkv, float *k_cache, float *v_cache, float *out,
                        const int32_t *state, float *scratch, const float *cos_t, const float *sin_t, int H, int hd,
                        int max_seq, unsigned *counters);
int64_t attn_decode_scratch_floats(int H, int hd);
// Decode attention that stops at per-split records [H][kAttnRecordSplits][hd + 4] = {max, sum, -, -, o[hd]};
// the consumer (Q8 matvec with the ATTN_MERGE prologue) merges them.  The maximum is in base-2 units (score *
// log2(e)): both sides use the hardware exp2.
constexpr int kAttnRecordSplits = 4;
void launch_attn_decode_records(hipStream_t s, const float *qkv, float *k_cache, float *v_cache, float *records,
                                const int32_t *state, const float *cos_t, const float *sin_t, int H, int hd,
                                int max_seq);
void launch_decode_next(hipStream_t s, const float *logits, int32_t *state, int32_t *tokens, int capacity,
                        const float *table, float *x, int vocab, int d, int n_positions);
int64_t attention_scratch_floats(int S, int H, int hd, int max_seq);

}  // namespace dj
