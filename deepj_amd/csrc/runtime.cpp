// Device runtime behind the C ABI: the buffer/residency manager, the command-stream
// interpreter and HIP-graph capture.  It takes the place of the reference's native
// library (native/deepj_metal_jni.mm:1350-2140: gBufferPool + the opcode switch) and
// keeps its observable contract: ids are chosen by the caller, allocating an existing
// id and releasing an unknown id are no-ops, uploads copy the caller's array length,
// and a stream is executed in program order.
//
// What is different by design:
//  * Tensors stay resident in HBM between flushes; released buffers go to a
//    size-class cache, so the "new output id + release the old id" pattern that
//    in-place ops arrive as (MetalBackend.java:400-411) costs no hipMalloc/hipFree.
//  * flush only enqueues on one in-order HIP stream; download is the single
//    synchronisation point (the reference waits for the GPU in every flush,
//    deepj_metal_jni.mm:2126-2127).
//  * The whole stream is validated on the host - opcode, stride, ids, buffer sizes,
//    shapes - before the first kernel is launched, so a malformed stream can never
//    make a kernel touch memory it does not own.
#include <algorithm>
#include <cstring>
#include <map>
#include <unordered_map>
#include <vector>

#include "dj_common.h"

namespace dj {

LaunchTiming g_launch_timing;

namespace {

struct Buffer {
    void *ptr = nullptr;
    size_t capacity = 0;      // bytes actually owned (size class)
    int64_t floats = 0;       // size the caller asked for
};

// A captured graph holds raw device addresses.  The buffers its stream named (id, address at capture time) and
// the workspace it used are remembered, and a replay is refused once any of them is gone or has moved.
struct Graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<std::pair<int32_t, void *>> refs;
    float *workspace = nullptr;       // set when the stream needs workspace
    // (weight id, prepared id) of every Q8_LINEAR that was captured reading a prepared copy the stream had not written
    // itself: once the copy stops standing for the weights (they were written again) a replay would use stale weights
    std::vector<std::pair<int32_t, int32_t>> prepared, self_prepared;
};

struct Runtime {
    bool ready = false;
    int device = 0;
    hipStream_t stream = nullptr;
    std::unordered_map<int32_t, Buffer> live;
    std::map<size_t, std::vector<void *>> cache;   // size class -> free blocks
    int64_t live_bytes = 0, cached_bytes = 0, driver_allocs = 0;
    size_t cache_limit = (size_t)16 << 30;
    float *workspace = nullptr;
    int64_t workspace_floats = 0;
    void *staging = nullptr;                       // pinned, for small uploads/downloads
    size_t staging_bytes = 0;
    bool capturing = false;
    std::unordered_map<int32_t, Graph> graphs;
    int32_t next_graph = 1;
    unsigned *attn_counters = nullptr;             // kAttnCounterHeads zeroed words: decode attention's split arrivals
    unsigned char *static_scratch = nullptr;       // device address of `scratch` below on g.device
    // Set by a K-sharing fp16 GEMM that also wrote the activations of the op right behind it in that op's layout
    // (GemmChain): which op of which stream, reading which buffer through which gain.  Good for that one op only.
    struct ChainSlot { const int32_t *cmd = nullptr; int32_t pos = -1, x_id = -1, gamma_id = -1; int64_t m = 0, k = 0; bool valid = false; } chain;
    bool no_alloc = false;                         // inside deepj_hip_flush_ops_noalloc: nothing may allocate
    std::vector<std::pair<int32_t, void *>> *track = nullptr;   // graph capture: buffers the dry pass resolves
    Graph *capture_into = nullptr;                               // graph capture: the graph the run pass records for
    struct Prepared { int32_t id; int k, rows; };
    std::unordered_map<int32_t, Prepared> prepared;   // Q8 weight buffer -> its copy in the fp16 GEMM's layout (OP_Q8_PREPARE)
};

Runtime g;
thread_local std::string g_error;

// Scratch memory of deepj_hip_flush_ops_noalloc, part of the loaded code object (each GPU the library runs on
// holds its own copy until the process ends): the arrival counters of the split decode attention, then the
// workspace that Q8_LINEAR's GEMM path writes its normalised activation rows to.  Host code never uses the
// symbol itself as an address: ensure_init() asks the runtime where the array lives on the current device.
constexpr size_t kStaticCounterBytes = (size_t)kAttnCounterHeads * sizeof(unsigned);
constexpr int64_t kStaticWorkspaceFloats = DEEPJ_HIP_NOALLOC_WORKSPACE_FLOATS;   // 8 MiB: e.g. 512 rows of 4096 floats
static __device__ __align__(256) unsigned char scratch[kStaticCounterBytes + (size_t)kStaticWorkspaceFloats * 4];

void ensure_init(int device = 0) {
    if (g.ready) return;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) fail("deepj_hip: no HIP device available");
    if (device < 0 || device >= count) fail("deepj_hip: bad device index " + std::to_string(device));
    DJ_HIP(hipSetDevice(device));
    DJ_HIP(hipStreamCreateWithFlags(&g.stream, hipStreamNonBlocking));
    g.staging_bytes = (size_t)1 << 20;
    DJ_HIP(hipHostMalloc(&g.staging, g.staging_bytes, hipHostMallocDefault));
    DJ_HIP(hipMalloc((void **)&g.attn_counters, kAttnCounterHeads * sizeof(unsigned)));
    DJ_HIP(hipMemset(g.attn_counters, 0, kAttnCounterHeads * sizeof(unsigned)));
    g.static_scratch = nullptr;
    DJ_HIP(hipGetSymbolAddress((void **)&g.static_scratch, HIP_SYMBOL(scratch)));
    if (!g.static_scratch) fail("deepj_hip: the static scratch array has no device address");
    DJ_HIP(hipMemset(g.static_scratch, 0, kStaticCounterBytes));
    q8_gemm_f16_configure();
    g.device = device;
    g.ready = true;
}

// A prepared copy stops standing for its Q8 buffer as soon as either is released or written.
void forget_prepared(int32_t id) {
    if (g.prepared.empty()) return;
    g.prepared.erase(id);
    for (auto it = g.prepared.begin(); it != g.prepared.end();) it = it->second.id == id ? g.prepared.erase(it) : std::next(it);
}

// 256 B granularity up to 64 KiB, then four classes per power of two (<= 25 % slack).
size_t size_class(size_t bytes) {
    if (bytes < 256) return 256;
    if (bytes <= (64u << 10)) return (bytes + 255) & ~(size_t)255;
    size_t p = (size_t)1 << (63 - __builtin_clzll(bytes));      // largest power of two <= bytes
    if (p == bytes) return bytes;
    size_t step = p >> 2;
    return (bytes + step - 1) / step * step;
}

void *pool_alloc(size_t cls) {
    auto it = g.cache.find(cls);
    if (it != g.cache.end() && !it->second.empty()) {
        void *p = it->second.back();
        it->second.pop_back();
        g.cached_bytes -= (int64_t)cls;
        return p;
    }
    if (g.capturing) fail("deepj_hip: device allocation requested while a graph is being captured");
    if (g.no_alloc) fail("deepj_hip: device allocation requested inside the allocation-free entry point");
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, cls);
    if (e != hipSuccess) {
        // give cached blocks back to the driver and retry once
        (void)hipGetLastError();
        DJ_HIP(hipStreamSynchronize(g.stream));
        for (auto &kv : g.cache) {
            for (void *q : kv.second) (void)hipFree(q);
            kv.second.clear();
        }
        g.cached_bytes = 0;
        e = hipMalloc(&p, cls);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            fail("Failed to allocate HIP buffer of " + std::to_string(cls) + " bytes: " + hipGetErrorString(e));
        }
    }
    g.driver_allocs++;
    return p;
}

void pool_free(void *p, size_t cls) {
    // Work already queued on the stream may still use the block; any later user is
    // queued behind it on the same in-order stream, so recycling needs no wait.
    if ((size_t)g.cached_bytes + cls > g.cache_limit) {
        DJ_HIP(hipStreamSynchronize(g.stream));
        DJ_HIP(hipFree(p));
        return;
    }
    g.cache[cls].push_back(p);
    g.cached_bytes += (int64_t)cls;
}

void ensure_workspace(int64_t floats) {
    if (g.no_alloc) {
        if (floats > kStaticWorkspaceFloats)
            fail("flush_ops_noalloc: the stream needs " + std::to_string(floats) + " floats of workspace, the static "
                 "scratch holds " + std::to_string(kStaticWorkspaceFloats) + " (use deepj_hip_flush_ops)");
        return;
    }
    if (floats <= g.workspace_floats) return;
    if (g.capturing) fail("deepj_hip: workspace would have to grow during graph capture; run the stream once first");
    DJ_HIP(hipStreamSynchronize(g.stream));
    if (g.workspace) DJ_HIP(hipFree(g.workspace));
    g.workspace = nullptr;
    g.workspace_floats = 0;
    int64_t want = std::max<int64_t>(floats, (int64_t)1 << 20);
    DJ_HIP(hipMalloc((void **)&g.workspace, (size_t)want * 4));
    g.driver_allocs++;
    g.workspace_floats = want;
}

// ── stream interpreter ──────────────────────────────────────────────────────

struct Cursor {
    const int32_t *cmd;
    int32_t len;
    int32_t pos;
    bool dry;          // validate only
    int64_t ws_need;   // workspace floats the stream needs (collected in the dry pass)
};

const char *op_name(int op);

int stride_of(int op) {
    switch (op) {
        case DJ_OP_SQRT: case DJ_OP_NEG: case DJ_OP_EXP: case DJ_OP_LOG: case DJ_OP_TANH: case DJ_OP_SIGMOID:
        case DJ_OP_RELU: case DJ_OP_GELU:
            return 4;
        case DJ_OP_ADD: case DJ_OP_SUBTRACT: case DJ_OP_MULTIPLY: case DJ_OP_DIVIDE: case DJ_OP_RELU_BACKWARD:
        case DJ_OP_GELU_BACKWARD: case DJ_OP_MULTIPLY_SCALAR: case DJ_OP_ADD_SCALAR: case DJ_OP_DIVIDE_SCALAR:
        case DJ_OP_TRANSPOSE: case DJ_OP_SUM_ROWS: case DJ_OP_MEAN_ALONG_ROWS: case DJ_OP_VARIANCE_ALONG_ROWS:
        case DJ_OP_SUM_ALONG_ROWS: case DJ_OP_MAX_ALONG_ROWS: case DJ_OP_SOFTMAX_ROWS: case DJ_OP_POW:
        case DJ_OP_SUM_ABS: case DJ_OP_SUM_SCALAR:
            return 5;
        case DJ_OP_CLAMP: case DJ_OP_CROSS_ENTROPY_LOSS: case DJ_OP_CROSS_ENTROPY_GRADIENT:
        case DJ_OP_SOFTMAX_BACKWARD: case DJ_OP_ADD_ROW_VECTOR: case DJ_OP_ADD_BROADCAST_COLS:
        case DJ_OP_SUBTRACT_BROADCAST_COLS: case DJ_OP_DIVIDE_BROADCAST_COLS: case DJ_OP_MULTIPLY_BROADCAST_ROWS:
        case DJ_OP_MULTIPLY_BROADCAST_COLS:
            return 6;
        case DJ_OP_MATMUL: case DJ_OP_LAYERNORM_BACKWARD: case DJ_OP_SCATTER_ADD_ROWS:
        case DJ_OP_SCATTER_ADD_ROWS_ATOMIC:
            return 7;
        case DJ_OP_ADAMW_UPDATE: return 13;
        case DJ_OP_Q8_QUANTIZE: case DJ_OP_Q8_DEQUANTIZE: return 8;
        case DJ_OP_Q8_LINEAR: return 12;
        case DJ_OP_RMSNORM: return 6;
        case DJ_OP_SILU_MUL: return 5;
        case DJ_OP_EMBED_GATHER: return 8;
        case DJ_OP_ROPE_KV_STORE: return 13;
        case DJ_OP_ATTENTION: return 12;
        case DJ_OP_ARGMAX_ROWS: return 5;
        case DJ_OP_DECODE_ADVANCE: return 6;
        case DJ_OP_COPY: return 6;
        case DJ_OP_FILL: return 4;
        case DJ_OP_ROPE_ROWS: return 13;
        case DJ_OP_ATTENTION_KV: return 14;
        case DJ_OP_DECODE_NEXT: return 10;
        case DJ_OP_ATTN_DECODE: return 13;
        case DJ_OP_APPEND_ROWS: return 8;
        case DJ_OP_Q8_LINEAR_DYN: return 10;
        case DJ_OP_LAYERNORM: return 7;
        case DJ_OP_ATTN_DECODE_RECORDS: return 12;
        case DJ_OP_ADD_POSITIONS: return 7;
        case DJ_OP_STREAM_READ: return 4;
        case DJ_OP_NOP: return 2;
        case DJ_OP_Q8_PREPARE: return 5;
        case DJ_OP_Q8_LINEAR_ROPE: return 20;
        default: return -1;
    }
}

float bits_to_float(int32_t b) { float f; std::memcpy(&f, &b, 4); return f; }

// Pointer to buffer `id`, after checking that it exists and holds >= floats floats.
float *buf(int32_t id, int64_t floats, int op, const char *role) {
    auto it = g.live.find(id);
    if (it == g.live.end())
        fail(std::string(op_name(op)) + ": missing GPU buffer id=" + std::to_string(id) + " (" + role + ")");
    if (floats < 0 || floats > it->second.floats)
        fail(std::string(op_name(op)) + ": buffer id=" + std::to_string(id) + " (" + role + ") holds " +
             std::to_string(it->second.floats) + " floats, op needs " + std::to_string(floats));
    if (g.track) g.track->emplace_back(id, it->second.ptr);
    return static_cast<float *>(it->second.ptr);
}
float *buf_opt(int32_t id, int64_t floats, int op, const char *role) {
    return id < 0 ? nullptr : buf(id, floats, op, role);
}

void need_positive(int op, const char *what, int64_t v) {
    if (v < 0) fail(std::string(op_name(op)) + ": negative " + what + " " + std::to_string(v));
}

void exec_one(Cursor &c) {
    const int32_t *w = c.cmd + c.pos;
    const int op = w[0];
    hipStream_t s = g.stream;
    const bool run = !c.dry;
    const Runtime::ChainSlot was = g.chain;
    if (run) g.chain.valid = false;
    // this op is the one a GemmChain's first launch prepared the activations of (x, gain, shape as it saw them)
    auto chained = [&](int32_t x_id, int32_t gamma_id, int flags, int64_t m, int64_t k) {
        return run && was.valid && was.cmd == c.cmd && was.pos == c.pos && was.x_id == x_id && was.gamma_id == gamma_id && was.m == m &&
               was.k == k && (flags & DJ_LIN_RMSNORM) && !(flags & DJ_LIN_LAYERNORM);
    };
    switch (op) {
        case DJ_OP_ADD: case DJ_OP_SUBTRACT: case DJ_OP_MULTIPLY: case DJ_OP_DIVIDE: case DJ_OP_RELU_BACKWARD:
        case DJ_OP_GELU_BACKWARD: {
            int64_t n = w[4]; need_positive(op, "n", n);
            const float *a = buf(w[1], n, op, "a"), *b = buf(w[2], n, op, "b");
            float *o = buf(w[3], n, op, "out");
            if (run) launch_binary(s, op, a, b, o, n);
            break;
        }
        case DJ_OP_SQRT: case DJ_OP_NEG: case DJ_OP_EXP: case DJ_OP_LOG: case DJ_OP_TANH: case DJ_OP_SIGMOID:
        case DJ_OP_RELU: case DJ_OP_GELU: {
            int64_t n = w[3]; need_positive(op, "n", n);
            const float *a = buf(w[1], n, op, "in");
            float *o = buf(w[2], n, op, "out");
            if (run) launch_unary(s, op, a, o, n);
            break;
        }
        case DJ_OP_MULTIPLY_SCALAR: case DJ_OP_ADD_SCALAR: case DJ_OP_DIVIDE_SCALAR: case DJ_OP_POW: {
            int64_t n = w[4]; need_positive(op, "n", n);
            const float *a = buf(w[1], n, op, "in");
            float *o = buf(w[2], n, op, "out");
            if (run) launch_scalar(s, op, a, o, bits_to_float(w[3]), 0.0f, n);
            break;
        }
        case DJ_OP_CLAMP: {
            int64_t n = w[5]; need_positive(op, "n", n);
            const float *a = buf(w[1], n, op, "in");
            float *o = buf(w[2], n, op, "out");
            if (run) launch_scalar(s, op, a, o, bits_to_float(w[3]), bits_to_float(w[4]), n);
            break;
        }
        case DJ_OP_MATMUL: {
            int64_t m = w[4], n = w[5], k = w[6];
            need_positive(op, "m", m); need_positive(op, "n", n); need_positive(op, "k", k);
            const float *a = buf(w[1], m * k, op, "a"), *b = buf(w[2], k * n, op, "b");
            float *o = buf(w[3], m * n, op, "out");
            if (run) launch_matmul_f32(s, a, b, o, (int)m, (int)n, (int)k);
            break;
        }
        case DJ_OP_TRANSPOSE: {
            int64_t rows = w[3], cols = w[4]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *a = buf(w[1], rows * cols, op, "in");
            float *o = buf(w[2], rows * cols, op, "out");
            if (run) launch_transpose(s, a, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_ADD_ROW_VECTOR: case DJ_OP_MULTIPLY_BROADCAST_ROWS: case DJ_OP_ADD_BROADCAST_COLS:
        case DJ_OP_SUBTRACT_BROADCAST_COLS: case DJ_OP_DIVIDE_BROADCAST_COLS: case DJ_OP_MULTIPLY_BROADCAST_COLS: {
            int64_t rows = w[4], cols = w[5]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            bool rowvec = (op == DJ_OP_ADD_ROW_VECTOR || op == DJ_OP_MULTIPLY_BROADCAST_ROWS);
            const float *a = buf(w[1], rows * cols, op, "a");
            const float *v = buf(w[2], rowvec ? cols : rows, op, "vector");
            float *o = buf(w[3], rows * cols, op, "out");
            if (run) launch_broadcast(s, op, a, v, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_SUM_ROWS: {
            int64_t rows = w[3], cols = w[4]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *a = buf(w[1], rows * cols, op, "in");
            float *o = buf(w[2], cols, op, "out");
            if (run) launch_sum_rows(s, a, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_SUM_ALONG_ROWS: case DJ_OP_MEAN_ALONG_ROWS: case DJ_OP_VARIANCE_ALONG_ROWS:
        case DJ_OP_MAX_ALONG_ROWS: case DJ_OP_SUM_ABS: {
            int64_t rows = w[3], cols = w[4]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *a = buf(w[1], rows * cols, op, "in");
            float *o = buf(w[2], rows, op, "out");
            if (run) launch_row_reduce(s, op, a, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_SUM_SCALAR: {
            int64_t rows = w[3], cols = w[4]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *a = buf(w[1], rows * cols, op, "in");
            float *o = buf(w[2], 1, op, "out");
            if (run) launch_sum_scalar(s, a, o, rows * cols);
            break;
        }
        case DJ_OP_SOFTMAX_ROWS: {
            int64_t rows = w[3], cols = w[4]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *a = buf(w[1], rows * cols, op, "in");
            float *o = buf(w[2], rows * cols, op, "out");
            if (run) launch_softmax_rows(s, a, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_SOFTMAX_BACKWARD: {
            int64_t rows = w[4], cols = w[5]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *gr = buf(w[1], rows * cols, op, "grad"), *sm = buf(w[2], rows * cols, op, "softmax");
            float *o = buf(w[3], rows * cols, op, "out");
            if (run) launch_softmax_backward(s, gr, sm, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_LAYERNORM_BACKWARD: {
            int64_t rows = w[5], cols = w[6]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *dx = buf(w[1], rows * cols, op, "dXHat"), *xh = buf(w[2], rows * cols, op, "xHat");
            const float *sd = buf(w[3], rows, op, "std");
            float *o = buf(w[4], rows * cols, op, "out");
            if (run) launch_layernorm_backward(s, dx, xh, sd, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_ADAMW_UPDATE: {
            int64_t n = w[12]; need_positive(op, "n", n);
            float *wt = buf(w[1], n, op, "w");
            const float *gr = buf(w[2], n, op, "g");
            float *mt = buf(w[3], n, op, "mt"), *vt = buf(w[4], n, op, "vt");
            if (run)
                launch_adamw(s, wt, gr, mt, vt, n, bits_to_float(w[5]), bits_to_float(w[6]), bits_to_float(w[7]),
                             bits_to_float(w[8]), bits_to_float(w[9]), bits_to_float(w[10]), bits_to_float(w[11]));
            break;
        }
        case DJ_OP_SCATTER_ADD_ROWS: case DJ_OP_SCATTER_ADD_ROWS_ATOMIC: {
            // Both opcodes accumulate atomically: the non-atomic variant is racy for
            // duplicate indices by construction (deepj_metal_jni.mm:559-577).
            int64_t trows = w[4], tcols = w[5], nidx = w[6];
            need_positive(op, "rows", trows); need_positive(op, "cols", tcols); need_positive(op, "indices", nidx);
            float *t = buf(w[1], trows * tcols, op, "target");
            const float *idx = buf(w[2], nidx, op, "indices");
            const float *gr = buf(w[3], nidx * tcols, op, "grad");
            if (run) launch_scatter_add(s, t, idx, gr, (int)trows, (int)tcols, (int)nidx);
            break;
        }
        case DJ_OP_CROSS_ENTROPY_LOSS: case DJ_OP_CROSS_ENTROPY_GRADIENT: {
            int64_t rows = w[4], cols = w[5]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            bool grad = op == DJ_OP_CROSS_ENTROPY_GRADIENT;
            const float *lg = buf(w[1], rows * cols, op, "logits"), *tg = buf(w[2], rows, op, "targets");
            float *o = buf(w[3], grad ? rows * cols : rows, op, "out");
            if (run) launch_cross_entropy(s, grad, lg, tg, o, (int)rows, (int)cols);
            break;
        }

        // ── fused inference opcodes ────────────────────────────────────────
        case DJ_OP_Q8_QUANTIZE: case DJ_OP_Q8_DEQUANTIZE: {
            int64_t k = w[3], n = w[4], off = w[5], step = w[6], total = w[7];
            if (k <= 0 || n <= 0 || total <= 0 || step <= 0 || off < 0) fail(std::string(op_name(op)) + ": bad shape");
            if (off + (n - 1) * step >= total) fail(std::string(op_name(op)) + ": rows fall outside the Q8 buffer");
            int64_t qfloats = (q8_bytes((int)k, (int)total) + 3) / 4;
            bool quant = op == DJ_OP_Q8_QUANTIZE;
            float *src = buf(w[1], quant ? k * n : qfloats, op, "src");
            float *dst = buf(w[2], quant ? qfloats : k * n, op, "dst");
            if (run) {
                forget_prepared(w[2]);
                if (quant) {
                    int8_t *q = reinterpret_cast<int8_t *>(dst);
                    float *sc = reinterpret_cast<float *>(q + q8_scale_offset_bytes((int)k, (int)total));
                    launch_q8_quantize(s, src, q, sc, (int)k, (int)n, (int)off, (int)step);
                } else {
                    const int8_t *q = reinterpret_cast<const int8_t *>(src);
                    const float *sc = reinterpret_cast<const float *>(q + q8_scale_offset_bytes((int)k, (int)total));
                    launch_q8_dequantize(s, q, sc, dst, (int)k, (int)n, (int)off, (int)step);
                }
            }
            break;
        }
        case DJ_OP_Q8_LINEAR: {
            int64_t m = w[4], k = w[5], n = w[6];
            int flags = w[7];
            if (m <= 0 || k <= 0 || n <= 0) fail("OP_Q8_LINEAR: bad shape");
            if (flags & ~127) fail("OP_Q8_LINEAR: unknown flag bits");
            const bool merge = flags & DJ_LIN_ATTN_MERGE;
            int64_t rec_hd = 0;
            if (merge) {
                // x holds decode-attention records [K / hd][kAttnRecordSplits][hd + 4]; hd travels in the gamma word
                rec_hd = w[8];
                if (flags & (DJ_LIN_RMSNORM | DJ_LIN_LAYERNORM | DJ_LIN_SWIGLU | DJ_LIN_GELU))
                    fail("OP_Q8_LINEAR: ATTN_MERGE cannot be combined with a norm prologue, SWIGLU or GELU");
                if (rec_hd != 32 && rec_hd != 64 && rec_hd != 128) fail("OP_Q8_LINEAR: ATTN_MERGE head dim must be 32, 64 or 128");
                if (m != 1 || k % rec_hd != 0) fail("OP_Q8_LINEAR: ATTN_MERGE needs M = 1 and K a multiple of the head dim");
                if (q8_linear_workspace_floats(1, (int)k, (int)n, 0) != 0 || k > 11 * 1024) fail("OP_Q8_LINEAR: ATTN_MERGE: K too large");
            }
            bool sw = flags & DJ_LIN_SWIGLU;
            bool ln = flags & DJ_LIN_LAYERNORM;
            if (sw && (flags & DJ_LIN_RESIDUAL)) fail("OP_Q8_LINEAR: SWIGLU cannot be combined with RESIDUAL");
            if (sw && (flags & (DJ_LIN_LAYERNORM | DJ_LIN_GELU))) fail("OP_Q8_LINEAR: SWIGLU cannot be combined with LAYERNORM or GELU");
            if (ln && (flags & DJ_LIN_RMSNORM)) fail("OP_Q8_LINEAR: RMSNORM and LAYERNORM are exclusive");
            int64_t rows = sw ? 2 * n : n;
            Q8Linear p;
            p.x = merge ? buf(w[1], (k / rec_hd) * kAttnRecordSplits * (rec_hd + 4), op, "attention records") : buf(w[1], m * k, op, "x");
            p.rec_hd = (int)rec_hd;
            const float *wq = buf(w[2], (q8_bytes((int)k, (int)rows) + 3) / 4, op, "weight");
            p.wq = reinterpret_cast<const int8_t *>(wq);
            p.scales = reinterpret_cast<const float *>(p.wq + q8_scale_offset_bytes((int)k, (int)rows));
            p.out = buf(w[3], m * n, op, "out");
            p.m = (int)m; p.k = (int)k; p.n = (int)n; p.flags = flags;
            p.gamma = (flags & (DJ_LIN_RMSNORM | DJ_LIN_LAYERNORM)) ? buf(w[8], k, op, "gamma") : nullptr;   // (ATTN_MERGE: w[8] = hd)
            p.beta = ln ? buf(w[10], k, op, "beta") : nullptr;
            p.bias = (flags & DJ_LIN_BIAS) ? buf(w[9], n, op, "bias") : nullptr;
            p.bias2 = ((flags & DJ_LIN_BIAS) && sw) ? buf(w[10], n, op, "bias2") : nullptr;
            p.residual = (flags & DJ_LIN_RESIDUAL) ? buf(w[11], m * n, op, "residual") : nullptr;
            // a workspace that may grow is sized for the kernel's fastest path; the fixed one for the smallest
            if (m > 1) {
                auto pit = g.prepared.find(w[2]);
                if (pit != g.prepared.end() && pit->second.k == k && pit->second.rows == rows)
                    p.prepared = buf(pit->second.id, q8_prepared_floats((int)k, (int)rows), op, "prepared weights");
                if (p.prepared && run && g.capture_into) {
                    const std::pair<int32_t, int32_t> pr(w[2], pit->second.id);
                    auto &own = g.capture_into->self_prepared;
                    if (std::find(own.begin(), own.end(), pr) == own.end()) g.capture_into->prepared.push_back(pr);
                }
            }
            int64_t ws = g.no_alloc ? q8_linear_workspace_floats((int)m, (int)k, (int)n, flags)
                                    : q8_linear_preferred_workspace_floats((int)m, (int)k, (int)n, flags, p.prepared != nullptr);
            if (c.dry) c.ws_need = std::max(c.ws_need, ws);
            // One rule for the allocation-free entry point, whatever happens to fit its fixed array: the many-row
            // fp16 GEMM (whose operands live in a workspace sized by the shape) is never taken there.
            p.small_workspace_only = g.no_alloc;
            GemmChain chain;
            int32_t next_gamma_id = -1;
            const int32_t next_pos = c.pos + stride_of(op);
            if (run && m > 1 && !g.no_alloc && !merge) {
                chain.planes_ready = chained(w[1], w[8], flags, m, k);
                // the op right behind this one normalises this output (RMSNorm) and multiplies it on the fp16 GEMM: the
                // launch may leave that op's activations ready (it does when this one shares its tiles' K)
                if (next_pos < c.len && !sw) {
                    const int32_t *nw = c.cmd + next_pos;
                    const bool n_rope = nw[0] == DJ_OP_Q8_LINEAR_ROPE;
                    if ((nw[0] == DJ_OP_Q8_LINEAR || n_rope) && nw[1] == w[3] && nw[4] == m && nw[5] == n && (nw[7] & DJ_LIN_RMSNORM) &&
                        !(nw[7] & (DJ_LIN_LAYERNORM | DJ_LIN_ATTN_MERGE))) {
                        const int64_t n_rows = n_rope ? 3 * (int64_t)nw[6] : ((nw[7] & DJ_LIN_SWIGLU) ? 2 * (int64_t)nw[6] : (int64_t)nw[6]);
                        if (n_rows > 0 && n_rows < (1 << 30) && (n_rope ? q8_gemm_f16_rope_ok((int)m, nw[6], (int)n) : q8_gemm_f16_shape_ok((int)m, (int)n_rows, (int)n))) {
                            next_gamma_id = nw[8];
                            chain.next_gamma = buf(next_gamma_id, n, op, "the next op's gamma");
                        }
                    }
                }
                p.chain = &chain;
            }
            if (run) launch_q8_linear(s, p, g.workspace, g.workspace_floats);
            if (chain.left_planes) {
                g.chain.cmd = c.cmd; g.chain.pos = next_pos; g.chain.x_id = w[3]; g.chain.gamma_id = next_gamma_id;
                g.chain.m = m; g.chain.k = n; g.chain.valid = true;
            }
            break;
        }
        case DJ_OP_Q8_LINEAR_ROPE: {
            // [op, x, weight, qOut, M, K, d, flags, gamma, bias, beta, kCache, vCache, state, cos, sin, H, hd, maxSeq, layer]
            const int64_t m = w[4], k = w[5], d = w[6], H = w[16], hd = w[17], max_seq = w[18], layer = w[19];
            const int flags = w[7];
            if (m <= 1 || k <= 0 || d <= 0 || H <= 0 || hd <= 0 || (hd & 3) || H * hd != d || max_seq <= 0 || layer < 0)
                fail("OP_Q8_LINEAR_ROPE: bad shape");
            if (flags & ~(DJ_LIN_RMSNORM | DJ_LIN_LAYERNORM | DJ_LIN_BIAS)) fail("OP_Q8_LINEAR_ROPE: only a norm prologue and a bias go with it");
            const bool ln = flags & DJ_LIN_LAYERNORM;
            if (ln && (flags & DJ_LIN_RMSNORM)) fail("OP_Q8_LINEAR_ROPE: RMSNORM and LAYERNORM are exclusive");
            if (g.no_alloc || !q8_gemm_f16_rope_ok((int)m, (int)d, (int)k))
                fail("OP_Q8_LINEAR_ROPE: this shape does not run on the fp16 GEMM (deepj_hip_q8_linear_rope_ok); use Q8_LINEAR + ROPE_KV_STORE");
            const int64_t rows = 3 * d, per_layer = H * max_seq * hd;
            Q8Linear p;
            p.x = buf(w[1], m * k, op, "x");
            const float *wq = buf(w[2], (q8_bytes((int)k, (int)rows) + 3) / 4, op, "weight");
            p.wq = reinterpret_cast<const int8_t *>(wq);
            p.scales = reinterpret_cast<const float *>(p.wq + q8_scale_offset_bytes((int)k, (int)rows));
            p.out = nullptr;
            p.m = (int)m; p.k = (int)k; p.n = (int)rows; p.flags = flags;
            p.gamma = (flags & (DJ_LIN_RMSNORM | DJ_LIN_LAYERNORM)) ? buf(w[8], k, op, "gamma") : nullptr;
            p.bias = (flags & DJ_LIN_BIAS) ? buf(w[9], rows, op, "bias") : nullptr;
            p.beta = ln ? buf(w[10], k, op, "beta") : nullptr;
            p.bias2 = nullptr; p.residual = nullptr;
            p.rope.q = buf(w[3], m * d, op, "qOut");
            p.rope.k_cache = buf(w[11], (layer + 1) * per_layer, op, "kCache") + layer * per_layer;
            p.rope.v_cache = buf(w[12], (layer + 1) * per_layer, op, "vCache") + layer * per_layer;
            p.rope.state = reinterpret_cast<const int32_t *>(buf(w[13], 4, op, "state"));
            p.rope.cos_t = buf(w[14], max_seq * (hd / 2), op, "cos");
            p.rope.sin_t = buf(w[15], max_seq * (hd / 2), op, "sin");
            p.rope.hd = (int)hd; p.rope.d = (int)d; p.rope.max_seq = (int)max_seq;
            auto pit = g.prepared.find(w[2]);
            if (pit != g.prepared.end() && pit->second.k == k && pit->second.rows == rows)
                p.prepared = buf(pit->second.id, q8_prepared_floats((int)k, (int)rows), op, "prepared weights");
            if (p.prepared && run && g.capture_into) {
                const std::pair<int32_t, int32_t> pr(w[2], pit->second.id);
                auto &own = g.capture_into->self_prepared;
                if (std::find(own.begin(), own.end(), pr) == own.end()) g.capture_into->prepared.push_back(pr);
            }
            const int64_t ws = q8_linear_preferred_workspace_floats((int)m, (int)k, (int)rows, flags, p.prepared != nullptr);
            if (c.dry) c.ws_need = std::max(c.ws_need, ws);
            GemmChain chain;
            chain.planes_ready = chained(w[1], w[8], flags, m, k);
            p.chain = &chain;
            if (run) launch_q8_linear(s, p, g.workspace, g.workspace_floats);
            break;
        }
        case DJ_OP_RMSNORM: {
            int64_t rows = w[4], cols = w[5]; need_positive(op, "rows", rows); need_positive(op, "cols", cols);
            const float *x = buf(w[1], rows * cols, op, "x"), *gm = buf(w[2], cols, op, "gamma");
            float *o = buf(w[3], rows * cols, op, "out");
            if (run) launch_rmsnorm(s, x, gm, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_LAYERNORM: {
            // [op, x, gamma, beta, out, rows, cols]
            int64_t rows = w[5], cols = w[6]; need_positive(op, "rows", rows);
            if (cols <= 0) fail("OP_LAYERNORM: bad shape");
            const float *x = buf(w[1], rows * cols, op, "x"), *gm = buf(w[2], cols, op, "gamma");
            const float *bt = buf(w[3], cols, op, "beta");
            float *o = buf(w[4], rows * cols, op, "out");
            if (run) launch_layernorm(s, x, gm, bt, o, (int)rows, (int)cols);
            break;
        }
        case DJ_OP_ADD_POSITIONS: {
            // [op, x, table, state, rows, d, maxSeq]
            int64_t rows = w[4], d = w[5], max_seq = w[6]; need_positive(op, "rows", rows);
            if (d <= 0 || max_seq <= 0) fail("OP_ADD_POSITIONS: bad shape");
            float *x = buf(w[1], rows * d, op, "x");
            const float *tb = buf(w[2], max_seq * d, op, "table");
            const float *st = buf(w[3], 4, op, "state");
            if (run) launch_add_positions(s, x, tb, reinterpret_cast<const int32_t *>(st), (int)rows, (int)d, (int)max_seq);
            break;
        }
        case DJ_OP_SILU_MUL: {
            int64_t n = w[4]; need_positive(op, "n", n);
            const float *a = buf(w[1], n, op, "gate"), *b = buf(w[2], n, op, "up");
            float *o = buf(w[3], n, op, "out");
            if (run) launch_silu_mul(s, a, b, o, n);
            break;
        }
        case DJ_OP_EMBED_GATHER: {
            int64_t nids = w[4], d = w[5], vocab = w[6], ids_off = w[7];
            if (nids < 0 || d <= 0 || vocab <= 0 || ids_off < 0) fail("OP_EMBED_GATHER: bad shape");
            const float *t = buf(w[1], vocab * d, op, "table");
            const float *ids = buf(w[2], ids_off + nids, op, "ids");
            float *o = buf(w[3], nids * d, op, "out");
            if (run)
                launch_embed_gather(s, t, reinterpret_cast<const int32_t *>(ids) + ids_off, o, (int)nids, (int)d,
                                    (int)vocab);
            break;
        }
        case DJ_OP_ROPE_KV_STORE: {
            int64_t S = w[8], H = w[9], hd = w[10], max_seq = w[11], layer = w[12];
            if (S <= 0 || H <= 0 || hd <= 0 || (hd & 3) || max_seq <= 0 || layer < 0) fail("OP_ROPE_KV_STORE: bad shape");
            int64_t d = H * hd, per_layer = H * max_seq * hd;
            const float *qkv = buf(w[1], S * 3 * d, op, "qkv");
            float *q_out = buf(w[2], S * d, op, "qOut");
            float *kc = buf(w[3], (layer + 1) * per_layer, op, "kCache");
            float *vc = buf(w[4], (layer + 1) * per_layer, op, "vCache");
            const float *st = buf(w[5], 4, op, "state");
            const float *ct = buf(w[6], max_seq * (hd / 2), op, "cos"), *sn = buf(w[7], max_seq * (hd / 2), op, "sin");
            if (run)
                launch_rope_kv_store(s, qkv, q_out, kc + layer * per_layer, vc + layer * per_layer,
                                     reinterpret_cast<const int32_t *>(st), ct, sn, (int)S, (int)H, (int)hd,
                                     (int)max_seq);
            break;
        }
        case DJ_OP_ROPE_ROWS: {
            // [op, x, out, state, cos, sin, rows, H, hd, maxSeq, posFromRow, rowStride, liveExtra]
            int64_t rows = w[6], H = w[7], hd = w[8], max_seq = w[9], stride = w[11], live_extra = w[12];
            if (rows <= 0 || H <= 0 || hd <= 0 || (hd & 1) || max_seq <= 0) fail("OP_ROPE_ROWS: bad shape");
            if (w[10] && rows > max_seq) fail("OP_ROPE_ROWS: more rows than RoPE table positions");
            if (stride == 0) stride = H * hd;
            if (stride < H * hd || (stride & 1) || live_extra < -1) fail("OP_ROPE_ROWS: bad row stride or live-row count");
            const float *x = buf(w[1], (rows - 1) * stride + H * hd, op, "x");
            float *o = buf(w[2], (rows - 1) * stride + H * hd, op, "out");
            const float *st = buf(w[3], 4, op, "state");
            const float *ct = buf(w[4], max_seq * (hd / 2), op, "cos"), *sn = buf(w[5], max_seq * (hd / 2), op, "sin");
            if (run)
                launch_rope_rows(s, x, o, reinterpret_cast<const int32_t *>(st), ct, sn, (int)rows, (int)H, (int)hd,
                                 (int)max_seq, w[10], (int)stride, (int)live_extra);
            break;
        }
        case DJ_OP_ATTENTION: case DJ_OP_ATTENTION_KV: {
            // ATTENTION    [op, q, kCache, vCache, out, state, scratch, S, H, hd, maxSeq, layer]  head-major cache
            // ATTENTION_KV [op, q, k, v, out, state, scratch, S, H, hd, maxSeq, 0, tokStride, vOff]  k,v token-major rows
            int64_t S = w[7], H = w[8], hd = w[9], max_seq = w[10], layer = w[11];
            if (S <= 0 || H <= 0 || max_seq <= 0 || layer < 0) fail(std::string(op_name(op)) + ": bad shape");
            if (hd != 32 && hd != 64 && hd != 128) fail(std::string(op_name(op)) + ": head dim must be 32, 64 or 128");
            int64_t d = H * hd, per_layer = H * max_seq * hd;
            AttnArgs a;
            a.q = buf(w[1], S * d, op, "q");
            bool cache = op == DJ_OP_ATTENTION;
            if (!cache && layer != 0) fail("OP_ATTENTION_KV: layer must be 0");
            int64_t tok = d, voff = 0;
            if (!cache) {
                tok = w[12] == 0 ? d : w[12];
                voff = w[13];
                if (tok < d || (tok & 3) || voff < 0 || (voff & 3)) fail("OP_ATTENTION_KV: bad token stride or value offset");
            }
            const float *kc = cache ? buf(w[2], (layer + 1) * per_layer, op, "k") : buf(w[2], (max_seq - 1) * tok + d, op, "k");
            const float *vc = cache ? buf(w[3], (layer + 1) * per_layer, op, "v")
                                    : buf(w[3], voff + (max_seq - 1) * tok + d, op, "v") + voff;
            a.k = kc + layer * per_layer; a.v = vc + layer * per_layer;
            a.k_tok_stride = cache ? hd : tok;
            a.k_head_stride = cache ? max_seq * hd : hd;
            a.out = buf(w[4], S * d, op, "out");
            a.state = reinterpret_cast<const int32_t *>(buf(w[5], 4, op, "state"));
            int64_t sf = attention_scratch_floats((int)S, (int)H, (int)hd, (int)max_seq);
            a.scratch = sf > 0 ? buf(w[6], sf, op, "scratch") : nullptr;
            a.scratch_floats = sf;
            a.counters = g.attn_counters;
            a.s = (int)S; a.h = (int)H; a.hd = (int)hd; a.max_seq = (int)max_seq;
            if (run) launch_attention(s, a);
            break;
        }
        case DJ_OP_ARGMAX_ROWS: {
            int64_t rows = w[3], cols = w[4];
            if (rows <= 0 || cols <= 0) fail("OP_ARGMAX_ROWS: bad shape");
            const float *a = buf(w[1], rows * cols, op, "logits");
            float *o = buf(w[2], rows, op, "out");
            if (run) launch_argmax_rows(s, a, reinterpret_cast<int32_t *>(o), (int)rows, (int)cols);
            break;
        }
        case DJ_OP_DECODE_ADVANCE: {
            // [op, state, token, tokens, capacity, nPositions]
            int64_t cap = w[4]; need_positive(op, "capacity", cap);
            need_positive(op, "positions", w[5]);
            float *st = buf(w[1], 4, op, "state");
            const float *tk = buf(w[2], 1, op, "token");
            float *out = buf(w[3], std::max<int64_t>(cap, 1), op, "tokens");
            if (run)
                launch_decode_advance(s, reinterpret_cast<int32_t *>(st), reinterpret_cast<const int32_t *>(tk),
                                      reinterpret_cast<int32_t *>(out), (int)cap, w[5]);
            break;
        }
        case DJ_OP_DECODE_NEXT: {
            // [op, logits, state, tokens, capacity, table, x, vocab, d, nPos]
            int64_t cap = w[4], vocab = w[7], d = w[8];
            if (cap < 0 || vocab <= 0 || d <= 0 || w[9] < 0) fail("OP_DECODE_NEXT: bad shape");
            const float *lg = buf(w[1], vocab, op, "logits");
            float *st = buf(w[2], 4, op, "state");
            float *tk = buf(w[3], std::max<int64_t>(cap, 1), op, "tokens");
            const float *tb = buf(w[5], vocab * d, op, "table");
            float *x = buf(w[6], d, op, "x");
            if (run)
                launch_decode_next(s, lg, reinterpret_cast<int32_t *>(st), reinterpret_cast<int32_t *>(tk), (int)cap,
                                   tb, x, (int)vocab, (int)d, w[9]);
            break;
        }
        case DJ_OP_ATTN_DECODE: {
            // [op, qkv, kCache, vCache, out, state, scratch, cos, sin, H, hd, maxSeq, layer]
            int64_t H = w[9], hd = w[10], max_seq = w[11], layer = w[12];
            if (H <= 0 || max_seq <= 0 || layer < 0) fail("OP_ATTN_DECODE: bad shape");
            if (hd != 32 && hd != 64 && hd != 128) fail("OP_ATTN_DECODE: head dim must be 32, 64 or 128");
            int64_t d = H * hd, per_layer = H * max_seq * hd;
            const float *qkv = buf(w[1], 3 * d, op, "qkv");
            float *kc = buf(w[2], (layer + 1) * per_layer, op, "kCache");
            float *vc = buf(w[3], (layer + 1) * per_layer, op, "vCache");
            float *o = buf(w[4], d, op, "out");
            const float *st = buf(w[5], 4, op, "state");
            float *sc = buf(w[6], attn_decode_scratch_floats((int)H, (int)hd), op, "scratch");
            const float *ct = buf(w[7], max_seq * (hd / 2), op, "cos"), *sn = buf(w[8], max_seq * (hd / 2), op, "sin");
            if (run)
                launch_attn_decode(s, qkv, kc + layer * per_layer, vc + layer * per_layer, o,
                                   reinterpret_cast<const int32_t *>(st), sc, ct, sn, (int)H, (int)hd, (int)max_seq,
                                   g.attn_counters);
            break;
        }
        case DJ_OP_ATTN_DECODE_RECORDS: {
            // [op, qkv, kCache, vCache, records, state, cos, sin, H, hd, maxSeq, layer]
            int64_t H = w[8], hd = w[9], max_seq = w[10], layer = w[11];
            if (H <= 0 || max_seq <= 0 || layer < 0) fail("OP_ATTN_DECODE_RECORDS: bad shape");
            if (hd != 32 && hd != 64 && hd != 128) fail("OP_ATTN_DECODE_RECORDS: head dim must be 32, 64 or 128");
            if (H > 65535) fail("OP_ATTN_DECODE_RECORDS: too many heads");
            int64_t d = H * hd, per_layer = H * max_seq * hd;
            const float *qkv = buf(w[1], 3 * d, op, "qkv");
            float *kc = buf(w[2], (layer + 1) * per_layer, op, "kCache");
            float *vc = buf(w[3], (layer + 1) * per_layer, op, "vCache");
            float *rec = buf(w[4], H * kAttnRecordSplits * (hd + 4), op, "records");
            const float *st = buf(w[5], 4, op, "state");
            const float *ct = buf(w[6], max_seq * (hd / 2), op, "cos"), *sn = buf(w[7], max_seq * (hd / 2), op, "sin");
            if (run)
                launch_attn_decode_records(s, qkv, kc + layer * per_layer, vc + layer * per_layer, rec,
                                           reinterpret_cast<const int32_t *>(st), ct, sn, (int)H, (int)hd, (int)max_seq);
            break;
        }
        case DJ_OP_APPEND_ROWS: {
            // [op, src, dst, state, rows, rowFloats, maxRows, dstOff]: dst[dstOff + (state[0]+i)*rowFloats ..] = src row i
            int64_t rows = w[4], rf = w[5], max_rows = w[6], off = w[7];
            if (rows <= 0 || rf <= 0 || max_rows <= 0 || off < 0) fail("OP_APPEND_ROWS: bad shape");
            const float *src = buf(w[1], rows * rf, op, "src");
            float *dst = buf(w[2], off + max_rows * rf, op, "dst");
            const float *st = buf(w[3], 4, op, "state");
            if (run) launch_append_rows(s, src, dst + off, reinterpret_cast<const int32_t *>(st), (int)rows, (int)rf, (int)max_rows);
            break;
        }
        case DJ_OP_Q8_LINEAR_DYN: {
            // [op, x, w, out, Mmax, K, N, state, extraRows, xOff]: rows [0, min(Mmax, state[0]+extraRows)) of x + xOff
            int64_t m = w[4], k = w[5], n = w[6], extra = w[8], xoff = w[9];
            if (m <= 0 || k <= 0 || n <= 0 || extra < 0 || xoff < 0) fail("OP_Q8_LINEAR_DYN: bad shape");
            Q8Linear p;
            p.x = buf(w[1], xoff + m * k, op, "x") + xoff;
            const float *wq = buf(w[2], (q8_bytes((int)k, (int)n) + 3) / 4, op, "weight");
            p.wq = reinterpret_cast<const int8_t *>(wq);
            p.scales = reinterpret_cast<const float *>(p.wq + q8_scale_offset_bytes((int)k, (int)n));
            p.out = buf(w[3], m * n, op, "out");
            p.m = (int)m; p.k = (int)k; p.n = (int)n; p.flags = 0;
            p.gamma = p.bias = p.bias2 = p.residual = nullptr;
            p.m_dev = reinterpret_cast<const int32_t *>(buf(w[7], 4, op, "state"));
            p.m_extra = (int)extra;
            if (run) launch_q8_linear(s, p, g.workspace, g.workspace_floats);
            break;
        }
        case DJ_OP_COPY: {
            int64_t n = w[3], so = w[4], dof = w[5];
            if (n < 0 || so < 0 || dof < 0) fail("OP_COPY: bad range");
            const float *a = buf(w[1], so + n, op, "src");
            float *o = buf(w[2], dof + n, op, "dst");
            if (run) { forget_prepared(w[2]); launch_copy(s, a + so, o + dof, n); }
            break;
        }
        case DJ_OP_Q8_PREPARE: {
            // [op, weight, prepared, K, rows]: writes the weights in the many-row GEMM's layout and lets that buffer
            // stand for them in later Q8_LINEARs with more than one row, until either buffer is released or written
            int64_t k = w[3], rows = w[4]; need_positive(op, "K", k); need_positive(op, "rows", rows);
            if (w[1] == w[2]) fail("OP_Q8_PREPARE: the prepared copy needs a buffer of its own");
            const float *wq = buf(w[1], (q8_bytes((int)k, (int)rows) + 3) / 4, op, "weight");
            float *prep = buf(w[2], q8_prepared_floats((int)k, (int)rows), op, "prepared");
            if (run) {
                const int8_t *q = reinterpret_cast<const int8_t *>(wq);
                launch_q8_prepare(s, q, reinterpret_cast<const float *>(q + q8_scale_offset_bytes((int)k, (int)rows)), prep, (int)k, (int)rows);
                forget_prepared(w[2]);
                g.prepared[w[1]] = Runtime::Prepared{w[2], (int)k, (int)rows};
                if (g.capture_into) g.capture_into->self_prepared.emplace_back(w[1], w[2]);   // every replay rewrites the copy
            }
            break;
        }
        case DJ_OP_STREAM_READ: {
            // [op, src, sink, n]: reads n floats of src and keeps nothing (sink holds >= 1 float)
            int64_t n = w[3]; need_positive(op, "n", n);
            const float *a = buf(w[1], n, op, "src");
            float *o = buf(w[2], 1, op, "sink");
            if (run) launch_stream_read(s, a, o, n);
            break;
        }
        case DJ_OP_NOP: {
            // [op, grid]: an empty kernel of `grid` workgroups of 256 threads
            if (w[1] < 1 || w[1] > 65535) fail("OP_NOP: grid must be 1..65535");
            if (run) launch_nop(s, w[1]);
            break;
        }
        case DJ_OP_FILL: {
            int64_t n = w[3]; need_positive(op, "n", n);
            float *o = buf(w[1], n, op, "dst");
            if (run) { forget_prepared(w[1]); launch_fill(s, reinterpret_cast<uint32_t *>(o), (uint32_t)w[2], n); }
            break;
        }
        default:
            fail("Unknown op code in graph: " + std::to_string(op));
    }
}

void walk(const int32_t *cmd, int32_t len, bool dry, int64_t *ws_need) {
    Cursor c{cmd, len, 0, dry, 0};
    g.chain.valid = false;          // nothing carries over from an earlier stream (or from one that ended in an error)
    while (c.pos < len) {
        int op = cmd[c.pos];
        int stride = stride_of(op);
        if (stride < 0) fail("Unknown op code in graph: " + std::to_string(op));
        if (c.pos + stride > len)
            fail(std::string(op_name(op)) + ": command stream truncated at word " + std::to_string(c.pos));
        exec_one(c);
        c.pos += stride;
    }
    if (ws_need) *ws_need = c.ws_need;
}

void run_stream(const int32_t *cmd, int32_t len) {
    if (len < 0) fail("flushOps: negative stream length");
    if (len > 0 && !cmd) fail("flushOps: null command stream");
    int64_t ws = 0;
    walk(cmd, len, true, &ws);      // validate everything first
    ensure_workspace(ws);
    walk(cmd, len, false, nullptr);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) fail(std::string("kernel launch failed: ") + hipGetErrorString(e));
}

const char *op_name(int op) {
    static const char *names[] = {
        "?", "OP_ADD", "OP_SUBTRACT", "OP_MULTIPLY", "OP_DIVIDE", "OP_MATMUL", "OP_MULTIPLY_SCALAR", "OP_SQRT",
        "OP_NEG", "OP_EXP", "OP_LOG", "OP_TANH", "OP_SIGMOID", "OP_RELU", "OP_RELU_BACKWARD", "OP_GELU",
        "OP_GELU_BACKWARD", "OP_SOFTMAX_ROWS", "OP_SOFTMAX_BACKWARD", "OP_LAYERNORM_BACKWARD", "OP_ADAMW_UPDATE",
        "OP_ADD_SCALAR", "OP_DIVIDE_SCALAR", "OP_TRANSPOSE", "OP_ADD_ROW_VECTOR", "OP_ADD_BROADCAST_COLS",
        "OP_SUBTRACT_BROADCAST_COLS", "OP_DIVIDE_BROADCAST_COLS", "OP_MULTIPLY_BROADCAST_ROWS", "OP_SUM_ROWS",
        "OP_MEAN_ALONG_ROWS", "OP_VARIANCE_ALONG_ROWS", "OP_MULTIPLY_BROADCAST_COLS", "OP_SUM_ALONG_ROWS",
        "OP_MAX_ALONG_ROWS", "OP_CLAMP", "OP_POW", "OP_SCATTER_ADD_ROWS", "OP_SUM_ABS", "OP_CROSS_ENTROPY_LOSS",
        "OP_CROSS_ENTROPY_GRADIENT", "OP_SUM_SCALAR", "OP_SCATTER_ADD_ROWS_ATOMIC"};
    if (op >= 1 && op <= 42) return names[op];
    switch (op) {
        case DJ_OP_Q8_QUANTIZE: return "OP_Q8_QUANTIZE";
        case DJ_OP_Q8_DEQUANTIZE: return "OP_Q8_DEQUANTIZE";
        case DJ_OP_Q8_LINEAR: return "OP_Q8_LINEAR";
        case DJ_OP_RMSNORM: return "OP_RMSNORM";
        case DJ_OP_LAYERNORM: return "OP_LAYERNORM";
        case DJ_OP_ATTN_DECODE_RECORDS: return "OP_ATTN_DECODE_RECORDS";
        case DJ_OP_ADD_POSITIONS: return "OP_ADD_POSITIONS";
        case DJ_OP_SILU_MUL: return "OP_SILU_MUL";
        case DJ_OP_EMBED_GATHER: return "OP_EMBED_GATHER";
        case DJ_OP_ROPE_KV_STORE: return "OP_ROPE_KV_STORE";
        case DJ_OP_Q8_LINEAR_ROPE: return "OP_Q8_LINEAR_ROPE";
        case DJ_OP_ATTENTION: return "OP_ATTENTION";
        case DJ_OP_ARGMAX_ROWS: return "OP_ARGMAX_ROWS";
        case DJ_OP_DECODE_ADVANCE: return "OP_DECODE_ADVANCE";
        case DJ_OP_COPY: return "OP_COPY";
        case DJ_OP_FILL: return "OP_FILL";
        case DJ_OP_ROPE_ROWS: return "OP_ROPE_ROWS";
        case DJ_OP_ATTENTION_KV: return "OP_ATTENTION_KV";
        case DJ_OP_DECODE_NEXT: return "OP_DECODE_NEXT";
        case DJ_OP_ATTN_DECODE: return "OP_ATTN_DECODE";
        case DJ_OP_APPEND_ROWS: return "OP_APPEND_ROWS";
        case DJ_OP_Q8_LINEAR_DYN: return "OP_Q8_LINEAR_DYN";
        case DJ_OP_STREAM_READ: return "OP_STREAM_READ";
        case DJ_OP_NOP: return "OP_NOP";
        case DJ_OP_Q8_PREPARE: return "OP_Q8_PREPARE";
        default: return "OP_?";
    }
}

template <class F> int guarded(F &&f) {
    try {
        f();
        g_error.clear();
        return 0;
    } catch (const std::exception &ex) {
        g_error = ex.what();
        return 1;
    } catch (...) {
        g_error = "deepj_hip: unknown native error";
        return 1;
    }
}

}  // namespace
}  // namespace dj

using namespace dj;

extern "C" {

int deepj_hip_init(int32_t device) {
    return guarded([&] { ensure_init(device); });
}

int deepj_hip_alloc_buffers(const int32_t *ids, const int32_t *sizes, int32_t count) {
    return guarded([&] {
        ensure_init();
        if (count < 0) fail("allocBuffers: negative count");
        if (count > 0 && (!ids || !sizes)) fail("allocBuffers: null array");
        for (int i = 0; i < count; i++) {
            if (g.live.count(ids[i])) continue;          // existing id: silent no-op
            if (sizes[i] < 0) fail("allocBuffers: negative size for id " + std::to_string(ids[i]));
            size_t bytes = (size_t)sizes[i] * 4;
            size_t cls = size_class(bytes);
            Buffer b;
            b.ptr = pool_alloc(cls);
            b.capacity = cls;
            b.floats = sizes[i];
            g.live.emplace(ids[i], b);
            g.live_bytes += (int64_t)cls;
        }
    });
}

int deepj_hip_upload(int32_t id, const float *src, int64_t n) {
    return guarded([&] {
        ensure_init();
        auto it = g.live.find(id);
        if (it == g.live.end()) fail("Buffer not found for upload");
        if (n < 0 || n > it->second.floats)
            fail("uploadBuffer: " + std::to_string(n) + " floats do not fit buffer id=" + std::to_string(id) + " of " +
                 std::to_string(it->second.floats));
        if (n == 0) return;
        if (!src) fail("uploadBuffer: null source");
        forget_prepared(id);
        size_t bytes = (size_t)n * 4;
        // The caller's array is only borrowed: the copy out of it has finished on return.
        if (bytes <= g.staging_bytes) {
            DJ_HIP(hipStreamSynchronize(g.stream));      // staging block may still be in flight
            std::memcpy(g.staging, src, bytes);
            DJ_HIP(hipMemcpyAsync(it->second.ptr, g.staging, bytes, hipMemcpyHostToDevice, g.stream));
        } else {
            DJ_HIP(hipMemcpyAsync(it->second.ptr, src, bytes, hipMemcpyHostToDevice, g.stream));
            DJ_HIP(hipStreamSynchronize(g.stream));
        }
    });
}

int deepj_hip_download(int32_t id, float *dst, int64_t n) {
    return guarded([&] {
        ensure_init();
        auto it = g.live.find(id);
        if (it == g.live.end()) fail("Buffer not found for download");
        if (n < 0 || n > it->second.floats)
            fail("downloadBuffer: " + std::to_string(n) + " floats exceed buffer id=" + std::to_string(id) + " of " +
                 std::to_string(it->second.floats));
        if (n > 0 && !dst) fail("downloadBuffer: null destination");
        if (n > 0) DJ_HIP(hipMemcpyAsync(dst, it->second.ptr, (size_t)n * 4, hipMemcpyDeviceToHost, g.stream));
        DJ_HIP(hipStreamSynchronize(g.stream));
    });
}

int deepj_hip_release(const int32_t *ids, int32_t count) {
    return guarded([&] {
        if (!g.ready) return;
        if (count > 0 && !ids) fail("releaseBuffers: null array");
        for (int i = 0; i < count; i++) {
            auto it = g.live.find(ids[i]);
            if (it == g.live.end()) continue;            // unknown id: silent no-op
            g.live_bytes -= (int64_t)it->second.capacity;
            pool_free(it->second.ptr, it->second.capacity);
            g.live.erase(it);
            forget_prepared(ids[i]);
        }
    });
}

int deepj_hip_flush_ops(const int32_t *cmd, int32_t len) {
    return guarded([&] {
        ensure_init();
        run_stream(cmd, len);
    });
}

// The same interpreter over the static scratch array instead of the runtime's own (growable) workspace and
// counters: no hipMalloc / hipFree on this path.  The counters are cleared by a fill kernel first (the array keeps
// whatever the last call left); calls that overlap on one GPU would share the array and race.
int deepj_hip_flush_ops_noalloc(const int32_t *cmd, int32_t len) {
    return guarded([&] {
        if (!g.ready)
            fail("flush_ops_noalloc: the runtime is not initialised (initialisation allocates: call deepj_hip_init first)");
        struct Scope {
            float *ws = g.workspace; int64_t wsf = g.workspace_floats; unsigned *ctr = g.attn_counters;
            Scope() {
                g.no_alloc = true;
                g.attn_counters = reinterpret_cast<unsigned *>(g.static_scratch);
                g.workspace = reinterpret_cast<float *>(g.static_scratch + kStaticCounterBytes);
                g.workspace_floats = kStaticWorkspaceFloats;
            }
            ~Scope() { g.no_alloc = false; g.workspace = ws; g.workspace_floats = wsf; g.attn_counters = ctr; }
        } scope;
        if (len < 0) fail("flushOps: negative stream length");
        if (len > 0 && !cmd) fail("flushOps: null command stream");
        int64_t ws = 0;
        walk(cmd, len, true, &ws);
        ensure_workspace(ws);           // only checks the need against the static size here
        launch_fill(g.stream, reinterpret_cast<uint32_t *>(g.attn_counters), 0u, kAttnCounterHeads);
        walk(cmd, len, false, nullptr);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) fail(std::string("kernel launch failed: ") + hipGetErrorString(e));
    });
}

const char *deepj_hip_last_error(void) { return g_error.c_str(); }

int deepj_hip_synchronize(void) {
    return guarded([&] {
        if (g.ready) DJ_HIP(hipStreamSynchronize(g.stream));
    });
}

int deepj_hip_trim(void) {
    return guarded([&] {
        if (!g.ready) return;
        DJ_HIP(hipStreamSynchronize(g.stream));
        for (auto &kv : g.cache) {
            for (void *p : kv.second) DJ_HIP(hipFree(p));
            kv.second.clear();
        }
        g.cached_bytes = 0;
    });
}

int deepj_hip_shutdown(void) {
    return guarded([&] {
        if (!g.ready) return;
        DJ_HIP(hipStreamSynchronize(g.stream));
        for (auto &kv : g.graphs) {
            if (kv.second.exec) (void)hipGraphExecDestroy(kv.second.exec);
            if (kv.second.graph) (void)hipGraphDestroy(kv.second.graph);
        }
        g.graphs.clear();
        for (auto &kv : g.live) (void)hipFree(kv.second.ptr);
        g.live.clear();
        for (auto &kv : g.cache)
            for (void *p : kv.second) (void)hipFree(p);
        g.cache.clear();
        if (g.workspace) (void)hipFree(g.workspace);
        g.workspace = nullptr; g.workspace_floats = 0;
        if (g.attn_counters) (void)hipFree(g.attn_counters);
        g.attn_counters = nullptr;
        g.prepared.clear();      // the association names buffer ids; a later session may reuse them for other things
        if (g.staging) (void)hipHostFree(g.staging);
        g.staging = nullptr;
        (void)hipStreamDestroy(g.stream);
        g.stream = nullptr;
        g.live_bytes = g.cached_bytes = 0;
        g.ready = false;
    });
}

int deepj_hip_pool_stats(int64_t out[4]) {
    return guarded([&] {
        if (!out) fail("pool_stats: null output");
        out[0] = (int64_t)g.live.size();
        out[1] = g.live_bytes;
        out[2] = g.cached_bytes;
        out[3] = g.driver_allocs;
    });
}

void *deepj_hip_stream(void) { return g.ready ? (void *)g.stream : nullptr; }

int32_t deepj_hip_attn_record_splits(void) { return kAttnRecordSplits; }

int64_t deepj_hip_attention_scratch_floats(int32_t S, int32_t H, int32_t hd, int32_t max_seq) {
    if (S <= 0 || H <= 0 || hd <= 0) return 0;
    return attention_scratch_floats(S, H, hd, max_seq);
}

int64_t deepj_hip_q8_floats(int32_t k, int32_t rows) {
    if (k <= 0 || rows <= 0) return 0;
    return (q8_bytes(k, rows) + 3) / 4;
}

int64_t deepj_hip_q8_prepared_floats(int32_t k, int32_t rows) {
    if (k <= 0 || rows <= 0) return 0;
    return q8_prepared_floats(k, rows);
}

int32_t deepj_hip_q8_gemm_path(int32_t m, int32_t k, int32_t rows) {
    if (m <= 1 || k <= 0 || rows <= 0) return 0;
    return q8_gemm_f16_tile_rows(m, rows, k);
}

void deepj_hip_q8_gemm_tile(int32_t m, int32_t k, int32_t rows, int32_t *tile_rows, int32_t *tile_cols, int32_t *k_shares) {
    int tr = 0, tc = 0, ks = 1;
    if (m > 1 && k > 0 && rows > 0) q8_gemm_f16_tile(m, rows, k, &tr, &tc, &ks);
    if (tile_rows) *tile_rows = tr;
    if (tile_cols) *tile_cols = tc;
    if (k_shares) *k_shares = ks;
}

void deepj_hip_q8_gemm_tile_prepared(int32_t m, int32_t k, int32_t rows, int32_t *tile_rows, int32_t *tile_cols, int32_t *k_shares) {
    int tr = 0, tc = 0, ks = 1;
    if (m > 1 && k > 0 && rows > 0) q8_gemm_f16_tile(m, rows, k, &tr, &tc, &ks, true);
    if (tile_rows) *tile_rows = tr;
    if (tile_cols) *tile_cols = tc;
    if (k_shares) *k_shares = ks;
}

int32_t deepj_hip_q8_linear_rope_ok(int32_t m, int32_t k, int32_t d) {
    if (m <= 1 || k <= 0 || d <= 0) return 0;
    return q8_gemm_f16_rope_ok(m, d, k) ? 1 : 0;
}

int32_t deepj_hip_q8_gemm_f16_extents(int32_t m, int32_t k, int32_t rows, int32_t tile_rows, int32_t tile_cols, int64_t *reach3, int64_t *size3) {
    if (m <= 1 || k <= 0 || rows <= 0 || !reach3 || !size3) return -1;
    int tr = tile_rows, tc = tile_cols;
    if (tr == 0) q8_gemm_f16_tile(m, rows, k, &tr, &tc, nullptr);
    if (!((tr == 128 || tr == 64) && (tc == 256 || tc == 192))) return -1;
    return q8_gemm_f16_extents(m, rows, k, tr, tc, reach3, size3) ? 1 : 0;
}

int deepj_hip_time_ops(const int32_t *cmd, int32_t len, int32_t iters, float *ms_total) {
    return guarded([&] {
        ensure_init();
        if (iters <= 0 || !ms_total) fail("time_ops: bad arguments");
        int64_t ws = 0;
        walk(cmd, len, true, &ws);
        ensure_workspace(ws);
        hipEvent_t e0, e1;
        DJ_HIP(hipEventCreate(&e0));
        DJ_HIP(hipEventCreate(&e1));
        DJ_HIP(hipEventRecord(e0, g.stream));
        for (int i = 0; i < iters; i++) walk(cmd, len, false, nullptr);
        DJ_HIP(hipEventRecord(e1, g.stream));
        DJ_HIP(hipEventSynchronize(e1));
        DJ_HIP(hipEventElapsedTime(ms_total, e0, e1));
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) fail(std::string("kernel launch failed: ") + hipGetErrorString(e));
    });
}

// The shader clock while a stream runs: a one-wavefront kernel on a second stream (default priority) samples
// (shader clock counter, 100 MHz wall clock) pairs while `cmd` runs `iters` times on the library's stream, bracketed by
// wall-clock stamps.  pairs receives 2 * samples counters, window the wall clock before and after the runs.  The
// sampler sleeps sleep_reps x 127 x 64 clocks between samples and ends by itself after `samples` of them.
int deepj_hip_clock_probe(const int32_t *cmd, int32_t len, int32_t iters, int32_t samples, int32_t sleep_reps,
                          uint64_t *pairs, uint64_t *window) {
    return guarded([&] {
        ensure_init();
        if (iters < 0 || samples <= 0 || samples > (1 << 20) || sleep_reps < 0 || sleep_reps > 4096 || !pairs || !window)
            fail("clock_probe: bad arguments");
        int64_t ws = 0;
        if (len > 0) walk(cmd, len, true, &ws);
        ensure_workspace(ws);
        hipStream_t side = nullptr;
        unsigned long long *d = nullptr;
        DJ_HIP(hipStreamCreateWithFlags(&side, hipStreamNonBlocking));
        const size_t bytes = ((size_t)2 * samples + 2) * sizeof(unsigned long long);
        hipError_t e = hipMalloc((void **)&d, bytes);
        if (e != hipSuccess) { (void)hipStreamDestroy(side); fail(std::string("clock_probe: hipMalloc: ") + hipGetErrorString(e)); }
        (void)hipMemset(d, 0, bytes);
        DJ_HIP(hipDeviceSynchronize());
        launch_clock_probe(side, d, samples, sleep_reps);
        launch_wall_stamp(g.stream, d + 2 * samples);
        for (int i = 0; i < iters && len > 0; i++) walk(cmd, len, false, nullptr);
        launch_wall_stamp(g.stream, d + 2 * samples + 1);
        e = hipStreamSynchronize(g.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(side);
        if (e == hipSuccess) e = hipMemcpy(pairs, d, (size_t)2 * samples * sizeof(unsigned long long), hipMemcpyDeviceToHost);
        if (e == hipSuccess) e = hipMemcpy(window, d + 2 * samples, 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost);
        (void)hipFree(d);
        (void)hipStreamDestroy(side);
        if (e != hipSuccess) fail(std::string("clock_probe: ") + hipGetErrorString(e));
    });
}

// Per-op kernel durations: every kernel dispatch of every op of the stream carries a start and a stop event, the
// stream runs `iters` times in order, and us_per_op[i] receives the mean over the passes of the summed begin-to-end
// times of op i's dispatches in microseconds (-1 for an op that launched nothing).  Optional outputs of the same
// length: us_longest[i], the longest single dispatch of the op (its main kernel), and dispatches[i], how many
// dispatches the op made (at most kMaxTimedLaunches of them are timed).
int deepj_hip_profile_ops(const int32_t *cmd, int32_t len, int32_t iters, float *us_per_op, int32_t capacity,
                          int32_t *n_ops, float *us_longest, int32_t *dispatches) {
    return guarded([&] {
        ensure_init();
        if (iters <= 0 || !us_per_op || capacity < 0) fail("profile_ops: bad arguments");
        int64_t ws = 0;
        walk(cmd, len, true, &ws);
        ensure_workspace(ws);
        std::vector<int32_t> starts;                 // word offset of every op
        for (int32_t pos = 0; pos < len; pos += stride_of(cmd[pos])) starts.push_back(pos);
        const int n = (int)starts.size();
        if (n_ops) *n_ops = n;
        if (n > capacity) fail("profile_ops: the stream holds " + std::to_string(n) + " ops, the output only " + std::to_string(capacity));
        constexpr int per_op = 2 * kMaxTimedLaunches;
        std::vector<hipEvent_t> ev((size_t)per_op * n, nullptr);
        std::vector<double> sum((size_t)n, 0.0), longest((size_t)n, 0.0);
        std::vector<int> count((size_t)n, 0), launches((size_t)n, 0);
        auto cleanup = [&] {
            g_launch_timing = LaunchTiming{};
            for (hipEvent_t e : ev) if (e) (void)hipEventDestroy(e);
        };
        try {
            for (auto &e : ev) DJ_HIP(hipEventCreate(&e));
            for (int it = 0; it < iters; it++) {
                g.chain.valid = false;
                for (int i = 0; i < n; i++) {
                    Cursor c{cmd, len, starts[(size_t)i], false, 0};
                    g_launch_timing.pairs = ev.data() + (size_t)per_op * i;
                    g_launch_timing.used = 0;
                    g_launch_timing.armed = true;
                    exec_one(c);
                    launches[(size_t)i] = g_launch_timing.used;
                    g_launch_timing.armed = false;
                }
                DJ_HIP(hipStreamSynchronize(g.stream));
                for (int i = 0; i < n; i++) {
                    if (!launches[(size_t)i]) continue;
                    double total = 0.0, top = 0.0;
                    for (int j = 0; j < launches[(size_t)i]; j++) {
                        float ms = 0.0f;
                        DJ_HIP(hipEventElapsedTime(&ms, ev[(size_t)per_op * i + 2 * j], ev[(size_t)per_op * i + 2 * j + 1]));
                        total += (double)ms * 1e3;
                        top = std::max(top, (double)ms * 1e3);
                    }
                    sum[(size_t)i] += total;
                    longest[(size_t)i] += top;
                    count[(size_t)i]++;
                }
            }
        } catch (...) {
            cleanup();
            throw;
        }
        cleanup();
        for (int i = 0; i < n; i++) {
            const bool ok = count[(size_t)i] > 0;
            us_per_op[i] = ok ? (float)(sum[(size_t)i] / count[(size_t)i]) : -1.0f;
            if (us_longest) us_longest[i] = ok ? (float)(longest[(size_t)i] / count[(size_t)i]) : -1.0f;
            if (dispatches) dispatches[i] = launches[(size_t)i];
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) fail(std::string("kernel launch failed: ") + hipGetErrorString(e));
    });
}

int deepj_hip_graph_capture(const int32_t *cmd, int32_t len, int32_t *handle) {
    return guarded([&] {
        ensure_init();
        if (!handle) fail("graph_capture: null handle");
        int64_t ws = 0;
        Graph gr;
        g.track = &gr.refs;
        try {
            walk(cmd, len, true, &ws);
        } catch (...) {
            g.track = nullptr;
            throw;
        }
        g.track = nullptr;
        std::sort(gr.refs.begin(), gr.refs.end());
        gr.refs.erase(std::unique(gr.refs.begin(), gr.refs.end()), gr.refs.end());
        ensure_workspace(ws);
        if (ws > 0) gr.workspace = g.workspace;
        DJ_HIP(hipStreamSynchronize(g.stream));
        DJ_HIP(hipStreamBeginCapture(g.stream, hipStreamCaptureModeThreadLocal));
        g.capturing = true;
        g.capture_into = &gr;
        try {
            walk(cmd, len, false, nullptr);
        } catch (...) {
            g.capturing = false;
            g.capture_into = nullptr;
            hipGraph_t tmp = nullptr;
            (void)hipStreamEndCapture(g.stream, &tmp);
            if (tmp) (void)hipGraphDestroy(tmp);
            throw;
        }
        g.capturing = false;
        g.capture_into = nullptr;
        DJ_HIP(hipStreamEndCapture(g.stream, &gr.graph));
        hipError_t e = hipGraphInstantiate(&gr.exec, gr.graph, nullptr, nullptr, 0);
        if (e != hipSuccess) {
            (void)hipGraphDestroy(gr.graph);
            fail(std::string("hipGraphInstantiate: ") + hipGetErrorString(e));
        }
        int32_t h = g.next_graph++;
        g.graphs.emplace(h, gr);
        *handle = h;
    });
}

int deepj_hip_graph_launch(int32_t handle, int32_t times) {
    return guarded([&] {
        auto it = g.graphs.find(handle);
        if (it == g.graphs.end()) fail("graph_launch: unknown graph handle " + std::to_string(handle));
        // the graph replays raw addresses: refuse when a buffer it names was released or now lives elsewhere,
        // or when the workspace it used has been replaced by a larger one
        for (const auto &ref : it->second.refs) {
            auto b = g.live.find(ref.first);
            if (b == g.live.end() || b->second.ptr != ref.second)
                fail("graph_launch: buffer id=" + std::to_string(ref.first) + " was released or reallocated after graph " +
                     std::to_string(handle) + " was captured; capture the stream again");
        }
        if (it->second.workspace && it->second.workspace != g.workspace)
            fail("graph_launch: the workspace was reallocated after graph " + std::to_string(handle) +
                 " was captured; capture the stream again");
        for (const auto &pr : it->second.prepared) {
            auto p = g.prepared.find(pr.first);
            if (p == g.prepared.end() || p->second.id != pr.second)
                fail("graph_launch: Q8 weights id=" + std::to_string(pr.first) + " were written after graph " + std::to_string(handle) +
                     " was captured with their prepared copy id=" + std::to_string(pr.second) + "; capture the stream again");
        }
        // Bounded run-ahead: at most kRing windows of kWindow replays are queued behind the one the
        // device is executing, so a long run never piles tens of thousands of dispatches (and their
        // kernel-argument blocks) into the queue; the device is never left idle by this.
        constexpr int kWindow = 16, kRing = 4;
        static hipEvent_t ring[kRing] = {};
        for (int i = 0; i < times; i++) {
            if (i % kWindow == 0) {
                int w = i / kWindow, slot = w % kRing;
                if (!ring[slot]) DJ_HIP(hipEventCreateWithFlags(&ring[slot], hipEventDisableTiming));
                if (w >= kRing) DJ_HIP(hipEventSynchronize(ring[slot]));
                if (w > 0) DJ_HIP(hipEventRecord(ring[(w - 1) % kRing], g.stream));
            }
            DJ_HIP(hipGraphLaunch(it->second.exec, g.stream));
        }
    });
}

int deepj_hip_graph_destroy(int32_t handle) {
    return guarded([&] {
        auto it = g.graphs.find(handle);
        if (it == g.graphs.end()) return;
        DJ_HIP(hipStreamSynchronize(g.stream));
        (void)hipGraphExecDestroy(it->second.exec);
        (void)hipGraphDestroy(it->second.graph);
        g.graphs.erase(it);
    });
}

}  // extern "C"
