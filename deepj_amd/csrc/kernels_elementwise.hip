// Element-wise, broadcast and data-movement kernels of the 42 primitive opcodes
// (semantics: CpuBackend.java:56-132,190-214,300-354,466-489,542-549 in the
// reference) plus the small fused inference helpers.  All of them are HBM
// bound: one pass, 128-bit accesses where the length allows it, grid sized to
// a multiple of the 256 CUs.
//
// Transcendentals follow the CPU backend's convention - evaluate in f64, cast
// to fp32 (CpuBackend.java:24-28) - so a GPU result differs from the CPU one by
// at most the last f64 bit of the math library, not by an fp32 approximation.
#include "dj_common.h"

namespace dj {
namespace {

constexpr int kThreads = 256;

inline int grid_for(int64_t work_items, int per_thread = 1) {
    int64_t blocks = (work_items + (int64_t)kThreads * per_thread - 1) / ((int64_t)kThreads * per_thread);
    if (blocks < 1) blocks = 1;
    if (blocks > 256 * 32) blocks = 256 * 32;      // grid-stride beyond 32 blocks per CU
    return (int)blocks;
}

__device__ __forceinline__ float d_exp(float x) { return (float)exp((double)x); }
__device__ __forceinline__ float d_log(float x) { return (float)log((double)x); }
__device__ __forceinline__ float d_tanh(float x) { return (float)tanh((double)x); }
__device__ __forceinline__ float d_pow(float x, float e) { return (float)pow((double)x, (double)e); }
__device__ __forceinline__ float d_sigmoid(float x) { return 1.0f / (1.0f + d_exp(-x)); }

__device__ __forceinline__ float d_gelu(float x) {
    float c = sqrtf(2.0f / 3.14159265358979323846f);
    float x3 = x * x * x;
    float t = c * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + d_tanh(t));
}
__device__ __forceinline__ float d_gelu_deriv(float x) {
    float c = sqrtf(2.0f / 3.14159265358979323846f);
    float x2 = x * x;
    float x3 = x2 * x;
    float t = c * (x + 0.044715f * x3);
    float th = d_tanh(t);
    float sech2 = 1.0f - th * th;
    float dtdx = c * (1.0f + 3.0f * 0.044715f * x2);
    return 0.5f * (1.0f + th) + 0.5f * x * sech2 * dtdx;
}

template <int OP> __device__ __forceinline__ float binary_op(float x, float y) {
    if constexpr (OP == DJ_OP_ADD) return x + y;
    if constexpr (OP == DJ_OP_SUBTRACT) return x - y;
    if constexpr (OP == DJ_OP_MULTIPLY) return x * y;
    if constexpr (OP == DJ_OP_DIVIDE) return x / y;
    if constexpr (OP == DJ_OP_RELU_BACKWARD) return x > 0.0f ? y : 0.0f;
    if constexpr (OP == DJ_OP_GELU_BACKWARD) return y * d_gelu_deriv(x);
    return 0.0f;
}

template <int OP> __device__ __forceinline__ float unary_op(float x) {
    if constexpr (OP == DJ_OP_SQRT) return sqrtf(x);          // correctly rounded, as (float)Math.sqrt
    if constexpr (OP == DJ_OP_NEG) return -x;
    if constexpr (OP == DJ_OP_EXP) return d_exp(x);
    if constexpr (OP == DJ_OP_LOG) return d_log(x);
    if constexpr (OP == DJ_OP_TANH) return d_tanh(x);
    if constexpr (OP == DJ_OP_SIGMOID) return d_sigmoid(x);
    if constexpr (OP == DJ_OP_RELU) return x > 0.0f ? x : (x != x ? x : 0.0f);
    if constexpr (OP == DJ_OP_GELU) return d_gelu(x);
    return 0.0f;
}

template <int OP> __device__ __forceinline__ float scalar_op(float x, float s0, float s1) {
    if constexpr (OP == DJ_OP_MULTIPLY_SCALAR) return x * s0;
    if constexpr (OP == DJ_OP_ADD_SCALAR) return x + s0;
    if constexpr (OP == DJ_OP_DIVIDE_SCALAR) return x / s0;
    if constexpr (OP == DJ_OP_POW) return d_pow(x, s0);
    if constexpr (OP == DJ_OP_CLAMP) {                         // Math.min(max, Math.max(min, x))
        float mx = x > s0 ? x : s0;
        if (x != x) mx = x;
        float mn = mx < s1 ? mx : s1;
        if (mx != mx) mn = mx;
        return mn;
    }
    return 0.0f;
}

template <int OP>
__global__ void __launch_bounds__(kThreads) k_binary(const float *__restrict__ a, const float *__restrict__ b,
                                                     float *__restrict__ out, int64_t n) {
    int64_t n4 = n >> 2;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const float4 *a4 = reinterpret_cast<const float4 *>(a);
    const float4 *b4 = reinterpret_cast<const float4 *>(b);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    for (int64_t i = tid; i < n4; i += stride) {
        float4 x = a4[i], y = b4[i], r;
        r.x = binary_op<OP>(x.x, y.x); r.y = binary_op<OP>(x.y, y.y);
        r.z = binary_op<OP>(x.z, y.z); r.w = binary_op<OP>(x.w, y.w);
        o4[i] = r;
    }
    for (int64_t i = (n4 << 2) + tid; i < n; i += stride) out[i] = binary_op<OP>(a[i], b[i]);
}

template <int OP>
__global__ void __launch_bounds__(kThreads) k_unary(const float *__restrict__ a, float *__restrict__ out, int64_t n) {
    int64_t n4 = n >> 2;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const float4 *a4 = reinterpret_cast<const float4 *>(a);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    for (int64_t i = tid; i < n4; i += stride) {
        float4 x = a4[i], r;
        r.x = unary_op<OP>(x.x); r.y = unary_op<OP>(x.y); r.z = unary_op<OP>(x.z); r.w = unary_op<OP>(x.w);
        o4[i] = r;
    }
    for (int64_t i = (n4 << 2) + tid; i < n; i += stride) out[i] = unary_op<OP>(a[i]);
}

template <int OP>
__global__ void __launch_bounds__(kThreads) k_scalar(const float *__restrict__ a, float *__restrict__ out,
                                                     float s0, float s1, int64_t n) {
    int64_t n4 = n >> 2;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const float4 *a4 = reinterpret_cast<const float4 *>(a);
    float4 *o4 = reinterpret_cast<float4 *>(out);
    for (int64_t i = tid; i < n4; i += stride) {
        float4 x = a4[i], r;
        r.x = scalar_op<OP>(x.x, s0, s1); r.y = scalar_op<OP>(x.y, s0, s1);
        r.z = scalar_op<OP>(x.z, s0, s1); r.w = scalar_op<OP>(x.w, s0, s1);
        o4[i] = r;
    }
    for (int64_t i = (n4 << 2) + tid; i < n; i += stride) out[i] = scalar_op<OP>(a[i], s0, s1);
}

// out[r,c] = a[r,c] (op) v[c]  (ROWVEC)  or  a[r,c] (op) v[r]  (column vector)
template <int OP, bool ROWVEC>
__global__ void __launch_bounds__(kThreads) k_broadcast(const float *__restrict__ a, const float *__restrict__ v,
                                                        float *__restrict__ out, int rows, int cols) {
    int64_t n = (int64_t)rows * cols;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int r = (int)(i / cols);
        int c = (int)(i - (int64_t)r * cols);
        float y = ROWVEC ? v[c] : v[r];
        out[i] = binary_op<OP>(a[i], y);
    }
}

// 32x32 tile through LDS (+1 padding: no bank conflicts on the transposed read).
__global__ void __launch_bounds__(256) k_transpose(const float *__restrict__ a, float *__restrict__ out, int rows,
                                                   int cols) {
    __shared__ float tile[32][33];
    int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;     // 32 x 8
    int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    for (int j = ty; j < 32; j += 8) {
        int r = r0 + j, c = c0 + tx;
        if (r < rows && c < cols) tile[j][tx] = a[(int64_t)r * cols + c];
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
        int c = c0 + j, r = r0 + tx;                       // out is [cols x rows]
        if (r < rows && c < cols) out[(int64_t)c * rows + r] = tile[tx][j];
    }
}

__global__ void __launch_bounds__(kThreads) k_adamw(float *__restrict__ w, const float *__restrict__ g,
                                                    float *__restrict__ mt, float *__restrict__ vt, int64_t n,
                                                    float lr, float beta1, float beta2, float eps, float wd,
                                                    float bc1, float bc2) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float grad = g[i];
        float m_new = beta1 * mt[i] + (1.0f - beta1) * grad;
        float v_new = beta2 * vt[i] + (1.0f - beta2) * (grad * grad);
        mt[i] = m_new;
        vt[i] = v_new;
        float m_hat = m_new / bc1;
        float v_hat = v_new / bc2;
        float update = (lr * m_hat) / (sqrtf(v_hat) + eps);
        if (wd != 0.0f) update += lr * wd * w[i];
        w[i] -= update;
    }
}

// target[idx[i], c] += grad[i, c]; indices arrive as floats (MetalBackend.java:43-54),
// rows outside the target are skipped (deepj_metal_jni.mm:606-607).
__global__ void __launch_bounds__(kThreads) k_scatter_add(float *__restrict__ target, const float *__restrict__ idx,
                                                          const float *__restrict__ grad, int target_rows, int cols,
                                                          int n_idx) {
    int64_t n = (int64_t)n_idx * cols;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += stride) {
        int i = (int)(t / cols);
        int c = (int)(t - (int64_t)i * cols);
        float fi = idx[i];
        if (!(fi >= 0.0f) || fi >= (float)target_rows) continue;
        int row = (int)fi;
        atomicAdd(&target[(int64_t)row * cols + c], grad[t]);
    }
}

__global__ void __launch_bounds__(kThreads) k_fill(uint32_t *__restrict__ dst, uint32_t bits, int64_t n) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = bits;
}

// Measurement floor of the HBM-bound decode kernels: the same bytes read with 128-bit loads, D in flight per lane,
// nothing computed but an AND over the words (so that no load can be dropped) and nothing stored unless every bit of
// the buffer is set.
template <int D>
__global__ void __launch_bounds__(kThreads) k_stream_read(const uint4 *__restrict__ src, uint32_t *__restrict__ sink,
                                                          int64_t n16, int64_t tail_from, const uint32_t *src_words,
                                                          int64_t n_words) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t acc = 0xffffffffu;
    for (; i + (D - 1) * stride < n16; i += D * stride) {
        uint4 v[D];
#pragma unroll
        for (int u = 0; u < D; u++) v[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < D; u++) acc &= v[u].x & v[u].y & v[u].z & v[u].w;
    }
    for (; i < n16; i += stride) { uint4 v = src[i]; acc &= v.x & v.y & v.z & v.w; }
    for (int64_t j = tail_from + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < n_words; j += stride) acc &= src_words[j];
    if (acc == 0xffffffffu && n_words > 0 && src_words[0] == 0xffffffffu) sink[0] = acc;     // practically never
}

__global__ void k_nop() {}

__global__ void __launch_bounds__(kThreads) k_copy(const float *__restrict__ src, float *__restrict__ dst, int64_t n) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// SiLU.java:20-24 then SwiGLULayer.java:69: (g * sigmoid(g)) * up
__global__ void __launch_bounds__(kThreads) k_silu_mul(const float *__restrict__ gate, const float *__restrict__ up,
                                                       float *__restrict__ out, int64_t n) {
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float g = gate[i];
        float sg = g * d_sigmoid(g);
        out[i] = sg * up[i];
    }
}

// Embedding.java:28-34 (Tensor.sliceRows): out[i,:] = table[ids[i],:].  Ids were range
// checked on the host when they came from the host; ids produced on the device
// (argmax) are always < vocab.  An out-of-range id writes NaN instead of reading.
__global__ void __launch_bounds__(kThreads) k_embed_gather(const float *__restrict__ table,
                                                           const int32_t *__restrict__ ids, float *__restrict__ out,
                                                           int n_ids, int d, int vocab) {
    int i = blockIdx.x;
    if (i >= n_ids) return;
    int id = ids[i];
    bool ok = id >= 0 && id < vocab;
    const float *src = table + (int64_t)(ok ? id : 0) * d;
    float *dst = out + (int64_t)i * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) dst[c] = ok ? src[c] : __builtin_nanf("");
}

// dst[(state[0] + i), :] = src[i, :] for i < rows: append to a cache whose fill level lives on the device.
__global__ void __launch_bounds__(kThreads) k_append_rows(const float *__restrict__ src, float *__restrict__ dst,
                                                          const int32_t *__restrict__ state, int rows, int row_floats,
                                                          int max_rows) {
    const int pos0 = state[0];
    int64_t n = (int64_t)rows * row_floats;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < n; t += stride) {
        int i = (int)(t / row_floats);
        int j = (int)(t - (int64_t)i * row_floats);
        int r = pos0 + i;
        if (r >= 0 && r < max_rows) dst[(int64_t)r * row_floats + j] = src[t];
    }
}

// state[0] = positions held in the cache, state[1] = current token, state[2] = tokens generated.
__global__ void k_decode_advance(int32_t *state, const int32_t *token, int32_t *tokens, int capacity,
                                 int n_positions) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        int32_t t = token[0];
        int32_t g = state[2];
        if (g < capacity) tokens[g] = t;
        state[1] = t;
        state[0] = state[0] + n_positions;
        state[2] = g + 1;
    }
}

}  // namespace

#define DJ_LAUNCH(kernel, grid, block, stream, ...) \
    launch_kernel(kernel, dim3(grid), dim3(block), 0, stream, __VA_ARGS__)

void launch_binary(hipStream_t s, int op, const float *a, const float *b, float *out, int64_t n) {
    if (n <= 0) return;
    int grid = grid_for(n, 4);
    switch (op) {
        case DJ_OP_ADD: DJ_LAUNCH(k_binary<DJ_OP_ADD>, grid, kThreads, s, a, b, out, n); break;
        case DJ_OP_SUBTRACT: DJ_LAUNCH(k_binary<DJ_OP_SUBTRACT>, grid, kThreads, s, a, b, out, n); break;
        case DJ_OP_MULTIPLY: DJ_LAUNCH(k_binary<DJ_OP_MULTIPLY>, grid, kThreads, s, a, b, out, n); break;
        case DJ_OP_DIVIDE: DJ_LAUNCH(k_binary<DJ_OP_DIVIDE>, grid, kThreads, s, a, b, out, n); break;
        case DJ_OP_RELU_BACKWARD: DJ_LAUNCH(k_binary<DJ_OP_RELU_BACKWARD>, grid, kThreads, s, a, b, out, n); break;
        case DJ_OP_GELU_BACKWARD: DJ_LAUNCH(k_binary<DJ_OP_GELU_BACKWARD>, grid, kThreads, s, a, b, out, n); break;
        default: fail("launch_binary: bad op");
    }
}

void launch_unary(hipStream_t s, int op, const float *a, float *out, int64_t n) {
    if (n <= 0) return;
    int grid = grid_for(n, 4);
    switch (op) {
        case DJ_OP_SQRT: DJ_LAUNCH(k_unary<DJ_OP_SQRT>, grid, kThreads, s, a, out, n); break;
        case DJ_OP_NEG: DJ_LAUNCH(k_unary<DJ_OP_NEG>, grid, kThreads, s, a, out, n); break;
        case DJ_OP_EXP: DJ_LAUNCH(k_unary<DJ_OP_EXP>, grid, kThreads, s, a, out, n); break;
        case DJ_OP_LOG: DJ_LAUNCH(k_unary<DJ_OP_LOG>, grid, kThreads, s, a, out, n); break;
        case DJ_OP_TANH: DJ_LAUNCH(k_unary<DJ_OP_TANH>, grid, kThreads, s, a, out, n); break;
        case DJ_OP_SIGMOID: DJ_LAUNCH(k_unary<DJ_OP_SIGMOID>, grid, kThreads, s, a, out, n); break;
        case DJ_OP_RELU: DJ_LAUNCH(k_unary<DJ_OP_RELU>, grid, kThreads, s, a, out, n); break;
        case DJ_OP_GELU: DJ_LAUNCH(k_unary<DJ_OP_GELU>, grid, kThreads, s, a, out, n); break;
        default: fail("launch_unary: bad op");
    }
}

void launch_scalar(hipStream_t s, int op, const float *a, float *out, float s0, float s1, int64_t n) {
    if (n <= 0) return;
    int grid = grid_for(n, 4);
    switch (op) {
        case DJ_OP_MULTIPLY_SCALAR: DJ_LAUNCH(k_scalar<DJ_OP_MULTIPLY_SCALAR>, grid, kThreads, s, a, out, s0, s1, n); break;
        case DJ_OP_ADD_SCALAR: DJ_LAUNCH(k_scalar<DJ_OP_ADD_SCALAR>, grid, kThreads, s, a, out, s0, s1, n); break;
        case DJ_OP_DIVIDE_SCALAR: DJ_LAUNCH(k_scalar<DJ_OP_DIVIDE_SCALAR>, grid, kThreads, s, a, out, s0, s1, n); break;
        case DJ_OP_POW: DJ_LAUNCH(k_scalar<DJ_OP_POW>, grid, kThreads, s, a, out, s0, s1, n); break;
        case DJ_OP_CLAMP: DJ_LAUNCH(k_scalar<DJ_OP_CLAMP>, grid, kThreads, s, a, out, s0, s1, n); break;
        default: fail("launch_scalar: bad op");
    }
}

void launch_broadcast(hipStream_t s, int op, const float *a, const float *v, float *out, int rows, int cols) {
    int64_t n = (int64_t)rows * cols;
    if (n <= 0) return;
    int grid = grid_for(n);
    switch (op) {
        case DJ_OP_ADD_ROW_VECTOR:
            DJ_LAUNCH((k_broadcast<DJ_OP_ADD, true>), grid, kThreads, s, a, v, out, rows, cols); break;
        case DJ_OP_MULTIPLY_BROADCAST_ROWS:
            DJ_LAUNCH((k_broadcast<DJ_OP_MULTIPLY, true>), grid, kThreads, s, a, v, out, rows, cols); break;
        case DJ_OP_ADD_BROADCAST_COLS:
            DJ_LAUNCH((k_broadcast<DJ_OP_ADD, false>), grid, kThreads, s, a, v, out, rows, cols); break;
        case DJ_OP_SUBTRACT_BROADCAST_COLS:
            DJ_LAUNCH((k_broadcast<DJ_OP_SUBTRACT, false>), grid, kThreads, s, a, v, out, rows, cols); break;
        case DJ_OP_DIVIDE_BROADCAST_COLS:
            DJ_LAUNCH((k_broadcast<DJ_OP_DIVIDE, false>), grid, kThreads, s, a, v, out, rows, cols); break;
        case DJ_OP_MULTIPLY_BROADCAST_COLS:
            DJ_LAUNCH((k_broadcast<DJ_OP_MULTIPLY, false>), grid, kThreads, s, a, v, out, rows, cols); break;
        default: fail("launch_broadcast: bad op");
    }
}

void launch_transpose(hipStream_t s, const float *a, float *out, int rows, int cols) {
    if (rows <= 0 || cols <= 0) return;
    dim3 grid((cols + 31) / 32, (rows + 31) / 32);
    launch_kernel(k_transpose, grid, dim3(256), 0, s, a, out, rows, cols);
}

void launch_adamw(hipStream_t s, float *w, const float *g, float *mt, float *vt, int64_t n, float lr, float beta1,
                  float beta2, float eps, float wd, float bc1, float bc2) {
    if (n <= 0) return;
    DJ_LAUNCH(k_adamw, grid_for(n), kThreads, s, w, g, mt, vt, n, lr, beta1, beta2, eps, wd, bc1, bc2);
}

void launch_scatter_add(hipStream_t s, float *target, const float *idx, const float *grad, int target_rows, int cols,
                        int n_idx) {
    int64_t n = (int64_t)n_idx * cols;
    if (n <= 0) return;
    DJ_LAUNCH(k_scatter_add, grid_for(n), kThreads, s, target, idx, grad, target_rows, cols, n_idx);
}

void launch_fill(hipStream_t s, uint32_t *dst, uint32_t bits, int64_t n) {
    if (n <= 0) return;
    DJ_LAUNCH(k_fill, grid_for(n), kThreads, s, dst, bits, n);
}

void launch_stream_read(hipStream_t s, const float *src, float *sink, int64_t n) {
    if (n <= 0) return;
    const int64_t n16 = n / 4, per_lane = (n16 + kThreads - 1) / kThreads;    // 128-bit loads a lane would issue in a grid of one
    // as many loads in flight per lane as leave at least two workgroups per CU, at most three (the matvec's grid)
    int depth = 8;
    while (depth > 1 && per_lane / depth < 512) depth >>= 1;
    int64_t grid = (per_lane + depth - 1) / depth;
    if (grid > 768) grid = 768;
    if (grid < 1) grid = 1;
    const uint4 *p = reinterpret_cast<const uint4 *>(src);
    uint32_t *o = reinterpret_cast<uint32_t *>(sink);
    const uint32_t *w = reinterpret_cast<const uint32_t *>(src);
    switch (depth) {
        case 8: launch_kernel(k_stream_read<8>, dim3((int)grid), dim3(kThreads), 0, s, p, o, n16, n16 * 4, w, n); break;
        case 4: launch_kernel(k_stream_read<4>, dim3((int)grid), dim3(kThreads), 0, s, p, o, n16, n16 * 4, w, n); break;
        case 2: launch_kernel(k_stream_read<2>, dim3((int)grid), dim3(kThreads), 0, s, p, o, n16, n16 * 4, w, n); break;
        default: launch_kernel(k_stream_read<1>, dim3((int)grid), dim3(kThreads), 0, s, p, o, n16, n16 * 4, w, n); break;
    }
}

// One wavefront that writes (shader clock counter, 100 MHz wall clock) pairs, `samples` of them, with naps of
// sleep_reps x 127 x 64 clocks in between: run beside other work, the pairs give the shader clock over time.  Both
// loops are bounded by arguments; nothing waits for anyone.
__global__ void __launch_bounds__(64) k_clock_probe(unsigned long long *out, int samples, int sleep_reps) {
    if (threadIdx.x != 0) return;
    for (int i = 0; i < samples; i++) {
        const unsigned long long c = clock64(), w = wall_clock64();
        __hip_atomic_store(out + 2 * i, c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(out + 2 * i + 1, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int j = 0; j < sleep_reps; j++) __builtin_amdgcn_s_sleep(127);
    }
}
// the wall clock at this point of a stream
__global__ void k_wall_stamp(unsigned long long *out) { if (threadIdx.x == 0) *out = wall_clock64(); }

void launch_clock_probe(hipStream_t s, unsigned long long *out, int samples, int sleep_reps) {
    hipLaunchKernelGGL(k_clock_probe, dim3(1), dim3(64), 0, s, out, samples, sleep_reps);
}
void launch_wall_stamp(hipStream_t s, unsigned long long *out) { hipLaunchKernelGGL(k_wall_stamp, dim3(1), dim3(64), 0, s, out); }

void launch_nop(hipStream_t s, int grid) {
    launch_kernel(k_nop, dim3(grid < 1 ? 1 : grid), dim3(kThreads), 0, s);
}

void launch_copy(hipStream_t s, const float *src, float *dst, int64_t n) {
    if (n <= 0) return;
    DJ_LAUNCH(k_copy, grid_for(n), kThreads, s, src, dst, n);
}

void launch_silu_mul(hipStream_t s, const float *gate, const float *up, float *out, int64_t n) {
    if (n <= 0) return;
    DJ_LAUNCH(k_silu_mul, grid_for(n), kThreads, s, gate, up, out, n);
}

void launch_append_rows(hipStream_t s, const float *src, float *dst, const int32_t *state, int rows, int row_floats,
                        int max_rows) {
    int64_t n = (int64_t)rows * row_floats;
    if (n <= 0) return;
    DJ_LAUNCH(k_append_rows, grid_for(n), kThreads, s, src, dst, state, rows, row_floats, max_rows);
}

void launch_embed_gather(hipStream_t s, const float *table, const int32_t *ids, float *out, int n_ids, int d,
                         int vocab) {
    if (n_ids <= 0) return;
    DJ_LAUNCH(k_embed_gather, n_ids, kThreads, s, table, ids, out, n_ids, d, vocab);
}

void launch_decode_advance(hipStream_t s, int32_t *state, const int32_t *token, int32_t *tokens, int capacity,
                           int n_positions) {
    DJ_LAUNCH(k_decode_advance, 1, 64, s, state, token, tokens, capacity, n_positions);
}

}  // namespace dj
