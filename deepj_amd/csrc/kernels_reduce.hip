// Row/column reductions, softmax family, cross entropy, fused RMSNorm and argmax.
// One 256-thread workgroup (4 wavefronts of 64) owns a row: lanes stride over the
// row with coalesced loads, reduce inside the wavefront with DPP/shuffle steps,
// then across the four wavefronts through 4 floats of LDS.  Reference semantics:
// CpuBackend.java:220-294 (reductions), :360-464 (softmax, cross entropy),
// :491-516 (layer-norm backward), RMSNorm1D.java:46-57.
#include "dj_common.h"

namespace dj {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Every thread of the block receives the result.
__device__ __forceinline__ float block_sum(float v, float *lds) {
    v = wave_sum(v);
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();                 // lds may still be read from a previous call
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float r = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; w++) r += lds[w];
    return r;
}
__device__ __forceinline__ float block_max(float v, float *lds) {
    v = wave_max(v);
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float r = lds[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) r = fmaxf(r, lds[w]);
    return r;
}

__device__ __forceinline__ float d_exp(float x) { return (float)exp((double)x); }

template <int OP>
__global__ void __launch_bounds__(kThreads) k_row_reduce(const float *__restrict__ a, float *__restrict__ out,
                                                         int rows, int cols) {
    __shared__ float lds[kWaves];
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        const float *row = a + (int64_t)r * cols;
        if constexpr (OP == DJ_OP_MAX_ALONG_ROWS) {
            float m = -INFINITY;
            for (int c = threadIdx.x; c < cols; c += kThreads) m = fmaxf(m, row[c]);
            m = block_max(m, lds);
            if (threadIdx.x == 0) out[r] = m;
        } else if constexpr (OP == DJ_OP_VARIANCE_ALONG_ROWS) {
            float s = 0.0f;
            for (int c = threadIdx.x; c < cols; c += kThreads) s += row[c];
            float inv = 1.0f / (float)cols;
            float mean = block_sum(s, lds) * inv;
            float acc = 0.0f;
            for (int c = threadIdx.x; c < cols; c += kThreads) { float d = row[c] - mean; acc += d * d; }
            acc = block_sum(acc, lds);
            if (threadIdx.x == 0) out[r] = acc * inv;
        } else {
            float s = 0.0f;
            for (int c = threadIdx.x; c < cols; c += kThreads) {
                float x = row[c];
                s += (OP == DJ_OP_SUM_ABS) ? fabsf(x) : x;
            }
            s = block_sum(s, lds);
            if (threadIdx.x == 0) out[r] = (OP == DJ_OP_MEAN_ALONG_ROWS) ? s * (1.0f / (float)cols) : s;
        }
    }
}

// Column sums [rows x cols] -> [1 x cols]: 64 columns per workgroup (coalesced
// 256 B rows), the four wavefronts take interleaved rows, LDS combines them.
__global__ void __launch_bounds__(kThreads) k_sum_rows(const float *__restrict__ a, float *__restrict__ out, int rows,
                                                       int cols) {
    __shared__ float part[kWaves][64];
    int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int c = blockIdx.x * 64 + lane;
    float s = 0.0f;
    if (c < cols)
        for (int r = wave; r < rows; r += kWaves) s += a[(int64_t)r * cols + c];
    part[wave][lane] = s;
    __syncthreads();
    if (wave == 0 && c < cols) out[c] = part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane];
}

// Whole-tensor sum into out[0]; one workgroup of 1024 threads (used for loss scalars).
__global__ void __launch_bounds__(1024) k_sum_scalar(const float *__restrict__ a, float *__restrict__ out, int64_t n) {
    __shared__ float lds[16];
    float s = 0.0f;
    for (int64_t i = threadIdx.x; i < n; i += 1024) s += a[i];
    s = wave_sum(s);
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) lds[wave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float r = 0.0f;
        for (int w = 0; w < 16; w++) r += lds[w];
        out[0] = r;
    }
}

// rowWriteSoftmax (CpuBackend.java:392-397): max, exp(x-max), sum of the same exps, divide.
__global__ void __launch_bounds__(kThreads) k_softmax_rows(const float *__restrict__ a, float *__restrict__ out,
                                                           int rows, int cols) {
    __shared__ float lds[kWaves];
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        const float *row = a + (int64_t)r * cols;
        float *orow = out + (int64_t)r * cols;
        float m = -INFINITY;
        for (int c = threadIdx.x; c < cols; c += kThreads) m = fmaxf(m, row[c]);
        m = block_max(m, lds);
        float s = 0.0f;
        for (int c = threadIdx.x; c < cols; c += kThreads) {
            float e = d_exp(row[c] - m);
            orow[c] = e;
            s += e;
        }
        s = block_sum(s, lds);
        for (int c = threadIdx.x; c < cols; c += kThreads) orow[c] = orow[c] / s;
    }
}

__global__ void __launch_bounds__(kThreads) k_softmax_backward(const float *__restrict__ g,
                                                               const float *__restrict__ sm, float *__restrict__ out,
                                                               int rows, int cols) {
    __shared__ float lds[kWaves];
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        int64_t base = (int64_t)r * cols;
        float dot = 0.0f;
        for (int c = threadIdx.x; c < cols; c += kThreads) dot += g[base + c] * sm[base + c];
        dot = block_sum(dot, lds);
        for (int c = threadIdx.x; c < cols; c += kThreads) out[base + c] = sm[base + c] * (g[base + c] - dot);
    }
}

__global__ void __launch_bounds__(kThreads) k_layernorm_backward(const float *__restrict__ dxhat,
                                                                 const float *__restrict__ xhat,
                                                                 const float *__restrict__ stdv,
                                                                 float *__restrict__ out, int rows, int cols) {
    __shared__ float lds[kWaves];
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        int64_t base = (int64_t)r * cols;
        float inv_std = 1.0f / stdv[r];
        float sd = 0.0f, sdx = 0.0f;
        for (int c = threadIdx.x; c < cols; c += kThreads) {
            float d = dxhat[base + c];
            sd += d;
            sdx += d * xhat[base + c];
        }
        sd = block_sum(sd, lds);
        sdx = block_sum(sdx, lds);
        float dim = (float)cols;
        for (int c = threadIdx.x; c < cols; c += kThreads) {
            float d = dxhat[base + c], xh = xhat[base + c];
            out[base + c] = inv_std * (d - sd / dim - xh * (sdx / dim));
        }
    }
}

// Per-row loss log(sum exp(x-max)) + max - x[target] (GRAD=false, out [rows x 1]) or
// (softmax - onehot)/rows (GRAD=true).  Targets arrive as floats; a target outside
// [0, cols) yields NaN for that row, as the reference's GPU kernels do
// (deepj_metal_jni.mm:472-476,497-503).
template <bool GRAD>
__global__ void __launch_bounds__(kThreads) k_cross_entropy(const float *__restrict__ logits,
                                                            const float *__restrict__ targets,
                                                            float *__restrict__ out, int rows, int cols) {
    __shared__ float lds[kWaves];
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        int64_t base = (int64_t)r * cols;
        float ft = targets[r];
        bool ok = ft >= 0.0f && ft < (float)cols;
        int target = ok ? (int)ft : 0;
        float m = -INFINITY;
        for (int c = threadIdx.x; c < cols; c += kThreads) m = fmaxf(m, logits[base + c]);
        m = block_max(m, lds);
        float s = 0.0f;
        for (int c = threadIdx.x; c < cols; c += kThreads) s += d_exp(logits[base + c] - m);
        s = block_sum(s, lds);
        if constexpr (GRAD) {
            float frows = (float)rows;
            for (int c = threadIdx.x; c < cols; c += kThreads) {
                float p = d_exp(logits[base + c] - m) / s;
                if (c == target) p -= 1.0f;
                out[base + c] = ok ? p / frows : __builtin_nanf("");
            }
        } else if (threadIdx.x == 0) {
            out[r] = ok ? (float)log((double)s) + m - logits[base + target] : __builtin_nanf("");
        }
    }
}

// out = gamma * (x / sqrt(mean(x*x) + 1e-6)) in one pass over the row
// (RMSNorm1D.java:46-57 folds six primitive ops and five temporaries into this).
// NV: 128-bit words a thread keeps of one row (rows of up to 1024 * NV floats stay in registers between the sum of
// squares and the scaling: one pass over memory); NV = 0: any width, two passes with scalar accesses.
template <int NV>
__global__ void __launch_bounds__(kThreads) k_rmsnorm(const float *__restrict__ x, const float *__restrict__ gamma,
                                                      float *__restrict__ out, int rows, int cols) {
    __shared__ float lds[kWaves];
    if constexpr (NV > 0) {
        const int n4 = cols >> 2;
        for (int r = blockIdx.x; r < rows; r += gridDim.x) {
            const float4 *row4 = reinterpret_cast<const float4 *>(x + (int64_t)r * cols);
            float4 *out4 = reinterpret_cast<float4 *>(out + (int64_t)r * cols);
            float4 v[NV], g[NV];
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int i = threadIdx.x + j * kThreads;
                v[j] = i < n4 ? row4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                g[j] = i < n4 ? reinterpret_cast<const float4 *>(gamma)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
                s += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
            }
            s = block_sum(s, lds);
            const float rms = sqrtf(s * (1.0f / (float)cols) + kRmsEps);
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int i = threadIdx.x + j * kThreads;
                if (i < n4)
                    out4[i] = make_float4((v[j].x / rms) * g[j].x, (v[j].y / rms) * g[j].y, (v[j].z / rms) * g[j].z,
                                          (v[j].w / rms) * g[j].w);
            }
        }
    } else {
        for (int r = blockIdx.x; r < rows; r += gridDim.x) {
            const float *row = x + (int64_t)r * cols;
            float *orow = out + (int64_t)r * cols;
            float s = 0.0f;
            for (int c = threadIdx.x; c < cols; c += kThreads) { float v = row[c]; s += v * v; }
            s = block_sum(s, lds);
            float rms = sqrtf(s * (1.0f / (float)cols) + kRmsEps);
            for (int c = threadIdx.x; c < cols; c += kThreads) orow[c] = (row[c] / rms) * gamma[c];
        }
    }
}

// out = ((x - mean) / sqrt(var + 1e-5)) * gamma + beta, population variance about the mean
// (LayerNorm1D.java:34-66 composes this from eight primitive ops).
__global__ void __launch_bounds__(kThreads) k_layernorm(const float *__restrict__ x, const float *__restrict__ gamma,
                                                        const float *__restrict__ beta, float *__restrict__ out,
                                                        int rows, int cols) {
    __shared__ float lds[kWaves];
    const float inv = 1.0f / (float)cols;
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        const float *row = x + (int64_t)r * cols;
        float *orow = out + (int64_t)r * cols;
        float s = 0.0f;
        for (int c = threadIdx.x; c < cols; c += kThreads) s += row[c];
        float mean = block_sum(s, lds) * inv;
        float v = 0.0f;
        for (int c = threadIdx.x; c < cols; c += kThreads) { float t = row[c] - mean; v += t * t; }
        float sd = sqrtf(block_sum(v, lds) * inv + kLayerNormEps);
        for (int c = threadIdx.x; c < cols; c += kThreads) orow[c] = ((row[c] - mean) / sd) * gamma[c] + beta[c];
    }
}

// x[i, :] += table[state[0] + i, :]: learned positions of rows that sit at state[0].. (GPTModel.java:52-54,
// PositionalEmbedding.java:26-33).  Rows whose position falls outside the table become NaN.
__global__ void __launch_bounds__(kThreads) k_add_positions(float *__restrict__ x, const float *__restrict__ table,
                                                            const int32_t *__restrict__ state, int rows, int d,
                                                            int max_seq) {
    const int p0 = state[0];
    const int64_t total = (int64_t)rows * d;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        int r = (int)(i / d);
        int c = (int)(i - (int64_t)r * d);
        int pos = p0 + r;
        x[i] = (pos >= 0 && pos < max_seq) ? x[i] + table[(int64_t)pos * d + c] : __builtin_nanf("");
    }
}

// Index of the row maximum, lowest index on ties: what topK=1 sampling reduces to
// (TextGenerator.java:110-114,163-170: stable descending sort, first element).
// NaN ranks above everything, as Float.compare orders it.
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
    bool vn = v != v, bn = bv != bv;
    if (vn != bn) return vn;
    if (!vn && v != bv) return v > bv;
    return i < bi;
}
// The same order for a candidate that is known to come AFTER the incumbent (i > bi), or for an empty incumbent
// (bi = INT_MAX): it wins only with a strictly larger value, or as the first NaN.
__device__ __forceinline__ bool better_later(float v, float bv, int bi) {
    return (v > bv) || ((v != v) && (bv == bv)) || bi == 0x7fffffff;
}
__global__ void __launch_bounds__(kThreads) k_argmax_rows(const float *__restrict__ a, int32_t *__restrict__ out,
                                                          int rows, int cols) {
    __shared__ float sv[kWaves];
    __shared__ int si[kWaves];
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        const float *row = a + (int64_t)r * cols;
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int c = threadIdx.x; c < cols; c += kThreads) {
            float v = row[c];
            if (better(v, c, bv, bi)) { bv = v; bi = c; }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            float ov = __shfl_xor(bv, off, 64);
            int oi = __shfl_xor(bi, off, 64);
            if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
        }
        int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
        __syncthreads();
        if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < kWaves; w++)
                if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
            out[r] = bi;
        }
    }
}

// End of a greedy decode step in one launch: argmax over the logits (ties -> lowest
// index), record the token, advance the position, and gather the token's embedding row
// as the next step's input (Embedding.java:28-34).
__global__ void __launch_bounds__(1024) k_decode_next(const float *__restrict__ logits, int32_t *__restrict__ state,
                                                      int32_t *__restrict__ tokens, int capacity,
                                                      const float *__restrict__ table, float *__restrict__ x,
                                                      int vocab, int d, int n_positions) {
    __shared__ float sv[16];
    __shared__ int si[16];
    __shared__ int s_tok;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    // the counters the last phase updates: requested now, used after the reduction
    int st_pos = 0, st_gen = 0;
    if (threadIdx.x == 0) { st_pos = state[0]; st_gen = state[2]; }
    // eight independent 128-bit loads per thread per round: one memory round trip per 32768 logits
    const int v4 = vocab >> 2;
    const float4 *l4 = reinterpret_cast<const float4 *>(logits);
    for (int base = 0; base < v4; base += 1024 * 8) {
        float4 t[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            int i = base + u * 1024 + threadIdx.x;
            t[u] = i < v4 ? l4[i] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            int c = (base + u * 1024 + threadIdx.x) * 4;
            if (c < (v4 << 2)) {                    // a thread meets its candidates in rising index order
                if (better_later(t[u].x, bv, bi)) { bv = t[u].x; bi = c; }
                if (better_later(t[u].y, bv, bi)) { bv = t[u].y; bi = c + 1; }
                if (better_later(t[u].z, bv, bi)) { bv = t[u].z; bi = c + 2; }
                if (better_later(t[u].w, bv, bi)) { bv = t[u].w; bi = c + 3; }
            }
        }
    }
    for (int c = (v4 << 2) + threadIdx.x; c < vocab; c += 1024) {
        float v = logits[c];
        if (better(v, c, bv, bi)) { bv = v; bi = c; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(bv, off, 64);
        int oi = __shfl_xor(bi, off, 64);
        if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++)
            if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        const int g = st_gen;
        if (g < capacity) tokens[g] = bi;
        state[1] = bi;
        state[0] = st_pos + n_positions;
        state[2] = g + 1;
        s_tok = bi;
    }
    __syncthreads();
    int tok = s_tok;
    bool ok = tok >= 0 && tok < vocab;
    const float *src = table + (int64_t)(ok ? tok : 0) * d;
    for (int c = threadIdx.x; c < d; c += 1024) x[c] = ok ? src[c] : __builtin_nanf("");
}

inline int row_grid(int rows) { return rows < 256 * 16 ? (rows < 1 ? 1 : rows) : 256 * 16; }

}  // namespace

void launch_row_reduce(hipStream_t s, int op, const float *a, float *out, int rows, int cols) {
    if (rows <= 0) return;
    dim3 grid(row_grid(rows)), block(kThreads);
    switch (op) {
        case DJ_OP_SUM_ALONG_ROWS: launch_kernel(k_row_reduce<DJ_OP_SUM_ALONG_ROWS>, grid, block, 0, s, a, out, rows, cols); break;
        case DJ_OP_MEAN_ALONG_ROWS: launch_kernel(k_row_reduce<DJ_OP_MEAN_ALONG_ROWS>, grid, block, 0, s, a, out, rows, cols); break;
        case DJ_OP_VARIANCE_ALONG_ROWS: launch_kernel(k_row_reduce<DJ_OP_VARIANCE_ALONG_ROWS>, grid, block, 0, s, a, out, rows, cols); break;
        case DJ_OP_MAX_ALONG_ROWS: launch_kernel(k_row_reduce<DJ_OP_MAX_ALONG_ROWS>, grid, block, 0, s, a, out, rows, cols); break;
        case DJ_OP_SUM_ABS: launch_kernel(k_row_reduce<DJ_OP_SUM_ABS>, grid, block, 0, s, a, out, rows, cols); break;
        default: fail("launch_row_reduce: bad op");
    }
}

void launch_sum_rows(hipStream_t s, const float *a, float *out, int rows, int cols) {
    if (cols <= 0) return;
    launch_kernel(k_sum_rows, dim3((cols + 63) / 64), dim3(kThreads), 0, s, a, out, rows, cols);
}

void launch_sum_scalar(hipStream_t s, const float *a, float *out, int64_t n) {
    launch_kernel(k_sum_scalar, dim3(1), dim3(1024), 0, s, a, out, n);
}

void launch_softmax_rows(hipStream_t s, const float *a, float *out, int rows, int cols) {
    if (rows <= 0) return;
    launch_kernel(k_softmax_rows, dim3(row_grid(rows)), dim3(kThreads), 0, s, a, out, rows, cols);
}

void launch_softmax_backward(hipStream_t s, const float *g, const float *sm, float *out, int rows, int cols) {
    if (rows <= 0) return;
    launch_kernel(k_softmax_backward, dim3(row_grid(rows)), dim3(kThreads), 0, s, g, sm, out, rows, cols);
}

void launch_layernorm_backward(hipStream_t s, const float *dxhat, const float *xhat, const float *stdv, float *out,
                               int rows, int cols) {
    if (rows <= 0) return;
    launch_kernel(k_layernorm_backward, dim3(row_grid(rows)), dim3(kThreads), 0, s, dxhat, xhat, stdv, out, rows,
                       cols);
}

void launch_cross_entropy(hipStream_t s, bool gradient, const float *logits, const float *targets, float *out,
                          int rows, int cols) {
    if (rows <= 0) return;
    if (gradient)
        launch_kernel(k_cross_entropy<true>, dim3(row_grid(rows)), dim3(kThreads), 0, s, logits, targets, out,
                           rows, cols);
    else
        launch_kernel(k_cross_entropy<false>, dim3(row_grid(rows)), dim3(kThreads), 0, s, logits, targets, out,
                           rows, cols);
}

void launch_rmsnorm(hipStream_t s, const float *x, const float *gamma, float *out, int rows, int cols) {
    if (rows <= 0) return;
    const dim3 grid(row_grid(rows)), block(kThreads);
    const int need = (cols & 3) == 0 ? (cols + 4 * kThreads - 1) / (4 * kThreads) : 0;     // 128-bit words per thread
    if (need >= 1 && need <= 2) launch_kernel(k_rmsnorm<2>, grid, block, 0, s, x, gamma, out, rows, cols);
    else if (need >= 3 && need <= 4) launch_kernel(k_rmsnorm<4>, grid, block, 0, s, x, gamma, out, rows, cols);
    else if (need >= 5 && need <= 6) launch_kernel(k_rmsnorm<6>, grid, block, 0, s, x, gamma, out, rows, cols);
    else if (need >= 7 && need <= 11) launch_kernel(k_rmsnorm<11>, grid, block, 0, s, x, gamma, out, rows, cols);
    else launch_kernel(k_rmsnorm<0>, grid, block, 0, s, x, gamma, out, rows, cols);
}

void launch_layernorm(hipStream_t s, const float *x, const float *gamma, const float *beta, float *out, int rows,
                      int cols) {
    if (rows <= 0) return;
    launch_kernel(k_layernorm, dim3(row_grid(rows)), dim3(kThreads), 0, s, x, gamma, beta, out, rows, cols);
}

void launch_add_positions(hipStream_t s, float *x, const float *table, const int32_t *state, int rows, int d,
                          int max_seq) {
    int64_t total = (int64_t)rows * d;
    if (total <= 0) return;
    int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 8192) blocks = 8192;
    launch_kernel(k_add_positions, dim3((int)blocks), dim3(kThreads), 0, s, x, table, state, rows, d, max_seq);
}

void launch_decode_next(hipStream_t s, const float *logits, int32_t *state, int32_t *tokens, int capacity,
                        const float *table, float *x, int vocab, int d, int n_positions) {
    launch_kernel(k_decode_next, dim3(1), dim3(1024), 0, s, logits, state, tokens, capacity, table, x, vocab, d,
                       n_positions);
}

void launch_argmax_rows(hipStream_t s, const float *a, int32_t *out, int rows, int cols) {
    if (rows <= 0) return;
    launch_kernel(k_argmax_rows, dim3(row_grid(rows)), dim3(kThreads), 0, s, a, out, rows, cols);
}

}  // namespace dj
