// What the GEMM kernels do to a finished sum before storing it (device code; included by the GEMM sources).
#pragma once
#include <cstdint>
#include <hip/hip_runtime.h>

namespace dj {

// RoPE and the cache append as the epilogue of the fused q | k | v projection (N = 3 d): row r is the token at position
// state[0] + r; columns [0, d) are its queries (rotated, to q), [d, 2 d) its keys (rotated, into the key cache), [2 d, 3 d)
// its values (into the value cache).  Rotation as RotaryEmbedding.java applies it: pairs (2 j, 2 j + 1) of a head by the
// table entry [position][j].
struct RopeStore {
    float *q = nullptr;             // [M x d]; null: no such epilogue
    float *k_cache = nullptr;       // one layer: [H][max_seq][hd]
    float *v_cache = nullptr;
    const int32_t *state = nullptr;
    const float *cos_t = nullptr, *sin_t = nullptr;   // [max_seq][hd / 2]
    int hd = 0, d = 0, max_seq = 0;
};

struct GemmEpilogue {
    const float *bias;      // [N] or null; with interleave: even col n -> bias[n/2], odd col -> bias2[n/2]
    const float *bias2;
    const float *residual;  // [M x N] or null
    int interleaved_bias;
    const int32_t *m_dev;   // when set, only rows < min(M, m_dev[0] + m_extra) exist (row count kept on the device)
    int m_extra;
    int gelu;               // GELU (tanh form, tensor/cpu/CpuBackend.java:338, used by activations/GELU.java:15-18) on acc + bias, before the residual
    int swiglu;             // Q8 GEMM only: columns are interleaved gate/up pairs; C is [M x N/2], C[r][j] = SiLU(gate_j) * up_j
    RopeStore rope;         // fp16 Q8 GEMM only
};

// A finished tile of a plain or SwiGLU epilogue leaves with streaming (non-temporal) stores: no workgroup of the launch
// reads it again, and lines a kernel leaves dirty in an XCD's L2 are written back when the kernel ends, with every
// compute unit waiting (the prompt's gate/up GEMM at 512 rows: 66.8 -> 65.8 us).  The consumer then reads from HBM
// rather than from the memory-side cache, which costs it about as much where it is a bandwidth-bound helper kernel (the
// sum of K shares) and more where it is the attention kernel - so the RoPE epilogue keeps ordinary stores (attention
// 21.7 -> 23.2 us with streaming ones).  Write-through (agent-scope) stores were slower throughout.
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_streaming(float *p, float4 v) { __builtin_nontemporal_store((floatx4){v.x, v.y, v.z, v.w}, reinterpret_cast<floatx4 *>(p)); }
__device__ __forceinline__ void store_streaming(float *p, float2 v) { __builtin_nontemporal_store((floatx2){v.x, v.y}, reinterpret_cast<floatx2 *>(p)); }

// Where the four columns col .. col + 3 of a q | k | v row go: fixed for a lane over the rows of its tile.
struct RopeColumn { int region, cc, head, within; };
__device__ __forceinline__ RopeColumn rope_column(const RopeStore &r, int col) {
    RopeColumn c;
    c.region = col / r.d;
    c.cc = col - c.region * r.d;
    c.head = c.cc / r.hd;
    c.within = c.cc - c.head * r.hd;
    return c;
}
// the table entries of row `row`'s two pairs (cos.x, cos.y, sin.x, sin.y); rows outside the cache read entry 0
__device__ __forceinline__ float4 rope_table(const RopeStore &r, const RopeColumn &c, int row, int pos0) {
    int pos = pos0 + row;
    if (pos < 0 || pos >= r.max_seq) pos = 0;
    const int64_t t = (int64_t)pos * (r.hd >> 1) + (c.within >> 1);
    const float2 cs = *reinterpret_cast<const float2 *>(r.cos_t + t), sn = *reinterpret_cast<const float2 *>(r.sin_t + t);
    return make_float4(cs.x, cs.y, sn.x, sn.y);
}
// v = the finished sums (bias added) of row `row`, columns col .. col + 3; pos0 = state[0]; tab = rope_table of the row
__device__ __forceinline__ void rope_store(const RopeStore &r, const RopeColumn &c, float4 v, int row, int pos0, float4 tab) {
    const int pos = pos0 + row;
    if (pos < 0 || pos >= r.max_seq) return;                 // never write outside the cache
    const int64_t at = ((int64_t)c.head * r.max_seq + pos) * r.hd + c.within;
    if (c.region == 2) { *reinterpret_cast<float4 *>(r.v_cache + at) = v; return; }
    const float4 o = make_float4(v.x * tab.x - v.y * tab.z, v.x * tab.z + v.y * tab.x, v.z * tab.y - v.w * tab.w, v.z * tab.w + v.w * tab.y);
    if (c.region == 0) *reinterpret_cast<float4 *>(r.q + (int64_t)row * r.d + c.cc) = o;
    else *reinterpret_cast<float4 *>(r.k_cache + at) = o;
}

__device__ __forceinline__ float gemm_gelu(float x) {
    float c = sqrtf(2.0f / 3.14159265358979323846f);
    float x3 = x * x * x;
    float t = c * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + (float)tanh((double)t));
}

}  // namespace dj
