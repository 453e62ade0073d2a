// Q8 weight path.
//
// Format (this library's own; the reference has no quantiser): a weight that the
// reference holds as fp32 [K x N] (Linear.java:13, y = x.W) is stored output-major,
//     q      [rows x Kp] int8,  Kp = K rounded up to 32, zero padded
//     scales [rows x Kp/32] fp32, one per 32 consecutive k of one output row
// with scale = max|w| / 127 over the group and q = rint(w / scale) clamped to
// [-127, 127]; dequantised weight = float(q) * scale (one fp32 rounding, so host
// and device agree bit for bit).  1.125 bytes per weight.
//
// Decode (M = 1): every weight byte is read from HBM exactly once.  One
// wavefront owns an output row at a time; its 64 lanes read the row with 128-bit
// loads (1 KiB per wave-load, fully coalesced), multiply them with the activation
// slice the lane keeps in VGPRs for the whole kernel, and reduce across the wavefront
// with DPP row operations.  The activation vector is staged once per workgroup through
// LDS, where the optional prologue is applied (RMSNorm, LayerNorm, or the merge of the
// decode attention's per-split records), so norm + projection (+ bias, + GELU,
// + residual, or the SwiGLU gate) is one launch.  The staged form is three planes of
// signed bytes per value (a 23-bit integer times a power of two per 16 values, XSlice
// below) that go into v_dot4_i32_i8 with the int8 weights as they are: the work left
// behind the last weight bytes to arrive is 19 instead of 33 instructions per 16 weights
// (decode 2430 -> 2448 tokens/s), at an error of 2^-23 of a slice's largest value.
// M > 1 goes to the MFMA GEMM in kernels_matmul.hip.
#include <cstdlib>
#include <type_traits>

#include "dj_common.h"
#include "dj_device.h"

namespace dj {

void launch_q8_gemm(hipStream_t s, const float *x, const int8_t *wq, const float *scales, float *out, int m,
                    int k, int n_rows, const float *bias, const float *bias2, const float *residual,
                    int interleaved_bias, const int32_t *m_dev, int m_extra, int gelu, int swiglu, float *workspace,
                    int64_t workspace_floats);
int64_t q8_gemm_workspace_floats(int m, int n_rows, int k);

namespace {
using namespace dev;

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

// Timeline of one launch, for tuning builds only (-DDJ_TRACE; never in the shipped library): every wavefront leaves
// 100 MHz time stamps at fixed points of the decode matvec.
#ifdef DJ_TRACE
__device__ unsigned long long g_mv_trace[8 * 16384];
#define DJ_STAMP(i) do { if (lane == 0 && wave_global < 16384) g_mv_trace[wave_global * 8 + (i)] = wall_clock64(); } while (0)
#else
#define DJ_STAMP(i) do {} while (0)
#endif

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// The epilogue sits on the critical path of every wavefront: single precision exp (about 1 ulp) instead of the
// double precision one the element-wise SIGMOID opcode uses; the difference is far inside the 1e-4 per-op bound.
__device__ __forceinline__ float d_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
// tensor/cpu/CpuBackend.java:338 (tanh form)
__device__ __forceinline__ float d_gelu(float x) {
    float c = sqrtf(2.0f / 3.14159265358979323846f);
    float x3 = x * x * x;
    float t = c * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + (float)tanh((double)t));
}

// ── quantise: grid (ceil(N/64), Kp/32); a workgroup takes 64 columns x one group ──
__global__ void __launch_bounds__(kThreads) k_q8_quantize(const float *__restrict__ w, int8_t *__restrict__ q,
                                                          float *__restrict__ scales, int k, int n, int kp,
                                                          int row_off, int row_step) {
    __shared__ float amax_part[4][64];
    int col = threadIdx.x & 63, kq = threadIdx.x >> 6;      // 4 slices of 8 k each
    int gn = blockIdx.x * 64 + col;
    int g = blockIdx.y;
    int k0 = g * kQ8Group + kq * 8;
    float v[8];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        int gk = k0 + j;
        v[j] = (gn < n && gk < k) ? w[(int64_t)gk * n + gn] : 0.0f;
        amax = fmaxf(amax, fabsf(v[j]));
    }
    amax_part[kq][col] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(amax_part[0][col], amax_part[1][col]), fmaxf(amax_part[2][col], amax_part[3][col]));
    if (gn >= n) return;
    float scale = amax / 127.0f;
    int64_t row = (int64_t)row_off + (int64_t)gn * row_step;
    if (kq == 0) scales[row * (kp / kQ8Group) + g] = scale;
    uint32_t packed[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; j++) {
        int qi = 0;
        if (scale != 0.0f) {
            float r = rintf(v[j] / scale);
            r = fminf(fmaxf(r, -127.0f), 127.0f);
            qi = (int)r;
        }
        packed[j >> 2] |= ((uint32_t)(qi & 0xff)) << (8 * (j & 3));
    }
    *reinterpret_cast<uint2 *>(q + row * kp + k0) = make_uint2(packed[0], packed[1]);
}

__global__ void __launch_bounds__(kThreads) k_q8_dequantize(const int8_t *__restrict__ q,
                                                            const float *__restrict__ scales, float *__restrict__ w,
                                                            int k, int n, int kp, int row_off, int row_step) {
    int64_t total = (int64_t)k * n;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        int gk = (int)(i / n);
        int gn = (int)(i - (int64_t)gk * n);
        int64_t row = (int64_t)row_off + (int64_t)gn * row_step;
        w[i] = (float)q[row * kp + gk] * scales[row * (kp / kQ8Group) + gk / kQ8Group];
    }
}

// ── decode matvec ──────────────────────────────────────────────────────────
struct MatvecArgs {
    const float *x; const int8_t *wq; const float *scales; float *out;
    int k, kp, n_out;                 // n_out outputs; SwiGLU: output o uses rows 2o, 2o+1
    const float *gamma, *bias, *bias2, *residual;
    const float *beta;                // set: LayerNorm prologue with gamma and beta (otherwise gamma alone = RMSNorm)
    int rec_hd;                       // ATTN_MERGE prologue: x holds attention records of heads this wide
};

// One batch of Q8 rows held in registers by a wavefront: R rows x NC chunks.
template <int NC, int R> struct RowBatch {
    int4 w[R][NC];
    float sc[R][NC];
    float ev;                         // epilogue operands of the batch: lane u holds the bias of output u, lane B + u its
                                      // second bias, lane 2B + u its residual (one load instruction for all of them)
};

// The epilogue operands of outputs o0 .. o0+B-1 are requested together with the weight rows, so the
// finished sums never wait for a bias or residual that is still in memory.
template <int NC, int R, int B, bool SWIGLU>
__device__ __forceinline__ void load_epilogue(RowBatch<NC, R> &b, const MatvecArgs &p, int o0) {
    // No load sits under a branch: an absent operand reads a valid dummy address instead (the value is never
    // used).  A conditional load would leave the number of loads in flight unknown at compile time, and every
    // later wait for an EARLIER load would have to be a wait for all of them.
    const float *bias = p.bias ? p.bias : p.scales, *bias2 = (SWIGLU && p.bias2) ? p.bias2 : p.scales;
    const float *residual = p.residual ? p.residual : p.scales;
    const int lane = threadIdx.x & 63;
    const int kind = lane / B, u = lane - kind * B;         // lanes past 3B repeat a valid address
    int o = o0 + u < p.n_out ? o0 + u : p.n_out - 1;
    o = o < 0 ? 0 : o;
    const float *src = kind == 1 ? bias2 : (kind == 2 ? residual : bias);
    b.ev = src[o];
}

// Loads are unconditional: rows past the wave's range are clamped to its last row and
// chunks past Kp to chunk 0 (their activations are zero), so no load sits under a branch.
template <int NC, int R>
__device__ __forceinline__ void load_batch(RowBatch<NC, R> &b, const MatvecArgs &p, int row0, int row_last, int lane,
                                           int groups) {
#pragma unroll
    for (int u = 0; u < R; u++) {
        int row = row0 + u < row_last ? row0 + u : row_last;
        const int8_t *wrow = p.wq + (int64_t)row * p.kp;
        const float *srow = p.scales + (int64_t)row * groups;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            int chunk = c * 64 + lane;
            if (chunk * 16 >= p.kp) chunk = 0;
            b.w[u][c] = *reinterpret_cast<const int4 *>(wrow + chunk * 16);
            b.sc[u][c] = srow[chunk >> 1];
        }
    }
}

// The activations of a lane's slice (16 consecutive k of each 1 KiB chunk) in the form the inner product wants.
// DIGITS: each value is t * 2^-shift of its slice with an integer |t| <= 2^22, held as three signed bytes
// t = d0 + 256 d1 + 65536 d2 (d0, d1 in [-128, 127], |d2| <= 64): one dword per four values and digit, so that
// v_dot4_i32_i8 multiplies four int8 weights by four digits at a time - 12 integer instructions per 16 weights and
// digit set, against 16 conversions and 16 multiply-adds on floats.  The integer sums are exact; they are put
// together in fp32 (k[0..2] = 2^-shift x {1, 256, 65536}).  A value is off by at most 2^-23 of its slice's largest.
template <int NC, bool DIGITS> struct XSlice;
template <int NC> struct XSlice<NC, false> { float f[NC][16]; };
template <int NC> struct XSlice<NC, true> { int d[NC][12]; float k[NC][3]; };

template <int NC>
__device__ __forceinline__ float dot_slice(const int4 &w, const XSlice<NC, false> &x, int c) { return dot16(w, x.f[c]); }
template <int NC>
__device__ __forceinline__ float dot_slice(const int4 &w, const XSlice<NC, true> &x, int c) {
    const int wd[4] = {w.x, w.y, w.z, w.w};
    int a0 = 0, a1 = 0, a2 = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a0 = __builtin_amdgcn_sdot4(wd[i], x.d[c][i], a0, false);
        a1 = __builtin_amdgcn_sdot4(wd[i], x.d[c][4 + i], a1, false);
        a2 = __builtin_amdgcn_sdot4(wd[i], x.d[c][8 + i], a2, false);
    }
    return fmaf((float)a2, x.k[c][2], fmaf((float)a1, x.k[c][1], (float)a0 * x.k[c][0]));
}

template <int NC, int B, bool SWIGLU, bool GELU, bool DIGITS>
__device__ __forceinline__ void finish_batch(const RowBatch<NC, B *(SWIGLU ? 2 : 1)> &b, const XSlice<NC, DIGITS> &xr,
                                             const MatvecArgs &p, int o0, int o_end, int lane, float rms) {
    constexpr int R = B * (SWIGLU ? 2 : 1);
    float acc[R];
#pragma unroll
    for (int u = 0; u < R; u++) {
        float a = 0.0f;
#pragma unroll
        for (int c = 0; c < NC; c++) a = fmaf(dot_slice<NC>(b.w[u][c], xr, c), b.sc[u][c], a);
        acc[u] = wave_sum_dpp(a) / rms;        // rms = 1 unless the RMSNorm scale was deferred to here
    }
    float eb[B], eb2[B], er[B];
#pragma unroll
    for (int u = 0; u < B; u++) {
        eb[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, b.ev), u));
        eb2[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, b.ev), B + u));
        er[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, b.ev), 2 * B + u));
    }
    if (lane == 0) {
#pragma unroll
        for (int u = 0; u < B; u++) {
            int o = o0 + u;
            if (o < o_end) {
                float v;
                if constexpr (SWIGLU) {
                    float gate = acc[2 * u], up = acc[2 * u + 1];
                    if (p.bias) gate = gate + eb[u];
                    if (p.bias2) up = up + eb2[u];
                    float sg = gate * d_sigmoid(gate);     // SiLU.java:20-24
                    v = sg * up;                            // SwiGLULayer.java:69
                } else {
                    v = acc[u];
                    if (p.bias) v = v + eb[u];
                    if constexpr (GELU) v = d_gelu(v);
                }
                if (p.residual) v = er[u] + v;
                p.out[o] = v;
            }
        }
    }
}

// LDS layout of the staged activation row, float form (rows whose length is not a multiple of 4).  A lane multiplies
// the 16 consecutive activations of "its" 16-byte weight chunk (chunk = 64 * c + lane) and reads them as four 128-bit
// words; stored in order, consecutive lanes would be 64 bytes apart and four of every sixteen lanes would hit the
// same banks on every read.  So the row is kept as planes: plane 4 * c + q holds the q-th word of every lane's slice
// of chunk row c, lane after lane (conflict free to read), and a plane is padded by 16 floats so that the staging
// writes - consecutive threads write the four words of one slice, i.e. to four planes - spread over the banks as well.
constexpr int kXsPlane = 64 * 4 + 16;                              // floats per plane
__host__ __device__ inline int xs_floats(int kp) { return ((kp + 1023) / 1024) * 4 * kXsPlane; }
// offset of activation e (any e < Kp rounded up to 1024)
__device__ __forceinline__ int xs_at(int e) {
    const int chunk = e >> 4, q = (e >> 2) & 3;
    return ((chunk >> 6) * 4 + q) * kXsPlane + (chunk & 63) * 4 + (e & 3);
}

// Digit form (XSlice<NC, true>), in the same LDS bytes: for chunk row c three planes of 256 dwords - plane
// 3 * c + digit holds, for slice l of the row (the one lane l multiplies), the four dwords of that digit at
// [4 l, 4 l + 4) - and behind all planes one shift per slice.  Thread t of the workgroup holds values
// 4 t .. 4 t + 3 of chunk row c, i.e. the dword t of each of its planes: writes and reads are both lane-consecutive.
// The four threads of a quad hold one slice; its shift puts the largest magnitude of the slice in [2^21, 2^22).
__device__ __forceinline__ int xd_plane(int c, int digit) { return (c * 3 + digit) * 256; }
template <int NC> __device__ __forceinline__ int xd_shift(int c) { return NC * 768 + c * 64; }
static_assert(768 + 64 <= 4 * kXsPlane, "the digit form fits in the float form's bytes");

__device__ __forceinline__ void stage_digits(float *xs, int plane0, int shift_at, int tid, float4 v) {
    // largest magnitude of the quad's 16 values, as bit patterns: an infinity or a NaN compares above every number
    uint32_t m = max(max(__float_as_uint(v.x) & 0x7fffffffu, __float_as_uint(v.y) & 0x7fffffffu),
                     max(__float_as_uint(v.z) & 0x7fffffffu, __float_as_uint(v.w) & 0x7fffffffu));
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xf, 0xf, false));      // quad_perm [1,0,3,2]
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xf, 0xf, false));      // quad_perm [2,3,0,1]
    // m = f * 2^e, f in [0.5, 1): values times 2^(22 - e) are below 2^22 in magnitude.  The shift stays where
    // 2^shift and 2^-shift are normal numbers (slices below 2^-98 keep fewer digits, of values that small).
    const int e = __builtin_amdgcn_frexp_expf(__uint_as_float(m));
    const int shift = min(22 - e, 120);
    const float up = ldexpf(1.0f, shift);
    // v * 2^shift + 1.5 * 2^23 rounds to an integer (to nearest even) and leaves it, as C + t with C = 0x4B400000,
    // in the bits of the sum.  t = b0 + 256 t1 with b0 the signed low byte means t1 = (t + 128) >> 8, and the same
    // once more for t1: the three digits are byte 0 of t, byte 1 of t + 128 and byte 2 of t + 128 + 32768 - and C
    // has no bits in its two low bytes, so only the last needs C taken off.
    const float magic = 12582912.0f;
    const uint32_t b[4] = {__float_as_uint(fmaf(v.x, up, magic)), __float_as_uint(fmaf(v.y, up, magic)),
                           __float_as_uint(fmaf(v.z, up, magic)), __float_as_uint(fmaf(v.w, up, magic))};
    uint32_t u[4], w[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { u[i] = b[i] + 128u; w[i] = b[i] + (32896u - 0x400000u); }
    // __builtin_amdgcn_perm(hi, lo, sel): result byte i is byte sel_i of the eight bytes {lo: 0-3, hi: 4-7}
    const uint32_t d0 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu), __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u), 0x07060100u);
    const uint32_t d1 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(u[3], u[2], 0x05010c0cu), __builtin_amdgcn_perm(u[1], u[0], 0x0c0c0501u), 0x07060100u);
    const uint32_t d2 = __builtin_amdgcn_perm(__builtin_amdgcn_perm(w[3], w[2], 0x06020c0cu), __builtin_amdgcn_perm(w[1], w[0], 0x0c0c0602u), 0x07060100u);
    uint32_t *xd = reinterpret_cast<uint32_t *>(xs);
    xd[plane0 + tid] = d0;
    xd[plane0 + 256 + tid] = d1;
    xd[plane0 + 512 + tid] = d2;
    // a slice with an infinity or a NaN in it: the sums of this slice become NaN (the float form would give NaN or
    // an infinity there)
    if ((tid & 3) == 0) xs[shift_at + (tid >> 2)] = m >= 0x7f800000u ? __uint_as_float(0x7fc00000u) : ldexpf(1.0f, -shift);
}

// NC: 1 KiB chunks of one row a lane visits (ceil(Kp/1024)); B: outputs per batch.
//
// Batches of outputs are dealt round-robin to the wavefronts.  The weight loads of a
// wavefront's first batch are issued before anything else - they do not depend on the activations - so
// the HBM stream is already running while the workgroup stages x through LDS and
// applies the RMSNorm prologue; after that the next batch is always in flight while
// the current one is multiplied (two register buffers used in turn).
// MODE (compile time, so that the other variants do not pay for its registers): 1 = GELU on the biased sum
// (its double-precision tanh costs some forty registers); 2 = ATTN_MERGE prologue: x is not the activation row
// but the per-split records [head][kAttnRecordSplits][hd + 4] = {max, sum, -, -, o[hd]} the decode attention
// kernel left, and the row is their merge  x[h*hd + j] = sum_s w_s o_s[j] / sum_s w_s l_s,  w_s = exp(max_s - max).
// PRO (compile time too: an operand that is not there must not be loaded - a workgroup's activation-sized loads
// are as many bytes as its weight rows): 0 = no prologue, 1 = RMSNorm (gamma), 2 = LayerNorm (gamma and beta).
// The operands arrive as separate kernel arguments, the ones every lane needs first in front: leading scalar
// arguments can be handed to a wavefront in registers at launch (a by-value struct is always fetched from the
// argument buffer, a dependent load ahead of every other load of the kernel).
// VEC (compile time): K is a multiple of 4 and the row is loaded as float4s.  A run-time choice between the two
// staging paths made the compiler merge their registers with copies placed right behind the first activation
// load - a wait for it ahead of every weight load.
template <int NC, int B, bool SWIGLU, int MODE, int PRO, bool VEC>
__global__ void __launch_bounds__(kThreads)
k_q8_matvec(const float *a_x, const int8_t *a_wq, const float *a_scales, float *a_out, int a_k, int a_grid, int a_n_out,
            int a_rec_hd, const float *a_gamma, const float *a_bias, const float *a_bias2, const float *a_residual,
            const float *a_beta) {
    // (the grid size comes as an argument: gridDim.x is one more value fetched from the argument buffer)
    const MatvecArgs p{a_x, a_wq, a_scales, a_out, a_k, (a_k + kQ8Group - 1) / kQ8Group * kQ8Group, a_n_out, a_gamma,
                       a_bias, a_bias2, a_residual, a_beta, a_rec_hd};
    constexpr bool GELU = MODE == 1;
    constexpr bool MERGE = MODE == 2;
    constexpr int NS = kAttnRecordSplits;
    extern __shared__ __align__(16) float xs[];   // the activation row, laid out by xs_at() below
    __shared__ float red[kWaves], red2[kWaves];
    constexpr int RPO = SWIGLU ? 2 : 1;           // Q8 rows per output
    constexpr int R = B * RPO;                    // rows per batch
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int groups = p.kp / kQ8Group;
    const int wave_global = blockIdx.x * kWaves + wave;
    const int wave_count = a_grid * kWaves;
    // Batches are dealt round-robin: batch j of wave w is batch w + j*wave_count of the
    // matrix, so at any moment the rows in flight across the chip are neighbours in memory.
    const int n_batches = (p.n_out + B - 1) / B;
    const bool has_work = wave_global < n_batches;    // wave-uniform
    const int row_last = p.n_out * RPO - 1;
    const int o_end = p.n_out;
    const int o_begin = wave_global * B;
    const int o_step = wave_count * B;
    DJ_STAMP(0);

    RowBatch<NC, R> ba, bb;
    bool deferred_norm = false;
    constexpr bool vec = VEC;
    float4 xv[NC], gv[NC], bv[NC];
    float2 rml[MERGE ? NC : 1][NS];
    float4 rov[MERGE ? NC : 1][NS];
    if constexpr (MERGE) {
        // the records of the head each float4 of the row belongs to: unconditional, issued before the weights
        const int rstride = p.rec_hd + 4;
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const int e = (tid + kThreads * j) * 4;
            const int ec = e < p.k ? e : 0;
            const int head = ec / p.rec_hd, off = ec - head * p.rec_hd;
            const float *r = p.x + (int64_t)head * NS * rstride;
#pragma unroll
            for (int sp = 0; sp < NS; sp++) {
                rml[j][sp] = *reinterpret_cast<const float2 *>(r + sp * rstride);
                rov[j][sp] = *reinterpret_cast<const float4 *>(r + sp * rstride + 4 + off);
            }
        }
    } else if (vec) {
        // The activation, gain and beta loads go out first: they hit in L2 and come back while the weight loads
        // issued right behind them are still on their way from HBM.  All of them are unconditional (clamped
        // address; which operands exist is known at compile time), so the wait for them is a counted one that
        // leaves the weight loads in flight.
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const int e = (tid + kThreads * j) * 4;
            const int ec = e < p.k ? e : 0;
            xv[j] = *reinterpret_cast<const float4 *>(p.x + ec);
            if constexpr (PRO >= 1) gv[j] = *reinterpret_cast<const float4 *>(p.gamma + ec);
            else gv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
            if constexpr (PRO == 2) bv[j] = *reinterpret_cast<const float4 *>(p.beta + ec);
            else bv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    asm volatile("" ::: "memory");      // the loads above are issued before the ones below ...
    {
        // waves without a batch load their (clamped) last row too: cheaper than a branch around the loads
        const int first = has_work ? o_begin : 0;
        load_batch<NC, R>(ba, p, first * RPO, row_last, lane, groups);
        load_epilogue<NC, R, B, SWIGLU>(ba, p, first);
    }
    asm volatile("" ::: "memory");
    if constexpr (MERGE) {
#pragma unroll
        for (int j = 0; j < NC; j++) {
            float m0 = rml[j][0].x;
            asm volatile("" : "+v"(m0));        // nothing consumes the records before the weight loads are out
            float mx = m0;
#pragma unroll
            for (int sp = 1; sp < NS; sp++) mx = fmaxf(mx, rml[j][sp].x);
            float lsum = 0.0f;
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int sp = 0; sp < NS; sp++) {
                const float ms = sp == 0 ? m0 : rml[j][sp].x;
                const float w = __builtin_amdgcn_exp2f(ms - mx);            // base-2 maxima; a split without keys: exp2(-inf) = 0
                lsum += rml[j][sp].y * w;
                acc.x += rov[j][sp].x * w; acc.y += rov[j][sp].y * w; acc.z += rov[j][sp].z * w; acc.w += rov[j][sp].w * w;
            }
            const bool ok = (tid + kThreads * j) * 4 < p.k;
            const float inv = 1.0f / lsum;
            xv[j] = ok ? make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv) : make_float4(0.f, 0.f, 0.f, 0.f);
            gv[j] = bv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    } else if (vec) {
#pragma unroll
        for (int j = 0; j < NC; j++) {
            // ... and nothing consumes them before the weight loads are out (the scheduler would otherwise park
            // the wavefront on the activations first and request the weights one L2 round trip later)
            float x0 = xv[j].x, x1 = xv[j].y, x2 = xv[j].z, x3 = xv[j].w;
            asm volatile("" : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3));
            const bool ok = (tid + kThreads * j) * 4 < p.k;
            const bool okg = ok && PRO >= 1;
            xv[j] = make_float4(ok ? x0 : 0.f, ok ? x1 : 0.f, ok ? x2 : 0.f, ok ? x3 : 0.f);
            gv[j] = make_float4(okg ? gv[j].x : 0.f, okg ? gv[j].y : 0.f, okg ? gv[j].z : 0.f, okg ? gv[j].w : 0.f);
            bv[j] = make_float4(ok ? bv[j].x : 0.f, ok ? bv[j].y : 0.f, ok ? bv[j].z : 0.f, ok ? bv[j].w : 0.f);
        }
    }

    // Stage the activation row through LDS (zero beyond K so padded weights meet zeros).
    // All global loads of the prologue - x and, for the RMSNorm prologue, gamma - were
    // issued together, so it costs one memory round trip, not one per element.
    if (vec && PRO == 2) {
        // LayerNorm prologue (LayerNorm1D.java:34-66): mean, then the population variance about it, then
        // ((x - mean) / sqrt(var + 1e-5)) * gamma + beta goes to LDS.
        const float inv_k = 1.0f / (float)p.k;
        float sm = 0.0f;
#pragma unroll
        for (int j = 0; j < NC; j++) sm += (xv[j].x + xv[j].y) + (xv[j].z + xv[j].w);
        sm = wave_sum_dpp(sm);
        if (lane == 0) red[wave] = sm;
        lds_barrier();
        const float mean = (red[0] + red[1] + red[2] + red[3]) * inv_k;
        float sv = 0.0f;
#pragma unroll
        for (int j = 0; j < NC; j++) {
            bool ok = (tid + kThreads * j) * 4 < p.k;
            float a = xv[j].x - mean, b = xv[j].y - mean, c = xv[j].z - mean, d = xv[j].w - mean;
            xv[j] = ok ? make_float4(a, b, c, d) : make_float4(0.f, 0.f, 0.f, 0.f);
            sv += ok ? (a * a + b * b) + (c * c + d * d) : 0.0f;
        }
        sv = wave_sum_dpp(sv);
        if (lane == 0) red2[wave] = sv;
        lds_barrier();
        const float sd = sqrtf((red2[0] + red2[1] + red2[2] + red2[3]) * inv_k + kLayerNormEps);
#pragma unroll
        for (int j = 0; j < NC; j++) {
            int e = (tid + kThreads * j) * 4;
            float4 y;
            y.x = (xv[j].x / sd) * gv[j].x + bv[j].x; y.y = (xv[j].y / sd) * gv[j].y + bv[j].y;
            y.z = (xv[j].z / sd) * gv[j].z + bv[j].z; y.w = (xv[j].w / sd) * gv[j].w + bv[j].w;
            (void)e;
            stage_digits(xs, xd_plane(j, 0), xd_shift<NC>(j), tid, y);         // e >= k: x, gamma and beta are all zero
        }
    } else if (vec) {
        if (PRO == 1) {
            // RMSNorm prologue (RMSNorm1D.java:46-57).  W.(g * x / rms) = (W.(g * x)) / rms: the staged row is
            // g * x, which needs no reduction, and the division by rms is applied to the finished sums, so the
            // sum of squares is reduced while the weight rows are still streaming in.
            float ss = 0.0f;
#pragma unroll
            for (int j = 0; j < NC; j++) ss += xv[j].x * xv[j].x + xv[j].y * xv[j].y + xv[j].z * xv[j].z + xv[j].w * xv[j].w;
            ss = wave_sum_dpp(ss);
            if (lane == 0) red[wave] = ss;
            deferred_norm = true;
#pragma unroll
            for (int j = 0; j < NC; j++) {
                xv[j].x = xv[j].x * gv[j].x; xv[j].y = xv[j].y * gv[j].y;
                xv[j].z = xv[j].z * gv[j].z; xv[j].w = xv[j].w * gv[j].w;
            }
        }
#pragma unroll
        for (int j = 0; j < NC; j++) stage_digits(xs, xd_plane(j, 0), xd_shift<NC>(j), tid, xv[j]);
    } else {
        float ss = 0.0f;
        for (int i = tid; i < p.kp; i += kThreads) {
            float v = i < p.k ? p.x[i] : 0.0f;
            xs[xs_at(i)] = v;
            ss += v * v;
        }
        if (p.beta) {
            float sm = 0.0f;
            for (int i = tid; i < p.k; i += kThreads) sm += p.x[i];
            sm = wave_sum_dpp(sm);
            if (lane == 0) red[wave] = sm;
            lds_barrier();
            float mean = (red[0] + red[1] + red[2] + red[3]) * (1.0f / (float)p.k);
            float sv = 0.0f;
            for (int i = tid; i < p.k; i += kThreads) { float c = xs[xs_at(i)] - mean; sv += c * c; }
            sv = wave_sum_dpp(sv);
            if (lane == 0) red2[wave] = sv;
            lds_barrier();
            float sd = sqrtf((red2[0] + red2[1] + red2[2] + red2[3]) * (1.0f / (float)p.k) + kLayerNormEps);
            for (int i = tid; i < p.k; i += kThreads) xs[xs_at(i)] = ((xs[xs_at(i)] - mean) / sd) * p.gamma[i] + p.beta[i];
        } else if (p.gamma) {
            ss = wave_sum_dpp(ss);
            if (lane == 0) red[wave] = ss;
            lds_barrier();
            float tot = red[0] + red[1] + red[2] + red[3];
            float rms = sqrtf(tot * (1.0f / (float)p.k) + kRmsEps);
            for (int i = tid; i < p.k; i += kThreads) xs[xs_at(i)] = (xs[xs_at(i)] / rms) * p.gamma[i];
        }
    }
    DJ_STAMP(1);
    lds_barrier();
    DJ_STAMP(2);
    if (!has_work) return;
    float rms = 1.0f;
    if (deferred_norm) {
        float tot = red[0] + red[1] + red[2] + red[3];
        rms = sqrtf(tot * (1.0f / (float)p.k) + kRmsEps);
    }

    // this lane's activation slice: 16 consecutive k of each 1 KiB chunk
    XSlice<NC, VEC> xr;
#pragma unroll
    for (int c = 0; c < NC; c++) {
        if constexpr (VEC) {
            const uint32_t *xd = reinterpret_cast<const uint32_t *>(xs);
#pragma unroll
            for (int g = 0; g < 3; g++) {
                const uint4 v = *reinterpret_cast<const uint4 *>(xd + xd_plane(c, g) + lane * 4);
                xr.d[c][4 * g] = (int)v.x; xr.d[c][4 * g + 1] = (int)v.y; xr.d[c][4 * g + 2] = (int)v.z; xr.d[c][4 * g + 3] = (int)v.w;
            }
            const float unit = xs[xd_shift<NC>(c) + lane];
            xr.k[c][0] = unit; xr.k[c][1] = unit * 256.0f; xr.k[c][2] = unit * 65536.0f;
        } else {
            int kb = (c * 64 + lane) * 16;
            bool active = kb < p.kp;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float4 v = active ? *reinterpret_cast<const float4 *>(xs + (c * 4 + j) * kXsPlane + lane * 4) : make_float4(0, 0, 0, 0);
                xr.f[c][4 * j] = v.x; xr.f[c][4 * j + 1] = v.y; xr.f[c][4 * j + 2] = v.z; xr.f[c][4 * j + 3] = v.w;
            }
        }
    }

    DJ_STAMP(3);
    for (int o0 = o_begin; o0 < o_end; o0 += 2 * o_step) {
        if (o0 + o_step < o_end) { load_batch<NC, R>(bb, p, (o0 + o_step) * RPO, row_last, lane, groups); load_epilogue<NC, R, B, SWIGLU>(bb, p, o0 + o_step); }
        finish_batch<NC, B, SWIGLU, GELU, VEC>(ba, xr, p, o0, o_end, lane, rms);
        if (o0 == o_begin) DJ_STAMP(4);
        if (o0 + o_step >= o_end) break;
        if (o0 + 2 * o_step < o_end) { load_batch<NC, R>(ba, p, (o0 + 2 * o_step) * RPO, row_last, lane, groups); load_epilogue<NC, R, B, SWIGLU>(ba, p, o0 + 2 * o_step); }
        finish_batch<NC, B, SWIGLU, GELU, VEC>(bb, xr, p, o0 + o_step, o_end, lane, rms);
    }
    DJ_STAMP(5);
}

constexpr int kMvGridCap = 768;          // three workgroups per CU
constexpr int kMvGridCapWide = 1024;     // four for the widest matrices (the LM head: two batches per wavefront instead of three, 14.7 -> 14.0 us)
inline int mv_grid_cap() { return kMvGridCap; }

template <int NC, int B, bool SW, int MODE = 0>
void launch_mv(hipStream_t s, const MatvecArgs &a) {
    if constexpr (B != 1 && MODE != 2) {
        if ((a.k & 3) != 0) { launch_mv<NC, 1, SW, MODE>(s, a); return; }
    }
    // Three workgroups (12 wavefronts) per CU when there are outputs for them; never
    // more wavefronts than outputs.
    int batches = (a.n_out + B - 1) / B;
    int grid = (batches + kWaves - 1) / kWaves;
    const int cap = a.n_out >= 16384 ? kMvGridCapWide : mv_grid_cap();
    if (grid > cap) {
        // every wavefront the same number of batches: fewer workgroups than the cap rather than a last, partly
        // filled round (gate/up: 704 workgroups of exactly two batches per wavefront instead of 768 with one or two)
        const int rounds = (batches + cap * kWaves - 1) / (cap * kWaves);
        grid = (batches + kWaves * rounds - 1) / (kWaves * rounds);
    }
    if (grid < 1) grid = 1;
    size_t lds = (size_t)xs_floats(a.kp) * sizeof(float);
    // the prologue the operands ask for: gamma and beta = LayerNorm, gamma alone = RMSNorm
    const int pro = a.gamma ? (a.beta ? 2 : 1) : 0;
    // ragged K (not a multiple of 4): the scalar staging path, built for one output per wavefront only
    const bool vec = (a.k & 3) == 0;
    auto go = [&](auto pro_tag) {
        constexpr int PRO = decltype(pro_tag)::value;
        if (vec) {
            launch_kernel(k_q8_matvec<NC, B, SW, MODE, PRO, true>, dim3(grid), dim3(kThreads), lds, s, a.x, a.wq,
                          a.scales, a.out, a.k, grid, a.n_out, a.rec_hd, a.gamma, a.bias, a.bias2, a.residual, a.beta);
        } else if constexpr (B == 1 && MODE != 2) {
            launch_kernel(k_q8_matvec<NC, B, SW, MODE, PRO, false>, dim3(grid), dim3(kThreads), lds, s, a.x, a.wq,
                          a.scales, a.out, a.k, grid, a.n_out, a.rec_hd, a.gamma, a.bias, a.bias2, a.residual, a.beta);
        } else {
            fail("q8_linear: no matvec kernel for this shape");     // launch_mv sends ragged K to B = 1
        }
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    using P2 = std::integral_constant<int, 2>;
    if constexpr (MODE == 2) {
        go(P0{});
    } else if constexpr (SW) {
        if (pro == 2) fail("q8_linear: SWIGLU cannot be combined with LAYERNORM");
        if (pro == 1) go(P1{});
        else go(P0{});
    } else {
        if (pro == 2) go(P2{});
        else if (pro == 1) go(P1{});
        else go(P0{});
    }
}

// Batch depth B (outputs a wavefront multiplies per step).  Small matrices want B = 1: every
// row gets its own wavefront, so the whole matrix is requested at once and the serial work
// after the data arrives is one row.  Large matrices want deeper batches (about eight 128-bit
// loads per lane in flight per buffer) so ~3000 resident wavefronts keep the HBM queues full.
inline int mv_target_waves() { return 3072; }

template <int NC>
void dispatch_mv(hipStream_t s, const MatvecArgs &a, bool swiglu, bool gelu) {
    if (a.rec_hd > 0) {           // ATTN_MERGE prologue (never with SwiGLU or GELU)
        // Every workgroup merges the whole row for itself, so fewer, deeper workgroups: two outputs per
        // wavefront even when that leaves wavefronts to spare (measured: +0.2 us over the plain kernel at
        // 2048 x 2048, +0.9 us with one output per wavefront).
        constexpr int BM = NC <= 4 ? 2 : 1;
        launch_mv<NC, BM, false, 2>(s, a);
        return;
    }
    constexpr int BMAX = NC == 1 ? 8 : (NC == 2 ? 4 : (NC <= 4 ? 2 : 1));
    int rows = swiglu ? 2 * a.n_out : a.n_out;
    int want = (rows + mv_target_waves() - 1) / mv_target_waves();      // rows per wavefront per step
    if (swiglu) {
        constexpr int BS = BMAX >= 2 ? BMAX / 2 : 1;
        if (BS >= 4 && want >= 8) launch_mv<NC, (BS >= 4 ? 4 : 1), true>(s, a);
        else if (BS >= 2 && want >= 4) launch_mv<NC, (BS >= 2 ? 2 : 1), true>(s, a);
        else launch_mv<NC, 1, true>(s, a);
    } else if (gelu) {
        if (BMAX >= 4 && want >= 4) launch_mv<NC, (BMAX >= 4 ? 4 : 1), false, 1>(s, a);
        else if (BMAX >= 2 && want >= 2) launch_mv<NC, (BMAX >= 2 ? 2 : 1), false, 1>(s, a);
        else launch_mv<NC, 1, false, 1>(s, a);
    } else {
        if (BMAX >= 8 && want >= 8) launch_mv<NC, (BMAX >= 8 ? 8 : 1), false>(s, a);
        else if (BMAX >= 4 && want >= 4) launch_mv<NC, (BMAX >= 4 ? 4 : 1), false>(s, a);
        else if (BMAX >= 2 && want >= 2) launch_mv<NC, (BMAX >= 2 ? 2 : 1), false>(s, a);
        else launch_mv<NC, 1, false>(s, a);
    }
}

}  // namespace

void launch_q8_quantize(hipStream_t s, const float *w, int8_t *q, float *scales, int k, int n, int row_off,
                        int row_step) {
    if (k <= 0 || n <= 0) return;
    int kp = q8_padded_k(k);
    dim3 grid((n + 63) / 64, kp / kQ8Group);
    launch_kernel(k_q8_quantize, grid, dim3(kThreads), 0, s, w, q, scales, k, n, kp, row_off, row_step);
}

void launch_q8_dequantize(hipStream_t s, const int8_t *q, const float *scales, float *w, int k, int n, int row_off,
                          int row_step) {
    int64_t total = (int64_t)k * n;
    if (total <= 0) return;
    int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 8192) blocks = 8192;
    launch_kernel(k_q8_dequantize, dim3((int)blocks), dim3(kThreads), 0, s, q, scales, w, k, n,
                       q8_padded_k(k), row_off, row_step);
}

static bool matvec_supported(int k) { return q8_padded_k(k) <= 11 * 1024; }

int64_t q8_linear_workspace_floats(int m, int k, int n, int flags) {
    bool mv = (m == 1) && matvec_supported(k);
    int64_t ws = 0;
    if (!mv) {
        if (flags & (DJ_LIN_RMSNORM | DJ_LIN_LAYERNORM)) ws += (int64_t)m * k;   // normalised activations
    }
    return ws;
}

int64_t q8_linear_preferred_workspace_floats(int m, int k, int n, int flags, bool prepared) {
    const int64_t ws = q8_linear_workspace_floats(m, k, n, flags);
    const int n_rows = (flags & DJ_LIN_SWIGLU) ? 2 * n : n;
    const bool mv = (m == 1) && matvec_supported(k);
    if (!mv && q8_gemm_f16_shape_ok(m, n_rows, k, prepared)) return std::max(ws, q8_gemm_f16_workspace_floats(m, n_rows, k, prepared));
    if (!mv) return ws + q8_gemm_workspace_floats(m, n_rows, k);      // the partial products of a K-sharing launch
    return ws;
}

void launch_q8_linear(hipStream_t s, const Q8Linear &p, float *workspace, int64_t workspace_floats) {
    if (p.m <= 0 || p.n <= 0) return;
    const bool swiglu = (p.flags & DJ_LIN_SWIGLU) != 0;
    const bool layernorm = (p.flags & DJ_LIN_LAYERNORM) != 0;
    const int gelu = (p.flags & DJ_LIN_GELU) ? 1 : 0;
    const float *gamma = (p.flags & (DJ_LIN_RMSNORM | DJ_LIN_LAYERNORM)) ? p.gamma : nullptr;
    const float *beta = layernorm ? p.beta : nullptr;
    const float *bias = (p.flags & DJ_LIN_BIAS) ? p.bias : nullptr;
    const float *bias2 = (p.flags & DJ_LIN_BIAS) && swiglu ? p.bias2 : nullptr;
    const float *residual = (p.flags & DJ_LIN_RESIDUAL) ? p.residual : nullptr;
    const int kp = q8_padded_k(p.k);

    if (p.m == 1 && !p.m_dev && matvec_supported(p.k)) {
        if (p.rope.q) fail("q8_linear: the RoPE epilogue exists on the fp16 GEMM only (deepj_hip_q8_linear_rope_ok says for which shapes)");
        const int rec_hd = (p.flags & DJ_LIN_ATTN_MERGE) ? p.rec_hd : 0;
        MatvecArgs a{p.x, p.wq, p.scales, p.out, p.k, kp, p.n, gamma, bias, bias2, residual, beta, rec_hd};
        int nc = (kp + 1023) / 1024;
        switch (nc) {
            case 1: dispatch_mv<1>(s, a, swiglu, gelu != 0); break;
            case 2: dispatch_mv<2>(s, a, swiglu, gelu != 0); break;
            case 3: dispatch_mv<3>(s, a, swiglu, gelu != 0); break;
            case 4: dispatch_mv<4>(s, a, swiglu, gelu != 0); break;
            case 5: dispatch_mv<5>(s, a, swiglu, gelu != 0); break;
            case 6: dispatch_mv<6>(s, a, swiglu, gelu != 0); break;
            case 7: dispatch_mv<7>(s, a, swiglu, gelu != 0); break;
            case 8: dispatch_mv<8>(s, a, swiglu, gelu != 0); break;
            case 9: dispatch_mv<9>(s, a, swiglu, gelu != 0); break;
            case 10: dispatch_mv<10>(s, a, swiglu, gelu != 0); break;
            default: dispatch_mv<11>(s, a, swiglu, gelu != 0); break;
        }
        return;
    }

    // GEMM path
    if (p.flags & DJ_LIN_ATTN_MERGE) fail("q8_linear: the ATTN_MERGE prologue exists for M = 1 only");
    if (workspace_floats < q8_linear_workspace_floats(p.m, p.k, p.n, p.flags)) fail("q8_linear: workspace too small");
    if (swiglu && residual) fail("q8_linear: SWIGLU with RESIDUAL is not supported");   // no caller combines them
    // many rows and enough tiles: the fp16 kernel, when the caller's workspace also holds its prepared operands; the
    // normalisation happens on the rows' way into that layout
    const int n_rows = swiglu ? 2 * p.n : p.n;
    const bool rope = p.rope.q != nullptr;
    if (!p.m_dev && !p.small_workspace_only && q8_gemm_f16_shape_ok(p.m, n_rows, p.k, p.prepared != nullptr) && workspace_floats >= q8_gemm_f16_workspace_floats(p.m, n_rows, p.k, p.prepared != nullptr)) {
        launch_q8_gemm_f16(s, p.x, gamma, beta, p.wq, p.scales, p.prepared, p.out, p.m, p.k, n_rows, bias, swiglu ? bias2 : nullptr,
                           swiglu ? nullptr : residual, swiglu ? 1 : 0, swiglu ? 0 : gelu, swiglu ? 1 : 0, workspace, workspace_floats,
                           rope ? &p.rope : nullptr, p.chain);
        return;
    }
    if (rope) fail("q8_linear: the RoPE epilogue exists on the fp16 GEMM only (deepj_hip_q8_linear_rope_ok says for which shapes)");
    const float *x = p.x;
    float *ws = workspace;
    if (gamma) {
        if (layernorm) launch_layernorm(s, p.x, gamma, beta, ws, p.m, p.k);
        else launch_rmsnorm(s, p.x, gamma, ws, p.m, p.k);
        x = ws;
        ws += (int64_t)p.m * p.k;
    }
    // what is left of the workspace takes the partial products when a few tiles share their K among several workgroups
    // (never with a workspace that cannot grow: one rule for the allocation-free entry point)
    float *part = p.small_workspace_only ? nullptr : ws;
    const int64_t part_floats = p.small_workspace_only ? 0 : workspace_floats - (ws - workspace);
    if (swiglu) {
        // the GEMM's epilogue pairs the interleaved gate/up columns, so the 2N-wide product never reaches memory
        launch_q8_gemm(s, x, p.wq, p.scales, p.out, p.m, p.k, 2 * p.n, bias, bias2, nullptr, 1, nullptr, 0, 0, 1, part, part_floats);
    } else {
        launch_q8_gemm(s, x, p.wq, p.scales, p.out, p.m, p.k, p.n, bias, nullptr, residual, 0, p.m_dev, p.m_extra, gelu, 0, part, part_floats);
    }
}

#ifdef DJ_TRACE
extern "C" int deepj_hip_debug_mv_trace(unsigned long long *out, int n) {
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_mv_trace), (size_t)n * sizeof(unsigned long long));
}
#endif

}  // namespace dj
