// Dense contractions on the fp32 matrix cores (v_mfma_f32_32x32x2_f32).
//
//   C[M x N] = A[M x K] . B      A fp32 row-major, fp32 accumulate
//
// B is either fp32 [K x N] row-major (OP_MATMUL; CpuBackend.java:168-188 in the
// reference) or a Q8 weight [N x Kp] int8 + one fp32 scale per 32-group, which is
// dequantised while it is staged into LDS (prefill-time Q8 GEMM: a dense
// contraction, so it belongs on MFMA; the M = 1 decode case is a separate
// HBM-bound kernel in kernels_q8.hip).
//
// Tiling: 256 threads = 4 wavefronts, workgroup tile 64 x 64, each wavefront owns
// one 32 x 32 accumulator (16 VGPRs), K advances 32 per step = one Q8 group.
// Both operand tiles sit k-major in LDS so the 64 lanes of an MFMA operand read
// 32 consecutive floats per half-wave (no bank conflicts).
#include "dj_common.h"

namespace dj {

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int BM = 64, BN = 64, BK = 32;
constexpr int PAD = 4;

struct GemmEpilogue {
    const float *bias;      // [N] or null; with interleave: even col n -> bias[n/2], odd col -> bias2[n/2]
    const float *bias2;
    const float *residual;  // [M x N] or null
    int interleaved_bias;
    const int32_t *m_dev;   // when set, only rows < min(M, m_dev[0] + m_extra) exist (row count kept on the device)
    int m_extra;
    int gelu;               // GELU (tanh form, tensor/cpu/CpuBackend.java:338, used by activations/GELU.java:15-18) on acc + bias, before the residual
};

__device__ __forceinline__ float gemm_gelu(float x) {
    float c = sqrtf(2.0f / 3.14159265358979323846f);
    float x3 = x * x * x;
    float t = c * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + (float)tanh((double)t));
}

template <bool Q8>
__global__ void __launch_bounds__(256) k_gemm(const float *__restrict__ A, const float *__restrict__ Bf,
                                              const int8_t *__restrict__ Bq, const float *__restrict__ Bs,
                                              float *__restrict__ C, int M, const int N, const int K, const int kp,
                                              GemmEpilogue ep) {
    __shared__ float As[BK][BM + PAD];
    __shared__ float Bl[BK][BN + PAD];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    if (ep.m_dev) {
        int live = ep.m_dev[0] + ep.m_extra;
        if (live < M) M = live;
        if (m0 >= M) return;                 // workgroup-uniform
    }

    floatx16 acc;
#pragma unroll
    for (int j = 0; j < 16; j++) acc[j] = 0.0f;

    const int a_row = t >> 2;            // 0..63
    const int a_k = (t & 3) * 8;         // 0,8,16,24
    const bool a_vec = (K & 3) == 0;

    // Register-staged software pipeline: the global loads of K-step i+1 are issued before the MFMAs of
    // step i, so their latency hides behind the matrix work instead of adding to every step.
    float va[8];                 // A: 8 consecutive k of one row
    float wb[8];                 // B fp32: 8 consecutive columns of one k
    int2 qraw = make_int2(0, 0); // B Q8: 8 consecutive k of one column
    float qsc = 0.0f;
    auto fetch = [&](int k0) {
        {
            int gr = m0 + a_row;
            if (gr < M && a_vec && k0 + a_k + 8 <= K) {
                const float4 *p = reinterpret_cast<const float4 *>(A + (int64_t)gr * K + k0 + a_k);
                float4 x = p[0], y = p[1];
                va[0] = x.x; va[1] = x.y; va[2] = x.z; va[3] = x.w; va[4] = y.x; va[5] = y.y; va[6] = y.z; va[7] = y.w;
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    int gk = k0 + a_k + j;
                    va[j] = (gr < M && gk < K) ? A[(int64_t)gr * K + gk] : 0.0f;
                }
            }
        }
        if constexpr (Q8) {
            int col = t >> 2, part = t & 3;          // 8 int8 per thread
            int gn = n0 + col;
            if (gn < N) {
                const int8_t *p = Bq + (int64_t)gn * kp + k0 + part * 8;   // kp is a multiple of 32: in bounds
                qraw = *reinterpret_cast<const int2 *>(p);
                qsc = Bs[(int64_t)gn * (kp / kQ8Group) + k0 / kQ8Group];
            } else {
                qraw = make_int2(0, 0);
                qsc = 0.0f;
            }
        } else {
            int bk = t >> 3, bn = (t & 7) * 8;       // 8 consecutive columns per thread
            int gk = k0 + bk;
            if (gk < K && (N & 3) == 0 && n0 + bn + 8 <= N) {
                const float4 *p = reinterpret_cast<const float4 *>(Bf + (int64_t)gk * N + n0 + bn);
                float4 x = p[0], y = p[1];
                wb[0] = x.x; wb[1] = x.y; wb[2] = x.z; wb[3] = x.w; wb[4] = y.x; wb[5] = y.y; wb[6] = y.z; wb[7] = y.w;
            } else {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    int gn = n0 + bn + j;
                    wb[j] = (gk < K && gn < N) ? Bf[(int64_t)gk * N + gn] : 0.0f;
                }
            }
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int j = 0; j < 8; j++) As[a_k + j][a_row] = va[j];
        if constexpr (Q8) {
            int col = t >> 2, part = t & 3;
            int r0 = qraw.x, r1 = qraw.y;
            float w[8];
            w[0] = (float)(int8_t)(r0 & 0xff) * qsc;         w[1] = (float)(int8_t)((r0 >> 8) & 0xff) * qsc;
            w[2] = (float)(int8_t)((r0 >> 16) & 0xff) * qsc; w[3] = (float)(int8_t)((r0 >> 24) & 0xff) * qsc;
            w[4] = (float)(int8_t)(r1 & 0xff) * qsc;         w[5] = (float)(int8_t)((r1 >> 8) & 0xff) * qsc;
            w[6] = (float)(int8_t)((r1 >> 16) & 0xff) * qsc; w[7] = (float)(int8_t)((r1 >> 24) & 0xff) * qsc;
#pragma unroll
            for (int j = 0; j < 8; j++) Bl[part * 8 + j][col] = w[j];
        } else {
            int bk = t >> 3, bn = (t & 7) * 8;
#pragma unroll
            for (int j = 0; j < 8; j++) Bl[bk][bn + j] = wb[j];
        }
    };

    if (K > 0) fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        stage();
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);

        // ── 16 MFMA steps of K = 2 ─────────────────────────────────────────
        const int half = lane >> 5, l32 = lane & 31;
#pragma unroll
        for (int kk = 0; kk < BK / 2; kk++) {
            float a = As[2 * kk + half][wm * 32 + l32];
            float b = Bl[2 * kk + half][wn * 32 + l32];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
        __syncthreads();
    }

    // ── epilogue: acc[j] is C[8*(j/4) + 4*(lane/32) + j%4][lane%32] of the wave tile ──
    const int col = n0 + wn * 32 + (lane & 31);
    if (col < N) {
        float badd = 0.0f;
        if (ep.bias) badd = ep.interleaved_bias ? ((col & 1) ? ep.bias2[col >> 1] : ep.bias[col >> 1]) : ep.bias[col];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            int row = m0 + wm * 32 + 8 * (j >> 2) + 4 * (lane >> 5) + (j & 3);
            if (row < M) {
                float v = acc[j];
                if (ep.bias) v = v + badd;
                if (ep.gelu) v = gemm_gelu(v);
                if (ep.residual) v = ep.residual[(int64_t)row * N + col] + v;
                C[(int64_t)row * N + col] = v;
            }
        }
    }
}

// ── 128 x 128 workgroup tile ────────────────────────────────────────────────
// Same data flow with each wavefront owning a 64 x 64 block (four 32 x 32 accumulators): every operand
// value read from LDS feeds two MFMAs instead of one, which is what the 64 x 64 kernel is bound by.
constexpr int BM2 = 128, BN2 = 128;

template <bool Q8>
__global__ void __launch_bounds__(256) k_gemm128(const float *__restrict__ A, const float *__restrict__ Bf,
                                                 const int8_t *__restrict__ Bq, const float *__restrict__ Bs,
                                                 float *__restrict__ C, int M, const int N, const int K, const int kp,
                                                 GemmEpilogue ep) {
    __shared__ float As[BK][BM2 + PAD];
    __shared__ float Bl[BK][BN2 + PAD];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM2, n0 = blockIdx.x * BN2;
    if (ep.m_dev) {
        int live = ep.m_dev[0] + ep.m_extra;
        if (live < M) M = live;
        if (m0 >= M) return;                 // workgroup-uniform
    }

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    const int a_row = t >> 1;            // 0..127
    const int a_k = (t & 1) * 16;        // 0,16
    const bool a_vec = (K & 3) == 0;

    float va[16];                // A: 16 consecutive k of one row
    float wb[16];                // B fp32: 16 consecutive columns of one k
    int4 qraw = make_int4(0, 0, 0, 0);   // B Q8: 16 consecutive k of one column (half a scale group)
    float qsc = 0.0f;
    auto fetch = [&](int k0) {
        {
            int gr = m0 + a_row;
            if (gr < M && a_vec && k0 + a_k + 16 <= K) {
                const float4 *p = reinterpret_cast<const float4 *>(A + (int64_t)gr * K + k0 + a_k);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    float4 x = p[q];
                    va[4 * q] = x.x; va[4 * q + 1] = x.y; va[4 * q + 2] = x.z; va[4 * q + 3] = x.w;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    int gk = k0 + a_k + j;
                    va[j] = (gr < M && gk < K) ? A[(int64_t)gr * K + gk] : 0.0f;
                }
            }
        }
        if constexpr (Q8) {
            int col = t >> 1, part = t & 1;
            int gn = n0 + col;
            if (gn < N) {
                const int8_t *p = Bq + (int64_t)gn * kp + k0 + part * 16;  // kp is a multiple of 32: in bounds
                qraw = *reinterpret_cast<const int4 *>(p);
                qsc = Bs[(int64_t)gn * (kp / kQ8Group) + k0 / kQ8Group];
            } else {
                qraw = make_int4(0, 0, 0, 0);
                qsc = 0.0f;
            }
        } else {
            int bk = t >> 3, bn = (t & 7) * 16;      // 16 consecutive columns per thread
            int gk = k0 + bk;
            if (gk < K && (N & 3) == 0 && n0 + bn + 16 <= N) {
                const float4 *p = reinterpret_cast<const float4 *>(Bf + (int64_t)gk * N + n0 + bn);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    float4 x = p[q];
                    wb[4 * q] = x.x; wb[4 * q + 1] = x.y; wb[4 * q + 2] = x.z; wb[4 * q + 3] = x.w;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    int gn = n0 + bn + j;
                    wb[j] = (gk < K && gn < N) ? Bf[(int64_t)gk * N + gn] : 0.0f;
                }
            }
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int j = 0; j < 16; j++) As[a_k + j][a_row] = va[j];
        if constexpr (Q8) {
            int col = t >> 1, part = t & 1;
            const int words[4] = {qraw.x, qraw.y, qraw.z, qraw.w};
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int r = words[q];
                Bl[part * 16 + 4 * q + 0][col] = (float)(int8_t)(r & 0xff) * qsc;
                Bl[part * 16 + 4 * q + 1][col] = (float)(int8_t)((r >> 8) & 0xff) * qsc;
                Bl[part * 16 + 4 * q + 2][col] = (float)(int8_t)((r >> 16) & 0xff) * qsc;
                Bl[part * 16 + 4 * q + 3][col] = (float)(int8_t)((r >> 24) & 0xff) * qsc;
            }
        } else {
            int bk = t >> 3, bn = (t & 7) * 16;
#pragma unroll
            for (int j = 0; j < 16; j++) Bl[bk][bn + j] = wb[j];
        }
    };

    if (K > 0) fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        stage();
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);
        const int half = lane >> 5, l32 = lane & 31;
#pragma unroll
        for (int kk = 0; kk < BK / 2; kk++) {
            float a0 = As[2 * kk + half][wm * 64 + l32], a1 = As[2 * kk + half][wm * 64 + 32 + l32];
            float b0 = Bl[2 * kk + half][wn * 64 + l32], b1 = Bl[2 * kk + half][wn * 64 + 32 + l32];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        __syncthreads();
    }

    // epilogue: acc[i][jn][e] is C[32*i + 8*(e/4) + 4*(lane/32) + e%4][32*jn + lane%32] of the wave's 64 x 64 block
#pragma unroll
    for (int jn = 0; jn < 2; jn++) {
        const int col = n0 + wn * 64 + 32 * jn + (lane & 31);
        if (col >= N) continue;
        float badd = 0.0f;
        if (ep.bias) badd = ep.interleaved_bias ? ((col & 1) ? ep.bias2[col >> 1] : ep.bias[col >> 1]) : ep.bias[col];
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                int row = m0 + wm * 64 + 32 * i + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (row < M) {
                    float v = acc[i][jn][e];
                    if (ep.bias) v = v + badd;
                    if (ep.gelu) v = gemm_gelu(v);
                    if (ep.residual) v = ep.residual[(int64_t)row * N + col] + v;
                    C[(int64_t)row * N + col] = v;
                }
            }
        }
    }
}

// The large tile needs enough workgroups to fill the chip; small problems keep the 64 x 64 tile.
inline bool use_big_tile(int m, int n) {
    return m >= 128 && n >= 128 && (int64_t)((m + BM2 - 1) / BM2) * ((n + BN2 - 1) / BN2) >= 256;
}

}  // namespace

void launch_matmul_f32(hipStream_t s, const float *a, const float *b, float *out, int m, int n, int k) {
    if (m <= 0 || n <= 0) return;
    if (k <= 0) { launch_fill(s, reinterpret_cast<uint32_t *>(out), 0u, (int64_t)m * n); return; }
    GemmEpilogue ep{nullptr, nullptr, nullptr, 0, nullptr, 0, 0};
    if (use_big_tile(m, n)) {
        dim3 grid2((n + BN2 - 1) / BN2, (m + BM2 - 1) / BM2);
        hipLaunchKernelGGL(k_gemm128<false>, grid2, dim3(256), 0, s, a, b, (const int8_t *)nullptr, (const float *)nullptr,
                           out, m, n, k, 0, ep);
        return;
    }
    dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM);
    hipLaunchKernelGGL(k_gemm<false>, grid, dim3(256), 0, s, a, b, (const int8_t *)nullptr, (const float *)nullptr,
                       out, m, n, k, 0, ep);
}

// Q8 GEMM used by launch_q8_linear for M > 1.  n_rows is the number of Q8 rows
// (= output columns of this launch; 2N for an interleaved gate/up weight).
void launch_q8_gemm(hipStream_t s, const float *x, const int8_t *wq, const float *scales, float *out, int m,
                    int k, int n_rows, const float *bias, const float *bias2, const float *residual,
                    int interleaved_bias, const int32_t *m_dev, int m_extra, int gelu) {
    if (m <= 0 || n_rows <= 0) return;
    GemmEpilogue ep{bias, bias2, residual, interleaved_bias, m_dev, m_extra, gelu};
    if (!m_dev && use_big_tile(m, n_rows)) {       // a device-side row count is usually far below m: keep small tiles
        dim3 grid2((n_rows + BN2 - 1) / BN2, (m + BM2 - 1) / BM2);
        hipLaunchKernelGGL(k_gemm128<true>, grid2, dim3(256), 0, s, x, (const float *)nullptr, wq, scales, out, m,
                           n_rows, k, q8_padded_k(k), ep);
        return;
    }
    dim3 grid((n_rows + BN - 1) / BN, (m + BM - 1) / BM);
    hipLaunchKernelGGL(k_gemm<true>, grid, dim3(256), 0, s, x, (const float *)nullptr, wq, scales, out, m, n_rows, k,
                       q8_padded_k(k), ep);
}

}  // namespace dj
