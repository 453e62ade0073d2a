// Dense contractions on the matrix cores.
//
//   C[M x N] = A[M x K] . B      A fp32 row-major, fp32 accumulate
//
// fp32 B [K x N] row-major (OP_MATMUL; CpuBackend.java:168-188 in the reference): v_mfma_f32_32x32x2_f32.
// 256 threads = 4 wavefronts; workgroup tile 64 x 64 (one 32 x 32 accumulator per wavefront) or 128 x 128 (four),
// K advances 32 per step.  Both operand tiles sit k-major in LDS so the 64 lanes of an MFMA operand read 32
// consecutive floats per half-wave (no bank conflicts).
//
// Q8 B [N x Kp] int8 + one fp32 scale per 32-group (prefill-time Q8 GEMM; the M = 1 decode case is the HBM-bound
// kernel in kernels_q8.hip): v_mfma_f32_32x32x16_bf16 at full fp32 accuracy.  An int8 weight is exact in bf16,
// and an fp32 activation is the exact sum of three bf16 numbers (its top, middle and bottom 8 significant bits,
// taken by truncation), so x . q = hi . q + mid . q + lo . q with every product exact and fp32 accumulation: three
// bf16 MFMAs of K = 16 replace eight fp32 MFMAs of K = 2 at four times the rate.  The group scale multiplies the
// finished 32-k partial sums (one scale per accumulator column per step).  Tile shapes (64 x 64, 64 x 128,
// 128 x 128), scale groups per step and wavefront sets per workgroup are template arguments chosen per problem
// shape by launch_q8_gemm; the epilogue adds bias / GELU / residual or pairs interleaved gate/up columns (SwiGLU).
#include <cstdlib>
#include "dj_common.h"
#include "gemm_epilogue.h"

namespace dj {

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int BM = 64, BN = 64, BK = 32;
constexpr int PAD = 4;

__global__ void __launch_bounds__(256) k_gemm(const float *__restrict__ A, const float *__restrict__ Bf,
                                              float *__restrict__ C, int M, const int N, const int K,
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
    float wb[8];                 // B: 8 consecutive columns of one k
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
        {
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
        {
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

__global__ void __launch_bounds__(256) k_gemm128(const float *__restrict__ A, const float *__restrict__ Bf,
                                                 float *__restrict__ C, int M, const int N, const int K,
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
    float wb[16];                // B: 16 consecutive columns of one k
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
        {
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
        {
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

// ── Q8 weights: three-way bf16 split of the activations ────────────────────
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// bf16(a) | bf16(b) << 16, both by truncation
__device__ __forceinline__ uint32_t pack_bf16_hi(float a, float b) {
    return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, b), __builtin_bit_cast(uint32_t, a), 0x07060302);
}
__device__ __forceinline__ float top_bits(float x) {      // the leading 8 significant bits of x: a bf16 value
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x) & 0xffff0000u);
}

// Workgroup tile 64 WTM x 64 WTN, WTM x WTN accumulators of 32 x 32 per wavefront (1 x 1: 64 x 64 tile; 2 x 2: 128 x 128).
// G: scale groups (of 32 k) per step.  A step costs two barriers and an LDS round trip whatever its size, and a
// 64 x 64 tile has only six products per wavefront and group to set against that, so it takes several groups a step.
// Operand element j of lane l is k = 16*step + 8*(l / 32) + j for A and B alike, so the pairing of the MFMA's
// k slots does not depend on how the hardware numbers them.
// KS: wavefront sets per workgroup (256 threads each).  Set s multiplies the groups s, s + KS, ... of every step
// into accumulators of its own and the sets are added through LDS at the end: with a grid of one small tile per
// CU this is what puts a second wavefront on every SIMD, so one set's conversions overlap the other's products.
template <int WTM, int WTN, int G, int KS>
__global__ void __launch_bounds__(256 * KS) k_gemm_q8(const float *__restrict__ A, const int8_t *__restrict__ Bq,
                                                 const float *__restrict__ Bs, float *__restrict__ C, int M,
                                                 const int N, const int K, const int kp, GemmEpilogue ep,
                                                 const int split_k, float *__restrict__ partial) {
    constexpr int TM = 64 * WTM, TN = 64 * WTN;
    constexpr int QBK = kQ8Group * G;        // k per step
    constexpr int LDK = QBK + 8;             // LDS row: the step's bf16 payload + 8 of padding (16-byte aligned, spreads banks)
    constexpr int NT = 256 * KS;
    constexpr int EL = TM * QBK / NT;        // activation floats a thread stages per step ...
    constexpr int TPR = QBK / EL;            // ... as one of TPR threads per tile row
    constexpr int ELB = TN * QBK / NT;       // weight bytes a thread stages per step ...
    constexpr int TPRB = QBK / ELB;          // ... as one of TPRB threads per tile column
    static_assert(EL >= 8 && EL <= kQ8Group && kQ8Group % EL == 0 && ELB >= 8 && ELB <= kQ8Group && kQ8Group % ELB == 0,
                  "a thread's share of a row lies inside one scale group");
    static_assert(G % KS == 0, "the step's groups divide over the sets");
    // One LDS block: the step's operands, and after the last step the sums the sets exchange.
    constexpr int kXsBytes = 3 * TM * LDK * 2, kWlBytes = TN * LDK * 2, kSsBytes = G * TN * 4;
    constexpr int kRedBytes = (KS - 1) * 4 * WTM * WTN * 16 * 64 * 4;
    constexpr int kOperandBytes = kXsBytes + kWlBytes + kSsBytes;
    __shared__ __align__(16) unsigned char lds[kOperandBytes > kRedBytes ? kOperandBytes : kRedBytes];
    uint16_t(*Xs)[TM][LDK] = reinterpret_cast<uint16_t(*)[TM][LDK]>(lds);             // hi / mid / lo pieces, k contiguous
    uint16_t(*Wl)[LDK] = reinterpret_cast<uint16_t(*)[LDK]>(lds + kXsBytes);          // weights as bf16, a row per output column
    float(*Ss)[TN] = reinterpret_cast<float(*)[TN]>(lds + kXsBytes + kWlBytes);       // the step's group scales per output column

    const int t = threadIdx.x;
    const int lane = t & 63, wave = (t >> 6) & 3, kset = t >> 8;
    const int wm = wave >> 1, wn = wave & 1;
    const int half = lane >> 5, l32 = lane & 31;
    const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    if (ep.m_dev) {
        int live = ep.m_dev[0] + ep.m_extra;
        if (live < M) M = live;
        if (m0 >= M) return;                 // workgroup-uniform
    }
    const int groups = kp / kQ8Group;

    floatx16 acc[WTM][WTN];
#pragma unroll
    for (int i = 0; i < WTM; i++)
#pragma unroll
        for (int j = 0; j < WTN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    const int s_row = t / TPR;               // tile row of A this thread stages, from k offset s_k
    const int s_k = (t % TPR) * EL;
    const int s_col = t / TPRB;              // tile column (row of B) this thread stages, from k offset s_kb
    const int s_kb = (t % TPRB) * ELB;
    const bool a_vec = (K & 3) == 0;

    float va[EL];
    int qraw[ELB / 4];
    float qsc = 0.0f;
    auto fetch = [&](int k0) {
        const int gr = m0 + s_row;
        if (gr < M && a_vec && k0 + s_k + EL <= K) {
            const float4 *p = reinterpret_cast<const float4 *>(A + (int64_t)gr * K + k0 + s_k);
#pragma unroll
            for (int q = 0; q < EL / 4; q++) {
                float4 x = p[q];
                va[4 * q] = x.x; va[4 * q + 1] = x.y; va[4 * q + 2] = x.z; va[4 * q + 3] = x.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < EL; j++) {
                int gk = k0 + s_k + j;
                va[j] = (gr < M && gk < K) ? A[(int64_t)gr * K + gk] : 0.0f;
            }
        }
        const int gn = n0 + s_col;
        if (gn < N && k0 + s_kb < kp) {
            const int *p = reinterpret_cast<const int *>(Bq + (int64_t)gn * kp + k0 + s_kb);  // kp is a multiple of 32: in bounds
#pragma unroll
            for (int q = 0; q < ELB / 4; q++) qraw[q] = p[q];
            qsc = Bs[(int64_t)gn * groups + (k0 + s_kb) / kQ8Group];
        } else {
#pragma unroll
            for (int q = 0; q < ELB / 4; q++) qraw[q] = 0;
            qsc = 0.0f;
        }
    };
    auto stage = [&]() {
        uint32_t ph[EL / 2], pm[EL / 2], pl[EL / 2], pw[ELB / 2];
#pragma unroll
        for (int j = 0; j < EL / 2; j++) {
            const float x0 = va[2 * j], x1 = va[2 * j + 1];
            const float h0 = top_bits(x0), h1 = top_bits(x1);
            const float r0 = x0 - h0, r1 = x1 - h1;              // exact: h is a prefix of x
            const float c0 = top_bits(r0), c1 = top_bits(r1);
            const float l0 = r0 - c0, l1 = r1 - c1;              // at most 8 significant bits left: a bf16 value
            ph[j] = pack_bf16_hi(h0, h1); pm[j] = pack_bf16_hi(c0, c1); pl[j] = pack_bf16_hi(l0, l1);
        }
#pragma unroll
        for (int q = 0; q < ELB / 4; q++) {
            const int r = qraw[q];
            pw[2 * q] = pack_bf16_hi((float)(int8_t)(r & 0xff), (float)(int8_t)((r >> 8) & 0xff));
            pw[2 * q + 1] = pack_bf16_hi((float)(int8_t)((r >> 16) & 0xff), (float)(int8_t)((r >> 24) & 0xff));
        }
#pragma unroll
        for (int q = 0; q < EL / 8; q++) {
            reinterpret_cast<uint4 *>(&Xs[0][s_row][s_k])[q] = make_uint4(ph[4 * q], ph[4 * q + 1], ph[4 * q + 2], ph[4 * q + 3]);
            reinterpret_cast<uint4 *>(&Xs[1][s_row][s_k])[q] = make_uint4(pm[4 * q], pm[4 * q + 1], pm[4 * q + 2], pm[4 * q + 3]);
            reinterpret_cast<uint4 *>(&Xs[2][s_row][s_k])[q] = make_uint4(pl[4 * q], pl[4 * q + 1], pl[4 * q + 2], pl[4 * q + 3]);
        }
#pragma unroll
        for (int q = 0; q < ELB / 8; q++)
            reinterpret_cast<uint4 *>(&Wl[s_col][s_kb])[q] = make_uint4(pw[4 * q], pw[4 * q + 1], pw[4 * q + 2], pw[4 * q + 3]);
        if (s_kb % kQ8Group == 0) Ss[s_kb / kQ8Group][s_col] = qsc;
    };

    // split_k > 0: gridDim.z workgroups share a tile's K, this one takes [k_begin, k_end) (split_k is a multiple of the
    // step) and leaves its bare sums in its own slab of `partial`; k_sum_partials_q8 adds the slabs in a fixed order
    const int k_begin = split_k > 0 ? (int)blockIdx.z * split_k : 0;
    const int k_end = split_k > 0 && k_begin + split_k < K ? k_begin + split_k : K;
    if (k_begin < k_end) fetch(k_begin);
    for (int k0 = k_begin; k0 < k_end; k0 += QBK) {
        stage();
        __syncthreads();
        if (k0 + QBK < k_end) fetch(k0 + QBK);     // next step's global loads fly while this step multiplies

        // (a run-time loop on purpose: unrolled, the products of consecutive groups get interleaved and the kernel
        // measured 4-10 % slower)
        for (int grp = kset; grp < G; grp += KS) {
        floatx16 g[WTM][WTN];                  // this group's unscaled partial sums
#pragma unroll
        for (int i = 0; i < WTM; i++)
#pragma unroll
            for (int j = 0; j < WTN; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) g[i][j][e] = 0.0f;
#pragma unroll
        for (int step = 0; step < kQ8Group / 16; step++) {
            const int kofs = grp * kQ8Group + step * 16 + half * 8;
            bf16x8 b[WTN];
#pragma unroll
            for (int tn = 0; tn < WTN; tn++) b[tn] = *reinterpret_cast<const bf16x8 *>(&Wl[wn * 32 * WTN + 32 * tn + l32][kofs]);
#pragma unroll
            for (int piece = 0; piece < 3; piece++) {
#pragma unroll
                for (int tm = 0; tm < WTM; tm++) {
                    const bf16x8 a = *reinterpret_cast<const bf16x8 *>(&Xs[piece][wm * 32 * WTM + 32 * tm + l32][kofs]);
#pragma unroll
                    for (int tn = 0; tn < WTN; tn++) g[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b[tn], g[tm][tn], 0, 0, 0);
                }
            }
        }
        // every accumulator entry of a lane belongs to one output column: one scale per lane and tile column
#pragma unroll
        for (int tn = 0; tn < WTN; tn++) {
            const float sc = Ss[grp][wn * 32 * WTN + 32 * tn + l32];
#pragma unroll
            for (int tm = 0; tm < WTM; tm++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[tm][tn][e] = fmaf(g[tm][tn][e], sc, acc[tm][tn][e]);
        }
        }
        __syncthreads();
    }

    if constexpr (KS > 1) {
        // add the sets' sums: every set but the first parks its accumulators in the (no longer read) piece buffers
        float *red = reinterpret_cast<float *>(lds);                // [KS - 1][4 wavefronts][WTM*WTN*16][64 lanes]
        if (kset > 0) {
#pragma unroll
            for (int i = 0; i < WTM; i++)
#pragma unroll
                for (int j = 0; j < WTN; j++)
#pragma unroll
                    for (int e = 0; e < 16; e++)
                        red[((((kset - 1) * 4 + wave) * WTM * WTN + i * WTN + j) * 16 + e) * 64 + lane] = acc[i][j][e];
        }
        __syncthreads();
        if (kset > 0) return;
#pragma unroll
        for (int ks = 1; ks < KS; ks++)
#pragma unroll
            for (int i = 0; i < WTM; i++)
#pragma unroll
                for (int j = 0; j < WTN; j++)
#pragma unroll
                    for (int e = 0; e < 16; e++)
                        acc[i][j][e] += red[((((ks - 1) * 4 + wave) * WTM * WTN + i * WTN + j) * 16 + e) * 64 + lane];
    }

    // epilogue: acc[i][jn][e] is C[32*i + 8*(e/4) + 4*(lane/32) + e%4][32*jn + lane%32] of the wavefront's block
    if (split_k > 0) {
        float *slab = partial + (int64_t)blockIdx.z * M * N;
#pragma unroll
        for (int jn = 0; jn < WTN; jn++) {
            const int col = n0 + wn * 32 * WTN + 32 * jn + l32;
            if (col >= N) continue;
#pragma unroll
            for (int i = 0; i < WTM; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int row = m0 + wm * 32 * WTM + 32 * i + 8 * (e >> 2) + 4 * half + (e & 3);
                    if (row < M) slab[(int64_t)row * N + col] = acc[i][jn][e];
                }
        }
        return;
    }
#pragma unroll
    for (int jn = 0; jn < WTN; jn++) {
        const int col = n0 + wn * 32 * WTN + 32 * jn + l32;
        if (col >= N) continue;
        float badd = 0.0f;
        if (ep.bias) badd = ep.interleaved_bias ? ((col & 1) ? ep.bias2[col >> 1] : ep.bias[col >> 1]) : ep.bias[col];
#pragma unroll
        for (int i = 0; i < WTM; i++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + wm * 32 * WTM + 32 * i + 8 * (e >> 2) + 4 * half + (e & 3);
                if (ep.swiglu) {
                    // gate and up of one output sit in neighbouring lanes (columns 2j, 2j + 1); N is even, so a
                    // pair is inside or outside the matrix together (SiLU.java:20-24, SwiGLULayer.java:69)
                    float v = acc[i][jn][e];
                    if (ep.bias) v = v + badd;
                    const float other = __shfl_xor(v, 1, 64);
                    if (row < M && (col & 1) == 0) {
                        const float sg = v * (1.0f / (1.0f + expf(-v)));
                        C[(int64_t)row * (N >> 1) + (col >> 1)] = sg * other;
                    }
                    continue;
                }
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

// C = epilogue(sum over the splits of partial[z]) for the K-sharing launches of k_gemm_q8: the same bias / GELU /
// residual / SwiGLU steps, in the same order, as the kernel's own epilogue (a fixed order of additions, so a run
// repeats bit for bit - which adding into C with atomics would not).  One thread per column pair of a row.
__global__ void __launch_bounds__(256) k_sum_partials_q8(const float *__restrict__ partial, float *__restrict__ C, int splits,
                                                        int M, int N, GemmEpilogue ep) {
    const int64_t pairs = (int64_t)M * (N >> 1), mn = (int64_t)M * N;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < pairs; i += (int64_t)gridDim.x * 256) {
        const int row = (int)(i / (N >> 1)), col = (int)(i % (N >> 1)) * 2;
        const int64_t at = (int64_t)row * N + col;
        float2 v = *reinterpret_cast<const float2 *>(partial + at);
        for (int z = 1; z < splits; z++) {
            const float2 p = *reinterpret_cast<const float2 *>(partial + (int64_t)z * mn + at);
            v.x += p.x; v.y += p.y;
        }
        if (ep.bias) {
            if (ep.interleaved_bias) { v.x = v.x + ep.bias[col >> 1]; v.y = v.y + ep.bias2[col >> 1]; }
            else { v.x = v.x + ep.bias[col]; v.y = v.y + ep.bias[col + 1]; }
        }
        if (ep.swiglu) {                        // SiLU.java:20-24, SwiGLULayer.java:69
            const float sg = v.x * (1.0f / (1.0f + expf(-v.x)));
            C[(int64_t)row * (N >> 1) + (col >> 1)] = sg * v.y;
            continue;
        }
        if (ep.gelu) { v.x = gemm_gelu(v.x); v.y = gemm_gelu(v.y); }
        if (ep.residual) {
            const float2 r = *reinterpret_cast<const float2 *>(ep.residual + at);
            v.x = r.x + v.x; v.y = r.y + v.y;
        }
        *reinterpret_cast<float2 *>(C + at) = v;
    }
}

constexpr int kFewTiles = 512, kGroupsFew = 4, kSetsFew = 4;
constexpr int kSetsBig = 1;
constexpr int kGroupsSmall = 2, kGroupsBig = 1;    // measured: 4 and 2 are slower (LDS per workgroup, registers)

// The large tile needs enough workgroups to fill the chip; small problems keep the 64 x 64 tile.
inline bool use_big_tile(int m, int n) {
    return m >= 128 && n >= 128 && (int64_t)((m + BM2 - 1) / BM2) * ((n + BN2 - 1) / BN2) >= 256;
}

}  // namespace

void launch_matmul_f32(hipStream_t s, const float *a, const float *b, float *out, int m, int n, int k) {
    if (m <= 0 || n <= 0) return;
    if (k <= 0) { launch_fill(s, reinterpret_cast<uint32_t *>(out), 0u, (int64_t)m * n); return; }
    GemmEpilogue ep{nullptr, nullptr, nullptr, 0, nullptr, 0, 0, 0};
    if (use_big_tile(m, n)) {
        dim3 grid2((n + BN2 - 1) / BN2, (m + BM2 - 1) / BM2);
        launch_kernel(k_gemm128, grid2, dim3(256), 0, s, a, b, out, m, n, k, ep);
        return;
    }
    dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM);
    launch_kernel(k_gemm, grid, dim3(256), 0, s, a, b, out, m, n, k, ep);
}

// Few tiles over a long K: how many workgroups share a tile's K (1: none).  A 64 x 64 tile's workgroup (1024 threads,
// its four wavefront sets already dividing every 128-k step) streams 64 weight rows; with fewer such workgroups than
// compute units the launch is as long as one workgroup's walk through K (64 rows x 2048 x 2048: 32 workgroups, 23 us,
// for 4.7 MB of weights; 11 us as 8 x 32).  Shares of at least two steps; one workgroup per compute unit at most (a
// second round of workgroups costs what the shorter walk saves: 64 x 5632 x 2048 16.1 us with 176 workgroups, 18.7 with 352).
int q8_gemm_k_shares(int m, int n_rows, int k) {
    if (n_rows & 1) return 1;
    if (use_big_tile(m, n_rows)) return 1;
    const int64_t tiles = (int64_t)((n_rows + BN - 1) / BN) * ((m + BM - 1) / BM);
    const int steps = (q8_padded_k(k) + kQ8Group * kGroupsFew - 1) / (kQ8Group * kGroupsFew);
    if (tiles > 128 || steps < 4) return 1;
    int shares = (int)std::min<int64_t>(std::min<int64_t>(8, 256 / tiles), steps / 2);
    if (shares < 2) return 1;
    const int per = (steps + shares - 1) / shares;
    return (steps + per - 1) / per;
}

int64_t q8_gemm_workspace_floats(int m, int n_rows, int k) {
    const int shares = q8_gemm_k_shares(m, n_rows, k);
    return shares > 1 ? (int64_t)shares * m * n_rows : 0;
}

// Q8 GEMM used by launch_q8_linear for M > 1.  n_rows is the number of Q8 rows
// (= output columns of this launch; 2N for an interleaved gate/up weight).  workspace: room for the partial products
// of a K-sharing launch (q8_gemm_workspace_floats), or less - then no K is shared.
void launch_q8_gemm(hipStream_t s, const float *x, const int8_t *wq, const float *scales, float *out, int m,
                    int k, int n_rows, const float *bias, const float *bias2, const float *residual,
                    int interleaved_bias, const int32_t *m_dev, int m_extra, int gelu, int swiglu, float *workspace,
                    int64_t workspace_floats) {
    if (m <= 0 || n_rows <= 0) return;
    if (swiglu && ((n_rows & 1) || residual || gelu)) fail("q8_gemm: the SwiGLU epilogue needs an even row count and takes no residual or GELU");
    GemmEpilogue ep{bias, bias2, residual, interleaved_bias, m_dev, m_extra, gelu, swiglu};
    if (!m_dev && use_big_tile(m, n_rows)) {       // a device-side row count is usually far below m: keep small tiles
        dim3 grid2((n_rows + BN2 - 1) / BN2, (m + BM2 - 1) / BM2);
        // Two 128 x 128 workgroups fit a CU, so the tiles run in rounds of 512; when the last round would be mostly
        // empty (352 or 704 tiles), 64 x 128 tiles - twice as many, three to four per CU - finish sooner
        // (512 x 11264 x 2048: 101 against 113 us; 1024 rows: 194 against 229 us).
        const int64_t tiles = (int64_t)grid2.x * grid2.y, rounds = (tiles + 511) / 512;
        if (tiles * 100 < rounds * 512 * 85) {
            dim3 gridw(grid2.x, (m + 63) / 64);
            launch_kernel((k_gemm_q8<1, 2, 2, 1>), gridw, dim3(256), 0, s, x, wq, scales, out, m, n_rows, k, q8_padded_k(k), ep, 0, nullptr);
            return;
        }
        launch_kernel((k_gemm_q8<2, 2, kGroupsBig, kSetsBig>), grid2, dim3(256 * kSetsBig), 0, s, x, wq, scales, out, m, n_rows, k, q8_padded_k(k), ep, 0, nullptr);
        return;
    }
    dim3 grid((n_rows + BN - 1) / BN, (m + BM - 1) / BM);
    const int shares = m_dev ? 1 : q8_gemm_k_shares(m, n_rows, k);
    if (shares > 1 && workspace && workspace_floats >= (int64_t)shares * m * n_rows) {
        constexpr int step = kQ8Group * kGroupsFew;
        const int steps = (q8_padded_k(k) + step - 1) / step, per = (steps + shares - 1) / shares;
        grid.z = shares;
        launch_kernel((k_gemm_q8<1, 1, kGroupsFew, kSetsFew>), grid, dim3(256 * kSetsFew), 0, s, x, wq, scales, out, m, n_rows, k, q8_padded_k(k), ep,
                      per * step, workspace);
        const int64_t pairs = (int64_t)m * (n_rows / 2);
        launch_kernel(k_sum_partials_q8, dim3((unsigned)std::min<int64_t>((pairs + 255) / 256, 4096)), dim3(256), 0, s, (const float *)workspace, out,
                      shares, m, n_rows, ep);
        return;
    }
    // few tiles (about one per CU): a workgroup brings its own second wavefront per SIMD
    if ((int64_t)grid.x * grid.y <= kFewTiles)
        launch_kernel((k_gemm_q8<1, 1, kGroupsFew, kSetsFew>), grid, dim3(256 * kSetsFew), 0, s, x, wq, scales, out, m, n_rows, k, q8_padded_k(k), ep, 0, nullptr);
    else
        launch_kernel((k_gemm_q8<1, 1, kGroupsSmall, 1>), grid, dim3(256), 0, s, x, wq, scales, out, m, n_rows, k, q8_padded_k(k), ep, 0, nullptr);
}

}  // namespace dj
