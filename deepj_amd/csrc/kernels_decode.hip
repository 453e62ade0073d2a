// Persistent greedy-decode kernel for the Llama block stack (batch 1, KV cache, Q8 weights).
//
// One launch runs `steps` whole tokens: every transformer block, the LM head, the arg-max and
// the embedding lookup of the chosen token (LlamaTransformerBlock.java:50-53,
// DecoderOnlyModel.java:58-64, TextGenerator.java:91-114 with topK = 1).  The grid is one
// workgroup of 512 threads per CU, all resident at once; the phases of a token
//     qkv = Wqkv.norm1(x) | attention | x2 = x + Wo.att | ff = SwiGLU(norm2(x2)) | x = x2 + Wd.ff
// are separated by grid-wide barriers (two-level arrival counters, bounded spinning) instead of
// kernel boundaries.
//
// Why: at batch 1 every matrix-vector product is a few microseconds of HBM streaming behind a
// few microseconds of launch, first-miss and drain latency.  Here a wavefront issues the loads of
// the Q8 rows it owns of the NEXT phase's matrix right after signalling the barrier that ends
// the current phase: the HBM stream runs while the workgroup waits for the other workgroups.
//
// Activations written in one phase are read by other workgroups in the next: they are written
// and read with agent-scope (device-coherent) accesses, and a workgroup waits for its stores
// to complete before it signals the barrier; weights, tables and KV rows of earlier positions
// use ordinary loads.  Plain HIP throughout: no inline assembly.
#include <cstdio>
#include <cstdlib>

#include "dj_common.h"
#include "dj_device.h"

namespace dj {
namespace {
using namespace dev;

constexpr int kDT = 512;                  // threads per workgroup
constexpr int kDW = kDT / 64;             // wavefronts per workgroup
constexpr unsigned kSpinLimit = 1u << 20;

// words of the sync buffer (uint32 index); every counter sits on its own 256-byte line
constexpr int SY_TOP = 0, SY_FAILED = 64, SY_EPOCH = 128, SY_GRP = 192, SY_REL = SY_GRP + 8 * 64,
              SY_HEAD = SY_REL + 8 * 64;
constexpr int kHeadStride = 16;
constexpr int kMaxHeads = 256;

// ── device-coherent accesses ────────────────────────────────────────────────
__device__ __forceinline__ unsigned ldc_u32(const unsigned *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void stc_u32(unsigned *p, unsigned v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ unsigned addc_u32(unsigned *p, unsigned v) { return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float ldc_f32(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void stc_f32(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float2 ldc_f2(const float *p) {
    unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__builtin_bit_cast(float, (unsigned)(v & 0xffffffffull)), __builtin_bit_cast(float, (unsigned)(v >> 32)));
}
// all of this wavefront's vector-memory operations (its stores in particular) have completed
__device__ __forceinline__ void wait_stores() { __builtin_amdgcn_s_waitcnt(0x0f70); }     // vmcnt(0)

__device__ __forceinline__ float d_sigmoid(float x) { return 1.0f / (1.0f + (float)exp((double)(-x))); }

// Float.compare order, ties to the lower index (TextGenerator.java:163-170)
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
    bool vn = v != v, bn = bv != bv;
    if (vn != bn) return vn;
    if (!vn && v != bv) return v > bv;
    return i < bi;
}

// ── Q8 rows in registers ────────────────────────────────────────────────────
// R rows x NC chunks of 16 int8 per lane (one 1 KiB stripe of a row per chunk) with their scales.
// One register store serves every matrix in turn: slot u * NC + c holds chunk c of row u.
constexpr int kSlots = 12;
struct Store {
    int4 w[kSlots];
    float sc[kSlots];
};

// outputs [ob, oe) of a matrix with n_out outputs that workgroup wg owns
__device__ __forceinline__ void wg_outputs(int n_out, int wg, int G, int &ob, int &oe) {
    ob = (int)(((long long)n_out * wg) / G);
    oe = (int)(((long long)n_out * (wg + 1)) / G);
}

// Loads rows row0 .. row0+R-1 of m (clamped to row_last); chunks past Kp read chunk 0 (their
// activations are zero), so no load sits under a branch.
template <int NC, int R>
__device__ __forceinline__ void load_batch(Store &b, const Q8Mat &m, int row0, int row_last, int lane) {
    static_assert(NC * R <= kSlots, "batch does not fit the register store");
    const int groups = m.kp / kQ8Group;
#pragma unroll
    for (int u = 0; u < R; u++) {
        int row = row0 + u < row_last ? row0 + u : row_last;
        const int8_t *wrow = m.w + (long long)row * m.kp;
        const float *srow = m.sc + (long long)row * groups;
#pragma unroll
        for (int c = 0; c < NC; c++) {
            int chunk = c * 64 + lane;
            if (chunk * 16 >= m.kp) chunk = 0;
            b.w[u * NC + c] = *reinterpret_cast<const int4 *>(wrow + chunk * 16);
            b.sc[u * NC + c] = srow[chunk >> 1];
        }
    }
}

// How a phase finishes its outputs.
struct Epilogue {
    float *out; const float *bias, *bias2, *residual;
    bool residual_coherent;
};

// The rows of matrix m this wavefront owns: batches of B outputs (RPO rows each) dealt
// round-robin to the 8 wavefronts of the workgroup inside the workgroup's output range.
template <int NC, int B, bool PAIRS> struct Work {
    static constexpr int RPO = PAIRS ? 2 : 1;
    static constexpr int R = B * RPO;
    using Regs = Store;

    // first batch of this wavefront into `b` (no-op when it has none)
    static __device__ __forceinline__ void prefetch(Regs &b, const Q8Mat &m, int wg, int G, int wave, int lane) {
        int ob, oe;
        wg_outputs(m.rows / RPO, wg, G, ob, oe);
        int o0 = ob + wave * B;
        if (o0 < oe) load_batch<NC, R>(b, m, o0 * RPO, oe * RPO - 1, lane);
    }

    // `b` holds the first batch (prefetch above); xs = staged activation row in LDS.
    static __device__ __forceinline__ void run(Regs &b, const Q8Mat &m, const float *xs, const Epilogue &ep, int wg, int G,
                                               int wave, int lane, float &best_v, int &best_i) {
        int ob, oe;
        wg_outputs(m.rows / RPO, wg, G, ob, oe);
        const int step = kDW * B;
        for (int o0 = ob + wave * B; o0 < oe; o0 += step) {
            // The lane's 16 activations of each 1 KiB stripe come from LDS stripe by stripe, so only
            // one stripe's worth is live in registers next to the weight batches.
            // bias / residual of this batch's outputs: requested now, used after the reduction
            float pb[B], pb2[B], pr[B];
#pragma unroll
            for (int u = 0; u < B; u++) {
                const int o = o0 + u < oe ? o0 + u : oe - 1;
                pb[u] = ep.bias ? ep.bias[o] : 0.0f;
                pb2[u] = (PAIRS && ep.bias2) ? ep.bias2[o] : 0.0f;
                pr[u] = ep.residual ? (ep.residual_coherent ? ldc_f32(ep.residual + o) : ep.residual[o]) : 0.0f;
            }
            float acc[R];
#pragma unroll
            for (int u = 0; u < R; u++) acc[u] = 0.0f;
#pragma unroll
            for (int c = 0; c < NC; c++) {
                const int kb = (c * 64 + lane) * 16;
                const bool active = kb < m.kp;
                float xc[16];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    float4 v = active ? *reinterpret_cast<const float4 *>(xs + kb + 4 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
                    xc[4 * j] = v.x; xc[4 * j + 1] = v.y; xc[4 * j + 2] = v.z; xc[4 * j + 3] = v.w;
                }
#pragma unroll
                for (int u = 0; u < R; u++) acc[u] = fmaf(dot16(b.w[u * NC + c], xc), b.sc[u * NC + c], acc[u]);
                __builtin_amdgcn_sched_barrier(0);     // keep one stripe of activations live at a time
            }
#pragma unroll
            for (int u = 0; u < R; u++) acc[u] = wave_sum_dpp(acc[u]);
            if (o0 + step < oe) load_batch<NC, R>(b, m, (o0 + step) * RPO, oe * RPO - 1, lane);   // next batch streams in
            if (lane == 0) {
#pragma unroll
                for (int u = 0; u < B; u++) {
                    int o = o0 + u;
                    if (o < oe) {
                        float v;
                        if (PAIRS) {
                            float gate = acc[2 * u], up = acc[2 * u + 1];
                            if (ep.bias) gate = gate + pb[u];
                            if (ep.bias2) up = up + pb2[u];
                            float sg = gate * d_sigmoid(gate);      // SiLU.java:20-24
                            v = sg * up;                             // SwiGLULayer.java:69
                        } else {
                            v = acc[u];
                            if (ep.bias) v = v + pb[u];
                        }
                        if (ep.residual) v = pr[u] + v;
                        stc_f32(ep.out + o, v);
                        if (better(v, o, best_v, best_i)) { best_v = v; best_i = o; }
                    }
                }
            }
        }
    }
};

// ── per-workgroup state ─────────────────────────────────────────────────────
struct Ctx {
    int wg, G, tid, lane, wave;
    unsigned epoch;            // grid barriers passed so far (all launches)
    bool failed;
    unsigned *sync;
    int *s_flag;               // LDS: [0] barrier failure, [1] last-split flag
};

// ── grid barrier, in two halves so that loads can be issued in between ──────
__device__ __forceinline__ void grid_arrive(Ctx &c) {
    wait_stores();
    __syncthreads();                       // every wavefront's activation stores are complete
    c.epoch++;
    if (c.tid == 0 && !c.failed) {
        const unsigned g = c.wg & 7;
        const unsigned ngroups = c.G < 8 ? c.G : 8;
        const unsigned gsize = (c.G - g + 7) >> 3;
        unsigned old = addc_u32(c.sync + SY_GRP + g * 64, 1u);
        if (old + 1 == c.epoch * gsize) {
            unsigned o2 = addc_u32(c.sync + SY_TOP, 1u);
            if (o2 + 1 == c.epoch * ngroups)
                for (unsigned i = 0; i < ngroups; i++) stc_u32(c.sync + SY_REL + i * 64, c.epoch);
        }
    }
}
__device__ __forceinline__ void grid_wait(Ctx &c) {
    if (c.tid == 0 && !c.failed) {
        const unsigned *p = c.sync + SY_REL + (c.wg & 7) * 64;
        unsigned spins = 0;
        while ((int)(ldc_u32(p) - c.epoch) < 0) {
            if (++spins > kSpinLimit || ldc_u32(c.sync + SY_FAILED)) {
                stc_u32(c.sync + SY_FAILED, 1u);
                c.s_flag[0] = 1;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    __syncthreads();
    if (c.s_flag[0]) c.failed = true;
}

// ── activation staging ──────────────────────────────────────────────────────
// xs[0..kp) = optional RMSNorm of src[0..k) (RMSNorm1D.java:46-57), zero beyond k.  All 512
// threads; NCX = ceil(kp / 1024).
// This thread's share of a gain vector, requested ahead of the phase that uses it.
template <int NCX>
__device__ __forceinline__ void load_gain(float2 (&gv)[NCX], const float *gamma, int k, int tid) {
#pragma unroll
    for (int j = 0; j < NCX; j++) {
        int e = (tid + kDT * j) * 2;
        gv[j] = make_float2(0.f, 0.f);
        if (e + 1 < k) gv[j] = *reinterpret_cast<const float2 *>(gamma + e);
        else if (e < k) gv[j].x = gamma[e];
    }
}

// gv = null: no RMSNorm.
template <int NCX>
__device__ __forceinline__ void stage_x(const Ctx &c, const float *src, bool coherent, int k, int kp, const float2 *gv,
                                        float *xs, float *red) {
    float2 xv[NCX];
#pragma unroll
    for (int j = 0; j < NCX; j++) {
        int e = (c.tid + kDT * j) * 2;
        xv[j] = make_float2(0.f, 0.f);
        if (e + 1 < k) xv[j] = coherent ? ldc_f2(src + e) : *reinterpret_cast<const float2 *>(src + e);
        else if (e < k) xv[j].x = coherent ? ldc_f32(src + e) : src[e];
    }
    if (gv) {
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < NCX; j++) ss += xv[j].x * xv[j].x + xv[j].y * xv[j].y;
        ss = wave_sum_dpp(ss);
        if (c.lane == 0) red[c.wave] = ss;
        __syncthreads();
        float tot = 0.0f;
#pragma unroll
        for (int w = 0; w < kDW; w++) tot += red[w];
        float rms = sqrtf(tot * (1.0f / (float)k) + kRmsEps);
#pragma unroll
        for (int j = 0; j < NCX; j++) {
            xv[j].x = (xv[j].x / rms) * gv[j].x;
            xv[j].y = (xv[j].y / rms) * gv[j].y;
        }
    }
#pragma unroll
    for (int j = 0; j < NCX; j++) {
        int e = (c.tid + kDT * j) * 2;
        if (e < kp) *reinterpret_cast<float2 *>(xs + e) = xv[j];
    }
    __syncthreads();
}

// ── attention for one (head, split) item ────────────────────────────────────
// Rotates q and the new key (RotaryEmbedding.java:112-122), appends the new key/value row,
// runs the online softmax over this split's keys (HeadOps.java:90-140 for one query row) and
// leaves a partial record; the last split of a head to finish merges the head's records.
template <int LPK>
__device__ __forceinline__ void attention_item(Ctx &c, const DecodeParams &P, int layer, int pos, int h, int split,
                                               float *aux) {
    constexpr int HD = LPK * 4;
    constexpr int KPW = 64 / LPK;
    constexpr int NSUB = kDW * KPW;
    float *s_m = aux;
    float *s_l = s_m + NSUB;
    float *s_o = s_l + NSUB;                               // [NSUB][HD]
    const int sub = c.lane / LPK, dl = c.lane % LPK;
    const int d = P.d, half = HD / 2, ns = P.nsplit;

    const int n_keys = pos + 1;
    const int per = (n_keys + ns - 1) / ns;
    const int k_begin = split * per;
    const int k_end = k_begin + per < n_keys ? k_begin + per : n_keys;

    const float2 c2 = *reinterpret_cast<const float2 *>(P.cos_t + (long long)pos * half + dl * 2);
    const float2 s2 = *reinterpret_cast<const float2 *>(P.sin_t + (long long)pos * half + dl * 2);
    const float2 qa = ldc_f2(P.qkv + h * HD + dl * 4), qb = ldc_f2(P.qkv + h * HD + dl * 4 + 2);
    const float4 qv = make_float4(qa.x * c2.x - qa.y * s2.x, qa.x * s2.x + qa.y * c2.x,
                                  qb.x * c2.y - qb.y * s2.y, qb.x * s2.y + qb.y * c2.y);
    const long long head_off = ((long long)layer * P.H + h) * P.max_seq * HD + dl * 4;
    float *kb = P.kc + head_off, *vb = P.vc + head_off;

    float m = -INFINITY, l = 0.0f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
    for (int key = k_begin + c.wave * KPW + sub; key < k_end; key += kDW * KPW) {
        float4 kk, vv;
        if (key == pos) {
            const float2 ka = ldc_f2(P.qkv + d + h * HD + dl * 4), kc2 = ldc_f2(P.qkv + d + h * HD + dl * 4 + 2);
            kk = make_float4(ka.x * c2.x - ka.y * s2.x, ka.x * s2.x + ka.y * c2.x,
                             kc2.x * c2.y - kc2.y * s2.y, kc2.x * s2.y + kc2.y * c2.y);
            const float2 va = ldc_f2(P.qkv + 2 * d + h * HD + dl * 4), vb2 = ldc_f2(P.qkv + 2 * d + h * HD + dl * 4 + 2);
            vv = make_float4(va.x, va.y, vb2.x, vb2.y);
            // the appended row is read by later tokens, possibly from another CU in this same launch
            stc_f32(kb + (long long)key * HD, kk.x); stc_f32(kb + (long long)key * HD + 1, kk.y);
            stc_f32(kb + (long long)key * HD + 2, kk.z); stc_f32(kb + (long long)key * HD + 3, kk.w);
            stc_f32(vb + (long long)key * HD, vv.x); stc_f32(vb + (long long)key * HD + 1, vv.y);
            stc_f32(vb + (long long)key * HD + 2, vv.z); stc_f32(vb + (long long)key * HD + 3, vv.w);
        } else {
            kk = *reinterpret_cast<const float4 *>(kb + (long long)key * HD);
            vv = *reinterpret_cast<const float4 *>(vb + (long long)key * HD);
        }
        float s = qv.x * kk.x + qv.y * kk.y + qv.z * kk.z + qv.w * kk.w;
#pragma unroll
        for (int off = LPK / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
        s *= P.scale;
        float mn = fmaxf(m, s);
        float corr = expf(m - mn);
        float p = expf(s - mn);
        l = l * corr + p;
        o.x = o.x * corr + p * vv.x; o.y = o.y * corr + p * vv.y;
        o.z = o.z * corr + p * vv.z; o.w = o.w * corr + p * vv.w;
        m = mn;
    }
    const int slot = c.wave * KPW + sub;
    if (dl == 0) { s_m[slot] = m; s_l[slot] = l; }
    *reinterpret_cast<float4 *>(s_o + slot * HD + dl * 4) = o;
    __syncthreads();
    float *rec = P.scratch + ((long long)h * ns + split) * (HD + 4);
    if (c.tid < HD) {
        float M = -INFINITY, L = 0.0f, O = 0.0f;
#pragma unroll 4
        for (int i = 0; i < NSUB; i++) M = fmaxf(M, s_m[i]);
        if (M != -INFINITY) {
#pragma unroll 2
            for (int i = 0; i < NSUB; i++) {
                float w = expf(s_m[i] - M);
                L += s_l[i] * w;
                O += s_o[i * HD + c.tid] * w;
            }
        }
        stc_f32(rec + 4 + c.tid, O);
        if (c.tid == 0) { stc_f32(rec, M); stc_f32(rec + 1, L); }
    }
    // this workgroup's stores (record, appended row) are complete before it counts itself in
    wait_stores();
    __syncthreads();
    if (c.tid == 0) {
        unsigned old = addc_u32(c.sync + SY_HEAD + h * kHeadStride, 1u);
        c.s_flag[1] = ((old + 1) % (unsigned)ns) == 0;
    }
    __syncthreads();
    if (c.s_flag[1] && c.tid < HD) {
        // all record loads are issued before the first use: one memory round trip (ns <= 16)
        const float *base = P.scratch + (long long)h * ns * (HD + 4);
        float rm[16], rl[16], ro[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float *r = base + (long long)(i < ns ? i : 0) * (HD + 4);
            rm[i] = ldc_f32(r); rl[i] = ldc_f32(r + 1); ro[i] = ldc_f32(r + 4 + c.tid);
        }
        float M = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) if (i < ns) M = fmaxf(M, rm[i]);
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (i < ns && rm[i] != -INFINITY) {
                float w = expf(rm[i] - M);
                L += rl[i] * w;
                O += ro[i] * w;
            }
        }
        stc_f32(P.att + h * HD + c.tid, O / L);
    }
    __syncthreads();                                       // aux is reused by the next item
}

__device__ __attribute__((noinline)) void attention_phase(Ctx &c, const DecodeParams &P, int layer, int pos, float *aux) {
    const int items = P.H * P.nsplit;
    for (int it = c.wg; it < items; it += c.G) {
        const int h = it / P.nsplit, split = it % P.nsplit;
        switch (P.hd) {
            case 32: attention_item<8>(c, P, layer, pos, h, split, aux); break;
            case 64: attention_item<16>(c, P, layer, pos, h, split, aux); break;
            default: attention_item<32>(c, P, layer, pos, h, split, aux); break;
        }
    }
}

// ── the kernel ──────────────────────────────────────────────────────────────
// ND = ceil(Kp(dModel) / 1024), NF = ceil(Kp(dFF) / 1024).  Rows a wavefront holds per matrix
// (sized for 256 workgroups; more rows than that simply take more than one batch):
template <int ND, int NF>
__global__ void __launch_bounds__(kDT) k_llama_decode(DecodeParams P) {
    constexpr int NX = ND > NF ? ND : NF;
    constexpr int B_QKV = (3 * ND + 1) / 2, B_WO = (ND + 1) / 2, B_GU = (NF + 1) / 2, B_DOWN = (ND + 1) / 2, B_LM = 4;
    static_assert(ND * B_QKV <= kSlots && ND * B_GU * 2 <= kSlots && NF * B_DOWN <= kSlots && ND * B_LM <= kSlots, "register store too small");
    using WQkv = Work<ND, B_QKV, false>;
    using WWo = Work<ND, B_WO, false>;
    using WGu = Work<ND, B_GU, true>;
    using WDown = Work<NF, B_DOWN, false>;
    using WLm = Work<ND, B_LM, false>;

    __shared__ __align__(16) float xs[NX * 1024];
    __shared__ __align__(16) float aux[2304];              // attention merge area: 2*NSUB + NSUB*HD floats <= 2176
    __shared__ float red[kDW];
    __shared__ int s_flag[2];
    __shared__ float sv[kDW];
    __shared__ int si[kDW];

    Ctx c;
    c.wg = blockIdx.x; c.G = gridDim.x; c.tid = threadIdx.x; c.lane = c.tid & 63; c.wave = c.tid >> 6;
    c.sync = P.sync;
    c.epoch = P.sync[SY_EPOCH];
    c.failed = false;
    c.s_flag = s_flag;
    if (c.tid == 0) { s_flag[0] = 0; s_flag[1] = 0; }
    __syncthreads();

    Store r;                                               // the next phase's rows of this wavefront
    float2 gain[ND];                                       // the next normalising phase's gain, this thread's share
    load_gain<ND>(gain, P.layers[0].g1, P.d, c.tid);
    WQkv::prefetch(r, P.layers[0].qkv, c.wg, c.G, c.wave, c.lane);

    const int pos0 = P.state[0], gen0 = P.state[2];
    int tok = P.state[1];
    float nb_v = -INFINITY; int nb_i = 0x7fffffff;         // unused arg-max trackers of the block phases
    int tix = 0;
#define DJ_STAMP() do { if (P.timing && c.wg == 0 && c.tid == 0 && step == P.steps - 1 && l == 1 && tix < 60) P.timing[tix++] = wall_clock64(); } while (0)
    for (int step = 0; step < P.steps && !c.failed; step++) {
        const int pos = pos0 + step < P.max_seq ? pos0 + step : P.max_seq - 1;
        const bool tok_ok = tok >= 0 && tok < P.vocab;
        const float *emb_row = P.emb + (long long)(tok_ok ? tok : 0) * P.d;
        for (int l = 0; l < P.L && !c.failed; l++) {
            const DecodeLayer &L = P.layers[l];
            const bool last = l + 1 == P.L;
            const float *xin = l == 0 ? emb_row : P.x;

            // qkv = norm1(x) . [Wq|Wk|Wv]
            stage_x<ND>(c, xin, l != 0, P.d, L.qkv.kp, gain, xs, red); DJ_STAMP();
            WQkv::run(r, L.qkv, xs, Epilogue{P.qkv, nullptr, nullptr, nullptr, false}, c.wg, c.G, c.wave, c.lane, nb_v, nb_i); DJ_STAMP();
            grid_arrive(c); DJ_STAMP();
            WWo::prefetch(r, L.wo, c.wg, c.G, c.wave, c.lane);          // streams in during the barrier and the attention
            load_gain<ND>(gain, L.g2, P.d, c.tid);
            grid_wait(c); DJ_STAMP();

            attention_phase(c, P, l, pos, aux); DJ_STAMP();
            grid_arrive(c); DJ_STAMP();
            grid_wait(c); DJ_STAMP();

            // x2 = x + att . Wo                                              LlamaTransformerBlock.java:51
            stage_x<ND>(c, P.att, true, P.d, L.wo.kp, nullptr, xs, red); DJ_STAMP();
            WWo::run(r, L.wo, xs, Epilogue{P.x2, nullptr, nullptr, xin, l != 0}, c.wg, c.G, c.wave, c.lane, nb_v, nb_i); DJ_STAMP();
            grid_arrive(c); DJ_STAMP();
            WGu::prefetch(r, L.gu, c.wg, c.G, c.wave, c.lane);
            grid_wait(c); DJ_STAMP();

            // ff = SiLU(gate(norm2(x2))) * up(norm2(x2))
            stage_x<ND>(c, P.x2, true, P.d, L.gu.kp, gain, xs, red); DJ_STAMP();
            WGu::run(r, L.gu, xs, Epilogue{P.ff, L.bg, L.bu, nullptr, false}, c.wg, c.G, c.wave, c.lane, nb_v, nb_i); DJ_STAMP();
            grid_arrive(c); DJ_STAMP();
            WDown::prefetch(r, L.down, c.wg, c.G, c.wave, c.lane);
            grid_wait(c); DJ_STAMP();

            // x = x2 + down(ff)                                              LlamaTransformerBlock.java:52
            stage_x<NF>(c, P.ff, true, P.dff, L.down.kp, nullptr, xs, red); DJ_STAMP();
            WDown::run(r, L.down, xs, Epilogue{P.x, L.bd, nullptr, P.x2, true}, c.wg, c.G, c.wave, c.lane, nb_v, nb_i); DJ_STAMP();
            grid_arrive(c); DJ_STAMP();
            if (last) { WLm::prefetch(r, P.lm, c.wg, c.G, c.wave, c.lane); load_gain<ND>(gain, P.gf, P.d, c.tid); }
            else { WQkv::prefetch(r, P.layers[l + 1].qkv, c.wg, c.G, c.wave, c.lane); load_gain<ND>(gain, P.layers[l + 1].g1, P.d, c.tid); }
            grid_wait(c); DJ_STAMP();
        }
        if (c.failed) break;
        // logits = norm(x) . Wlm + blm, arg-max of this workgroup's rows       DecoderOnlyModel.java:58-64
        float bv = -INFINITY; int bi = 0x7fffffff;
        stage_x<ND>(c, P.x, true, P.d, P.lm.kp, gain, xs, red);
        WLm::run(r, P.lm, xs, Epilogue{P.logits, P.blm, nullptr, nullptr, false}, c.wg, c.G, c.wave, c.lane, bv, bi);
        bv = __shfl(bv, 0, 64); bi = __shfl(bi, 0, 64);    // lane 0 tracked the wavefront's rows
        if (c.lane == 0) { sv[c.wave] = bv; si[c.wave] = bi; }
        __syncthreads();
        if (c.tid == 0) {
            for (int w = 1; w < kDW; w++)
                if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
            stc_f32(P.argbuf + 2 * c.wg, bv);
            stc_u32(reinterpret_cast<unsigned *>(P.argbuf) + 2 * c.wg + 1, (unsigned)bi);
        }
        grid_arrive(c);
        if (step + 1 < P.steps) {                          // next token's first rows
            WQkv::prefetch(r, P.layers[0].qkv, c.wg, c.G, c.wave, c.lane);
            load_gain<ND>(gain, P.layers[0].g1, P.d, c.tid);
        }
        grid_wait(c);
        if (c.failed) break;
        // every workgroup reduces the per-workgroup winners to the same token
        bv = -INFINITY; bi = 0x7fffffff;
        if (c.tid < c.G) {
            bv = ldc_f32(P.argbuf + 2 * c.tid);
            bi = (int)ldc_u32(reinterpret_cast<const unsigned *>(P.argbuf) + 2 * c.tid + 1);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            float ov = __shfl_xor(bv, off, 64);
            int oi = __shfl_xor(bi, off, 64);
            if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
        }
        if (c.lane == 0) { sv[c.wave] = bv; si[c.wave] = bi; }
        __syncthreads();
        bv = sv[0]; bi = si[0];
        for (int w = 1; w < kDW; w++)
            if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
        tok = bi;
        __syncthreads();
        if (c.wg == 0 && c.tid == 0 && gen0 + step < P.capacity) P.tokens[gen0 + step] = tok;
    }
    // Leave x = embedding row of the token to process next, as the per-token stream does
    // (Embedding.java:28-34), so the two decode paths can be mixed within a sequence.
    if (c.wg == 0 && !c.failed) {
        const bool ok = tok >= 0 && tok < P.vocab;
        const float *src = P.emb + (long long)(ok ? tok : 0) * P.d;
        for (int i = c.tid; i < P.d; i += kDT) P.x[i] = ok ? src[i] : __builtin_nanf("");
    }
    if (c.wg == 0 && c.tid == 0) {
        P.state[0] = pos0 + P.steps;
        P.state[1] = tok;
        P.state[2] = gen0 + P.steps;
        P.state[3] = (c.failed || ldc_u32(P.sync + SY_FAILED)) ? 1 : 0;
        P.sync[SY_EPOCH] = c.epoch;
    }
}

}  // namespace

// ── host side ───────────────────────────────────────────────────────────────
int64_t llama_decode_sync_words() { return SY_HEAD + kMaxHeads * kHeadStride; }

static int decode_grid() {
    static int cus = [] {
        int dev = 0, n = 0;
        DJ_HIP(hipGetDevice(&dev));
        DJ_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
        return n;
    }();
    return cus < 256 ? cus : 256;
}

void llama_decode_plan(int H, int hd, int *grid, int *nsplit, int64_t *scratch_floats, int64_t *argbuf_floats) {
    int g = decode_grid();
    int ns = g / (H > 0 ? H : 1);
    if (ns < 1) ns = 1;
    if (ns > 16) ns = 16;
    if (grid) *grid = g;
    if (nsplit) *nsplit = ns;
    if (scratch_floats) *scratch_floats = (int64_t)H * ns * (hd + 4);
    if (argbuf_floats) *argbuf_floats = 2 * (int64_t)g;
}

bool llama_decode_supported(int d, int dff) {
    int nd = (q8_padded_k(d) + 1023) / 1024, nf = (q8_padded_k(dff) + 1023) / 1024;
    return (nd == 1 && nf == 1) || (nd <= 2 && nf <= 6);
}

// The caller has filled every pointer and dimension; this derives the launch geometry.
void launch_llama_decode(hipStream_t s, DecodeParams &p) {
    if (p.hd != 32 && p.hd != 64 && p.hd != 128) fail("llama_decode: head dim must be 32, 64 or 128");
    if (p.H < 1 || p.H > kMaxHeads || p.H * p.hd != p.d) fail("llama_decode: bad head count");
    if (!llama_decode_supported(p.d, p.dff)) fail("llama_decode: dModel above 2048 or dFF above 6144 is not supported");
    if (p.steps <= 0) return;
    int grid = 0, ns = 0;
    llama_decode_plan(p.H, p.hd, &grid, &ns, nullptr, nullptr);
    p.nsplit = ns;
    p.scale = (float)(1.0 / sqrt((double)p.hd));
    p.slot_count = 0; p.xs_bytes = 0;
    static unsigned long long *timing = nullptr;
    const bool want_timing = getenv("DJ_DECODE_TIMING") != nullptr;
    if (want_timing && !timing) { DJ_HIP(hipMalloc((void **)&timing, 64 * 8)); }
    if (want_timing) DJ_HIP(hipMemsetAsync(timing, 0, 64 * 8, s));
    p.timing = want_timing ? timing : nullptr;
    int nd = (q8_padded_k(p.d) + 1023) / 1024, nf = (q8_padded_k(p.dff) + 1023) / 1024;
    if (nd == 1 && nf == 1) hipLaunchKernelGGL((k_llama_decode<1, 1>), dim3(grid), dim3(kDT), 0, s, p);
    else hipLaunchKernelGGL((k_llama_decode<2, 6>), dim3(grid), dim3(kDT), 0, s, p);
    if (want_timing) {
        unsigned long long h[64];
        DJ_HIP(hipStreamSynchronize(s));
        DJ_HIP(hipMemcpy(h, timing, sizeof(h), hipMemcpyDeviceToHost));
        fprintf(stderr, "decode phase stamps (us since first):");
        for (int i = 0; i < 64 && h[i]; i++) fprintf(stderr, " %.2f", (double)(h[i] - h[0]) / 100.0);
        fprintf(stderr, "\n");
    }
}

}  // namespace dj
