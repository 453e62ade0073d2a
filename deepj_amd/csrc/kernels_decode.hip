// Persistent greedy-decode kernel for the Llama block stack (batch 1, KV cache, Q8 weights).
//
// One launch runs `steps` whole tokens: every transformer block, the LM head, the arg-max
// and the embedding lookup of the chosen token (LlamaTransformerBlock.java:50-53,
// DecoderOnlyModel.java:58-64, TextGenerator.java:91-114 with topK = 1).  The grid is one
// workgroup per CU, all resident at once; the phases of a token
//     qkv = Wqkv.norm1(x) | attention | x2 = x + Wo.att | ff = SwiGLU(norm2(x2)) | x = x2 + Wd.ff
// are separated by grid-wide barriers (two-level arrival counters, bounded spinning) instead
// of kernel boundaries.
//
// Why: at batch 1 every matrix-vector product is a few microseconds of HBM streaming behind a
// few microseconds of launch, first-miss and drain latency.  Here the Q8 rows a workgroup will
// need next are already on their way into LDS (asynchronous global->LDS loads, four ring slots)
// while it finishes the current phase and waits at the barrier, so the HBM stream does not stop
// at phase boundaries.
//
// Division of labour inside a workgroup (8 wavefronts): wavefronts 0-6 issue the weight
// prefetches; all 8 multiply rows out of LDS; wavefront 7 alone touches activations in global
// memory (loads x, applies RMSNorm, stages it in LDS; adds bias/residual/SwiGLU and stores the
// outputs).  Its vector-memory counter therefore never contains a prefetch, and the prefetching
// wavefronts never wait for anything but the chunk they are about to read.
//
// Activations written in one phase are read by other workgroups in the next: they are written
// and read with agent-scope (device-coherent) accesses; weights, tables and KV rows of earlier
// positions use ordinary loads.
#include "dj_common.h"

namespace dj {
namespace {

constexpr int kDT = 512;                  // threads per workgroup
constexpr int kDW = kDT / 64;             // wavefronts per workgroup
constexpr int kIssuers = kDW - 1;         // wavefronts 0..6 issue weight prefetches
constexpr unsigned kSlotBytes = 32768;    // one ring slot (14 rows of K = 2048 with their scales)
constexpr unsigned kAuxBytes = 10240;     // attention merge area / output staging
constexpr unsigned kLdsLimit = 160 * 1024;
constexpr unsigned kSpinLimit = 1u << 20;
constexpr int kMaxSlots = 4;

// words of the sync buffer (uint32 index); every counter sits on its own 256-byte line
constexpr int SY_TOP = 0, SY_FAILED = 64, SY_EPOCH = 128, SY_GRP = 192, SY_REL = SY_GRP + 8 * 64,
              SY_HEAD = SY_REL + 8 * 64;
constexpr int kHeadStride = 16;
constexpr int kMaxHeads = 256;
constexpr int kMaxChunkRows = 112;        // staged sums per chunk (two buffers of 128 floats in aux)

using Mat = Q8Mat;
using DecLayer = DecodeLayer;


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
__device__ __forceinline__ void stc_f2(float *p, float2 v) {
    unsigned long long u = (unsigned long long)__builtin_bit_cast(unsigned, v.x) | ((unsigned long long)__builtin_bit_cast(unsigned, v.y) << 32);
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 16 bytes per lane from global memory straight into LDS at lds_off + lane * 16 (lds_off wave-uniform).
__device__ __forceinline__ void dma16(const void *g, unsigned lds_off) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_off) : "memory", "m0");
}

// wait until at most n of this wavefront's vector-memory operations are outstanding
__device__ __forceinline__ void wait_vm(unsigned n) {
    switch (n) {
#define DJ_W(i) case i: asm volatile("s_waitcnt vmcnt(" #i ")" ::: "memory"); break;
        DJ_W(1) DJ_W(2) DJ_W(3) DJ_W(4) DJ_W(5) DJ_W(6) DJ_W(7) DJ_W(8) DJ_W(9) DJ_W(10) DJ_W(11) DJ_W(12)
        DJ_W(13) DJ_W(14) DJ_W(15) DJ_W(16) DJ_W(17) DJ_W(18) DJ_W(19) DJ_W(20) DJ_W(21) DJ_W(22) DJ_W(23) DJ_W(24)
#undef DJ_W
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
}

// workgroup barrier that leaves vector-memory operations (the prefetches) in flight
__device__ __forceinline__ void wg_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

__device__ __forceinline__ float d_sigmoid(float x) { return 1.0f / (1.0f + (float)exp((double)(-x))); }

__device__ __forceinline__ float wave_sum_dpp(float v) {
#define DJ_DPP_ADD(ctrl, row_mask) \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, row_mask, 0xf, false))
    DJ_DPP_ADD(0xB1, 0xf);
    DJ_DPP_ADD(0x4E, 0xf);
    DJ_DPP_ADD(0x141, 0xf);
    DJ_DPP_ADD(0x140, 0xf);
    DJ_DPP_ADD(0x142, 0xa);
    DJ_DPP_ADD(0x143, 0xc);
#undef DJ_DPP_ADD
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float dot16(const int4 &w, const float *xr) {
    float d = 0.0f;
    const int words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int v = words[i];
        d = fmaf(xr[4 * i + 0], (float)(int8_t)(v & 0xff), d);
        d = fmaf(xr[4 * i + 1], (float)(int8_t)((v >> 8) & 0xff), d);
        d = fmaf(xr[4 * i + 2], (float)(int8_t)((v >> 16) & 0xff), d);
        d = fmaf(xr[4 * i + 3], (float)(v >> 24), d);
    }
    return d;
}

// Float.compare order, ties to the lower index (TextGenerator.java:163-170)
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
    bool vn = v != v, bn = bv != bv;
    if (vn != bn) return vn;
    if (!vn && v != bv) return v > bv;
    return i < bi;
}

// ── per-workgroup view of the kernel ────────────────────────────────────────
struct Ctx {
    const DecodeParams &P;
    unsigned char *lds;        // dynamic LDS
    unsigned lds_base;         // its LDS byte address (for M0)
    float *xs;                 // staged activation row [kp]
    unsigned char *aux;
    int wg, G, tid, lane, wave;
    unsigned epoch;            // grid barriers passed so far (all launches)
    bool failed;
};

// rows of a matrix owned by workgroup wg, in units of `unit` rows
__device__ __forceinline__ void wg_rows(const Mat &m, int unit, int wg, int G, int &r0, int &r1) {
    int units = m.rows / unit;
    r0 = (int)(((long long)units * wg) / G) * unit;
    r1 = (int)(((long long)units * (wg + 1)) / G) * unit;
}
// rows per ring slot: as many as fit, a multiple of `unit`
__device__ __forceinline__ int rows_per_chunk(const Mat &m, int unit) {
    int r = (int)(kSlotBytes / (unsigned)(m.kp + m.kp / 8));
    if (r > kMaxChunkRows) r = kMaxChunkRows;
    r -= r % unit;
    return r < unit ? unit : r;
}

// ── weight prefetch ring ────────────────────────────────────────────────────
// The chunk sequence of a workgroup is a pure function of (step, layer, matrix, row), so the
// prefetching side and the consuming side each walk it with their own cursor.
struct Cursor { int step, layer, kind, row; };     // kind 0 qkv, 1 wo, 2 gate/up, 3 down, 4 LM head; row < 0: not entered

__device__ __forceinline__ const Mat &mat_of(const DecodeParams &P, int layer, int kind) {
    if (kind == 4) return P.lm;
    const DecLayer &L = P.layers[layer];
    return kind == 0 ? L.qkv : (kind == 1 ? L.wo : (kind == 2 ? L.gu : L.down));
}

struct Pipe {
    Cursor cur;
    unsigned issued, consumed;
    unsigned nload0, nload1, nload2, nload3;    // prefetch loads this wavefront issued for the chunk in each slot

    __device__ __forceinline__ unsigned get_nload(unsigned s) const { return s == 0 ? nload0 : (s == 1 ? nload1 : (s == 2 ? nload2 : nload3)); }
    __device__ __forceinline__ void set_nload(unsigned s, unsigned v) {
        if (s == 0) nload0 = v; else if (s == 1) nload1 = v; else if (s == 2) nload2 = v; else nload3 = v;
    }

    // next chunk of the sequence; false when all steps are done
    __device__ __forceinline__ bool next(const Ctx &c, const int8_t *&w, const float *&sc, int &rows, int &kp) {
        const DecodeParams &P = c.P;
        while (cur.step < P.steps) {
            const Mat &m = mat_of(P, cur.layer, cur.kind);
            const int unit = cur.kind == 2 ? 2 : 1;
            int r0, r1;
            wg_rows(m, unit, c.wg, c.G, r0, r1);
            if (cur.row < 0) cur.row = r0;
            if (cur.row < r1) {
                int rpc = rows_per_chunk(m, unit);
                rows = r1 - cur.row < rpc ? r1 - cur.row : rpc;
                kp = m.kp;
                w = m.w + (long long)cur.row * m.kp;
                sc = m.sc + (long long)cur.row * (m.kp / kQ8Group);
                cur.row += rows;
                return true;
            }
            cur.row = -1;
            if (cur.kind == 4) { cur.kind = 0; cur.layer = 0; cur.step++; }
            else if (cur.kind == 3) {
                if (cur.layer + 1 < P.L) { cur.layer++; cur.kind = 0; }
                else cur.kind = 4;
            } else cur.kind++;
        }
        return false;
    }

    __device__ __forceinline__ void top_up(const Ctx &c) {
        const unsigned slots = c.P.slot_count;
        while (issued - consumed < slots) {
            const int8_t *w; const float *sc; int rows, kp;
            if (!next(c, w, sc, rows, kp)) break;
            const unsigned slot = issued % slots;
            const unsigned base = c.lds_base + slot * kSlotBytes;
            unsigned n = 0;
            if (c.wave < kIssuers) {
                const unsigned wbytes = (unsigned)rows * (unsigned)kp;
                const unsigned sbytes = (unsigned)rows * (unsigned)(kp / kQ8Group) * 4u;
                for (unsigned p = c.wave; p * 1024u < wbytes; p += kIssuers) {
                    unsigned off = p * 1024u + c.lane * 16u;
                    if (off < wbytes) dma16(reinterpret_cast<const unsigned char *>(w) + off, __builtin_amdgcn_readfirstlane(base + p * 1024u));
                    n++;
                }
                for (unsigned p = c.wave; p * 1024u < sbytes; p += kIssuers) {
                    unsigned off = p * 1024u + c.lane * 16u;
                    if (off < sbytes) dma16(reinterpret_cast<const unsigned char *>(sc) + off, __builtin_amdgcn_readfirstlane(base + wbytes + p * 1024u));
                    n++;
                }
            }
            set_nload(slot, n);
            issued++;
        }
    }

    // LDS byte offset of the oldest chunk once all of it has landed
    __device__ __forceinline__ unsigned acquire(const Ctx &c) {
        const unsigned slots = c.P.slot_count;
        unsigned younger = 0;
        for (unsigned i = consumed + 1; i < issued; i++) younger += get_nload(i % slots);
        if (c.wave < kIssuers) wait_vm(younger);
        wg_sync();
        return (consumed % slots) * kSlotBytes;
    }
    // every wavefront has finished reading the oldest chunk (callers sync before this)
    __device__ __forceinline__ void release(const Ctx &c) {
        consumed++;
        top_up(c);
    }
};

// ── grid barrier ────────────────────────────────────────────────────────────
__device__ __forceinline__ bool spin_until(Ctx &c, const unsigned *p, unsigned target) {
    unsigned spins = 0;
    while ((int)(ldc_u32(p) - target) < 0) {
        if (++spins > kSpinLimit || ldc_u32(c.P.sync + SY_FAILED)) {
            stc_u32(c.P.sync + SY_FAILED, 1u);
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    return true;
}

// Called by all threads.  Wavefront 7 has no prefetch in flight, so its vmcnt(0) only covers
// the activation stores of this phase.
__device__ __forceinline__ void grid_sync(Ctx &c) {
    c.epoch++;
    if (c.wave == kDW - 1) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (c.lane == 0 && !c.failed) {
            unsigned *sy = c.P.sync;
            const unsigned g = c.wg & 7;
            const unsigned ngroups = c.G < 8 ? c.G : 8;
            const unsigned gsize = (c.G - g + 7) >> 3;
            unsigned old = addc_u32(sy + SY_GRP + g * 64, 1u);
            if (old + 1 == c.epoch * gsize) {
                unsigned o2 = addc_u32(sy + SY_TOP, 1u);
                if (o2 + 1 == c.epoch * ngroups)
                    for (unsigned i = 0; i < ngroups; i++) stc_u32(sy + SY_REL + i * 64, c.epoch);
            }
            if (!spin_until(c, sy + SY_REL + g * 64, c.epoch)) *reinterpret_cast<volatile int *>(c.aux + kAuxBytes - 4) = 1;
        }
    }
    wg_sync();
    if (*reinterpret_cast<volatile int *>(c.aux + kAuxBytes - 4)) c.failed = true;
}

// ── activation staging (wavefront 7) ────────────────────────────────────────
// xs[0..kp) = optional RMSNorm of src[0..k) (RMSNorm1D.java:46-57), zero beyond k.
__device__ __forceinline__ void stage_x(Ctx &c, const float *src, const bool COHERENT, int k, int kp, const float *gamma) {
    if (c.wave != kDW - 1) return;
    // lane handles 16 consecutive floats of each 1024-float block
    float ss = 0.0f;
    for (int kb = c.lane * 16; kb < kp; kb += 1024) {
        float v[16];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            int e = kb + 2 * j;
            float2 t = make_float2(0.f, 0.f);
            if (e + 1 < k) t = COHERENT ? ldc_f2(src + e) : *reinterpret_cast<const float2 *>(src + e);
            else if (e < k) t.x = COHERENT ? ldc_f32(src + e) : src[e];
            v[2 * j] = t.x; v[2 * j + 1] = t.y;
            ss += t.x * t.x + t.y * t.y;
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            *reinterpret_cast<float4 *>(c.xs + kb + 4 * j) = make_float4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3]);
    }
    if (gamma) {
        float tot = wave_sum_dpp(ss);
        float rms = sqrtf(tot * (1.0f / (float)k) + kRmsEps);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        for (int kb = c.lane * 16; kb < kp; kb += 1024) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                int e = kb + 4 * j;
                float4 t = *reinterpret_cast<float4 *>(c.xs + e);
                float4 g = make_float4(0.f, 0.f, 0.f, 0.f);
                if (e + 3 < k) g = *reinterpret_cast<const float4 *>(gamma + e);
                else { if (e < k) g.x = gamma[e]; if (e + 1 < k) g.y = gamma[e + 1]; if (e + 2 < k) g.z = gamma[e + 2]; }
                t.x = (t.x / rms) * g.x; t.y = (t.y / rms) * g.y; t.z = (t.z / rms) * g.z; t.w = (t.w / rms) * g.w;
                *reinterpret_cast<float4 *>(c.xs + e) = t;
            }
        }
    }
}

// ── one matrix-vector phase ─────────────────────────────────────────────────
// kind selects the epilogue wavefront 7 applies when it stores a chunk's outputs:
//   0 qkv: plain; 1 wo: + residual; 2 gate/up: SiLU(gate + bg) * (up + bu); 3 down: + bd + residual;
//   4 LM head: + blm, tracks the arg-max.
struct Epilogue {
    float *out; const float *bias, *bias2, *residual;
    bool residual_coherent;
    float best_v; int best_i;      // kind 4, wavefront 7
};

template <int NC, bool PAIRS>
__device__ __forceinline__ void run_matrix(Ctx &c, Pipe &pipe, const Mat &m, Epilogue &ep) {
    constexpr int unit = PAIRS ? 2 : 1;
    int r0, r1;
    wg_rows(m, unit, c.wg, c.G, r0, r1);
    const int kp = m.kp, groups = kp / kQ8Group;
    const int rpc = rows_per_chunk(m, unit);
    float *stage = reinterpret_cast<float *>(c.aux);          // two buffers of 128 floats

    // this lane's slice of the staged activation row
    float xr[NC][16];
#pragma unroll
    for (int cc = 0; cc < NC; cc++) {
        int kb = (cc * 64 + c.lane) * 16;
        bool active = kb < kp;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float4 v = active ? *reinterpret_cast<const float4 *>(c.xs + kb + 4 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
            xr[cc][4 * j] = v.x; xr[cc][4 * j + 1] = v.y; xr[cc][4 * j + 2] = v.z; xr[cc][4 * j + 3] = v.w;
        }
    }

    int parity = 0;
    for (int row = r0; row < r1; row += rpc, parity ^= 1) {
        const int rows = r1 - row < rpc ? r1 - row : rpc;
        const unsigned slot = pipe.acquire(c);
        const unsigned char *wl = c.lds + slot;
        const float *sl = reinterpret_cast<const float *>(c.lds + slot + (unsigned)rows * (unsigned)kp);
        float *st = stage + parity * 128;
        for (int u = c.wave * unit; u < rows; u += kDW * unit) {
            float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
            for (int cc = 0; cc < NC; cc++) {
                int chunk = cc * 64 + c.lane;
                if (chunk * 16 >= kp) chunk = 0;          // its activations are zero
                int4 w0 = *reinterpret_cast<const int4 *>(wl + (unsigned)u * kp + chunk * 16);
                float s0 = sl[u * groups + (chunk >> 1)];
                a0 = fmaf(dot16(w0, xr[cc]), s0, a0);
                if (PAIRS) {
                    int4 w1 = *reinterpret_cast<const int4 *>(wl + (unsigned)(u + 1) * kp + chunk * 16);
                    float s1 = sl[(u + 1) * groups + (chunk >> 1)];
                    a1 = fmaf(dot16(w1, xr[cc]), s1, a1);
                }
            }
            a0 = wave_sum_dpp(a0);
            if (PAIRS) a1 = wave_sum_dpp(a1);
            if (c.lane == 0) {
                st[u] = a0;
                if (PAIRS) st[u + 1] = a1;
            }
        }
        wg_sync();                                     // chunk fully read, staged sums visible
        pipe.release(c);
        if (c.wave == kDW - 1) {
            const int n_out = rows / unit;
            for (int i = c.lane; i < n_out; i += 64) {
                const int o = (row / unit) + i;
                float v;
                if (PAIRS) {
                    float gate = st[2 * i], up = st[2 * i + 1];
                    if (ep.bias) gate = gate + ep.bias[o];
                    if (ep.bias2) up = up + ep.bias2[o];
                    float sg = gate * d_sigmoid(gate);          // SiLU.java:20-24
                    v = sg * up;                                 // SwiGLULayer.java:69
                } else {
                    v = st[i];
                    if (ep.bias) v = v + ep.bias[o];
                }
                if (ep.residual) v = (ep.residual_coherent ? ldc_f32(ep.residual + o) : ep.residual[o]) + v;
                stc_f32(ep.out + o, v);
                if (better(v, o, ep.best_v, ep.best_i)) { ep.best_v = v; ep.best_i = o; }
            }
        }
    }
}

template <bool PAIRS>
__device__ __forceinline__ void run_matrix_nc(Ctx &c, Pipe &pipe, const Mat &m, Epilogue &ep) {
    const int nc = (m.kp + 1023) / 1024;
    if (nc <= 1) run_matrix<1, PAIRS>(c, pipe, m, ep);
    else if (nc <= 2) run_matrix<2, PAIRS>(c, pipe, m, ep);
    else if (nc <= 4) run_matrix<4, PAIRS>(c, pipe, m, ep);
    else if (nc <= 6) run_matrix<6, PAIRS>(c, pipe, m, ep);
    else if (nc <= 8) run_matrix<8, PAIRS>(c, pipe, m, ep);
    else run_matrix<11, PAIRS>(c, pipe, m, ep);
}

// ── attention for one (head, split) item ────────────────────────────────────
// Rotates q and the new key (RotaryEmbedding.java:112-122), appends the new key/value row,
// runs the online softmax over this split's keys (HeadOps.java:90-140 for one query row) and
// leaves a partial record; the last split of a head to finish merges the head's records.
template <int LPK>
__device__ __forceinline__ void attention_item(Ctx &c, int layer, int pos, int h, int split) {
    const DecodeParams &P = c.P;
    constexpr int HD = LPK * 4;
    constexpr int KPW = 64 / LPK;
    constexpr int NSUB = kDW * KPW;
    float *s_m = reinterpret_cast<float *>(c.aux);
    float *s_l = s_m + NSUB;
    float *s_o = s_l + NSUB;                               // [NSUB][HD]
    int *s_last = reinterpret_cast<int *>(c.aux + kAuxBytes - 8);
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
    for (int key = k_begin + c.wave * KPW + sub; key < k_end; key += kDW * KPW) {
        float4 kk, vv;
        if (key == pos) {
            const float2 ka = ldc_f2(P.qkv + d + h * HD + dl * 4), kc2 = ldc_f2(P.qkv + d + h * HD + dl * 4 + 2);
            kk = make_float4(ka.x * c2.x - ka.y * s2.x, ka.x * s2.x + ka.y * c2.x,
                             kc2.x * c2.y - kc2.y * s2.y, kc2.x * s2.y + kc2.y * c2.y);
            const float2 va = ldc_f2(P.qkv + 2 * d + h * HD + dl * 4), vb2 = ldc_f2(P.qkv + 2 * d + h * HD + dl * 4 + 2);
            vv = make_float4(va.x, va.y, vb2.x, vb2.y);
            stc_f2(kb + (long long)key * HD, make_float2(kk.x, kk.y));
            stc_f2(kb + (long long)key * HD + 2, make_float2(kk.z, kk.w));
            stc_f2(vb + (long long)key * HD, make_float2(vv.x, vv.y));
            stc_f2(vb + (long long)key * HD + 2, make_float2(vv.z, vv.w));
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
    wg_sync();
    float *rec = P.scratch + ((long long)h * ns + split) * (HD + 4);
    if (c.tid < HD) {
        float M = -INFINITY, L = 0.0f, O = 0.0f;
#pragma unroll 8
        for (int i = 0; i < NSUB; i++) M = fmaxf(M, s_m[i]);
        if (M != -INFINITY) {
#pragma unroll 8
            for (int i = 0; i < NSUB; i++) {
                float w = expf(s_m[i] - M);
                L += s_l[i] * w;
                O += s_o[i * HD + c.tid] * w;
            }
        }
        stc_f32(rec + 4 + c.tid, O);
        if (c.tid == 0) { stc_f32(rec, M); stc_f32(rec + 1, L); }
    }
    // all of this workgroup's stores (record, appended row) must be complete before it counts itself in
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    wg_sync();
    if (c.tid == 0) {
        unsigned old = addc_u32(P.sync + SY_HEAD + h * kHeadStride, 1u);
        *s_last = ((old + 1) % (unsigned)ns) == 0;
    }
    wg_sync();
    if (*reinterpret_cast<volatile int *>(s_last) && c.tid < HD) {
        const float *base = P.scratch + (long long)h * ns * (HD + 4);
        float M = -INFINITY;
        for (int i = 0; i < ns; i++) M = fmaxf(M, ldc_f32(base + (long long)i * (HD + 4)));
        float L = 0.0f, O = 0.0f;
        for (int i = 0; i < ns; i++) {
            const float *r = base + (long long)i * (HD + 4);
            float mi = ldc_f32(r);
            if (mi != -INFINITY) {
                float w = expf(mi - M);
                L += ldc_f32(r + 1) * w;
                O += ldc_f32(r + 4 + c.tid) * w;
            }
        }
        stc_f32(P.att + h * HD + c.tid, O / L);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the merged head is in memory before the workgroup moves on
    wg_sync();                                             // aux is reused by the next item / phase
}

__device__ __forceinline__ void attention_phase(Ctx &c, int layer, int pos) {
    const DecodeParams &P = c.P;
    const int items = P.H * P.nsplit;
    for (int it = c.wg; it < items; it += c.G) {
        const int h = it / P.nsplit, split = it % P.nsplit;
        switch (P.hd) {
            case 32: attention_item<8>(c, layer, pos, h, split); break;
            case 64: attention_item<16>(c, layer, pos, h, split); break;
            default: attention_item<32>(c, layer, pos, h, split); break;
        }
    }
}

// ── the kernel ──────────────────────────────────────────────────────────────
__global__ void __launch_bounds__(kDT) k_llama_decode(DecodeParams P) {
    extern __shared__ __align__(16) unsigned char lds[];
    Ctx c{P};
    c.lds = lds;
    c.lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
    c.xs = reinterpret_cast<float *>(lds + P.slot_count * kSlotBytes);
    c.aux = lds + P.slot_count * kSlotBytes + P.xs_bytes;
    c.wg = blockIdx.x; c.G = gridDim.x; c.tid = threadIdx.x; c.lane = c.tid & 63; c.wave = c.tid >> 6;
    c.epoch = P.sync[SY_EPOCH];
    c.failed = false;
    if (c.tid == 0) { *reinterpret_cast<volatile int *>(c.aux + kAuxBytes - 4) = 0; *reinterpret_cast<volatile int *>(c.aux + kAuxBytes - 8) = 0; }
    wg_sync();

    Pipe pipe;
    pipe.cur = Cursor{0, 0, 0, -1};
    pipe.issued = pipe.consumed = 0;
    pipe.nload0 = pipe.nload1 = pipe.nload2 = pipe.nload3 = 0;
    pipe.top_up(c);

    const int pos0 = P.state[0], gen0 = P.state[2];
    int tok = P.state[1];
    Epilogue ep;
    const int phases = 5 * P.L + 1;                  // five per block, then the LM head
    for (int step = 0; step < P.steps && !c.failed; step++) {
        const int pos = pos0 + step;
        const bool tok_ok = tok >= 0 && tok < P.vocab && pos < P.max_seq;
        const float *emb_row = P.emb + (long long)(tok_ok ? tok : 0) * P.d;
        for (int item = 0; item < phases && !c.failed; item++) {
            const int l = item / 5, ph = item - 5 * l;
            if (l < P.L && ph == 1) {
                attention_phase(c, l, pos < P.max_seq ? pos : P.max_seq - 1);
                grid_sync(c);
                continue;
            }
            // what this phase multiplies, from where, and how its outputs are finished
            const Mat *m; const float *src, *gamma = nullptr; int k; bool coherent = true, pairs = false;
            if (l == P.L) {                          // logits = norm(x) . Wlm + blm        DecoderOnlyModel.java:58-64
                m = &P.lm; src = P.x; k = P.d; gamma = P.gf;
                ep = Epilogue{P.logits, P.blm, nullptr, nullptr, false, -INFINITY, 0x7fffffff};
            } else {
                const DecLayer &L = P.layers[l];
                const float *xin = l == 0 ? emb_row : P.x;
                if (ph == 0) {                       // qkv = norm1(x) . [Wq|Wk|Wv]
                    m = &L.qkv; src = xin; k = P.d; gamma = L.g1; coherent = l != 0;
                    ep = Epilogue{P.qkv, nullptr, nullptr, nullptr, false, -INFINITY, 0x7fffffff};
                } else if (ph == 2) {                // x2 = x + att . Wo                  LlamaTransformerBlock.java:51
                    m = &L.wo; src = P.att; k = P.d;
                    ep = Epilogue{P.x2, nullptr, nullptr, xin, l != 0, -INFINITY, 0x7fffffff};
                } else if (ph == 3) {                // ff = SiLU(gate(norm2(x2))) * up(norm2(x2))
                    m = &L.gu; src = P.x2; k = P.d; gamma = L.g2; pairs = true;
                    ep = Epilogue{P.ff, L.bg, L.bu, nullptr, false, -INFINITY, 0x7fffffff};
                } else {                             // x = x2 + down(ff)                  LlamaTransformerBlock.java:52
                    m = &L.down; src = P.ff; k = P.dff;
                    ep = Epilogue{P.x, L.bd, nullptr, P.x2, true, -INFINITY, 0x7fffffff};
                }
            }
            stage_x(c, src, coherent, k, m->kp, gamma);
            wg_sync();
            if (pairs) run_matrix_nc<true>(c, pipe, *m, ep);
            else run_matrix_nc<false>(c, pipe, *m, ep);
            if (l == P.L && c.wave == kDW - 1) {     // this workgroup's best logit
                float bv = ep.best_v; int bi = ep.best_i;
#pragma unroll
                for (int off = 32; off > 0; off >>= 1) {
                    float ov = __shfl_xor(bv, off, 64);
                    int oi = __shfl_xor(bi, off, 64);
                    if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
                }
                if (c.lane == 0) { stc_f32(P.argbuf + 2 * c.wg, bv); stc_u32(reinterpret_cast<unsigned *>(P.argbuf) + 2 * c.wg + 1, (unsigned)bi); }
            }
            grid_sync(c);
        }
        // every workgroup reduces the per-workgroup winners to the same token
        {
            float bv = -INFINITY; int bi = 0x7fffffff;
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
            float *sv = reinterpret_cast<float *>(c.aux);
            int *si = reinterpret_cast<int *>(c.aux) + kDW;
            if (c.lane == 0) { sv[c.wave] = bv; si[c.wave] = bi; }
            wg_sync();
            bv = sv[0]; bi = si[0];
            for (int w = 1; w < kDW; w++)
                if (better(sv[w], si[w], bv, bi)) { bv = sv[w]; bi = si[w]; }
            tok = bi;
            wg_sync();
        }
        if (c.wg == 0 && c.tid == 0 && gen0 + step < P.capacity) P.tokens[gen0 + step] = tok;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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

// The caller has filled every pointer and dimension; this derives the launch geometry.
void launch_llama_decode(hipStream_t s, DecodeParams &p) {
    if (p.hd != 32 && p.hd != 64 && p.hd != 128) fail("llama_decode: head dim must be 32, 64 or 128");
    if (p.H < 1 || p.H > kMaxHeads || p.H * p.hd != p.d) fail("llama_decode: bad head count");
    if (p.steps <= 0) return;
    int grid = 0, ns = 0;
    llama_decode_plan(p.H, p.hd, &grid, &ns, nullptr, nullptr);
    p.nsplit = ns;
    p.scale = (float)(1.0 / sqrt((double)p.hd));
    int kp_max = p.lm.kp;
    auto check = [&](const Q8Mat &m, int unit) {
        if (m.kp > 11 * 1024) fail("llama_decode: inner dimension above 11264 is not supported");
        if ((int64_t)(m.kp + m.kp / 8) * unit > (int64_t)kSlotBytes) fail("llama_decode: row does not fit a prefetch slot");
        if (m.rows % unit) fail("llama_decode: odd gate/up row count");
        if (m.kp > kp_max) kp_max = m.kp;
    };
    check(p.lm, 1);
    for (int l = 0; l < p.L; l++) {
        check(p.layers_host[l].qkv, 1); check(p.layers_host[l].wo, 1); check(p.layers_host[l].gu, 2); check(p.layers_host[l].down, 1);
    }
    p.xs_bytes = (unsigned)round_up((int64_t)kp_max * 4, 1024);
    int64_t room = (int64_t)kLdsLimit - kAuxBytes - p.xs_bytes;
    int slots = (int)(room / kSlotBytes);
    if (slots > kMaxSlots) slots = kMaxSlots;
    if (slots < 2) fail("llama_decode: not enough LDS for the prefetch ring");
    p.slot_count = (unsigned)slots;
    size_t lds = (size_t)slots * kSlotBytes + p.xs_bytes + kAuxBytes;
    static bool attr_set = false;
    if (!attr_set) {
        DJ_HIP(hipFuncSetAttribute((const void *)k_llama_decode, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsLimit));
        attr_set = true;
    }
    hipLaunchKernelGGL(k_llama_decode, dim3(grid), dim3(kDT), lds, s, p);
}

}  // namespace dj
