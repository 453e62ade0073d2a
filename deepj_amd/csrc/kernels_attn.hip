// RoPE + KV-cache store, and causal softmax attention over a device-resident
// KV cache (fp32).  Semantics follow the reference's Java composition:
//   RotaryEmbedding.java:63-70,112-122   interleaved pairs (2i, 2i+1), tables via f64
//   HeadOps.java:90-140                  s = (q.k) * scale, causal mask, softmax, p.v
//   MultiHeadSelfAttention.java:45       scale = (float)(1/sqrt(headDim))
// but nothing is materialised: no [H*S x S] score tensor, no mask tensor, no head
// split/merge copies.  Keys later than the query position are simply not read
// (the reference adds -1e9 to them, which makes their probability exactly 0).
//
// Cache layout (per layer): K and V as [H][maxSeq][hd] fp32, so one head's keys
// are a single contiguous stream.  A key row is read by hd/4 lanes as float4
// (a wavefront load covers 64/(hd/4) whole keys = 1 KiB, fully coalesced).
//
// Decode (S = 1) is one fused op: the query and the new key are rotated in registers,
// the new key/value row is appended to the cache by the workgroup that owns it, the key
// range is split evenly (computed on the device from the live position, so a captured
// graph stays valid as the cache grows) over gridDim.y workgroups per head so the
// HBM-bound KV read is spread over all CUs, and a second tiny kernel merges the
// per-split (max, sum, weighted V) records.
#include <cstdlib>
#include <type_traits>

#include "dj_common.h"
#include "dj_device.h"

namespace dj {
namespace {
using namespace dev;

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kAttnFullGrid = 512;        // workgroups that give every CU one

// ── RoPE on the fused projection + cache append ─────────────────────────────
// qkv [S x 3d]: Q | K | V.  Row i sits at position state[0] + i.
__global__ void __launch_bounds__(kThreads) k_rope_kv_store(const float *__restrict__ qkv, float *__restrict__ q_out,
                                                            float *__restrict__ k_cache, float *__restrict__ v_cache,
                                                            const int32_t *__restrict__ state,
                                                            const float *__restrict__ cos_t,
                                                            const float *__restrict__ sin_t, int S, int H, int hd,
                                                            int max_seq) {
    const int half = hd >> 1, d = H * hd;
    const int pos0 = state[0];
    int64_t total = (int64_t)S * H * half;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        int j = (int)(t % half);
        int h = (int)((t / half) % H);
        int i = (int)(t / ((int64_t)half * H));
        int pos = pos0 + i;
        if (pos < 0 || pos >= max_seq) continue;          // never write outside the cache
        float c = cos_t[(int64_t)pos * half + j], s = sin_t[(int64_t)pos * half + j];
        const float *row = qkv + (int64_t)i * 3 * d;
        int e = h * hd + 2 * j;
        float2 q = *reinterpret_cast<const float2 *>(row + e);
        float2 k = *reinterpret_cast<const float2 *>(row + d + e);
        float2 v = *reinterpret_cast<const float2 *>(row + 2 * d + e);
        float2 qr = make_float2(q.x * c - q.y * s, q.x * s + q.y * c);
        float2 kr = make_float2(k.x * c - k.y * s, k.x * s + k.y * c);
        *reinterpret_cast<float2 *>(q_out + (int64_t)i * d + e) = qr;
        int64_t ce = ((int64_t)h * max_seq + pos) * hd + 2 * j;
        *reinterpret_cast<float2 *>(k_cache + ce) = kr;
        *reinterpret_cast<float2 *>(v_cache + ce) = v;
    }
}

// RoPE on token-major rows [rows x H*hd]; position = row (pos_from_row) or state[0] + row.
__global__ void __launch_bounds__(kThreads) k_rope_rows(const float *x, float *out,   // may alias (in place)
                                                        const int32_t *__restrict__ state,
                                                        const float *__restrict__ cos_t,
                                                        const float *__restrict__ sin_t, int rows, int H, int hd,
                                                        int max_seq, int pos_from_row, int row_stride, int live_extra) {
    const int half = hd >> 1, d = row_stride;
    const int pos0 = pos_from_row ? 0 : state[0];
    if (live_extra >= 0) {                        // only the rows a growing cache holds so far
        int live = state[0] + live_extra;
        rows = rows < live ? rows : live;
    }
    int64_t total = (int64_t)rows * H * half;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += stride) {
        int j = (int)(t % half);
        int h = (int)((t / half) % H);
        int i = (int)(t / ((int64_t)half * H));
        int pos = pos0 + i;
        if (pos < 0 || pos >= max_seq) continue;
        float c = cos_t[(int64_t)pos * half + j], s = sin_t[(int64_t)pos * half + j];
        int64_t e = (int64_t)i * d + h * hd + 2 * j;
        float2 v = *reinterpret_cast<const float2 *>(x + e);
        *reinterpret_cast<float2 *>(out + e) = make_float2(v.x * c - v.y * s, v.x * s + v.y * c);
    }
}

// ── attention, several query rows (prefill) ─────────────────────────────────
// grid (H, S).  LPK = hd/4 lanes cooperate on one key; a wavefront handles 64/LPK keys per
// step; the 4*(64/LPK) running softmax states of a workgroup are merged through LDS.
struct AttnKernelArgs {
    const float *q; const float *k; const float *v; float *out;
    const int32_t *state;
    int64_t tok_stride, head_stride;
    int S, H, hd, max_seq;
    float scale;
    float *partial = nullptr;   // key-sharing launches of the tiled kernel: records [row][head][share][hd + 4]
};

template <int LPK>
__global__ void __launch_bounds__(kThreads) k_attention(AttnKernelArgs a) {
    constexpr int HD = LPK * 4;
    constexpr int KPW = 64 / LPK;                 // keys per wavefront step
    constexpr int NSUB = kWaves * KPW;            // independent running softmaxes per workgroup
    __shared__ float s_m[NSUB], s_l[NSUB];
    __shared__ __align__(16) float s_o[NSUB][HD];

    const int h = blockIdx.x, qi = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane / LPK, dl = lane % LPK;
    const int d = a.H * HD;

    const int pos = a.state[0] + qi;              // this query's position; keys 0..pos
    int n_keys = pos + 1;
    if (n_keys > a.max_seq) n_keys = a.max_seq;

    const float4 qv = *reinterpret_cast<const float4 *>(a.q + (int64_t)qi * d + h * HD + dl * 4);
    const float *kb = a.k + (int64_t)h * a.head_stride + dl * 4;
    const float *vb = a.v + (int64_t)h * a.head_stride + dl * 4;

    float m = -INFINITY, l = 0.0f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int key = wave * KPW + sub; key < n_keys; key += kWaves * KPW) {
        float4 kk = *reinterpret_cast<const float4 *>(kb + (int64_t)key * a.tok_stride);
        float4 vv = *reinterpret_cast<const float4 *>(vb + (int64_t)key * a.tok_stride);
        float s = qv.x * kk.x + qv.y * kk.y + qv.z * kk.z + qv.w * kk.w;
#pragma unroll
        for (int off = LPK / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
        s *= a.scale;
        float mn = fmaxf(m, s);
        float corr = expf(m - mn);                // 0 when m = -inf
        float p = expf(s - mn);
        l = l * corr + p;
        o.x = o.x * corr + p * vv.x; o.y = o.y * corr + p * vv.y;
        o.z = o.z * corr + p * vv.z; o.w = o.w * corr + p * vv.w;
        m = mn;
    }
    const int slot = wave * KPW + sub;
    if (dl == 0) { s_m[slot] = m; s_l[slot] = l; }
    *reinterpret_cast<float4 *>(&s_o[slot][dl * 4]) = o;
    __syncthreads();
    if (tid < HD) {
        float M = -INFINITY, L = 0.0f, O = 0.0f;
#pragma unroll
        for (int i = 0; i < NSUB; i++) M = fmaxf(M, s_m[i]);
#pragma unroll
        for (int i = 0; i < NSUB; i++) {
            float w = expf(s_m[i] - M);           // empty slots: exp(-inf) = 0
            L += s_l[i] * w;
            O += s_o[i][tid] * w;
        }
        a.out[(int64_t)qi * d + h * HD + tid] = O / L;
    }
}

// ── attention, many query rows: tiled on the matrix cores ────────────────────
// grid (H, ceil(S / 128)): a workgroup takes one head and 128 query rows, 32 per wavefront, and walks the
// keys in tiles of 32 that all four wavefronts share through LDS (K as three bf16 planes, V as is).  Per tile and
// wavefront two products run on the matrix cores:
//     S^T = K . Q^T      v_mfma_f32_32x32x16_bf16 on split planes (split3 above): 32 keys x 32 queries; a lane ends up
//                        with ONE query column and 16 of its keys, so the running soft-max state (max, sum) is one
//                        scalar pair per lane.  A key row is HD bf16 values per plane, its 16-byte chunks XOR-ed with
//                        the key's low bits so that the 32 rows an operand read touches spread over all banks
//     O^T += V^T . P     either v_mfma_f32_32x32x2_f32 with P consumed straight from the accumulator registers of the first
//                        product, or (PVB) the bf16 instruction again on split planes of P and of the value tile, which is
//                        staged transposed - [element][key slot] - into the bytes the key planes have just left: the
//                        key order of the contraction is chosen to be the order in which a lane holds them
// Causal masking (HeadOps.java:105-126) excludes key j for query position p when j > p; a tile that lies
// beyond every query of a wavefront is skipped by it.
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// An fp32 value is the exact sum of three bf16 pieces: its leading 8 significant bits, the next 8, the last 8 (each by
// truncation; the remainders are exact).  A product of two such values on the bf16 matrix cores takes the six piece
// products whose weights reach 2^-24 of the largest - hi.hi, hi.mid, mid.hi, hi.lo, lo.hi, mid.mid - accumulated in
// fp32: fp32 accuracy at three eighths of the fp32 matrix instructions' time (32 x 32 x 16 in 32 cycles against
// 32 x 32 x 2 in 64).
__device__ __forceinline__ float top_bits(float x) { return __uint_as_float(__float_as_uint(x) & 0xffff0000u); }
// bf16(a) | bf16(b) << 16 of values that are bf16 numbers already
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) { return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u); }
__device__ __forceinline__ void split3(float x0, float x1, uint32_t &hi, uint32_t &mid, uint32_t &lo) {
    const float h0 = top_bits(x0), h1 = top_bits(x1);
    const float r0 = x0 - h0, r1 = x1 - h1;
    const float c0 = top_bits(r0), c1 = top_bits(r1);
    hi = pack_bf16(h0, h1); mid = pack_bf16(c0, c1); lo = pack_bf16(r0 - c0, r1 - c1);
}

// The hardware's base-2 exponential (exp2(-inf) = 0).  Soft-max weights are exp2((s - max) log2 e): scores are carried
// multiplied by log2(e), one instruction per weight where the library's expf takes some twenty.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
constexpr float kLog2e = 1.44269504088896340736f;

// KSETS = 2 or 4 (for grids that would leave CUs idle): a workgroup takes 64 or 32 query rows; its wavefronts are
// 2 or 4 sets that walk every KSETS-th key tile for the SAME queries, KSETS tiles are staged per round, and the
// sets' partial soft-max states are merged through LDS at the end - more workgroups and fewer rounds.
// SHARE: the gridDim.z workgroups of a (head, query tile) take the rounds of key tiles in turn (round r goes to
// r % gridDim.z, so the shares are even whatever the position, which only the device knows) and leave their
// unnormalised states as records; k_attention_merge_shares finishes the rows.  For a handful of query rows over a
// long context, where (head, query tile) alone are far fewer workgroups than compute units.
template <int HD, int KSETS, bool SHARE = false, bool PVB = false>
__global__ void __launch_bounds__(256) k_attention_tiled(AttnKernelArgs a) {
    constexpr int KT = 32, NT = HD / 32;
    constexpr int QW = 4 / KSETS;                           // wavefronts that hold distinct query rows
    constexpr int QWG = 32 * QW;                            // query rows per workgroup
    constexpr int KSTEPS = HD / 16;                         // bf16 matrix instructions (K = 16) along the head dimension
    constexpr int CH = HD / 8;                              // 16-byte chunks of a key row of one plane
    constexpr int VP = KT + 8;                              // bf16 values per row of the transposed value tile: 32 keys + 16 bytes
    constexpr int kKbFloats = KSETS * 3 * KT * HD / 2, kVtFloats = KSETS * 3 * HD * VP / 2, kVsFloats = KSETS * KT * HD;
    // PVB: the key planes and the value planes use the same bytes in turn (scores first, then values); else the value
    // tile sits behind the key planes as fp32 rows
    constexpr int kStageFloats = PVB ? (kKbFloats > kVtFloats ? kKbFloats : kVtFloats) : kKbFloats + kVsFloats;
    constexpr int kMergeFloats = (KSETS - 1) * QW * 64 * (NT * 16 + 2);
    __shared__ __align__(16) float lds[kStageFloats > kMergeFloats ? kStageFloats : kMergeFloats];
    uint16_t(*Kb)[3][KT][HD] = reinterpret_cast<uint16_t(*)[3][KT][HD]>(lds);          // [set][plane][key][j], chunks swizzled
    uint16_t(*Vt)[3][HD][VP] = reinterpret_cast<uint16_t(*)[3][HD][VP]>(lds);          // PVB: [set][plane][j][key slot], transposed
    float(*Vs)[KT][HD] = reinterpret_cast<float(*)[KT][HD]>(lds + kKbFloats);          // else: [set][key][j]

    // Causal work grows with the query tile.  The second half of the tiles is taken in reverse, so that the workgroups
    // that become resident together on a compute unit (index i and i + half the grid) are a short and a long one.
    const int h = blockIdx.x, y_half = gridDim.y >> 1;
    const int qt = (int)blockIdx.y < y_half ? (int)blockIdx.y : (int)gridDim.y - 1 - ((int)blockIdx.y - y_half);
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, half = lane >> 5, l32 = lane & 31;
    const int qw = wave % QW, kset = wave / QW;
    const int d = a.H * HD;
    int pos0 = a.state[0];
    if (pos0 < 0) pos0 = 0;
    const int q_wave0 = qt * QWG + qw * 32;
    const int qi = q_wave0 + l32;                           // this lane's query row
    const bool q_ok = qi < a.S;
    int qpos = pos0 + qi;                                   // its position: keys 0 .. qpos
    if (qpos >= a.max_seq) qpos = a.max_seq - 1;
    const int q_end_wg = a.S < qt * QWG + QWG ? a.S : qt * QWG + QWG;
    const int q_end_wave = a.S < q_wave0 + 32 ? a.S : q_wave0 + 32;
    int wg_last = pos0 + q_end_wg - 1;                      // last key any query of the workgroup sees
    if (wg_last >= a.max_seq) wg_last = a.max_seq - 1;
    const int wave_last = q_end_wave > q_wave0 ? pos0 + q_end_wave - 1 : -1;

    // this lane's query row as the B operand of the score products: for step s its eight k slots are the elements
    // 16 s + 8 half .. + 7 (the same numbering the key operand uses), three planes
    bf16x8 qv[3][KSTEPS];
    {
        const float *qrow = a.q + (int64_t)(q_ok ? qi : 0) * d + h * HD;
#pragma unroll
        for (int sidx = 0; sidx < KSTEPS; sidx++) {
            const float4 v0 = *reinterpret_cast<const float4 *>(qrow + 16 * sidx + 8 * half);
            const float4 v1 = *reinterpret_cast<const float4 *>(qrow + 16 * sidx + 8 * half + 4);
            uint32_t hi[4], mid[4], lo[4];
            split3(v0.x, v0.y, hi[0], mid[0], lo[0]); split3(v0.z, v0.w, hi[1], mid[1], lo[1]);
            split3(v1.x, v1.y, hi[2], mid[2], lo[2]); split3(v1.z, v1.w, hi[3], mid[3], lo[3]);
            qv[0][sidx] = __builtin_bit_cast(bf16x8, make_uint4(hi[0], hi[1], hi[2], hi[3]));
            qv[1][sidx] = __builtin_bit_cast(bf16x8, make_uint4(mid[0], mid[1], mid[2], mid[3]));
            qv[2][sidx] = __builtin_bit_cast(bf16x8, make_uint4(lo[0], lo[1], lo[2], lo[3]));
        }
    }
    floatx16 acc[NT];
#pragma unroll
    for (int i = 0; i < NT; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
    float m = -INFINITY, l = 0.0f;

    const float *kbase = a.k + (int64_t)h * a.head_stride;
    const float *vbase = a.v + (int64_t)h * a.head_stride;
    // Value staging: a thread takes a pair of neighbouring keys (2 vkp, 2 vkp + 1) and four elements 4 vq .. 4 vq + 3 of
    // their rows, and writes each element's pair - neighbours in the transposed row - as one dword per plane.  Slot of key
    // kk in a row: the order in which the lanes hold their 16 scores of a tile (key 8 (e / 4) + 4 half + e % 4 in st[e]),
    // product mm = e / 8 taking slots 16 mm + 8 half + e % 8.  (Thread bits chosen so that the writes of a wavefront
    // spread over the banks two to a bank; an 80-byte row pitch makes the operand reads conflict free.)
    constexpr int VREP = HD >= 64 ? HD / 64 : 1;
    const int vq = (t & 3) | ((t >> 6) << 2), vkp = (t >> 2) & 15;
    const bool v_ok = 4 * vq < HD;
    const int vslot = 16 * (vkp >> 3) + 8 * ((vkp >> 1) & 1) + 4 * ((vkp >> 2) & 1) + 2 * (vkp & 1);
    const int k_first = SHARE ? (int)blockIdx.z * KT * KSETS : 0;
    const int k_stride = SHARE ? (int)gridDim.z * KT * KSETS : KT * KSETS;
    for (int k0 = k_first; k0 <= wg_last; k0 += k_stride) {
#pragma unroll
        for (int ks = 0; ks < KSETS; ks++) {
            // stage the key tile as bf16 planes and the value tile; rows past the last key repeat it (masked below)
            constexpr int PART = HD / 8;
            int key = k0 + ks * KT + (t & 31);
            if (key > wg_last) key = wg_last;
            const float *kr = kbase + (int64_t)key * a.tok_stride + (t >> 5) * PART;
#pragma unroll
            for (int j = 0; j < PART; j += 4) {
                float4 v = *reinterpret_cast<const float4 *>(kr + j);
                const int c = (t >> 5) * PART + j;                                       // first of four elements of the row
                const int at = ((((c >> 3) ^ (t & 31)) & (CH - 1)) << 3) + (c & 7);       // chunk c / 8 lives at (c / 8) ^ key
                uint32_t hi[2], mid[2], lo[2];
                split3(v.x, v.y, hi[0], mid[0], lo[0]); split3(v.z, v.w, hi[1], mid[1], lo[1]);
                *reinterpret_cast<uint2 *>(&Kb[ks][0][t & 31][at]) = make_uint2(hi[0], hi[1]);
                *reinterpret_cast<uint2 *>(&Kb[ks][1][t & 31][at]) = make_uint2(mid[0], mid[1]);
                *reinterpret_cast<uint2 *>(&Kb[ks][2][t & 31][at]) = make_uint2(lo[0], lo[1]);
            }
        }
        // PVB: the value rows are requested now and fly while the scores are computed; else the value tile is staged as it is
        float4 va[PVB ? KSETS : 1][VREP], vb[PVB ? KSETS : 1][VREP];
        if constexpr (!PVB) {
#pragma unroll
            for (int ks = 0; ks < KSETS; ks++) {
                constexpr int PART = HD / 8;
                int vkey = k0 + ks * KT + (t >> 3);
                if (vkey > wg_last) vkey = wg_last;
                const float *vr = vbase + (int64_t)vkey * a.tok_stride + (t & 7) * PART;
#pragma unroll
                for (int j = 0; j < PART; j += 4)
                    *reinterpret_cast<float4 *>(&Vs[ks][t >> 3][(t & 7) * PART + j]) = *reinterpret_cast<const float4 *>(vr + j);
            }
        }
#pragma unroll
        for (int ks = 0; ks < (PVB ? KSETS : 0); ks++) {
            int key_a = k0 + ks * KT + 2 * vkp, key_b = key_a + 1;
            if (key_a > wg_last) key_a = wg_last;
            if (key_b > wg_last) key_b = wg_last;
#pragma unroll
            for (int rep = 0; rep < VREP; rep++) {
                const int j0 = v_ok ? 4 * (vq + 16 * rep) : 0;
                va[ks][rep] = *reinterpret_cast<const float4 *>(vbase + (int64_t)key_a * a.tok_stride + j0);
                vb[ks][rep] = *reinterpret_cast<const float4 *>(vbase + (int64_t)key_b * a.tok_stride + j0);
            }
        }
        __syncthreads();
        const int kb0 = k0 + kset * KT;                     // this wavefront's tile of the round
        const bool active = kb0 <= wave_last;               // wave-uniform
        floatx16 st;
        if (active) {
#pragma unroll
            for (int e = 0; e < 16; e++) st[e] = 0.0f;
#pragma unroll
            for (int sidx = 0; sidx < KSTEPS; sidx++) {
                const int at = (((2 * sidx + half) ^ l32) & (CH - 1)) << 3;
                const bf16x8 k_hi = *reinterpret_cast<const bf16x8 *>(&Kb[kset][0][l32][at]);
                const bf16x8 k_mid = *reinterpret_cast<const bf16x8 *>(&Kb[kset][1][l32][at]);
                const bf16x8 k_lo = *reinterpret_cast<const bf16x8 *>(&Kb[kset][2][l32][at]);
                // the small terms first
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_lo, qv[0][sidx], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_hi, qv[2][sidx], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_mid, qv[1][sidx], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_mid, qv[0][sidx], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_hi, qv[1][sidx], st, 0, 0, 0);
                st = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_hi, qv[0][sidx], st, 0, 0, 0);
            }
            // st[e] = q . k for key kb0 + 8*(e/4) + 4*half + e%4 and this lane's query
            float tmax = -INFINITY;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                int key = kb0 + 8 * (e >> 2) + 4 * half + (e & 3);
                float sv = (q_ok && key <= qpos) ? (st[e] * a.scale) * kLog2e : -INFINITY;      // scale after the product, then the change of base
                st[e] = sv;
                tmax = fmaxf(tmax, sv);
            }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const float mn = fmaxf(m, tmax);
            const float corr = (mn == -INFINITY) ? 1.0f : fast_exp2(m - mn);
            float psum = 0.0f;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                float p = (st[e] == -INFINITY) ? 0.0f : fast_exp2(st[e] - mn);
                st[e] = p;
                psum += p;
            }
            l = l * corr + psum;
            m = mn;
#pragma unroll
            for (int i = 0; i < NT; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][e] *= corr;
            if constexpr (!PVB) {
                // O^T += V^T . P on the fp32 matrix instruction, P straight from the registers the scores arrived in
#pragma unroll
                for (int kk = 0; kk < 16; kk++) {
                    const int key = 8 * (kk >> 2) + 4 * half + (kk & 3);
#pragma unroll
                    for (int i = 0; i < NT; i++)
                        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(Vs[kset][key][32 * i + l32], st[kk], acc[i], 0, 0, 0);
                }
            }
        }
        __syncthreads();                                    // every wavefront has read its keys (PVB: the bytes now take the values)
        if constexpr (!PVB) continue;
#pragma unroll
        for (int ks = 0; ks < (PVB ? KSETS : 0); ks++) {
            if (!v_ok) break;
#pragma unroll
            for (int rep = 0; rep < VREP; rep++) {
                const float ca[4] = {va[ks][rep].x, va[ks][rep].y, va[ks][rep].z, va[ks][rep].w};
                const float cb[4] = {vb[ks][rep].x, vb[ks][rep].y, vb[ks][rep].z, vb[ks][rep].w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t hi, mid, lo;                   // (key, key + 1) of one element: neighbours in the row
                    split3(ca[i], cb[i], hi, mid, lo);
                    const int j = 4 * (vq + 16 * rep) + i;
                    *reinterpret_cast<uint32_t *>(&Vt[ks][0][j][vslot]) = hi;
                    *reinterpret_cast<uint32_t *>(&Vt[ks][1][j][vslot]) = mid;
                    *reinterpret_cast<uint32_t *>(&Vt[ks][2][j][vslot]) = lo;
                }
            }
        }
        __syncthreads();
        if (active) {
            // O^T += V^T . P: the k slots of product mm are the keys the lane holds in st[8 mm .. 8 mm + 7]
#pragma unroll
            for (int mm = 0; mm < 2; mm++) {
                uint32_t ph[4], pm[4], pl[4];
#pragma unroll
                for (int i = 0; i < 4; i++) split3(st[8 * mm + 2 * i], st[8 * mm + 2 * i + 1], ph[i], pm[i], pl[i]);
                const bf16x8 p_hi = __builtin_bit_cast(bf16x8, make_uint4(ph[0], ph[1], ph[2], ph[3]));
                const bf16x8 p_mid = __builtin_bit_cast(bf16x8, make_uint4(pm[0], pm[1], pm[2], pm[3]));
                const bf16x8 p_lo = __builtin_bit_cast(bf16x8, make_uint4(pl[0], pl[1], pl[2], pl[3]));
#pragma unroll
                for (int i = 0; i < NT; i++) {
                    const int j = 32 * i + l32, at = 16 * mm + 8 * half;
                    const bf16x8 v_hi = *reinterpret_cast<const bf16x8 *>(&Vt[kset][0][j][at]);
                    const bf16x8 v_mid = *reinterpret_cast<const bf16x8 *>(&Vt[kset][1][j][at]);
                    const bf16x8 v_lo = *reinterpret_cast<const bf16x8 *>(&Vt[kset][2][j][at]);
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_lo, p_hi, acc[i], 0, 0, 0);
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_hi, p_lo, acc[i], 0, 0, 0);
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_mid, p_mid, acc[i], 0, 0, 0);
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_mid, p_hi, acc[i], 0, 0, 0);
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_hi, p_mid, acc[i], 0, 0, 0);
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_hi, p_hi, acc[i], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }
    if constexpr (KSETS > 1) {
        // merge the key sets' states of the same queries: every set but the first parks (m, l, acc) lane by lane,
        // set 0 adds them
        constexpr int REC = NT * 16 + 2;
        if (kset > 0) {
            float *mg = lds + (int64_t)(((kset - 1) * QW + qw) * 64 + lane) * REC;
            mg[0] = m; mg[1] = l;
#pragma unroll
            for (int i = 0; i < NT; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) mg[2 + i * 16 + e] = acc[i][e];
        }
        __syncthreads();
        if (kset > 0) return;
#pragma unroll
        for (int ks = 1; ks < KSETS; ks++) {
            const float *mg = lds + (int64_t)(((ks - 1) * QW + qw) * 64 + lane) * REC;
            const float m1 = mg[0], l1 = mg[1];
            const float mn = fmaxf(m, m1);
            const float w0 = (m == -INFINITY) ? 0.0f : fast_exp2(m - mn), w1 = (m1 == -INFINITY) ? 0.0f : fast_exp2(m1 - mn);
            l = l * w0 + l1 * w1;
            m = mn;
#pragma unroll
            for (int i = 0; i < NT; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][e] = acc[i][e] * w0 + mg[2 + i * 16 + e] * w1;
        }
    }
    l += __shfl_xor(l, 32, 64);
    if constexpr (SHARE) {
        if (q_ok) {
            float *rec = a.partial + (((int64_t)qi * a.H + h) * gridDim.z + blockIdx.z) * (HD + 4);
            if (half == 0) { rec[0] = m; rec[1] = l; }
#pragma unroll
            for (int i = 0; i < NT; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) rec[4 + 32 * i + 8 * (e >> 2) + 4 * half + (e & 3)] = acc[i][e];
        }
        return;
    }
    if (q_ok) {
        float *orow = a.out + (int64_t)qi * d + h * HD;
#pragma unroll
        for (int i = 0; i < NT; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) orow[32 * i + 8 * (e >> 2) + 4 * half + (e & 3)] = acc[i][e] / l;
    }
}

// out[row, h, :] = sum_z w_z o_z / sum_z w_z l_z,  w_z = exp2(m_z - max m) (the maxima are in base-2 units), over the `shares` records of (row, head);
// grid (H, S), one thread per output element.  A share without keys left m = -inf, l = 0.
__global__ void __launch_bounds__(128) k_attention_merge_shares(const float *__restrict__ partial, float *__restrict__ out, int H,
                                                               int hd, int shares) {
    const int h = blockIdx.x, row = blockIdx.y, j = threadIdx.x;
    if (j >= hd) return;
    const float *rec = partial + ((int64_t)row * H + h) * shares * (hd + 4);
    float M = -INFINITY;
    for (int z = 0; z < shares; z++) M = fmaxf(M, rec[(int64_t)z * (hd + 4)]);
    float L = 0.0f, O = 0.0f;
    for (int z = 0; z < shares; z++) {
        const float *r = rec + (int64_t)z * (hd + 4);
        if (r[0] == -INFINITY) continue;
        const float w = fast_exp2(r[0] - M);
        L += r[1] * w;
        O += r[4 + j] * w;
    }
    out[((int64_t)row * H + h) * hd + j] = O / L;
}

// ── fused decode attention ──────────────────────────────────────────────────
// Record layout in scratch, per (head, split): [max, sum, pad, pad, o[hd]].
struct DecodeArgs {
    const float *qkv;          // FUSED: [3d] q | k | v of the new token (not rotated); else q [d], rotated
    float *k_cache, *v_cache;  // keys / values: element (key, h, j) at [h*head_stride + key*tok_stride + j]
    int64_t tok_stride, head_stride;
    float *out;                // [d]
    const int32_t *state;
    float *scratch;
    const float *cos_t, *sin_t;
    int H, hd, max_seq, nsplit;
    float scale;
    unsigned *counters;        // one arrival counter per head, zero between launches
};

// FUSED: rotate q and the new key in registers and append the new key/value row to the cache.
template <int LPK, bool FUSED>
__global__ void __launch_bounds__(kThreads) k_attn_decode_partial(DecodeArgs a) {
    constexpr int HD = LPK * 4;
    constexpr int KPW = 64 / LPK;
    constexpr int NSUB = kWaves * KPW;
    __shared__ float s_m[NSUB], s_l[NSUB];
    __shared__ __align__(16) float s_o[NSUB][HD];

    const int h = blockIdx.x, split = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane / LPK, dl = lane % LPK;
    const int d = a.H * HD, half = HD / 2;

    int pos = a.state[0];
    if (pos < 0) pos = 0;
    if (pos >= a.max_seq) pos = a.max_seq - 1;             // the host never lets this happen; stay in bounds
    const int n_keys = pos + 1;
    const int per = (n_keys + a.nsplit - 1) / a.nsplit;
    const int k_begin = split * per;
    const int k_end = k_begin + per < n_keys ? k_begin + per : n_keys;

    // rotate this lane's two (even, odd) pairs of q and of the new k
    float2 c2 = make_float2(1.f, 1.f), s2 = make_float2(0.f, 0.f);
    if constexpr (FUSED) {
        c2 = *reinterpret_cast<const float2 *>(a.cos_t + (int64_t)pos * half + dl * 2);
        s2 = *reinterpret_cast<const float2 *>(a.sin_t + (int64_t)pos * half + dl * 2);
    }
    const float4 q0 = *reinterpret_cast<const float4 *>(a.qkv + h * HD + dl * 4);
    const float4 qv = FUSED ? make_float4(q0.x * c2.x - q0.y * s2.x, q0.x * s2.x + q0.y * c2.x,
                                          q0.z * c2.y - q0.w * s2.y, q0.z * s2.y + q0.w * c2.y)
                            : q0;
    float *kb = a.k_cache + (int64_t)h * a.head_stride + dl * 4;
    float *vb = a.v_cache + (int64_t)h * a.head_stride + dl * 4;

    float m = -INFINITY, l = 0.0f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    // Four keys per lane group per round: their rows are requested together (clamped, never under a
    // branch), so a split of up to 4 * 64 / LPK * 4 keys costs one memory round trip.  The new token's
    // row is not in memory yet: it is rotated in registers, used, and appended.
    constexpr int U = 4;
    constexpr int STRIDE = kWaves * KPW;
    float4 nk = make_float4(0.f, 0.f, 0.f, 0.f), nv = nk;
    if (FUSED) {
        const float4 k0 = *reinterpret_cast<const float4 *>(a.qkv + d + h * HD + dl * 4);
        nk = make_float4(k0.x * c2.x - k0.y * s2.x, k0.x * s2.x + k0.y * c2.x,
                         k0.z * c2.y - k0.w * s2.y, k0.z * s2.y + k0.w * c2.y);
        nv = *reinterpret_cast<const float4 *>(a.qkv + 2 * d + h * HD + dl * 4);
    }
    for (int base = k_begin + wave * KPW + sub; base < k_end; base += U * STRIDE) {
        float4 kk[U], vv[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            int key = base + u * STRIDE;
            int row = (key < k_end && !(FUSED && key == pos)) ? key : k_begin;     // any row of the cache is readable
            kk[u] = *reinterpret_cast<const float4 *>(kb + (int64_t)row * a.tok_stride);
            vv[u] = *reinterpret_cast<const float4 *>(vb + (int64_t)row * a.tok_stride);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            int key = base + u * STRIDE;
            bool valid = key < k_end;                       // uniform over the LPK lanes of a key
            if (FUSED && valid && key == pos) {
                kk[u] = nk; vv[u] = nv;
                *reinterpret_cast<float4 *>(kb + (int64_t)key * a.tok_stride) = nk;
                *reinterpret_cast<float4 *>(vb + (int64_t)key * a.tok_stride) = nv;
            }
            float s = group_sum<LPK>(qv.x * kk[u].x + qv.y * kk[u].y + qv.z * kk[u].z + qv.w * kk[u].w);
            if (valid) {
                s *= a.scale;
                float mn = fmaxf(m, s);
                float corr = expf(m - mn);
                float p = expf(s - mn);
                l = l * corr + p;
                o.x = o.x * corr + p * vv[u].x; o.y = o.y * corr + p * vv[u].y;
                o.z = o.z * corr + p * vv[u].z; o.w = o.w * corr + p * vv[u].w;
                m = mn;
            }
        }
    }
    const int slot = wave * KPW + sub;
    if (dl == 0) { s_m[slot] = m; s_l[slot] = l; }
    *reinterpret_cast<float4 *>(&s_o[slot][dl * 4]) = o;
    __syncthreads();
    if (tid < HD) {
        float M = -INFINITY, L = 0.0f, O = 0.0f;
#pragma unroll
        for (int i = 0; i < NSUB; i++) M = fmaxf(M, s_m[i]);
        if (M != -INFINITY) {
#pragma unroll
            for (int i = 0; i < NSUB; i++) {
                float w = expf(s_m[i] - M);
                L += s_l[i] * w;
                O += s_o[i][tid] * w;
            }
        }
        // The record is written through to memory (agent-scope stores) so that the split that
        // finishes last can read every record of its head without a cache flush.
        float *rec = a.scratch + ((int64_t)h * a.nsplit + split) * (HD + 4);
        __hip_atomic_store(rec + 4 + tid, O, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid == 0) {
            __hip_atomic_store(rec, M, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(rec + 1, L, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // Last split of the head to arrive merges the head's records: out[h*hd + j] = sum_i w_i o_i[j] / sum_i w_i l_i.
    __shared__ int s_last;
    __builtin_amdgcn_s_waitcnt(0x0f70);            // vmcnt(0): this workgroup's record and appended row are in memory
    __syncthreads();
    if (tid == 0) {
        unsigned *counter = a.counters + h;
        unsigned old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bool last = old + 1 == (unsigned)a.nsplit;
        if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = last ? 1 : 0;
    }
    __syncthreads();
    if (s_last && tid < HD) {
        const float *base = a.scratch + (int64_t)h * a.nsplit * (HD + 4);
        float m[16], l[16], o[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float *r = base + (int64_t)(i < a.nsplit ? i : 0) * (HD + 4);
            m[i] = __hip_atomic_load(r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            l[i] = __hip_atomic_load(r + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            o[i] = __hip_atomic_load(r + 4 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        float M = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; i++) if (i < a.nsplit) M = fmaxf(M, m[i]);
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (i < a.nsplit && m[i] != -INFINITY) {
                float w = expf(m[i] - M);
                L += l[i] * w;
                O += o[i] * w;
            }
        }
        a.out[h * HD + tid] = O / L;
    }
}

// ── decode attention that leaves the split merge to its consumer ───────────
// Same work as the fused kernel above (rotate q and the new key, append the new row, online softmax over this
// split's keys), but it stops at the per-split record [max, sum, -, -, o[hd]]: merging records across workgroups
// inside one kernel costs a store acknowledgement, an atomic and a reload - three trips to memory in a row - while
// the next kernel reads them across the kernel boundary for free (the Q8 matvec's ATTN_MERGE prologue does the
// merge while its weight rows are in flight).
//
// What the kernel is built around: a launch of this size is bound by memory round trips and by its own serial
// tail, not by bytes.
//  * Keys are dealt to the kAttnRecordSplits splits of a head in TILES of kRecWaves * (64 / LPK) consecutive keys,
//    tile t to split t % splits: every split has work from the first tiles on, whatever the position.
//  * The running softmax is updated once per round of kRecU keys, not once per key: one maximum, one correction,
//    kRecU weights - and in base 2 with the hardware exponential (scores are multiplied by log2(e), the records hold
//    the maximum in that unit): a dozen instructions per round where the library expf took sixty.
//  * Four splits of 512 threads: eight splits shorten this kernel by 0.9 us at 1500 keys and cost the Wo matvec,
//    every workgroup of which reads all records, 0.7 us.  (Requesting the first tiles before the position is known
//    - rows past it are readable, being inside the cache buffer - gained nothing: measured 2435 against 2443 tok/s.)
constexpr int kRecThreads = 512;
constexpr int kRecWaves = kRecThreads / 64;
constexpr int kRecU = 4;          // key tiles a workgroup requests per round (2: 2437, 4: 2443, 8: 2411 tok/s)

// Timeline of one launch, for tuning builds only (-DDJ_TRACE; never in the shipped library).
#ifdef DJ_TRACE
__device__ unsigned long long g_at_trace[8 * 8192];
#define DJ_STAMP(i) do { if (lane == 0) g_at_trace[((blockIdx.y * gridDim.x + blockIdx.x) * kRecWaves + wave) * 8 + (i)] = wall_clock64(); } while (0)
#else
#define DJ_STAMP(i) do {} while (0)
#endif

// Separate scalar arguments, the ones the first loads need in front (they can reach a wavefront in registers at
// launch; a by-value struct is always fetched from the argument buffer first).
template <int LPK>
__global__ void __launch_bounds__(kRecThreads)
k_attn_decode_records(const int32_t *a_state, float *a_k_cache, float *a_v_cache, const float *a_qkv,
                      const float *a_cos_t, const float *a_sin_t, int a_max_seq, int a_H, float *a_records,
                      float a_scale) {
    constexpr int HD = LPK * 4;
    constexpr int KPW = 64 / LPK;                  // keys a wavefront handles at a time
    constexpr int TILE = kRecWaves * KPW;          // consecutive keys of one tile
    constexpr int U = kRecU;
    constexpr int NS = kAttnRecordSplits;
    __shared__ float s_m[kRecWaves], s_l[kRecWaves];
    __shared__ __align__(16) float s_o[kRecWaves][HD];

    const int h = blockIdx.x, split = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sub = lane / LPK, dl = lane % LPK;
    const int d = a_H * HD, half = HD / 2;
    const int64_t head_stride = (int64_t)a_max_seq * HD;
    DJ_STAMP(0);

    float *kb = a_k_cache + (int64_t)h * head_stride + dl * 4;
    float *vb = a_v_cache + (int64_t)h * head_stride + dl * 4;
    const int key0 = split * TILE + wave * KPW + sub;          // this lane group's key in tile 0 of the split
    const int row_cap = a_max_seq - 1;
    int pos = a_state[0];
    if (pos < 0) pos = 0;
    if (pos > row_cap) pos = row_cap;                      // the host never lets this happen; stay in bounds
    DJ_STAMP(1);
    // Round r of a split: tiles r * U .. r * U + U - 1 of its own, i.e. keys key0 + (r * U + u) * NS * TILE.  Loads are
    // unconditional (row 0 for keys past the position: an L2 hit), so waits for them are counted ones.
    auto load_round = [&](float4 (&K)[U], float4 (&V)[U], int t0) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int key = key0 + (t0 + u) * NS * TILE;
            const int row = key < pos ? key : 0;
            K[u] = *reinterpret_cast<const float4 *>(kb + (int64_t)row * HD);
            V[u] = *reinterpret_cast<const float4 *>(vb + (int64_t)row * HD);
        }
    };
    auto has_keys = [&](int t0) { return (t0 * NS + split) * TILE <= pos; };    // workgroup-uniform
    // The small operands (L2 hits) go out first and the first two rounds of keys and values right behind them: the
    // rotation below then waits for the small ones only while the key/value rows are on their way from HBM.
    const float2 c2 = *reinterpret_cast<const float2 *>(a_cos_t + (int64_t)pos * half + dl * 2);
    const float2 s2 = *reinterpret_cast<const float2 *>(a_sin_t + (int64_t)pos * half + dl * 2);
    float4 q0 = *reinterpret_cast<const float4 *>(a_qkv + h * HD + dl * 4);
    const float4 k0 = *reinterpret_cast<const float4 *>(a_qkv + d + h * HD + dl * 4);
    const float4 nv = *reinterpret_cast<const float4 *>(a_qkv + 2 * d + h * HD + dl * 4);
    float4 ka[U], va[U];
    load_round(ka, va, 0);
    asm volatile("" ::: "memory");
    asm volatile("" : "+v"(q0.x), "+v"(q0.y), "+v"(q0.z), "+v"(q0.w));
    const float4 qr = make_float4(q0.x * c2.x - q0.y * s2.x, q0.x * s2.x + q0.y * c2.x,
                                  q0.z * c2.y - q0.w * s2.y, q0.z * s2.y + q0.w * c2.y);
    const float4 nk = make_float4(k0.x * c2.x - k0.y * s2.x, k0.x * s2.x + k0.y * c2.x,
                                  k0.z * c2.y - k0.w * s2.y, k0.z * s2.y + k0.w * c2.y);

    float m = -INFINITY, l = 0.0f;
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    auto compute_round = [&](float4 (&K)[U], float4 (&V)[U], int t0) {
        float sc[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int key = key0 + (t0 + u) * NS * TILE;
            const bool valid = key <= pos;                  // uniform over the LPK lanes of a key
            if (key == pos) {                               // the new row: used from registers, and appended
                K[u] = nk; V[u] = nv;
                *reinterpret_cast<float4 *>(kb + (int64_t)key * HD) = nk;
                *reinterpret_cast<float4 *>(vb + (int64_t)key * HD) = nv;
            }
            // (q.k) * scale as the reference computes it (HeadOps.java:96-99), then the change of base
            const float dot = group_sum<LPK>(qr.x * K[u].x + qr.y * K[u].y + qr.z * K[u].z + qr.w * K[u].w);
            sc[u] = valid ? (dot * a_scale) * kLog2e : -INFINITY;
            if (!valid) V[u] = make_float4(0.f, 0.f, 0.f, 0.f);       // whatever the row held, it adds nothing
        }
        float mn = m;
#pragma unroll
        for (int u = 0; u < U; u++) mn = fmaxf(mn, sc[u]);
        if (mn > -INFINITY) {
            const float corr = fast_exp2(m - mn);           // m = -inf: 0
            l *= corr; o.x *= corr; o.y *= corr; o.z *= corr; o.w *= corr;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float p = fast_exp2(sc[u] - mn);
                l += p;
                o.x += p * V[u].x; o.y += p * V[u].y; o.z += p * V[u].z; o.w += p * V[u].w;
            }
            m = mn;
        }
    };
    // (Requesting round r + 1 before round r is used - two register sets in turn - was slower: 2419 against 2441 tok/s.)
    for (int t0 = 0;;) {
        compute_round(ka, va, t0);
        if (t0 == 0) DJ_STAMP(2);
        t0 += U;
        if (!has_keys(t0)) break;
        load_round(ka, va, t0);
    }
    DJ_STAMP(3);
    // the KPW lane groups of a wavefront first (shuffles), then the wavefronts (LDS)
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) {
        const float m2 = __shfl_xor(m, off, 64), l2 = __shfl_xor(l, off, 64);
        const float4 o2 = make_float4(__shfl_xor(o.x, off, 64), __shfl_xor(o.y, off, 64), __shfl_xor(o.z, off, 64),
                                      __shfl_xor(o.w, off, 64));
        const float mn = fmaxf(m, m2);
        const float w1 = mn == -INFINITY ? 0.0f : fast_exp2(m - mn), w2 = mn == -INFINITY ? 0.0f : fast_exp2(m2 - mn);
        l = l * w1 + l2 * w2;
        o.x = o.x * w1 + o2.x * w2; o.y = o.y * w1 + o2.y * w2; o.z = o.z * w1 + o2.z * w2; o.w = o.w * w1 + o2.w * w2;
        m = mn;
    }
    if (lane == 0) { s_m[wave] = m; s_l[wave] = l; }
    if (sub == 0) *reinterpret_cast<float4 *>(&s_o[wave][dl * 4]) = o;
    __syncthreads();
    DJ_STAMP(4);
    if (tid < HD) {
        float M = -INFINITY, L = 0.0f, O = 0.0f;
#pragma unroll
        for (int i = 0; i < kRecWaves; i++) M = fmaxf(M, s_m[i]);
        if (M != -INFINITY) {
#pragma unroll
            for (int i = 0; i < kRecWaves; i++) {
                const float w = fast_exp2(s_m[i] - M);
                L += s_l[i] * w;
                O += s_o[i][tid] * w;
            }
        }
        float *rec = a_records + ((int64_t)h * NS + split) * (HD + 4);
        rec[4 + tid] = O;
        if (tid == 0) { rec[0] = M; rec[1] = L; }
    }
    DJ_STAMP(5);
}


inline int fused_decode_splits(int H) {
    int ns = 512 / H;
    if (ns < 1) ns = 1;
    if (ns > 16) ns = 16;
    return ns;
}

}  // namespace

void launch_rope_kv_store(hipStream_t s, const float *qkv, float *q_out, float *k_cache, float *v_cache,
                          const int32_t *state, const float *cos_t, const float *sin_t, int S, int H, int hd,
                          int max_seq) {
    int64_t total = (int64_t)S * H * (hd / 2);
    if (total <= 0) return;
    int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 4096) blocks = 4096;
    launch_kernel(k_rope_kv_store, dim3((int)blocks), dim3(kThreads), 0, s, qkv, q_out, k_cache, v_cache, state,
                       cos_t, sin_t, S, H, hd, max_seq);
}

void launch_rope_rows(hipStream_t s, const float *x, float *out, const int32_t *state, const float *cos_t,
                      const float *sin_t, int rows, int H, int hd, int max_seq, int pos_from_row, int row_stride,
                      int live_extra) {
    int64_t total = (int64_t)rows * H * (hd / 2);
    if (total <= 0) return;
    int64_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 4096) blocks = 4096;
    launch_kernel(k_rope_rows, dim3((int)blocks), dim3(kThreads), 0, s, x, out, state, cos_t, sin_t, rows, H, hd,
                       max_seq, pos_from_row, row_stride > 0 ? row_stride : H * hd, live_extra);
}

// One row uses the split decode kernel (scratch: attn_decode_scratch_floats); 2 to kAttnShareRows rows - a short
// continuation of a cached prefix - the matrix-core kernel with the key rounds dealt to kAttnKeyShares workgroups
// (scratch: their records); more rows need no scratch.
constexpr int kAttnShareRows = 32;
int attention_key_shares(int S, int H) {
    if (S < 2 || S > kAttnShareRows) return 1;
    int z = 256 / H;                                   // about one workgroup per compute unit
    return z < 1 ? 1 : (z > 8 ? 8 : z);
}
int64_t attention_scratch_floats(int S, int H, int hd, int max_seq) {
    (void)max_seq;
    if (S == 1) return attn_decode_scratch_floats(H, hd);
    const int z = attention_key_shares(S, H);
    return z > 1 ? (int64_t)S * H * z * (hd + 4) : 0;
}

int64_t attn_decode_scratch_floats(int H, int hd) { return (int64_t)H * fused_decode_splits(H) * (hd + 4); }

template <bool FUSED>
static void launch_decode_kernels(hipStream_t s, DecodeArgs &a) {
    a.nsplit = fused_decode_splits(a.H);
    a.scale = (float)(1.0 / sqrt((double)a.hd));
    dim3 grid(a.H, a.nsplit);
    switch (a.hd) {
        case 32: launch_kernel((k_attn_decode_partial<8, FUSED>), grid, dim3(kThreads), 0, s, a); break;
        case 64: launch_kernel((k_attn_decode_partial<16, FUSED>), grid, dim3(kThreads), 0, s, a); break;
        case 128: launch_kernel((k_attn_decode_partial<32, FUSED>), grid, dim3(kThreads), 0, s, a); break;
        default: fail("attention: head dim must be 32, 64 or 128");
    }
}

void launch_attn_decode(hipStream_t s, const float *qkv, float *k_cache, float *v_cache, float *out,
                        const int32_t *state, float *scratch, const float *cos_t, const float *sin_t, int H, int hd,
                        int max_seq, unsigned *counters) {
    if (H > kAttnCounterHeads) fail("attention: more than 1024 heads");
    DecodeArgs a;
    a.counters = counters;
    a.qkv = qkv; a.k_cache = k_cache; a.v_cache = v_cache; a.out = out; a.state = state; a.scratch = scratch;
    a.tok_stride = hd; a.head_stride = (int64_t)max_seq * hd;
    a.cos_t = cos_t; a.sin_t = sin_t; a.H = H; a.hd = hd; a.max_seq = max_seq;
    launch_decode_kernels<true>(s, a);
}

void launch_attn_decode_records(hipStream_t s, const float *qkv, float *k_cache, float *v_cache, float *records,
                                const int32_t *state, const float *cos_t, const float *sin_t, int H, int hd,
                                int max_seq) {
    const float scale = (float)(1.0 / sqrt((double)hd));
    dim3 grid(H, kAttnRecordSplits);
    auto go = [&](auto kernel) {
        launch_kernel(kernel, grid, dim3(kRecThreads), 0, s, state, k_cache, v_cache, qkv, cos_t, sin_t, max_seq, H,
                      records, scale);
    };
    switch (hd) {
        case 32: go(k_attn_decode_records<8>); break;
        case 64: go(k_attn_decode_records<16>); break;
        case 128: go(k_attn_decode_records<32>); break;
        default: fail("attention: head dim must be 32, 64 or 128");
    }
}

void launch_attention(hipStream_t s, const AttnArgs &p) {
    if (p.s <= 0) return;
    if (p.s == 1) {
        if (p.scratch_floats < attn_decode_scratch_floats(p.h, p.hd)) fail("attention: scratch buffer too small");
        DecodeArgs a;
        a.qkv = p.q; a.k_cache = const_cast<float *>(p.k); a.v_cache = const_cast<float *>(p.v); a.out = p.out;
        a.state = p.state; a.scratch = p.scratch; a.tok_stride = p.k_tok_stride; a.head_stride = p.k_head_stride;
        a.cos_t = a.sin_t = nullptr; a.H = p.h; a.hd = p.hd; a.max_seq = p.max_seq;
        if (p.h > kAttnCounterHeads) fail("attention: more than 1024 heads");
        a.counters = p.counters;
        launch_decode_kernels<false>(s, a);
        return;
    }
    AttnKernelArgs a;
    a.q = p.q; a.k = p.k; a.v = p.v; a.out = p.out; a.state = p.state;
    a.tok_stride = p.k_tok_stride; a.head_stride = p.k_head_stride;
    a.S = p.s; a.H = p.h; a.hd = p.hd; a.max_seq = p.max_seq;
    a.scale = (float)(1.0 / sqrt((double)p.hd));
    const int shares = attention_key_shares(p.s, p.h);
    if (shares > 1) {
        // A handful of rows after a long prefix: one 32-row query tile per head, its key rounds dealt to `shares`
        // workgroups.  (32 heads of 64, 2 to 31 rows after 1500 cached ones: 15 to 17 us with the merge, against 34 us
        // for one workgroup per row (2 to 15 rows) and 55 us for the unshared matrix-core kernel (16 to 31); after 500:
        // 10 to 12 us against 13 and 25.  A fresh prompt of so few rows pays 6 us for it.)
        if (p.scratch_floats < attention_scratch_floats(p.s, p.h, p.hd, p.max_seq)) fail("attention: scratch buffer too small");
        a.partial = p.scratch;
        dim3 tgz(p.h, 1, shares);
        switch (p.hd) {
            case 32: launch_kernel((k_attention_tiled<32, 4, true>), tgz, dim3(256), 0, s, a); break;
            case 64: launch_kernel((k_attention_tiled<64, 4, true>), tgz, dim3(256), 0, s, a); break;
            case 128: launch_kernel((k_attention_tiled<128, 4, true>), tgz, dim3(256), 0, s, a); break;
            default: fail("attention: head dim must be 32, 64 or 128");
        }
        launch_kernel(k_attention_merge_shares, dim3(p.h, p.s), dim3(128), 0, s, (const float *)p.scratch, p.out, p.h, p.hd, shares);
        return;
    }
    if (p.s >= 16) {                     // enough rows to share key tiles: matrix-core kernel
        // the value products on bf16 planes (PVB) or on the fp32 matrix instruction: DEEPJ_HIP_ATTN_PVB=0 / 1 forces one
        static const int forced = [] { const char *e = getenv("DEEPJ_HIP_ATTN_PVB"); return e ? atoi(e) : -1; }();
        auto go = [&](auto hd_tag, auto sets_tag, dim3 grid, bool pvb) {
            constexpr int HD = decltype(hd_tag)::value, KSETS = decltype(sets_tag)::value;
            if (pvb) launch_kernel((k_attention_tiled<HD, KSETS, false, true>), grid, dim3(256), 0, s, a);
            else launch_kernel((k_attention_tiled<HD, KSETS, false, false>), grid, dim3(256), 0, s, a);
        };
        auto by_hd = [&](auto sets_tag, dim3 grid) {
            constexpr int KSETS = decltype(sets_tag)::value;
            // measured: wide heads gain from the bf16 value products (2048 rows, 128-wide: 328 -> 294 us per block); 64-wide
            // heads with four key sets lose (20.9 -> 23.8 us at 512 rows: the second staging pass and its barriers)
            const bool pvb = forced >= 0 ? forced != 0 : (p.hd == 128 || KSETS == 1);
            switch (p.hd) {
                case 32: go(std::integral_constant<int, 32>{}, sets_tag, grid, pvb); break;
                case 64: go(std::integral_constant<int, 64>{}, sets_tag, grid, pvb); break;
                case 128: go(std::integral_constant<int, 128>{}, sets_tag, grid, pvb); break;
                default: fail("attention: head dim must be 32, 64 or 128");
            }
        };
        dim3 tg(p.h, (p.s + 127) / 128);
        if ((int64_t)tg.x * tg.y * 2 < kAttnFullGrid)        // far too few workgroups for the chip: 32 rows each, keys in four sets
            by_hd(std::integral_constant<int, 4>{}, dim3(p.h, (p.s + 31) / 32));
        else if ((int64_t)tg.x * tg.y < kAttnFullGrid)      // too few: 64 rows each, keys in two sets
            by_hd(std::integral_constant<int, 2>{}, dim3(p.h, (p.s + 63) / 64));
        else
            by_hd(std::integral_constant<int, 1>{}, tg);
        return;
    }
    dim3 grid(p.h, p.s);
    switch (p.hd) {
        case 32: launch_kernel(k_attention<8>, grid, dim3(kThreads), 0, s, a); break;
        case 64: launch_kernel(k_attention<16>, grid, dim3(kThreads), 0, s, a); break;
        case 128: launch_kernel(k_attention<32>, grid, dim3(kThreads), 0, s, a); break;
        default: fail("attention: head dim must be 32, 64 or 128");
    }
}

#ifdef DJ_TRACE
extern "C" int deepj_hip_debug_attn_trace(unsigned long long *out, int n) {
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_at_trace), (size_t)n * sizeof(unsigned long long));
}
#endif

}  // namespace dj
