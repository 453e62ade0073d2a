// Q8 GEMM for many rows (prefill): C[M x N] = X[M x K] . dequant(W)^T, W int8 [N x Kp] with one fp32 scale per 32 k.
//
// Arithmetic.  An int8 weight is exact in fp16.  A row of activations is multiplied by a power of two that brings its
// largest magnitude into [2^14, 2^15) (exact, undone at the end) and every element is then written as hi + lo, two
// fp16 numbers: hi = fp16(v) by round-to-nearest, lo = fp16(v - hi).  hi carries 11 significant bits and lo the next 11
// (down to 2^-24 in the scaled units, i.e. 2^-38 of the row's largest value, where fp16 subnormals end), so hi + lo holds v to
// about 2^-23 relative - the fp32
// value itself for all practical rows - and x . q = hi . q + lo . q with exact products and fp32 accumulation: two
// v_mfma_f32_32x32x16_f16 per 16 k instead of three bf16 ones.  The group scale multiplies the finished 32-k partial
// sum, as in the reference's dequantise-then-multiply (Q8 layout: q8_format notes in dj_common.h).
//
// Data path.  Both operands are prepared in global memory in the exact byte layout the matrix cores want: two fp16
// planes of X (k_split_f16) and an fp16 copy of W with its scales transposed to [group][row] (k_q8_to_f16).  The GEMM
// kernel then moves them with direct global -> LDS loads (global_load_lds_dwordx4: no vector registers, no LDS
// store instructions), three stages deep, and spends its vector instructions on the per-group scaling only.
//
// Kernels.  k_gemm_q8_f16 (128 x 256 workgroup tile, described next) for problems with many tiles; k_gemm_q8_f16_m64
// (64 x 256 or 64 x 192, further down) for those whose large tiles would leave compute units idle, optionally with a
// tile's K shared by several workgroups and k_sum_partials adding their partial products in a fixed order;
// q8_gemm_f16_plan chooses.  A workgroup's tile follows from its index so that the workgroups of one column tile
// run on one XCD (tile_of_workgroup), and those of one K share too where K is shared (tile_of_share).
//
// Shape.  Workgroup tile 128 x 256, 256 threads = 4 wavefronts (2 x 2), one wavefront per SIMD; a wavefront owns
// 64 x 128 of C = 8 MFMA tiles of 32 x 32 = 128 fp32 accumulators per lane, kept in ordinary vector registers because
// the scaling reads and writes them with vector instructions.  All MFMA operands are in ordinary vector registers as
// well: products whose A/B operands sit in the accumulation registers run at about two thirds of the rate here.
// That budget (128 accumulators + 32 partial sums + 64 operand registers of 256) fixes the schedule: a K step of
// 32 is 8 passes of one 32 x 32 tile (4 dependent MFMAs: 2 K halves x hi/lo), two partial-sum tiles alternate, and in
// the shadow of a pass's MFMAs the wavefront issues the previous tile's 16 multiply-adds, the LDS reads of the
// operands it needs next, and its share of the loads for the step after next.  __builtin_amdgcn_sched_barrier pins
// that interleaving; the compiler still allocates registers and inserts the MFMA hazard waits.
//
// Stages and barriers.  Stage s % 3 holds K step s.  During step s a wavefront reads stage s (the second tile row,
// column 3) and, after a mid-step barrier, stage s + 1 (the next step's first tile row, columns 0-2, scales); the
// loads of step s + 2 are issued in the first half of step s into the stage that step s - 1 used, which every
// wavefront has left by the barrier at the top of step s.  Loads past the last step are clamped to it and land in a
// stage nobody reads again, so every step issues the same number of loads and the wait counts are constants.
// The direct loads are inline assembly (the compiler would otherwise wait for ALL of them before any LDS read), and
// the matching s_waitcnt vmcnt are written by hand; the kernel contains no other vector memory loads before its
// epilogue, so the compiler's own counting is not disturbed.
//
// Epilogue.  A wavefront passes its accumulators through its own quarter of LDS to turn the MFMA layout (a lane owns a
// column) into rows, then applies the row's power of two, bias / GELU / residual or the SwiGLU pairing on float4s and
// stores 16 bytes per lane.
#include "dj_common.h"
#include "gemm_epilogue.h"
#include <cstdlib>
#include <type_traits>

namespace dj {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));

namespace {

constexpr int TM = 128, TN = 256;
constexpr int kXs = 2 * TM * 64;            // bytes of the two activation planes of one stage: [plane][row][32 k] fp16
constexpr int kStages = 3;

struct GemmF16Args {
    const uint16_t *planes;     // [2][m_pad][pitch] fp16: hi plane, lo plane
    const uint16_t *w16;        // [n_pad][pitch] fp16
    const float *scales_t;      // [kp / 32][n_pad]
    const float *unscale;       // [m_pad]: 2^-s of the row
    float *out;
    int m, n, m_pad, n_pad, kp, pitch;
    int m_tiles, n_tiles;       // tiles of the launched kernel's size along M and N
    GemmEpilogue ep;
    int split_steps;            // 64-row kernel only: K steps per share of a tile (0: all of K, no partial sums); gridDim.z shares
    float *partial;             // [gridDim.z][m][n] partial products when split_steps > 0
};

// 64 lanes x 16 bytes from base + off[lane] into LDS bytes [dst, dst + 1024), lane order.  The statements write M0
// and say so in their clobber lists, so that the compiler never carries a value of its own in M0 across them (it
// initialises M0 itself for some LDS and message instructions); clang notes that M0 is a reserved register, which
// is the point of listing it.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load_to_lds16(const void *base, uint32_t off, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void load_to_lds4(const void *base, uint32_t off, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(dst), "v"(off), "s"(base) : "memory", "m0");
}
#pragma clang diagnostic pop

// Timeline of one launch, for tuning builds only (-DDJ_TRACE; never in the shipped library): every wavefront leaves
// 100 MHz time stamps at its start, at its first product, after its K loop and after its epilogue.
#ifdef DJ_TRACE
__device__ unsigned long long g_gemm_trace[4 * 16384];
#define DJ_GSTAMP(i) do { const int wg_ = (blockIdx.z * gridDim.x + blockIdx.x) * 4 + wave; if (lane == 0 && wg_ < 16384) g_gemm_trace[wg_ * 4 + (i)] = wall_clock64(); } while (0)
#else
#define DJ_GSTAMP(i) do {} while (0)
#endif

// Workgroup -> tile.  Workgroups go to the eight XCDs (each with its own L2) round-robin by their linear index, so index L
// runs on XCD L % 8.  All row tiles of one column tile get indices that agree mod 8: the column tile's weights - the
// bulk of the traffic - are then fetched into one L2 instead of up to eight.  Groups of eight column tiles; the grid is
// padded to whole groups and the surplus workgroups leave at once.
__device__ __forceinline__ bool tile_of_workgroup(int m_tiles, int n_tiles, int &m_tile, int &n_tile) {
    const int per_group = 8 * m_tiles, g = blockIdx.x / per_group, r = blockIdx.x % per_group;
    n_tile = g * 8 + (r & 7);
    m_tile = r >> 3;
    return n_tile < n_tiles;
}

// The same for a launch whose tiles share K among gridDim.z workgroups (share z takes K steps [z, z + 1) * split_steps).
// With the mapping above every XCD would run all shares and all row tiles of its column tiles and so fetch ALL activation
// planes - eight times the planes in all.  When the share count divides eight, an XCD instead takes ONE share and every
// (8 / shares)-th column tile: it fetches that share's quarter (half, eighth) of the planes and an eighth of the weights,
// as before.
__device__ __forceinline__ bool tile_of_share(int m_tiles, int n_tiles, int &m_tile, int &n_tile, int &z) {
    const int shares = gridDim.z;
    if (shares == 1 || (8 % shares) != 0) {
        z = blockIdx.z;
        return tile_of_workgroup(m_tiles, n_tiles, m_tile, n_tile);
    }
    const int idx = blockIdx.z * gridDim.x + blockIdx.x, c = idx & 7, r = idx >> 3;     // gridDim.x is a multiple of 8: XCD c
    z = c % shares;
    n_tile = c / shares + (8 / shares) * (r / m_tiles);
    m_tile = r % m_tiles;
    return n_tile < n_tiles;
}

// One tile row of a wavefront's block: acc[tn][e] is C[row0 + 8 (e / 4) + 4 half + e % 4][col0 + 32 tn + l32], TNW tiles
// wide.  The 32 x 32 TNW floats go through LDS that belongs to this wavefront alone (16 KB) and come back as rows of
// float4 (8 TNW lanes per row, two rows per round), which get bias / GELU / residual or the SwiGLU pairing; the row's
// power of two is applied before the trip through LDS.
// The powers of two of the 16 rows a lane holds of the tile row at row0 (four runs of four rows): requested together
// and applied on the way into LDS, so that the row loop holds no load a store would wait for.
struct RowFactors { float4 run[4]; };
__device__ __forceinline__ RowFactors load_row_factors(const GemmF16Args &a, int row0, int lane) {
    RowFactors f;
#pragma unroll
    for (int j = 0; j < 4; j++) f.run[j] = *reinterpret_cast<const float4 *>(a.unscale + row0 + 8 * j + 4 * (lane >> 5));
    return f;
}

template <int TNW, bool ROPE = false>
__device__ __forceinline__ void store_tile_row(const GemmF16Args &a, float *stage_f, const float (&acc)[TNW][16], int row0, int col0, int lane) {
    const RowFactors factors = load_row_factors(a, row0, lane);
    constexpr int W = 32 * TNW, LPR = 8 * TNW;                         // floats per row; lanes per row
    const GemmEpilogue &ep = a.ep;
    const int out_n = ep.swiglu ? a.n >> 1 : a.n;
    const int half = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int tn = 0; tn < TNW; tn++)
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const float4 u = factors.run[e >> 2];
            const float us = (e & 3) == 0 ? u.x : (e & 3) == 1 ? u.y : (e & 3) == 2 ? u.z : u.w;
            stage_f[(8 * (e >> 2) + 4 * half + (e & 3)) * W + 32 * tn + l32] = acc[tn][e] * us;
        }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int rsel = lane / LPR, c4 = lane % LPR;                      // this lane's row of the pair, and its float4 in the row
    const bool active = rsel < 2;
    const int col = col0 + c4 * 4;                                     // first of this lane's four columns
    float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active && ep.bias && col < a.n) {
        if (ep.interleaved_bias) {                                     // even column n: bias[n / 2], odd: bias2[n / 2]
            const float2 be = *reinterpret_cast<const float2 *>(ep.bias + (col >> 1)), bo = *reinterpret_cast<const float2 *>(ep.bias2 + (col >> 1));
            b4 = make_float4(be.x, bo.x, be.y, bo.y);
        } else {
            b4 = *reinterpret_cast<const float4 *>(ep.bias + col);
        }
    }
    constexpr bool rope = ROPE;      // (a compile-time variant: its sixteen table entries would cost every other launch registers)
    RopeColumn rc{0, 0, 0, 0};
    int pos0 = 0;
    float4 tab[ROPE ? 16 : 1];                                         // the rotation's table entries of the lane's 16 rows, requested together
    if (rope && active && col < a.n) {
        rc = rope_column(ep.rope, col);
        pos0 = ep.rope.state[0];
        if (rc.region < 2) {
#pragma unroll
            for (int i = 0; i < 16; i++) tab[i] = rope_table(ep.rope, rc, min(row0 + i * 2 + rsel, a.m - 1), pos0);
        }
    }
#pragma unroll(ROPE ? 16 : 4)
    for (int i = 0; i < 16; i++) {
        const int rl = i * 2 + rsel, row = row0 + rl;
        if (!active || row >= a.m || col >= a.n) continue;
        float4 v = *reinterpret_cast<const float4 *>(stage_f + rl * W + c4 * 4);
        if (ep.bias) { v.x = v.x + b4.x; v.y = v.y + b4.y; v.z = v.z + b4.z; v.w = v.w + b4.w; }
        if constexpr (ROPE) { rope_store(ep.rope, rc, v, row, pos0, tab[i]); continue; }
        if (ep.swiglu) {
            // (gate, up) pairs in neighbouring columns (SiLU.java:20-24, SwiGLULayer.java:69)
            float2 o;
            o.x = v.x * (1.0f / (1.0f + expf(-v.x))) * v.y;
            o.y = v.z * (1.0f / (1.0f + expf(-v.z))) * v.w;
            store_streaming(a.out + (int64_t)row * out_n + (col >> 1), o);
            continue;
        }
        if (ep.gelu) { v.x = gemm_gelu(v.x); v.y = gemm_gelu(v.y); v.z = gemm_gelu(v.z); v.w = gemm_gelu(v.w); }
        if (ep.residual) {
            const float4 r = *reinterpret_cast<const float4 *>(ep.residual + (int64_t)row * a.n + col);
            v.x = r.x + v.x; v.y = r.y + v.y; v.z = r.z + v.z; v.w = r.w + v.w;
        }
        store_streaming(a.out + (int64_t)row * a.n + col, v);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                  // the rows are in registers before anything overwrites them
}

// TNW: 32-column MFMA tiles per wavefront along N - 4 (workgroup tile 128 x 256, the shape described at the top) or 3
// (128 x 192: 512 rows against 11264 output rows are 176 tiles of the former on 256 compute units, 236 of the latter).
// A K step is 2 TNW passes; the schedule below places the same kinds of work in both.
constexpr int stage128_bytes(int tnw) { return kXs + 64 * tnw * 64 + 1024; }     // X planes, W rows, 256 scales

template <int TNW, bool ROPE = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) k_gemm_q8_f16(const GemmF16Args a) {
    static_assert(TNW == 3 || TNW == 4, "the slots of the schedule are written out for these");
    constexpr int kTn = 64 * TNW, kW = kTn * 64, kStageB = stage128_bytes(TNW);
    constexpr int kPasses = 2 * TNW;
    constexpr int kLoadsB = 5 + TNW;            // direct loads per wavefront per stage: 4 of X, TNW of W, 1 of scales
    extern __shared__ __align__(16) unsigned char lds[];
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1, half = lane >> 5, l32 = lane & 31;
    int m_tile, n_tile;
    if (!tile_of_workgroup(a.m_tiles, a.n_tiles, m_tile, n_tile)) return;
    DJ_GSTAMP(0);
    const int m0 = m_tile * TM, n0 = n_tile * kTn;
    const int64_t plane_elems = (int64_t)a.m_pad * a.pitch;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
    float acc[2][TNW][16];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < TNW; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.f;

    // A stage is made of 1 KB blocks of 16 rows x 4 chunks of 16 bytes (8 fp16); row r keeps chunk c at slot
    // c ^ ((r >> 2) & 3), which spreads the 32 rows an MFMA operand read touches over all LDS banks.  A direct load
    // writes lane order, so lane p fetches the chunk that belongs at slot p & 3 of row p >> 2.  The lane's byte
    // offset is the same in every block; a block's origin is wave-uniform.
    const int prow = lane >> 2, pchunk = (lane & 3) ^ ((prow >> 2) & 3);
    const uint32_t op_lane = (uint32_t)((prow * a.pitch + pchunk * 8) * 2), s_lane = lane * 4;
    const unsigned char *x_base[4], *w_base[TNW];
    uint32_t x_dst[4], w_dst[TNW];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int blk = wave * 4 + i, pl = blk >> 3, rb = blk & 7;      // X: 2 planes x 8 row blocks
        x_base[i] = reinterpret_cast<const unsigned char *>(a.planes) + (pl * plane_elems + (int64_t)(m0 + rb * 16) * a.pitch) * 2;
        x_dst[i] = pl * TM * 64 + rb * 1024;
    }
#pragma unroll
    for (int i = 0; i < TNW; i++) {
        const int blk = wave * TNW + i;                                 // W: 4 TNW row blocks
        w_base[i] = reinterpret_cast<const unsigned char *>(a.w16) + (int64_t)(n0 + blk * 16) * a.pitch * 2;
        w_dst[i] = kXs + blk * 1024;
    }
    // every wavefront fetches 64 scales; with TNW = 3 the last 64 belong to the next column tile and are never read
    const unsigned char *s_base = reinterpret_cast<const unsigned char *>(a.scales_t) + (int64_t)(n0 + wave * 64) * 4;
    const uint32_t s_dst = kXs + kW + wave * 256;
    const int steps = a.kp / 32, last = steps - 1;
    auto load_one = [&](int i, int step, int stage) {
        const uint32_t sb = lds0 + stage * kStageB;
        step = min(step, last);
        if (i < 4) load_to_lds16(x_base[i] + (int64_t)step * 64, op_lane, sb + x_dst[i]);
        else if (i < 4 + TNW) load_to_lds16(w_base[i - 4] + (int64_t)step * 64, op_lane, sb + w_dst[i - 4]);
        else load_to_lds4(s_base + (int64_t)step * a.n_pad * 4, s_lane, sb + s_dst);
    };

    // MFMA operand addresses: lane l32 + 32 * half reads row l32, K chunk 2 * sub + half of its tile
    const int sw = (l32 >> 2) & 3;
    const int lane_sub0 = (l32 << 6) + (((0 + half) ^ sw) << 4), lane_sub1 = (l32 << 6) + (((2 + half) ^ sw) << 4);
    const int x_wave = wm * 64 * 64, w_wave = kXs + wn * (32 * TNW) * 64, s_wave = kXs + kW + wn * (32 * TNW) * 4 + l32 * 4;
    const floatx16 z16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    halfx8 fx[2][2][2];                 // [tile row][K half][hi, lo]
    halfx8 fw[2][TNW];                  // [K half][tile column]
    float sc[TNW];                      // [tile column]
    floatx16 g[2] = {z16, z16};         // partial sums of the tile in flight and of the one being scaled
#pragma unroll
    for (int j = 0; j < TNW; j++) sc[j] = 0.f;
    struct Addr { const unsigned char *x0, *x1, *w0, *w1, *s; };
    auto addr_of = [&](int stage) {
        const unsigned char *sb = lds + stage * kStageB;
        return Addr{sb + x_wave + lane_sub0, sb + x_wave + lane_sub1, sb + w_wave + lane_sub0, sb + w_wave + lane_sub1, sb + s_wave};
    };
    auto read_x = [&](int tm, int q, const Addr &ad) {      // q = K half * 2 + piece
        const int sub = q >> 1, piece = q & 1;
        fx[tm][sub][piece] = *reinterpret_cast<const halfx8 *>((sub ? ad.x1 : ad.x0) + piece * TM * 64 + tm * 2048);
    };
    auto read_w = [&](int sub, int tn, const Addr &ad) { fw[sub][tn] = *reinterpret_cast<const halfx8 *>((sub ? ad.w1 : ad.w0) + tn * 2048); };

    auto k_step = [&](int step, int stage) {
        const int sy = stage == 2 ? 0 : stage + 1, sz = sy == 2 ? 0 : sy + 1;
        const Addr ax = addr_of(stage);
        const int dy = (sy - stage) * kStageB;
        __builtin_amdgcn_s_barrier();                                  // every wavefront has left stage sz
        asm volatile("" ::: "memory");
#pragma unroll
        for (int k = 0; k < kPasses; k++) {
            const int tm = k / TNW, tn = k % TNW, par = k & 1;
            const int pk = (k + kPasses - 1) % kPasses, ptm = pk / TNW, ptn = pk % TNW;   // the tile finished by the previous pass
            if (k == TNW) {
                // this wavefront's loads of step + 1 have landed (all but the kLoadsB of step + 2 it has issued since) ...
                if (TNW == 4) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
                __builtin_amdgcn_s_barrier();                          // ... and so have everyone's
                asm volatile("" ::: "memory");
            }
            const Addr ay = Addr{ax.x0 + dy, ax.x1 + dy, ax.w0 + dy, ax.w1 + dy, ax.s + dy};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int sub = i >> 1, piece = i & 1;
                g[par] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fx[tm][sub][piece], fw[sub][tn], i == 0 ? z16 : g[par], 0, 0, 0);
                // the previous tile's scaling, one slot away from the MFMA that completed it
                const int f0 = i <= 1 ? 0 : i == 2 ? 6 : 11, f1 = i == 0 ? 0 : i == 1 ? 6 : i == 2 ? 11 : 16;
#pragma unroll
                for (int f = f0; f < f1; f++) acc[ptm][ptn][f] = fmaf(g[1 - par][f], sc[ptn], acc[ptm][ptn][f]);
                // the last column of this step (operands, scale) in pass 0 - its registers were in use until the end of the
                // previous step; the other columns of the next step as this step leaves them, from pass TNW + 1 on
                if (k == 0 && i < 2) read_w(i, TNW - 1, ax);
                if (k >= TNW + 1 && i < 2) read_w(i, k - (TNW + 1), ay);
                if (k == 0 && i == 3) sc[TNW - 1] = *reinterpret_cast<const float *>(ax.s + (TNW - 1) * 128);
                if (k >= TNW + 1 && i == 3) sc[k - (TNW + 1)] = *reinterpret_cast<const float *>(ay.s + (k - (TNW + 1)) * 128);
                // the four operand reads of this step's second tile row in its first half, of the next step's first
                // tile row in its second half; the loads of step + 2 in the first half
                if constexpr (TNW == 4) {
                    if (k < 4 && i == 2) read_x(1, k, ax);
                    if (k >= 4 && i == 2) read_x(0, k - 4, ay);
                    if (k < 4 && (i == 1 || i == 3)) load_one(k * 2 + (i >> 1), step + 2, sz);
                    if (k == 3 && i == 0) load_one(8, step + 2, sz);
                } else {
                    if (k < 3 && i == 2) read_x(1, k, ax);
                    if (k == 2 && i == 0) read_x(1, 3, ax);
                    if (k >= 3 && i == 2) read_x(0, k - 3, ay);
                    if (k == 3 && i == 0) read_x(0, 3, ay);
                    if (k < 3 && (i == 1 || i == 3)) load_one(k * 2 + (i >> 1), step + 2, sz);
                    if (k == 1 && i == 0) load_one(6, step + 2, sz);
                    if (k == 2 && i == 2) load_one(7, step + 2, sz);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    for (int s = 0; s < 2; s++)
        for (int i = 0; i < kLoadsB; i++) load_one(i, s, s);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    {
        const Addr a0 = addr_of(0);
        for (int q = 0; q < 4; q++) read_x(0, q, a0);
        for (int tn = 0; tn < TNW - 1; tn++) { read_w(0, tn, a0); read_w(1, tn, a0); }
        for (int tn = 0; tn < TNW - 1; tn++) sc[tn] = *reinterpret_cast<const float *>(a0.s + tn * 128);
    }
    DJ_GSTAMP(1);
    int stage = 0;
    for (int step = 0; step < steps; step++) {
        k_step(step, stage);
        stage = stage == 2 ? 0 : stage + 1;
    }
    DJ_GSTAMP(2);
    // the last tile's scaling; its scale (the last column of the last step) is still in place
#pragma unroll
    for (int e = 0; e < 16; e++) acc[1][TNW - 1][e] = fmaf(g[1][e], sc[TNW - 1], acc[1][TNW - 1][e]);
    // no direct load may still be writing LDS when the epilogue reuses it or the workgroup ends
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    float *stage_f = reinterpret_cast<float *>(lds + wave * (32 * 128 * 4));
#pragma unroll
    for (int tm = 0; tm < 2; tm++) store_tile_row<TNW, ROPE>(a, stage_f, acc[tm], m0 + wm * 64 + 32 * tm, n0 + wn * (32 * TNW), lane);
    DJ_GSTAMP(3);
}

// The same product on a 64-row workgroup tile, 256 (TNW = 4) or 192 (TNW = 3) columns wide, for problems whose 128-row
// tiles would leave most of the chip idle (a 512-row prompt against 6144 output rows is 96 such tiles on 256 compute
// units, 192 of 64 x 256 and exactly 256 of 64 x 192).  A wavefront owns one tile row (32 rows x 32 TNW columns, 16 TNW
// accumulators), which leaves registers for two complete operand sets: everything step s + 1 needs is read from its
// stage during step s, a stage is only ever read during the step before its own, and the loads of step s + 3 go into
// the stage of step s at the top of step s, behind one barrier per step - two steps of distance for the direct loads
// instead of one.  Stage: 8 KB of X (2 planes x 64 rows), 4 TNW KB of W, 1 KB of scales (every wavefront fetches 64 of
// them; with TNW = 3 the last 64 belong to the next column tile and are never read).
constexpr int TM64 = 64;
constexpr int kXs64 = 2 * TM64 * 64;
constexpr int stage64_bytes(int tnw) { return kXs64 + 64 * tnw * 64 + 1024; }
constexpr int kMinSplitSteps = 8;           // K steps a workgroup must at least have when several share a tile's K

template <int TNW, bool ROPE = false>
__global__ void __launch_bounds__(256) k_gemm_q8_f16_m64(const GemmF16Args a) {
    constexpr int kTn = 64 * TNW, kW = kTn * 64, kStage64 = stage64_bytes(TNW);
    constexpr int kLoads64 = TNW + 3;           // per wavefront per stage: 2 of X, TNW of W, 1 of scales
    constexpr int kReads = 4 + 3 * TNW, kSlots = 4 * TNW;
    static_assert(TNW == 3 || TNW == 4, "the wait counts below are written out for these");
    extern __shared__ __align__(16) unsigned char lds[];
    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1, half = lane >> 5, l32 = lane & 31;
    int m_tile, n_tile, share;
    if (!tile_of_share(a.m_tiles, a.n_tiles, m_tile, n_tile, share)) return;
    DJ_GSTAMP(0);
    const int m0 = m_tile * TM64, n0 = n_tile * kTn;
    const int64_t plane_elems = (int64_t)a.m_pad * a.pitch;
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
    float acc[TNW][16];
#pragma unroll
    for (int j = 0; j < TNW; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[j][e] = 0.f;

    const int prow = lane >> 2, pchunk = (lane & 3) ^ ((prow >> 2) & 3);
    const uint32_t op_lane = (uint32_t)((prow * a.pitch + pchunk * 8) * 2), s_lane = lane * 4;
    const unsigned char *x_base[2], *w_base[TNW];
    uint32_t x_dst[2], w_dst[TNW];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int blk = wave * 2 + i, pl = blk >> 2, rb = blk & 3;      // X: 2 planes x 4 row blocks
        x_base[i] = reinterpret_cast<const unsigned char *>(a.planes) + (pl * plane_elems + (int64_t)(m0 + rb * 16) * a.pitch) * 2;
        x_dst[i] = pl * TM64 * 64 + rb * 1024;
    }
#pragma unroll
    for (int i = 0; i < TNW; i++) {
        const int blk = wave * TNW + i;                                 // W: 4 TNW row blocks
        w_base[i] = reinterpret_cast<const unsigned char *>(a.w16) + (int64_t)(n0 + blk * 16) * a.pitch * 2;
        w_dst[i] = kXs64 + blk * 1024;
    }
    const unsigned char *s_base = reinterpret_cast<const unsigned char *>(a.scales_t) + (int64_t)(n0 + wave * 64) * 4;
    const uint32_t s_dst = kXs64 + kW + wave * 256;
    // this workgroup's share of K: all of it, or split_steps steps from share * split_steps (a partial product)
    const int all_steps = a.kp / 32, first = a.split_steps ? share * a.split_steps : 0;
    const int steps = a.split_steps ? min(a.split_steps, all_steps - first) : all_steps, last = first + steps - 1;
    auto load_one = [&](int i, int step, int stage) {
        const uint32_t sb = lds0 + stage * kStage64;
        step = min(first + step, last);
        if (i < 2) load_to_lds16(x_base[i] + (int64_t)step * 64, op_lane, sb + x_dst[i]);
        else if (i < 2 + TNW) load_to_lds16(w_base[i - 2] + (int64_t)step * 64, op_lane, sb + w_dst[i - 2]);
        else load_to_lds4(s_base + (int64_t)step * a.n_pad * 4, s_lane, sb + s_dst);
    };

    const int sw = (l32 >> 2) & 3;
    const int lane_sub0 = (l32 << 6) + (((0 + half) ^ sw) << 4), lane_sub1 = (l32 << 6) + (((2 + half) ^ sw) << 4);
    const int x_wave = wm * 32 * 64, w_wave = kXs64 + wn * (32 * TNW) * 64, s_wave = kXs64 + kW + wn * (32 * TNW) * 4 + l32 * 4;
    const floatx16 z16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    halfx8 fx[2][2][2];                 // [set][K half][hi, lo]
    halfx8 fw[2][2][TNW];               // [set][K half][tile column]
    float sc[2][TNW];                   // [set][tile column]
    floatx16 g[2] = {z16, z16};
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < TNW; j++) sc[i][j] = 0.f;
    // read n of the kReads LDS reads that fetch a step's operands, in the order of their first use
    auto read_one = [&](auto set_c, int n, const unsigned char *x0, const unsigned char *x1, const unsigned char *w0, const unsigned char *w1, const unsigned char *sp) {
        constexpr int set = decltype(set_c)::value;
        if (n < 4) fx[set][n >> 1][n & 1] = *reinterpret_cast<const halfx8 *>(((n >> 1) ? x1 : x0) + (n & 1) * TM64 * 64);
        else if (n < 4 + 2 * TNW) { const int tn = (n - 4) >> 1, sub = (n - 4) & 1; fw[set][sub][tn] = *reinterpret_cast<const halfx8 *>((sub ? w1 : w0) + tn * 2048); }
        else sc[set][n - 4 - 2 * TNW] = *reinterpret_cast<const float *>(sp + (n - 4 - 2 * TNW) * 128);
    };
    auto k_step = [&](auto set_c, int step, int stage) {
        constexpr int set = decltype(set_c)::value;
        // step + 1 has landed (step + 2 may be in flight); this step's operands are in registers
        if (TNW == 4) asm volatile("s_waitcnt vmcnt(7) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const int next = stage == 2 ? 0 : stage + 1;
        const unsigned char *nb = lds + next * kStage64;
        const unsigned char *x0 = nb + x_wave + lane_sub0, *x1 = nb + x_wave + lane_sub1, *w0 = nb + w_wave + lane_sub0, *w1 = nb + w_wave + lane_sub1, *sp = nb + s_wave;
#pragma unroll
        for (int tn = 0; tn < TNW; tn++) {
            // the partial-sum registers alternate from tile to tile, across the step boundary as well
            const int par = (set * TNW + tn) & 1, ptn = (tn + TNW - 1) % TNW, pset = tn == 0 ? 1 - set : set;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int sub = i >> 1, piece = i & 1, slot = tn * 4 + i;
                g[par] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fx[set][sub][piece], fw[set][sub][tn], i == 0 ? z16 : g[par], 0, 0, 0);
                const int f0 = i <= 1 ? 0 : i == 2 ? 6 : 11, f1 = i == 0 ? 0 : i == 1 ? 6 : i == 2 ? 11 : 16;
#pragma unroll
                for (int f = f0; f < f1; f++) acc[ptn][f] = fmaf(g[1 - par][f], sc[pset][ptn], acc[ptn][f]);
                // the next step's operands: two reads per slot at first, so that the last slots have none in flight
                // when the next step begins by waiting for them
                constexpr int kDouble = kReads - (kSlots - 4);         // slots that carry two reads
                if (slot < kDouble) {
                    read_one(std::integral_constant<int, 1 - set>{}, 2 * slot, x0, x1, w0, w1, sp);
                    read_one(std::integral_constant<int, 1 - set>{}, 2 * slot + 1, x0, x1, w0, w1, sp);
                } else if (slot < kSlots - 4) {
                    read_one(std::integral_constant<int, 1 - set>{}, slot + kDouble, x0, x1, w0, w1, sp);
                }
                if ((slot & 1) && (slot >> 1) < kLoads64) load_one(slot >> 1, step + 3, stage);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    for (int s = 0; s < 3; s++)
        for (int i = 0; i < kLoads64; i++) load_one(i, s, s);
    if (TNW == 4) asm volatile("s_waitcnt vmcnt(14)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    {
        const unsigned char *x0 = lds + x_wave + lane_sub0, *x1 = lds + x_wave + lane_sub1, *w0 = lds + w_wave + lane_sub0, *w1 = lds + w_wave + lane_sub1, *sp = lds + s_wave;
        for (int n = 0; n < kReads; n++) read_one(std::integral_constant<int, 0>{}, n, x0, x1, w0, w1, sp);
    }
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    DJ_GSTAMP(1);
    int stage = 0, step = 0;
    for (; step + 1 < steps; step += 2) {
        const int st1 = stage == 2 ? 0 : stage + 1;
        k_step(S0{}, step, stage);
        k_step(S1{}, step + 1, st1);
        stage = st1 == 2 ? 0 : st1 + 1;
    }
    if (step < steps) k_step(S0{}, step, stage);
    DJ_GSTAMP(2);
    // the last tile's scaling: the last column of the last step, whose set (and partial-sum register) follow that step's parity
    {
        const bool odd = (steps - 1) & 1;
        const bool in_g1 = ((odd ? TNW : 0) + TNW - 1) & 1;
#pragma unroll
        for (int e = 0; e < 16; e++) acc[TNW - 1][e] = fmaf(in_g1 ? g[1][e] : g[0][e], odd ? sc[1][TNW - 1] : sc[0][TNW - 1], acc[TNW - 1][e]);
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    float *stage_f = reinterpret_cast<float *>(lds + wave * (32 * 128 * 4));
    if (a.split_steps) {
        // a partial product: the bare sums (times the row's power of two) into this split's slab; k_sum_partials finishes them
        GemmF16Args b = a;
        b.out = a.partial + (int64_t)share * a.m * a.n;
        b.ep = GemmEpilogue{nullptr, nullptr, nullptr, 0, nullptr, 0, 0, 0};
        store_tile_row<TNW>(b, stage_f, acc, m0 + wm * 32, n0 + wn * 32 * TNW, lane);
        DJ_GSTAMP(3);
        return;
    }
    store_tile_row<TNW, ROPE>(a, stage_f, acc, m0 + wm * 32, n0 + wn * 32 * TNW, lane);
    DJ_GSTAMP(3);
}

// out = epilogue(sum over the splits of partial[z]) on float4s: bias, GELU, residual or the SwiGLU pairing as in
// store_tile_row (a fixed order of additions, so a run repeats bit for bit - which adding into C with atomics would not)
__global__ void __launch_bounds__(256) k_sum_partials(const float *__restrict__ partial, float *__restrict__ out, int splits, int64_t mn4, int n4,
                                                     const GemmEpilogue ep) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < mn4; i += (int64_t)gridDim.x * 256) {
        float4 v = reinterpret_cast<const float4 *>(partial)[i];
        for (int z = 1; z < splits; z++) {
            const float4 p = reinterpret_cast<const float4 *>(partial)[(int64_t)z * mn4 + i];
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        const int c4 = (int)(i % n4);                                   // this float4's place in its row
        if (ep.bias) {
            float4 b;
            if (ep.interleaved_bias) {                                  // even column n: bias[n / 2], odd: bias2[n / 2]
                const float2 be = reinterpret_cast<const float2 *>(ep.bias)[c4], bo = reinterpret_cast<const float2 *>(ep.bias2)[c4];
                b = make_float4(be.x, bo.x, be.y, bo.y);
            } else {
                b = reinterpret_cast<const float4 *>(ep.bias)[c4];
            }
            v.x = v.x + b.x; v.y = v.y + b.y; v.z = v.z + b.z; v.w = v.w + b.w;
        }
        if (ep.swiglu) {                                                // (gate, up) pairs in neighbouring columns
            float2 o;
            o.x = v.x * (1.0f / (1.0f + expf(-v.x))) * v.y;
            o.y = v.z * (1.0f / (1.0f + expf(-v.z))) * v.w;
            reinterpret_cast<float2 *>(out)[i] = o;                     // row * (n / 2) + col / 2 = 2 i floats in
            continue;
        }
        if (ep.gelu) { v.x = gemm_gelu(v.x); v.y = gemm_gelu(v.y); v.z = gemm_gelu(v.z); v.w = gemm_gelu(v.w); }
        if (ep.residual) {
            const float4 r = reinterpret_cast<const float4 *>(ep.residual)[i];
            v.x = r.x + v.x; v.y = r.y + v.y; v.z = r.z + v.z; v.w = r.w + v.w;
        }
        reinterpret_cast<float4 *>(out)[i] = v;
    }
}

// One workgroup per row of X: the row's normalisation if asked for (NORM 1: gamma * x / sqrt(mean(x^2) + 1e-6),
// RMSNorm1D.java:46-57; NORM 2: gamma * (x - mean) / sqrt(var + 1e-5) + beta, LayerNorm1D.java:34-66; the same formulas
// and unfused multiply-adds as the stand-alone kernels), the largest magnitude of the result, then the two fp16 planes
// of it times 2^s.  Rows of up to 8192 floats stay in registers in between; longer or ragged ones are read three or four
// times, from L2 after the first.  Columns [k, kp) are written as zeros
// (the weights' padding is zero as well, but 0 x garbage could be a NaN).  The grid covers the rows the GEMM's tiles
// read, which may go past m: those rows only feed output rows that are never stored, and are written as zeros so that
// the GEMM never multiplies what an earlier user of the workspace left there.
// SUM: the row is not read from x but put together first - the sum over `splits` slabs of partial products of a
// K-sharing GEMM, plus bias and residual in the order that GEMM's own epilogue uses - and written to sum_out as that
// GEMM's result; what follows is the next GEMM's prologue on it.  One kernel where the two GEMMs would otherwise launch
// one each (the sum of the slabs, the split of the rows).  Rows that fit the register path only.
struct SplitSum { const float *partial; int splits; int64_t slab; const float *bias, *residual; float *sum_out; };

template <int NORM, bool SUM = false>
__global__ void __launch_bounds__(256) k_split_f16(const float *__restrict__ x, const float *__restrict__ gamma, const float *__restrict__ beta,
                                                   uint16_t *__restrict__ planes, float *__restrict__ unscale, int m, int k, int kp, int pitch,
                                                   int64_t plane_elems, const SplitSum sum) {
#pragma clang fp contract(off)
    __shared__ float red[4];
    const int row = blockIdx.x, t = threadIdx.x;
    if (row >= m) {
        uint32_t *hi32 = reinterpret_cast<uint32_t *>(planes + (int64_t)row * pitch), *lo32 = hi32 + plane_elems / 2;
        for (int c = t; c < kp / 2; c += 256) { hi32[c] = 0u; lo32[c] = 0u; }
        if (t == 0) unscale[row] = 0.f;
        return;
    }
    const float *xr = x + (int64_t)row * k;
    auto block_reduce = [&](float v, bool is_max) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { const float u = __shfl_xor(v, o, 64); v = is_max ? fmaxf(v, u) : v + u; }
        __syncthreads();
        if ((t & 63) == 0) red[t >> 6] = v;
        __syncthreads();
        return is_max ? fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])) : ((red[0] + red[1]) + red[2]) + red[3];
    };
    auto scale_of = [&](float mx) {
        // mx = f * 2^e with f in [0.5, 1): s = 15 - e puts it in [2^14, 2^15).  Zero, infinite or NaN rows stay
        // unscaled; s is kept where 2^s and 2^-s are both normal numbers.
        int s = 0;
        if (mx > 0.f && mx < __builtin_inff()) {
            int e;
            (void)frexpf(mx, &e);
            s = max(-126, min(126, 15 - e));
        }
        if (t == 0) unscale[row] = ldexpf(1.0f, -s);
        return ldexpf(1.0f, s);
    };
    auto halves = [](float v, uint16_t &h, uint16_t &l) {
        const _Float16 hh = (_Float16)v;
        const _Float16 ll = (_Float16)(v - (float)hh);
        h = __builtin_bit_cast(uint16_t, hh);
        l = __builtin_bit_cast(uint16_t, ll);
    };
    uint16_t *hi = planes + (int64_t)row * pitch, *lo = hi + plane_elems;
    constexpr int NV = 8;                                            // 128-bit words a thread keeps of one row
    if (SUM || ((k & 3) == 0 && k == kp && k <= 256 * 4 * NV)) {
        // the row stays in registers: one pass over memory
        const int n4 = k >> 2;
        const float4 *row4 = reinterpret_cast<const float4 *>(xr);
        float4 v[NV];
        float s1 = 0.f;
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = t + j * 256;
            if constexpr (SUM) {
                v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (i < n4) {
                    const float4 *p4 = reinterpret_cast<const float4 *>(sum.partial + (int64_t)row * k) + i;
                    float4 a = *p4;
                    for (int z = 1; z < sum.splits; z++) {
                        const float4 q = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p4) + (int64_t)z * sum.slab);
                        a.x += q.x; a.y += q.y; a.z += q.z; a.w += q.w;
                    }
                    if (sum.bias) {
                        const float4 b = reinterpret_cast<const float4 *>(sum.bias)[i];
                        a.x = a.x + b.x; a.y = a.y + b.y; a.z = a.z + b.z; a.w = a.w + b.w;
                    }
                    if (sum.residual) {
                        const float4 r = reinterpret_cast<const float4 *>(sum.residual + (int64_t)row * k)[i];
                        a.x = r.x + a.x; a.y = r.y + a.y; a.z = r.z + a.z; a.w = r.w + a.w;
                    }
                    reinterpret_cast<float4 *>(sum.sum_out + (int64_t)row * k)[i] = a;
                    v[j] = a;
                }
                if (NORM == 1) s1 += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
                if (NORM == 2) s1 += (v[j].x + v[j].y) + (v[j].z + v[j].w);
                continue;
            }
            v[j] = i < n4 ? row4[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            if (NORM == 1) s1 += v[j].x * v[j].x + v[j].y * v[j].y + v[j].z * v[j].z + v[j].w * v[j].w;
            if (NORM == 2) s1 += (v[j].x + v[j].y) + (v[j].z + v[j].w);
        }
        if (NORM == 1) {
            const float rms = sqrtf(block_reduce(s1, false) * (1.0f / (float)k) + kRmsEps);
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int i = t + j * 256;
                if (i >= n4) continue;
                const float4 g = reinterpret_cast<const float4 *>(gamma)[i];
                v[j] = make_float4((v[j].x / rms) * g.x, (v[j].y / rms) * g.y, (v[j].z / rms) * g.z, (v[j].w / rms) * g.w);
            }
        } else if (NORM == 2) {
            const float inv = 1.0f / (float)k, mean = block_reduce(s1, false) * inv;
            float var = 0.f;
#pragma unroll
            for (int j = 0; j < NV; j++) {
                if (t + j * 256 >= n4) continue;
                const float a = v[j].x - mean, b = v[j].y - mean, c = v[j].z - mean, d = v[j].w - mean;
                var += (a * a + b * b) + (c * c + d * d);
            }
            const float sd = sqrtf(block_reduce(var, false) * inv + kLayerNormEps);
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int i = t + j * 256;
                if (i >= n4) continue;
                const float4 g = reinterpret_cast<const float4 *>(gamma)[i], bt = reinterpret_cast<const float4 *>(beta)[i];
                v[j] = make_float4(((v[j].x - mean) / sd) * g.x + bt.x, ((v[j].y - mean) / sd) * g.y + bt.y,
                                   ((v[j].z - mean) / sd) * g.z + bt.z, ((v[j].w - mean) / sd) * g.w + bt.w);
            }
        }
        float mx = 0.f;
#pragma unroll
        for (int j = 0; j < NV; j++) mx = fmaxf(mx, fmaxf(fmaxf(fabsf(v[j].x), fabsf(v[j].y)), fmaxf(fabsf(v[j].z), fabsf(v[j].w))));
        const float up = scale_of(block_reduce(mx, true));
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = t + j * 256;
            if (i >= n4) continue;
            uint16_t h[4], l[4];
            halves(v[j].x * up, h[0], l[0]); halves(v[j].y * up, h[1], l[1]); halves(v[j].z * up, h[2], l[2]); halves(v[j].w * up, h[3], l[3]);
            reinterpret_cast<uint2 *>(hi)[i] = make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
            reinterpret_cast<uint2 *>(lo)[i] = make_uint2(l[0] | ((uint32_t)l[1] << 16), l[2] | ((uint32_t)l[3] << 16));
        }
        return;
    }
    float mean = 0.f, denom = 1.f;
    if (NORM == 1) {
        float ss = 0.f;
        for (int c = t; c < k; c += 256) { const float v = xr[c]; ss += v * v; }
        denom = sqrtf(block_reduce(ss, false) * (1.0f / (float)k) + kRmsEps);
    } else if (NORM == 2) {
        const float inv = 1.0f / (float)k;
        float sm = 0.f;
        for (int c = t; c < k; c += 256) sm += xr[c];
        mean = block_reduce(sm, false) * inv;
        float var = 0.f;
        for (int c = t; c < k; c += 256) { const float d = xr[c] - mean; var += d * d; }
        denom = sqrtf(block_reduce(var, false) * inv + kLayerNormEps);
    }
    auto value = [&](int c) {
        const float v = xr[c];
        if (NORM == 1) return (v / denom) * gamma[c];
        if (NORM == 2) return ((v - mean) / denom) * gamma[c] + beta[c];
        return v;
    };
    float mx = 0.f;
    for (int c = t; c < k; c += 256) mx = fmaxf(mx, fabsf(value(c)));
    const float up = scale_of(block_reduce(mx, true));
    for (int c = t; c < kp; c += 256) {
        uint16_t h, l;
        halves(c < k ? value(c) * up : 0.f, h, l);
        hi[c] = h;
        lo[c] = l;
    }
}

// int8 weights [rows x kp] -> fp16 [rows x pitch] (8 per thread), scales [rows x groups] -> [groups x n_pad]; rows
// [rows, rows_read) - what a last column tile of either width reads past the weight - become zeros
__global__ void __launch_bounds__(256) k_q8_to_f16(const int8_t *__restrict__ wq, const float *__restrict__ scales, uint16_t *__restrict__ w16,
                                                   float *__restrict__ scales_t, int rows, int rows_read, int kp, int pitch, int n_pad) {
    const int chunks = kp >> 3;
    const int64_t total = (int64_t)rows_read * chunks;
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int row = (int)(idx / chunks), c = (int)(idx % chunks);
        if (row >= rows) {                                   // rows the last column tile reads past the weight: zeros
            *reinterpret_cast<uint4 *>(w16 + (int64_t)row * pitch + c * 8) = make_uint4(0u, 0u, 0u, 0u);
            if ((c & 3) == 0) scales_t[(int64_t)(c >> 2) * n_pad + row] = 0.f;
            continue;
        }
        const int2 q = *reinterpret_cast<const int2 *>(wq + (int64_t)row * kp + c * 8);
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int w = j < 2 ? q.x : q.y, sh = (j & 1) * 16;
            const _Float16 a = (_Float16)(float)(int8_t)((w >> sh) & 0xff), b = (_Float16)(float)(int8_t)((w >> (sh + 8)) & 0xff);
            o[j] = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
        }
        *reinterpret_cast<uint4 *>(w16 + (int64_t)row * pitch + c * 8) = make_uint4(o[0], o[1], o[2], o[3]);
        if ((c & 3) == 0) scales_t[(int64_t)(c >> 2) * n_pad + row] = scales[(int64_t)row * (kp >> 5) + (c >> 2)];
    }
}

}  // namespace

// How these kernels take a problem: the workgroup tile (rows 128 or 64, columns 256 or 192; rows 0: not at all), and for
// the 64-row kernel the number of workgroups that share K (1: none).  A compute unit runs one workgroup at a time, so
// what counts is how many of the 256 a launch keeps busy and for how many rounds.
struct GemmF16Plan { int tile_rows, tile_cols, splits; };

constexpr int kNPad = 768;      // weight rows of a prepared buffer are padded to a multiple of both tile widths

constexpr int kMinRowsPrepared = 16;     // fewer rows than this stay on the bf16 kernels even with prepared weights

GemmF16Plan q8_gemm_f16_plan(int m, int n_rows, int k, bool prepared) {
    // DEEPJ_HIP_GEMM_F16=0 keeps every GEMM on the bf16 kernels; =128, =128192, =64 or =192 force the 128 x 256,
    // 128 x 192, 64 x 256 or 64 x 192 tile (for comparisons)
    static const int forced = [] { const char *e = getenv("DEEPJ_HIP_GEMM_F16"); return e ? atoi(e) : -1; }();
    if (forced == 0) return {0, 0, 1};
    // four columns per lane in the epilogue need n_rows % 4 == 0
    if ((n_rows & 3) != 0 || k < 64) return {0, 0, 1};
    // Fewer than 256 rows: only when the weights are already in these kernels' layout - a conversion per call costs more
    // than the launch gains.
    if (m < 256 && (!prepared || m < kMinRowsPrepared || forced > 0)) return {0, 0, 1};
    const int64_t rows128 = (m + TM - 1) / TM, rows64 = (m + TM64 - 1) / TM64, cols256 = (n_rows + 255) / 256, cols192 = (n_rows + 191) / 192;
    const int64_t t128 = rows128 * cols256, t128n = rows128 * cols192, t64 = rows64 * cols256, t64n = rows64 * cols192;
    if (forced == 128 || forced == 128192 || forced == 64 || forced == 192) {
        if (t64 < 128) return {0, 0, 1};
        return forced == 128 ? GemmF16Plan{128, 256, 1} : forced == 128192 ? GemmF16Plan{128, 192, 1} : forced == 64 ? GemmF16Plan{64, 256, 1} : GemmF16Plan{64, 192, 1};
    }
    // Enough tiles for several rounds: the large tile.  Around one round the time is rounds x one tile's time, and a
    // tile's time goes with its area over its efficiency (measured at 512 rows, K 2048: a 128 x 256 tile 58 us of K
    // loop + 11 us of prologue and epilogue, 64 x 256 35 + 10, 64 x 192 27 + 9; a 128 x 192 tile takes almost as long as
    // a 128 x 256 one - 236 of them 66.2 us where 176 of those take 67.6 - so it only wins where it saves a round or
    // fills idle compute units): take the cheapest.
    if (t128 >= 512) return {128, 256, 1};
    auto rounds = [](int64_t tiles) { return (tiles + 255) / 256; };
    const double c128 = rounds(t128) * 1.00, c128n = rounds(t128n) * 0.98, c64 = rounds(t64) * 0.65, c64n = rounds(t64n) * 0.52;
    if (t64 >= 128) {
        if (t128n >= 160 && c128n < c128 && c128n < c64 && c128n < c64n) return {128, 192, 1};
        if (t128 >= 160 && c128 <= c64 && c128 <= c64n) return {128, 256, 1};
        return c64n < c64 ? GemmF16Plan{64, 192, 1} : GemmF16Plan{64, 256, 1};
    }
    // Few tiles: several workgroups per tile, each with a share of K of at least kMinSplitSteps steps, their partial
    // products summed by a second kernel - as many workgroups as that allows, on the tile width that gives more of them
    // (the wider one unless the narrower gives 5 % more).  Worth it when there is enough work to stream: K of 1536 or more
    // (512 x 2048 over K 1024: 25 us against 17.5 on the bf16 kernels) and 48 narrow tiles or more, or 40 with a long K.  Measured against the bf16 kernels (us, prepared weights): 512 x 2048 over K 5632
    // 44 / 68; 512 x 2048 over K 2048 29 / 28; 256 x 6144 over K 2048 (two shares) 29 / 49; 320 x 2048 over K 2048 (six
    // shares) 23 / 26; 64 x 11008 over K 4096 28 / 47; 128 x 11264 over K 2048 27 / 48; 255 x 2048 over K 5632 30 / 45.
    // Below those bounds the partial products cost more than the launch gains (256 x 2048 over K 2048: 23 / 19; 64 x 2048
    // over K 2048, eight shares: 16 / 12).
    const int steps = q8_padded_k(k) / 32;
    if (steps < 48 || !(t64n >= 48 || (t64n >= 40 && steps >= 128))) return {0, 0, 1};
    auto shares_of = [&](int64_t tiles) { return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(8, 256 / tiles), steps / kMinSplitSteps)); };
    const int sw = shares_of(t64), sn = shares_of(t64n);
    return (double)(t64n * sn) > 1.05 * (double)(t64 * sw) ? GemmF16Plan{64, 192, sn} : GemmF16Plan{64, 256, sw};
}

int q8_gemm_f16_tile_rows(int m, int n_rows, int k, bool prepared) { return q8_gemm_f16_plan(m, n_rows, k, prepared).tile_rows; }
// the fused q | k | v projection with RoPE and the cache append as its epilogue: on these kernels, K not shared
bool q8_gemm_f16_rope_ok(int m, int d, int k) {
    const GemmF16Plan p = q8_gemm_f16_plan(m, 3 * d, k, false);      // (256 rows and more: whatever the weights' state)
    return p.tile_rows != 0 && p.splits == 1;
}
bool q8_gemm_f16_shape_ok(int m, int n_rows, int k, bool prepared) { return q8_gemm_f16_tile_rows(m, n_rows, k, prepared) != 0; }
void q8_gemm_f16_tile(int m, int n_rows, int k, int *tile_rows, int *tile_cols, int *k_shares, bool prepared) {
    const GemmF16Plan p = q8_gemm_f16_plan(m, n_rows, k, prepared);
    if (tile_rows) *tile_rows = p.tile_rows;
    if (tile_cols) *tile_cols = p.tile_cols;
    if (k_shares) *k_shares = p.splits;
}

// weight rows a column tile of either width (256 or 192) may read: the prepared buffer holds zeros from n_rows up to here
static int q8_prepared_rows_read(int n_rows) { return (int)std::max(round_up(n_rows, 256), round_up(n_rows, 192)); }

// the weights in this kernel's layout: fp16 rows, then the transposed scales (each part 256-byte aligned)
int64_t q8_prepared_floats(int k, int n_rows) {
    const int64_t kp = q8_padded_k(k), pitch = kp + 64, n_pad = round_up(n_rows, kNPad);
    return round_up(n_pad * pitch / 2, 64) + round_up((kp / 32) * n_pad, 64) + 64;     // + the scale fetch's reach past the last tile
}

// floats of workspace: planes, row factors and, unless the caller holds prepared weights, those
int64_t q8_gemm_f16_workspace_floats(int m, int n_rows, int k, bool prepared) {
    const int64_t kp = q8_padded_k(k), pitch = kp + 64, m_pad = round_up(m, TM);
    const int splits = q8_gemm_f16_plan(m, n_rows, k, prepared).splits;
    return round_up(m_pad * pitch, 64) + round_up(m_pad, 64) + (prepared ? 0 : q8_prepared_floats(k, n_rows)) +
           (splits > 1 ? round_up((int64_t)splits * m * n_rows, 64) : 0);
}

// What the direct global -> LDS loads of one launch reach, against what the buffers hold, in bytes from the start of
// the planes, of the fp16 weights and of the transposed scales.  A lane's load is 16 bytes (4 for a scale) at
// base + lane offset + step * 64: the last one of the activations is plane 1, the last row of the last row tile, the
// last K step; of the weights the last row of the last column tile; of the scales the 256 floats that the four
// wavefronts fetch from the last column tile's first row on (with 192-column tiles the last 64 of them lie past the
// tile, are fetched and never read).  Loads past a workgroup's last step are clamped to it, so the last step bounds
// every address.  Pure host arithmetic: a CPU test runs it over the shape space, and every launch checks it.
bool q8_gemm_f16_extents(int m, int n_rows, int k, int tile_rows, int tile_cols, int64_t reach[3], int64_t size[3]) {
    const int64_t kp = q8_padded_k(k), pitch = kp + 64, m_pad = round_up(m, TM), n_pad = round_up(n_rows, kNPad), steps = kp / 32;
    const int64_t m_read = round_up(m, tile_rows), n_read = round_up(n_rows, tile_cols);
    reach[0] = 2 * (m_pad * pitch + (m_read - 1) * pitch + kp);
    size[0] = 2 * 2 * m_pad * pitch;
    reach[1] = 2 * ((n_read - 1) * pitch + kp);
    size[1] = 2 * std::min<int64_t>(n_pad, q8_prepared_rows_read(n_rows)) * pitch;      // the rows that hold weights or zeros
    reach[2] = 4 * ((steps - 1) * n_pad + (n_read - tile_cols) + 256);
    size[2] = 4 * (round_up(steps * n_pad, 64) + 64);
    return m_read <= m_pad && reach[0] <= size[0] && reach[1] <= size[1] && reach[2] <= size[2];
}

void launch_q8_prepare(hipStream_t s, const int8_t *wq, const float *scales, float *prepared, int k, int n_rows) {
    if (k <= 0 || n_rows <= 0) return;
    const int kp = q8_padded_k(k), pitch = kp + 64, n_pad = (int)round_up(n_rows, kNPad);
    uint16_t *w16 = reinterpret_cast<uint16_t *>(prepared);
    float *scales_t = prepared + round_up((int64_t)n_pad * pitch / 2, 64);
    const int rows_read = q8_prepared_rows_read(n_rows);
    if (rows_read > n_pad) fail("q8_prepare: the column tiles reach past the padded rows");
    const int64_t items = (int64_t)rows_read * (kp / 8);
    launch_kernel(k_q8_to_f16, dim3((unsigned)std::min<int64_t>((items + 255) / 256, 8192)), dim3(256), 0, s, wq, scales, w16, scales_t, n_rows, rows_read, kp, pitch, n_pad);
}

// The kernels' LDS (three stages) is above the 64 KB a kernel gets without asking; called once per device at start-up
// (not at the first launch, which may sit inside a graph capture).
void q8_gemm_f16_configure() {
    auto lds = [](const void *kernel, int bytes, const char *what) { hip_check(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes), what); };
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16<4>), kStages * stage128_bytes(4), "hipFuncSetAttribute(k_gemm_q8_f16<4>)");
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16<3>), kStages * stage128_bytes(3), "hipFuncSetAttribute(k_gemm_q8_f16<3>)");
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16<4, true>), kStages * stage128_bytes(4), "hipFuncSetAttribute(k_gemm_q8_f16<4, rope>)");
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16<3, true>), kStages * stage128_bytes(3), "hipFuncSetAttribute(k_gemm_q8_f16<3, rope>)");
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16_m64<4>), kStages * stage64_bytes(4), "hipFuncSetAttribute(k_gemm_q8_f16_m64<4>)");
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16_m64<3>), kStages * stage64_bytes(3), "hipFuncSetAttribute(k_gemm_q8_f16_m64<3>)");
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16_m64<4, true>), kStages * stage64_bytes(4), "hipFuncSetAttribute(k_gemm_q8_f16_m64<4, rope>)");
    lds(reinterpret_cast<const void *>(k_gemm_q8_f16_m64<3, true>), kStages * stage64_bytes(3), "hipFuncSetAttribute(k_gemm_q8_f16_m64<3, rope>)");
}

void launch_q8_gemm_f16(hipStream_t s, const float *x, const float *gamma, const float *beta, const int8_t *wq, const float *scales,
                        const float *prepared, float *out, int m, int k, int n_rows, const float *bias, const float *bias2,
                        const float *residual, int interleaved_bias, int gelu, int swiglu, float *workspace, int64_t workspace_floats,
                        const RopeStore *rope, GemmChain *chain) {
    if (!q8_gemm_f16_shape_ok(m, n_rows, k, prepared != nullptr)) fail("q8_gemm_f16: shape outside this kernel's range");
    if (workspace_floats < q8_gemm_f16_workspace_floats(m, n_rows, k, prepared != nullptr)) fail("q8_gemm_f16: workspace too small");
    if (swiglu && ((n_rows & 1) || residual || gelu)) fail("q8_gemm_f16: the SwiGLU epilogue needs an even row count and takes no residual or GELU");
    const int kp = q8_padded_k(k), pitch = kp + 64, m_pad = (int)round_up(m, TM), n_pad = (int)round_up(n_rows, kNPad);
    const GemmF16Plan plan = q8_gemm_f16_plan(m, n_rows, k, prepared != nullptr);
    if (rope && (plan.splits > 1 || swiglu || gelu || residual || n_rows != 3 * rope->d || (rope->hd & 3) || rope->d % rope->hd))
        fail("q8_gemm_f16: the RoPE epilogue needs an unshared K, N = 3 d and no other epilogue than a bias");
    int64_t reach[3], size[3];
    if (!q8_gemm_f16_extents(m, n_rows, k, plan.tile_rows, plan.tile_cols, reach, size)) fail("q8_gemm_f16: a tile's loads would reach past its buffer");
    const int m_read = (int)round_up(m, plan.tile_rows);                // rows the row tiles read: [m, m_read) are zeros
    float *w = workspace;
    uint16_t *planes = reinterpret_cast<uint16_t *>(w); w += round_up((int64_t)m_pad * pitch, 64);
    float *unscale = w;                                  w += round_up(m_pad, 64);
    // gamma alone: RMSNorm of the rows first; gamma and beta: LayerNorm
    auto split = !gamma ? k_split_f16<0> : beta ? k_split_f16<2> : k_split_f16<1>;
    // (the helpers are ordinary launches: per-kernel timing of this op, launch_kernel's business, is the GEMM's)
    // (a K-sharing GEMM right before this one may have left these rows here already: GemmChain)
    if (!(chain && chain->planes_ready))
        launch_kernel(split, dim3(m_read), dim3(256), 0, s, x, gamma, beta, planes, unscale, m, k, kp, pitch, (int64_t)m_pad * pitch, SplitSum{});
    if (!prepared) {
        launch_q8_prepare(s, wq, scales, w, k, n_rows);
        prepared = w;
        w += q8_prepared_floats(k, n_rows);
    }
    const uint16_t *w16 = reinterpret_cast<const uint16_t *>(prepared);
    const float *scales_t = prepared + round_up((int64_t)n_pad * pitch / 2, 64);
    const int split_steps = plan.splits > 1 ? (kp / 32 + plan.splits - 1) / plan.splits : 0;
    const int n_tiles = (n_rows + plan.tile_cols - 1) / plan.tile_cols, m_tiles = plan.tile_rows == 64 ? (m + TM64 - 1) / TM64 : m_pad / TM;
    const unsigned grid_x = (unsigned)((n_tiles + 7) / 8 * 8 * m_tiles);
    GemmF16Args a{planes, w16, scales_t, unscale, out, m, n_rows, m_pad, n_pad, kp, pitch, m_tiles, n_tiles,
                  GemmEpilogue{bias, bias2, residual, interleaved_bias, nullptr, 0, gelu, swiglu, rope ? *rope : RopeStore{}}, split_steps, w};
    const bool roped = rope != nullptr;
    if (plan.tile_rows == 64) {
        const dim3 grid(grid_x, 1, plan.splits);
        if (plan.tile_cols == 192) {
            if (roped) launch_kernel((k_gemm_q8_f16_m64<3, true>), grid, dim3(256), (size_t)kStages * stage64_bytes(3), s, a);
            else launch_kernel((k_gemm_q8_f16_m64<3>), grid, dim3(256), (size_t)kStages * stage64_bytes(3), s, a);
        } else {
            if (roped) launch_kernel((k_gemm_q8_f16_m64<4, true>), grid, dim3(256), (size_t)kStages * stage64_bytes(4), s, a);
            else launch_kernel((k_gemm_q8_f16_m64<4>), grid, dim3(256), (size_t)kStages * stage64_bytes(4), s, a);
        }
        // The next GEMM of the stream normalises this one's output (RMSNorm) and runs on these kernels too: the sum of
        // the K shares and that GEMM's activation split are one row-wise kernel, which leaves the planes where the next
        // launch looks for them - at the start of the workspace, below this launch's slabs.
        const int kp_next = q8_padded_k(n_rows);
        const int64_t next_floats = round_up((int64_t)m_pad * (kp_next + 64), 64) + round_up(m_pad, 64);
        if (plan.splits > 1 && chain && chain->next_gamma && !gelu && !swiglu && !interleaved_bias && (n_rows & 3) == 0 &&
            n_rows == kp_next && n_rows <= 8192 && w - workspace >= next_floats) {
            uint16_t *planes_next = reinterpret_cast<uint16_t *>(workspace);
            float *unscale_next = workspace + round_up((int64_t)m_pad * (kp_next + 64), 64);
            launch_kernel((k_split_f16<1, true>), dim3(m_pad), dim3(256), 0, s, (const float *)nullptr, chain->next_gamma, (const float *)nullptr,
                          planes_next, unscale_next, m, n_rows, kp_next, kp_next + 64, (int64_t)m_pad * (kp_next + 64),
                          SplitSum{w, plan.splits, (int64_t)m * n_rows, bias, residual, out});
            chain->left_planes = true;
        } else if (plan.splits > 1) {
            const int64_t mn4 = (int64_t)m * n_rows / 4;
            launch_kernel(k_sum_partials, dim3((unsigned)std::min<int64_t>((mn4 + 255) / 256, 4096)), dim3(256), 0, s, (const float *)w, out, plan.splits,
                               mn4, n_rows / 4, a.ep);
        }
    } else if (plan.tile_cols == 192) {
        if (roped) launch_kernel((k_gemm_q8_f16<3, true>), dim3(grid_x), dim3(256), (size_t)kStages * stage128_bytes(3), s, a);
        else launch_kernel((k_gemm_q8_f16<3>), dim3(grid_x), dim3(256), (size_t)kStages * stage128_bytes(3), s, a);
    } else {
        if (roped) launch_kernel((k_gemm_q8_f16<4, true>), dim3(grid_x), dim3(256), (size_t)kStages * stage128_bytes(4), s, a);
        else launch_kernel((k_gemm_q8_f16<4>), dim3(grid_x), dim3(256), (size_t)kStages * stage128_bytes(4), s, a);
    }
}

#ifdef DJ_TRACE
extern "C" int deepj_hip_debug_gemm_trace(unsigned long long *out, int n) {
    return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_gemm_trace), (size_t)n * sizeof(unsigned long long));
}
#endif

}  // namespace dj
