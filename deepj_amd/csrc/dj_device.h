// Device-side helpers shared by the decode kernels (Q8 matvec and decode attention).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace dj {
namespace dev {

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding global
// load (its workgroup-scope fence needs vmcnt(0)), which here would park the workgroup until the weight rows
// already requested from HBM have arrived; the staged activations only need the LDS writes to be complete.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
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

// Sum over the 64 lanes with DPP row operations (no LDS traffic); every lane gets the total.
__device__ __forceinline__ float wave_sum_dpp(float v) {
#define DJ_DPP_ADD(ctrl, row_mask)                                                                        \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, row_mask, 0xf, false))
    DJ_DPP_ADD(0xB1, 0xf);    // quad_perm [1,0,3,2]
    DJ_DPP_ADD(0x4E, 0xf);    // quad_perm [2,3,0,1]
    DJ_DPP_ADD(0x141, 0xf);   // row_half_mirror
    DJ_DPP_ADD(0x140, 0xf);   // row_mirror: every lane of a 16-lane row holds the row sum
    DJ_DPP_ADD(0x142, 0xa);   // row_bcast:15 into rows 1 and 3
    DJ_DPP_ADD(0x143, 0xc);   // row_bcast:31 into rows 2 and 3: lane 63 holds the total
#undef DJ_DPP_ADD
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Sum over the LPK (8, 16 or 32) consecutive lanes that share a key; every lane of the group gets the total.
// DPP row operations instead of shuffles: a shuffle is an LDS-crossbar round trip with a wait behind it, and the
// score of every key needs log2(LPK) of them in a row.
template <int LPK>
__device__ __forceinline__ float group_sum(float v) {
#define DJ_DPP_ADD(ctrl) \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, false))
    DJ_DPP_ADD(0xB1);                             // quad_perm [1,0,3,2]
    DJ_DPP_ADD(0x4E);                             // quad_perm [2,3,0,1]: quad sums
    if constexpr (LPK >= 8) DJ_DPP_ADD(0x141);    // row_half_mirror: 8 lanes
    if constexpr (LPK >= 16) DJ_DPP_ADD(0x140);   // row_mirror: 16 lanes
#undef DJ_DPP_ADD
    if constexpr (LPK == 32) v += __shfl_xor(v, 16, 64);
    return v;
}

}  // namespace dev
}  // namespace dj
