// What the GEMM kernels do to a finished sum before storing it (device code; included by the GEMM sources).
#pragma once
#include <cstdint>
#include <hip/hip_runtime.h>

namespace dj {

struct GemmEpilogue {
    const float *bias;      // [N] or null; with interleave: even col n -> bias[n/2], odd col -> bias2[n/2]
    const float *bias2;
    const float *residual;  // [M x N] or null
    int interleaved_bias;
    const int32_t *m_dev;   // when set, only rows < min(M, m_dev[0] + m_extra) exist (row count kept on the device)
    int m_extra;
    int gelu;               // GELU (tanh form, tensor/cpu/CpuBackend.java:338, used by activations/GELU.java:15-18) on acc + bias, before the residual
    int swiglu;             // Q8 GEMM only: columns are interleaved gate/up pairs; C is [M x N/2], C[r][j] = SiLU(gate_j) * up_j
};

__device__ __forceinline__ float gemm_gelu(float x) {
    float c = sqrtf(2.0f / 3.14159265358979323846f);
    float x3 = x * x * x;
    float t = c * (x + 0.044715f * x3);
    return 0.5f * x * (1.0f + (float)tanh((double)t));
}

}  // namespace dj
