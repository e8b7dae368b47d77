// SwiGLU gate: out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i], silu(x) = x / (1 + exp(-x)).
// Computed in float32, rounded once.
#include "common.h"

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int intermediate) {
    const int token = blockIdx.x;
    const int i = blockIdx.y * blockDim.x + threadIdx.x;
    if (i >= intermediate) return;
    const T* row = gate_up + static_cast<size_t>(token) * 2 * intermediate;
    const float g = to_float(row[i]);
    const float u = to_float(row[intermediate + i]);
    out[static_cast<size_t>(token) * intermediate + i] = from_float<T>((g / (1.0f + expf(-g))) * u);
}

CIE_API int cie_silu_mul(void* stream, int dtype, const void* gate_up, void* out, int tokens,
                         int intermediate) {
    if (tokens < 0 || intermediate <= 0 || (intermediate + 255) / 256 > 65535) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(tokens, (intermediate + 255) / 256);
    if (dtype == CIE_F32)
        silu_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), intermediate);
    else if (dtype == CIE_BF16)
        silu_mul_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), intermediate);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
