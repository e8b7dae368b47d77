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

// Eight elements per thread with 16-byte loads and stores (bf16, intermediate a multiple of 8).
__global__ void silu_mul_vec8_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int intermediate) {
    const int token = blockIdx.x;
    const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
    if (i >= intermediate) return;
    const bf16_t* row = gate_up + static_cast<size_t>(token) * 2 * intermediate;
    const uint4 graw = *reinterpret_cast<const uint4*>(row + i);
    const uint4 uraw = *reinterpret_cast<const uint4*>(row + intermediate + i);
    const uint32_t gw[4] = {graw.x, graw.y, graw.z, graw.w};
    const uint32_t uw[4] = {uraw.x, uraw.y, uraw.z, uraw.w};
    uint32_t packed[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float g0 = __uint_as_float(gw[q] << 16), g1 = __uint_as_float(gw[q] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[q] << 16), u1 = __uint_as_float(uw[q] & 0xffff0000u);
        packed[q] = pack_bf16((g0 / (1.0f + expf(-g0))) * u0, (g1 / (1.0f + expf(-g1))) * u1);
    }
    *reinterpret_cast<uint4*>(out + static_cast<size_t>(token) * intermediate + i) =
        uint4{packed[0], packed[1], packed[2], packed[3]};
}

CIE_API int cie_silu_mul(void* stream, int dtype, const void* gate_up, void* out, int tokens,
                         int intermediate) {
    if (tokens < 0 || intermediate <= 0 || (intermediate + 255) / 256 > 65535) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(tokens, (intermediate + 255) / 256);
    if (dtype == CIE_BF16 && intermediate % 8 == 0) {
        dim3 vec_grid(tokens, (intermediate / 8 + 255) / 256);
        silu_mul_vec8_kernel<<<vec_grid, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), intermediate);
        return cie_after_launch();
    }
    if (dtype == CIE_F32)
        silu_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), intermediate);
    else if (dtype == CIE_BF16)
        silu_mul_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), intermediate);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
