// SwiGLU gate: out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i], silu(x) = x / (1 + exp(-x)).
// Computed in float32, rounded once.
// With `row_sumsq` the rows of gate_up come from a product whose input rows lacked the 1/rms of an
// RMSNorm (a product is linear in its rows): both halves are first multiplied by
// rsqrt(sum of the row's `parts` partial sums of squares / hidden + eps).
#include "common.h"

// the row's factor, made by the whole workgroup; 1 without row_sumsq
__device__ __forceinline__ float row_factor(const float* __restrict__ row_sumsq, int parts, int hidden, float eps,
                                            int token, float* scratch) {
    if (!row_sumsq) return 1.f;  // (the same for every thread: no barrier is skipped by some)
    float s = 0.f;
    for (int p = threadIdx.x; p < parts; p += blockDim.x) s += row_sumsq[static_cast<size_t>(token) * parts + p];
    return 1.0f / sqrtf(block_sum(s, scratch) / static_cast<float>(hidden) + eps);
}

template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int intermediate,
                                const float* __restrict__ row_sumsq, int parts, int hidden, float eps) {
    __shared__ float scratch[16];
    const int token = blockIdx.x;
    const float factor = row_factor(row_sumsq, parts, hidden, eps, token, scratch);
    const int i = blockIdx.y * blockDim.x + threadIdx.x;
    if (i >= intermediate) return;
    const T* row = gate_up + static_cast<size_t>(token) * 2 * intermediate;
    const float g = to_float(row[i]) * factor;
    const float u = to_float(row[intermediate + i]) * factor;
    out[static_cast<size_t>(token) * intermediate + i] = from_float<T>((g / (1.0f + expf(-g))) * u);
}

// Eight elements per thread with 16-byte loads and stores (bf16, intermediate a multiple of 8).
__global__ void silu_mul_vec8_kernel(const bf16_t* __restrict__ gate_up, bf16_t* __restrict__ out, int intermediate,
                                     const float* __restrict__ row_sumsq, int parts, int hidden, float eps) {
    __shared__ float scratch[16];
    const int token = blockIdx.x;
    const float factor = row_factor(row_sumsq, parts, hidden, eps, token, scratch);
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
        const float g0 = __uint_as_float(gw[q] << 16) * factor, g1 = __uint_as_float(gw[q] & 0xffff0000u) * factor;
        const float u0 = __uint_as_float(uw[q] << 16) * factor, u1 = __uint_as_float(uw[q] & 0xffff0000u) * factor;
        packed[q] = pack_bf16((g0 / (1.0f + expf(-g0))) * u0, (g1 / (1.0f + expf(-g1))) * u1);
    }
    *reinterpret_cast<uint4*>(out + static_cast<size_t>(token) * intermediate + i) =
        uint4{packed[0], packed[1], packed[2], packed[3]};
}

CIE_API int cie_silu_mul(void* stream, int dtype, const void* gate_up, void* out, int tokens,
                         int intermediate, const float* row_sumsq, int parts, int hidden, float eps) {
    if (tokens < 0 || intermediate <= 0 || (intermediate + 255) / 256 > 65535) return CIE_BAD_ARGUMENT;
    if (row_sumsq && (parts < 1 || hidden < 1 || !(eps > 0.f))) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(tokens, (intermediate + 255) / 256);
    if (dtype == CIE_BF16 && intermediate % 8 == 0) {
        dim3 vec_grid(tokens, (intermediate / 8 + 255) / 256);
        silu_mul_vec8_kernel<<<vec_grid, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), intermediate,
                                                     row_sumsq, parts, hidden, eps);
        return cie_after_launch();
    }
    if (dtype == CIE_F32)
        silu_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), intermediate,
                                                   row_sumsq, parts, hidden, eps);
    else if (dtype == CIE_BF16)
        silu_mul_kernel<bf16_t><<<grid, 256, 0, s>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), intermediate,
                                                    row_sumsq, parts, hidden, eps);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
