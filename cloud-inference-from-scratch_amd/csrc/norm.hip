// Fused residual-add + RMSNorm.
//
//   x   = residual[row] (+ branch[row])        float32
//   var = mean(x^2);  y = x * (1 / sqrt(var + eps)) * weight
//
// The statistics, the scaling and the residual sum are float32; the output is
// rounded once to the activation type.  With `rows` given, only those rows are
// normalised (the rows whose logits are wanted) and the residual is not written
// back.  One workgroup per output row; the row is staged in LDS, so hidden*4
// bytes must fit in 64 KB.
#include "common.h"

template <typename T, typename W>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ branch,
                                   const W* __restrict__ weight, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps,
                                   int write_residual) {
    extern __shared__ float staged[];
    __shared__ float scratch[16];
    const int out_row = blockIdx.x;
    const int row = rows ? rows[out_row] : out_row;
    float* res = residual + static_cast<size_t>(row) * hidden;
    const T* add = branch ? branch + static_cast<size_t>(row) * hidden : nullptr;
    float sum_sq = 0.f;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) {
        float x = res[h];
        if (add) {
            x += to_float(add[h]);
            if (write_residual) res[h] = x;
        }
        staged[h] = x;
        sum_sq += x * x;
    }
    const float total = block_sum(sum_sq, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    T* dst = out + static_cast<size_t>(out_row) * hidden;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x)
        dst[h] = from_float<T>((staged[h] * inv) * to_float(weight[h]));
}

// bf16 activations and weight, hidden a multiple of 8: eight elements per thread, 16-byte accesses.
__global__ void add_rmsnorm_vec8_kernel(float* __restrict__ residual, const bf16_t* __restrict__ branch,
                                        const bf16_t* __restrict__ weight, bf16_t* __restrict__ out,
                                        int hidden, float eps) {
    extern __shared__ float staged[];
    __shared__ float scratch[16];
    const int row = blockIdx.x;
    float* res = residual + static_cast<size_t>(row) * hidden;
    const bf16_t* add = branch ? branch + static_cast<size_t>(row) * hidden : nullptr;
    float sum_sq = 0.f;
    for (int h = threadIdx.x * 8; h < hidden; h += blockDim.x * 8) {
        float4 x0 = *reinterpret_cast<const float4*>(res + h);
        float4 x1 = *reinterpret_cast<const float4*>(res + h + 4);
        if (add) {
            const uint4 raw = *reinterpret_cast<const uint4*>(add + h);
            x0.x += __uint_as_float(raw.x << 16); x0.y += __uint_as_float(raw.x & 0xffff0000u);
            x0.z += __uint_as_float(raw.y << 16); x0.w += __uint_as_float(raw.y & 0xffff0000u);
            x1.x += __uint_as_float(raw.z << 16); x1.y += __uint_as_float(raw.z & 0xffff0000u);
            x1.z += __uint_as_float(raw.w << 16); x1.w += __uint_as_float(raw.w & 0xffff0000u);
            *reinterpret_cast<float4*>(res + h) = x0;
            *reinterpret_cast<float4*>(res + h + 4) = x1;
        }
        *reinterpret_cast<float4*>(staged + h) = x0;
        *reinterpret_cast<float4*>(staged + h + 4) = x1;
        sum_sq += (x0.x * x0.x + x0.y * x0.y) + (x0.z * x0.z + x0.w * x0.w) + (x1.x * x1.x + x1.y * x1.y) +
                  (x1.z * x1.z + x1.w * x1.w);
    }
    const float total = block_sum(sum_sq, scratch);
    const float inv = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    bf16_t* dst = out + static_cast<size_t>(row) * hidden;
    for (int h = threadIdx.x * 8; h < hidden; h += blockDim.x * 8) {
        const float4 x0 = *reinterpret_cast<const float4*>(staged + h);
        const float4 x1 = *reinterpret_cast<const float4*>(staged + h + 4);
        const uint4 raw = *reinterpret_cast<const uint4*>(weight + h);
        uint4 packed;
        packed.x = pack_bf16((x0.x * inv) * __uint_as_float(raw.x << 16), (x0.y * inv) * __uint_as_float(raw.x & 0xffff0000u));
        packed.y = pack_bf16((x0.z * inv) * __uint_as_float(raw.y << 16), (x0.w * inv) * __uint_as_float(raw.y & 0xffff0000u));
        packed.z = pack_bf16((x1.x * inv) * __uint_as_float(raw.z << 16), (x1.y * inv) * __uint_as_float(raw.z & 0xffff0000u));
        packed.w = pack_bf16((x1.z * inv) * __uint_as_float(raw.w << 16), (x1.w * inv) * __uint_as_float(raw.w & 0xffff0000u));
        *reinterpret_cast<uint4*>(dst + h) = packed;
    }
}

template <typename T, typename W>
static int launch_norm(hipStream_t s, float* residual, const void* branch, const void* weight,
                       void* out, const int* rows, int n_out, int hidden, float eps,
                       int write_residual) {
    add_rmsnorm_kernel<T, W><<<n_out, n_out <= 64 ? 1024 : 256, hidden * sizeof(float), s>>>(
        residual, static_cast<const T*>(branch), static_cast<const W*>(weight), static_cast<T*>(out),
        rows, hidden, eps, write_residual);
    return cie_after_launch();
}

// RMSNorm of rows whose partial sums of squares are already known (left by the product that wrote the
// residual): no reduction over the row is needed, so a row is spread over several workgroups.
template <typename T, typename W>
__global__ void __launch_bounds__(256)
rmsnorm_from_sumsq_kernel(const float* __restrict__ residual, const float* __restrict__ sumsq, int parts,
                          const W* __restrict__ weight, T* __restrict__ out, int hidden, float eps) {
    __shared__ float scratch[16];
    const int row = blockIdx.y;
    float s = 0.f;
    for (int p = threadIdx.x; p < parts; p += blockDim.x) s += sumsq[static_cast<size_t>(row) * parts + p];
    const float inv = 1.0f / sqrtf(block_sum(s, scratch) / static_cast<float>(hidden) + eps);
    const int h = blockIdx.x * blockDim.x + threadIdx.x;
    if (h < hidden)
        out[static_cast<size_t>(row) * hidden + h] =
            from_float<T>((residual[static_cast<size_t>(row) * hidden + h] * inv) * to_float(weight[h]));
}

CIE_API int cie_rmsnorm_from_sumsq(void* stream, int wdtype, const float* residual, const float* sumsq, int parts,
                                   const void* weight, void* out, int rows, int hidden, float eps) {
    if (rows < 0 || rows > 65535 || hidden <= 0 || parts < 1 || !(eps > 0.f)) return CIE_BAD_ARGUMENT;
    if (rows == 0) return CIE_OK;
    dim3 grid((hidden + 255) / 256, rows);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (wdtype == CIE_BF16)
        rmsnorm_from_sumsq_kernel<bf16_t, bf16_t><<<grid, 256, 0, s>>>(
            residual, sumsq, parts, static_cast<const bf16_t*>(weight), static_cast<bf16_t*>(out), hidden, eps);
    else if (wdtype == CIE_F32)
        rmsnorm_from_sumsq_kernel<bf16_t, float><<<grid, 256, 0, s>>>(
            residual, sumsq, parts, static_cast<const float*>(weight), static_cast<bf16_t*>(out), hidden, eps);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

// dtype: activation type of branch/out; wdtype: storage type of the weight.
CIE_API int cie_add_rmsnorm(void* stream, int dtype, int wdtype, float* residual, const void* branch,
                            const void* weight, void* out, const int* rows, int n_out, int hidden,
                            float eps, int write_residual) {
    if (n_out < 0 || hidden <= 0 || hidden * sizeof(float) > 64 * 1024 || !(eps > 0.f))
        return CIE_BAD_ARGUMENT;
    if (rows && write_residual) return CIE_BAD_ARGUMENT;
    if (n_out == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32 && wdtype == CIE_F32)
        return launch_norm<float, float>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    if (dtype == CIE_BF16 && wdtype == CIE_BF16 && !rows && write_residual && hidden % 8 == 0) {
        add_rmsnorm_vec8_kernel<<<n_out, n_out <= 64 ? 1024 : 256, hidden * sizeof(float), s>>>(
            residual, static_cast<const bf16_t*>(branch), static_cast<const bf16_t*>(weight), static_cast<bf16_t*>(out),
            hidden, eps);
        return cie_after_launch();
    }
    if (dtype == CIE_BF16 && wdtype == CIE_BF16)
        return launch_norm<bf16_t, bf16_t>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    if (dtype == CIE_BF16 && wdtype == CIE_F32)
        return launch_norm<bf16_t, float>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    return CIE_BAD_ARGUMENT;
}
