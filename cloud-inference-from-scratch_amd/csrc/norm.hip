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

template <typename T, typename W>
static int launch_norm(hipStream_t s, float* residual, const void* branch, const void* weight,
                       void* out, const int* rows, int n_out, int hidden, float eps,
                       int write_residual) {
    add_rmsnorm_kernel<T, W><<<n_out, 256, hidden * sizeof(float), s>>>(
        residual, static_cast<const T*>(branch), static_cast<const W*>(weight), static_cast<T*>(out),
        rows, hidden, eps, write_residual);
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
    if (dtype == CIE_BF16 && wdtype == CIE_BF16)
        return launch_norm<bf16_t, bf16_t>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    if (dtype == CIE_BF16 && wdtype == CIE_F32)
        return launch_norm<bf16_t, float>(s, residual, branch, weight, out, rows, n_out, hidden, eps, write_residual);
    return CIE_BAD_ARGUMENT;
}
