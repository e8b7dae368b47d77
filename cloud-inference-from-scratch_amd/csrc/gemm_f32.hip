// True float32 matrix product for the 32-bit path: C = A * W^T (+ bias).
//   A [M, K] row-major (row stride lda), W [N, K] row-major (a Linear's weight), C [M, N].
// Plain fused multiply-adds in float32, no matrix-core reduced-precision mode.
// Every output element is a sum over k in one fixed order (blocks of 256 k summed one after the other, the
// blocks' sums added in turn: the rounding error grows with 256 + K/256 terms, not with K), so a row's result
// does not depend on how many other rows are in the batch.
// 64x64 output tile per workgroup, 16-deep k slices through LDS, 4x4 per thread.
#include "common.h"

namespace {
constexpr int BM = 64, BN = 64, BK = 16;
constexpr int kSlicesPerBlock = 16;  // 256 k: a block's sum joins the total
}

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W,
                const float* __restrict__ bias, float* __restrict__ C, int M, int N, int K,
                int lda, int ldc) {
    __shared__ float a_tile[BK][BM + 4];
    __shared__ float w_tile[BK][BN + 4];
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * BN;
    const int tx = threadIdx.x % 16;
    const int ty = threadIdx.x / 16;
    float acc[4][4] = {}, total[4][4] = {};
    int slice = 0;
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int idx = threadIdx.x + 256 * r;
            const int row = idx / BK;
            const int kk = idx % BK;
            const int k = k0 + kk;
            const int m = m0 + row;
            const int n = n0 + row;
            a_tile[kk][row] = (m < M && k < K) ? A[static_cast<size_t>(m) * lda + k] : 0.f;
            w_tile[kk][row] = (n < N && k < K) ? W[static_cast<size_t>(n) * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = a_tile[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = w_tile[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        if (++slice == kSlicesPerBlock) {
            slice = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    total[i][j] += acc[i][j];
                    acc[i][j] = 0.f;
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[static_cast<size_t>(m) * ldc + n] = (total[i][j] + acc[i][j]) + (bias ? bias[n] : 0.f);
        }
    }
}

CIE_API int cie_gemm_f32(void* stream, const float* A, const float* W, const float* bias, float* C,
                         int M, int N, int K, int lda, int ldc) {
    if (M < 0 || N <= 0 || K <= 0 || lda < K || ldc < N) return CIE_BAD_ARGUMENT;
    if (M == 0) return CIE_OK;
    const int grid_y = (M + BM - 1) / BM;
    if (grid_y > 65535) return CIE_BAD_ARGUMENT;
    dim3 grid((N + BN - 1) / BN, grid_y);
    gemm_f32_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(A, W, bias, C, M, N, K, lda, ldc);
    return cie_after_launch();
}
