// bfloat16 matrix product on the matrix cores for few rows (decode steps, logits):
//   C = A * W^T (+ bias),  A [M, K] bf16, W [N, K] bf16 (a Linear's weight),
//   C [M, N] float32 or bf16, accumulated in float32.
//
// The product is bound by streaming W once.  A workgroup of 4 waves owns 64
// columns of C (each wave 16 of them = 16 rows of W) and up to 64 rows of A; it
// walks K in slices of 128.  Every lane loads 64 contiguous bytes of its W row
// straight into the B operand of four v_mfma_f32_16x16x32_bf16; the A slice is
// staged once per workgroup in LDS and read as A operands by all four waves.
// The order in which a slice's k values are spread over the lanes is the same
// for A and W, which is all the dot product needs.
//
// Output element (m, n) of a 16x16 tile sits in lane (n % 16) + 16 * (m / 4),
// register m % 4.
#include "common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kSliceK = 128;           // k values per slice
constexpr int kLdsStride = kSliceK + 8;  // bf16 elements per staged A row (padding against bank conflicts)

template <int MT, typename OutT>
__global__ void __launch_bounds__(256)
gemm_bf16_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W,
                        const bf16_t* __restrict__ bias, OutT* __restrict__ C, int M, int N, int K,
                        int lda, int ldc) {
    __shared__ __attribute__((aligned(16))) uint16_t a_lds[MT * 16 * kLdsStride];
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane % 16;
    const int g = lane / 16;
    const int m0 = blockIdx.y * (MT * 16);
    const int n0 = blockIdx.x * 64 + wave * 16;
    const int w_row = min(n0 + r, N - 1);  // rows past N are computed from a valid row and not stored
    const bf16_t* w_ptr = W + static_cast<size_t>(w_row) * K + g * 32;

    floatx4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < K; k0 += kSliceK) {
        // This lane's 32 k values of its W row; zero past K.
        uint4 b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + g * 32 + j * 8;
            b[j] = (k < K) ? *reinterpret_cast<const uint4*>(w_ptr + k0 + j * 8) : uint4{0, 0, 0, 0};
        }
        __syncthreads();  // the previous slice's readers are done with a_lds
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int piece = threadIdx.x + 256 * i;  // 16 pieces of 8 k values per row
            const int row = piece / 16;
            const int col = (piece % 16) * 8;
            const int m = m0 + row;
            const int k = k0 + col;
            const uint4 v = (m < M && k < K)
                                ? *reinterpret_cast<const uint4*>(A + static_cast<size_t>(m) * lda + k)
                                : uint4{0, 0, 0, 0};
            *reinterpret_cast<uint4*>(&a_lds[row * kLdsStride + col]) = v;
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < MT; ++t) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint4 a = *reinterpret_cast<const uint4*>(
                    &a_lds[(t * 16 + r) * kLdsStride + g * 32 + j * 8]);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b[j]), acc[t], 0, 0, 0);
            }
        }
    }

    const int n = n0 + r;
    if (n >= N) return;
    const float add = bias ? to_float(bias[n]) : 0.f;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + t * 16 + g * 4 + i;
            if (m < M) C[static_cast<size_t>(m) * ldc + n] = from_float<OutT>(acc[t][i] + add);
        }
    }
}

template <typename OutT>
int launch_skinny(hipStream_t s, const bf16_t* A, const bf16_t* W, const bf16_t* bias, OutT* C, int M,
                  int N, int K, int lda, int ldc) {
    const int n_blocks = (N + 63) / 64;
    if (M <= 16) {
        gemm_bf16_skinny_kernel<1, OutT><<<dim3(n_blocks, 1), 256, 0, s>>>(A, W, bias, C, M, N, K, lda, ldc);
    } else if (M <= 32) {
        gemm_bf16_skinny_kernel<2, OutT><<<dim3(n_blocks, 1), 256, 0, s>>>(A, W, bias, C, M, N, K, lda, ldc);
    } else {
        const int m_blocks = (M + 63) / 64;
        if (m_blocks > 65535) return CIE_BAD_ARGUMENT;
        gemm_bf16_skinny_kernel<4, OutT><<<dim3(n_blocks, m_blocks), 256, 0, s>>>(A, W, bias, C, M, N, K, lda, ldc);
    }
    return cie_after_launch();
}

}  // namespace

// out_dtype: CIE_F32 or CIE_BF16.  K and lda must be multiples of 8 (16-byte loads).
CIE_API int cie_gemm_bf16(void* stream, const void* A, const void* W, const void* bias, void* C,
                          int out_dtype, int M, int N, int K, int lda, int ldc) {
    if (M < 0 || N <= 0 || K <= 0 || K % 8 || lda % 8 || lda < K || ldc < N) return CIE_BAD_ARGUMENT;
    if (M == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bf16_t* a = static_cast<const bf16_t*>(A);
    const bf16_t* w = static_cast<const bf16_t*>(W);
    const bf16_t* b = static_cast<const bf16_t*>(bias);
    if (out_dtype == CIE_F32) return launch_skinny<float>(s, a, w, b, static_cast<float*>(C), M, N, K, lda, ldc);
    if (out_dtype == CIE_BF16) return launch_skinny<bf16_t>(s, a, w, b, static_cast<bf16_t*>(C), M, N, K, lda, ldc);
    return CIE_BAD_ARGUMENT;
}
