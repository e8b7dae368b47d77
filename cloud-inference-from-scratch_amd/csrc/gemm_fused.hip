// Decode-step matrix products on the matrix cores, fused with what surrounds them.
//
//   C = A * W^T     A [M, K] with few rows (M <= 64 per workgroup row), W [N, K] bf16
//
// A step with few tokens is bound by streaming W once and by the number of
// kernel launches, so this kernel takes over its neighbours' work:
//
//   prologue  NORM   A is not given; it is made on the fly from the float32
//                    residual stream: A[m,k] = bf16(residual[m,k] * inv_rms[m] * norm_w[k]),
//                    inv_rms[m] = 1/sqrt(sum_p sumsq[m,p] / K + eps), where sumsq holds
//                    partial sums of squares of the row that the producer of the
//                    residual left (one per 16 columns).
//   epilogue  PLAIN  C[m,n] = acc + bias[n], bf16 or float32
//             SILU   W stacks gate rows over up rows: C[m,n] = silu(acc_gate) * acc_up, bf16
//             RESID  residual[m,n] += acc (float32, in place) and the partial sums of
//                    squares of the new residual rows are written for the next NORM.
//             PARTIAL  K is cut into grid.z parts, each workgroup writes its float32 partial
//                    product to C[part, m, n]; the consumer (the add + norm kernel) sums the
//                    parts.  For products with few columns and a long K, where one
//                    workgroup per column tile cannot pull the weight fast enough.
//
// Work split: one workgroup owns NT tiles of 16 columns (NT = 2 only for SILU:
// a gate tile and its up tile) and all rows; its WAVES waves cut K into slices of
// 128 and take them round-robin.  Every lane streams its W row(s) with 16-byte
// loads straight into B operands of v_mfma_f32_16x16x32_bf16 and loads (or
// makes) its own row of A for the same k values; nothing is shared until the
// end, when the waves' partial tiles are summed through LDS in wave order and
// wave 0 runs the epilogue.  No workgroup ever waits for another one: on this
// GPU a device-wide fence between workgroups costs more than the whole product.
// Sums are float32 throughout.
#include "common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

enum { EPI_PLAIN_BF16 = 0, EPI_PLAIN_F32 = 1, EPI_SILU = 2, EPI_RESID = 3, EPI_PARTIAL = 4 };

struct FusedArgs {
    // A: either a bf16 matrix, or residual + norm
    const bf16_t* a;
    int lda;
    const float* residual_in;   // [M, K] float32 (NORM)
    const float* sumsq_in;      // [M, parts_in]
    int parts_in;
    const void* norm_w;         // [K] bf16 or float32
    int norm_w_f32;
    float eps;
    const bf16_t* w;            // [N, K]
    const bf16_t* bias;         // [N] or null
    void* c;                    // PLAIN: [M, N]; SILU: [M, N/2]
    float* residual_out;        // RESID: [M, N] float32, accumulated in place
    float* sumsq_out;           // RESID: [M, N/16]
    int M, N, K;
    int second_tile_offset;     // rows of W between a workgroup's first and second tile (NT == 2)
    int k_per_part;             // PARTIAL: k values per grid.z part (a multiple of 128); otherwise K
};

template <int WAVES, int MT, int NT, int EPI, bool NORM, bool HALF>
__global__ void __launch_bounds__(WAVES * 64) gemm_fused_kernel(FusedArgs a) {
    // HALF: the workgroup owns 8 columns only (lanes r and r + 8 read the same row of W and compute the
    // same column; the upper copies are dropped).  Twice as many workgroups for products with few columns.
    constexpr int TILE_N = HALF ? 8 : 16;
    constexpr int ROWS = 16 * MT;
    __shared__ float reduce[WAVES > 1 ? (WAVES - 1) * MT * NT * 64 * 4 : 1];
    __shared__ float inv_rms[ROWS];

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int m0 = blockIdx.y * ROWS;
    const int n_first = blockIdx.x * TILE_N;
    const int col = HALF ? (r & 7) : r;  // column of this lane within the tile

    if (NORM) {
        for (int m = wave; m < ROWS; m += WAVES) {
            float s = 0.f;
            if (m0 + m < a.M)
                for (int p = lane; p < a.parts_in; p += kWave) s += a.sumsq_in[static_cast<size_t>(m0 + m) * a.parts_in + p];
            s = wave_sum(s);
            if (lane == 0) inv_rms[m] = 1.0f / sqrtf(s / static_cast<float>(a.K) + a.eps);
        }
        __syncthreads();
    }

    const bf16_t* w_row[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) w_row[t] = a.w + static_cast<size_t>(n_first + t * a.second_tile_offset + col) * a.K + g * 8;

    floatx4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

    // U slices of 128 k values are in flight per wave: the loads of all of them are issued before the
    // first matrix product, which is what keeps enough bytes in flight to cover the memory latency
    constexpr int U = (MT == 1) ? (NT == 1 ? 4 : 2) : 1;
    const int k_begin = blockIdx.z * a.k_per_part;
    const int k_end = min(a.K, k_begin + a.k_per_part);
    for (int kbase = k_begin + wave * 128; kbase < k_end; kbase += U * WAVES * 128) {
        uint4 b[U][NT][4];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int k0 = kbase + u * WAVES * 128;
                    // the four lane groups read one contiguous 64-byte piece of each row per load
                    const int k = k0 + j * 32 + g * 8;
                    b[u][t][j] = (k < k_end) ? *reinterpret_cast<const uint4*>(w_row[t] + k0 + j * 32) : uint4{0, 0, 0, 0};
                }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = kbase + u * WAVES * 128;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int m = m0 + mt * 16 + r;
                uint4 av[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int k = k0 + j * 32 + g * 8;
                    av[j] = uint4{0, 0, 0, 0};
                    if (m < a.M && k < k_end) {
                        if (NORM) {
                            const float* src = a.residual_in + static_cast<size_t>(m) * a.K + k;
                            const float4 x0 = *reinterpret_cast<const float4*>(src);
                            const float4 x1 = *reinterpret_cast<const float4*>(src + 4);
                            float wv[8];
                            if (a.norm_w_f32) {
                                const float* wp = static_cast<const float*>(a.norm_w) + k;
                                const float4 w0 = *reinterpret_cast<const float4*>(wp);
                                const float4 w1 = *reinterpret_cast<const float4*>(wp + 4);
                                wv[0] = w0.x; wv[1] = w0.y; wv[2] = w0.z; wv[3] = w0.w;
                                wv[4] = w1.x; wv[5] = w1.y; wv[6] = w1.z; wv[7] = w1.w;
                            } else {
                                const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const bf16_t*>(a.norm_w) + k);
                                const uint32_t ww[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                                for (int q = 0; q < 4; ++q) {
                                    wv[2 * q] = __uint_as_float(ww[q] << 16);
                                    wv[2 * q + 1] = __uint_as_float(ww[q] & 0xffff0000u);
                                }
                            }
                            const float inv = inv_rms[mt * 16 + r];
                            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                            uint32_t packed[4];
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const uint32_t lo = bf16_bits_from_float((x[2 * q] * inv) * wv[2 * q]);
                                const uint32_t hi = bf16_bits_from_float((x[2 * q + 1] * inv) * wv[2 * q + 1]);
                                packed[q] = lo | (hi << 16);
                            }
                            av[j] = uint4{packed[0], packed[1], packed[2], packed[3]};
                        } else {
                            av[j] = *reinterpret_cast<const uint4*>(a.a + static_cast<size_t>(m) * a.lda + k);
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int t = 0; t < NT; ++t)
                        acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8, av[j]), __builtin_bit_cast(bf16x8, b[u][t][j]), acc[mt][t], 0, 0, 0);
            }
        }
    }

    // ---- sum the waves' partial tiles in wave order; wave 0 keeps the result
    if (WAVES > 1) {
        if (wave > 0) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        reduce[((((wave - 1) * MT + mt) * NT + t) * 4 + i) * 64 + lane] = acc[mt][t][i];
        }
        __syncthreads();
        if (wave > 0) return;
        for (int w = 1; w < WAVES; ++w)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[mt][t][i] += reduce[((((w - 1) * MT + mt) * NT + t) * 4 + i) * 64 + lane];
    }

    // ---- epilogue (wave 0): lane (r, g) holds rows g*4+i of column r of each tile
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (HALF && r >= 8) continue;
        if (EPI == EPI_SILU) {
            const int n = n_first + r;  // column of the gate tile = column of the output
            const int out_cols = a.second_tile_offset;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + mt * 16 + g * 4 + i;
                if (m < a.M) {
                    const float gate = acc[mt][0][i];
                    const float up = acc[mt][NT - 1][i];
                    static_cast<bf16_t*>(a.c)[static_cast<size_t>(m) * out_cols + n] =
                        from_float<bf16_t>((gate / (1.0f + __expf(-gate))) * up);
                }
            }
        } else {
            const int n = n_first + r;
            const float add = (a.bias && blockIdx.z == 0) ? to_float(a.bias[n]) : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + mt * 16 + g * 4 + i;
                const bool ok = m < a.M;
                float v = acc[mt][0][i] + add;
                if (EPI == EPI_RESID) {
                    float* dst = a.residual_out + static_cast<size_t>(m) * a.N + n;
                    if (ok) {
                        v += *dst;
                        *dst = v;
                    } else {
                        v = 0.f;
                    }
                    // sum of squares over the tile's 16 columns (the lanes that share g)
                    float sq = v * v;
                    sq += __shfl_xor(sq, 1, kWave);
                    sq += __shfl_xor(sq, 2, kWave);
                    sq += __shfl_xor(sq, 4, kWave);
                    if (!HALF) sq += __shfl_xor(sq, 8, kWave);
                    if (r == 0 && ok) a.sumsq_out[static_cast<size_t>(m) * (a.N / TILE_N) + blockIdx.x] = sq;
                } else if (ok) {
                    if (EPI == EPI_PARTIAL)
                        static_cast<float*>(a.c)[(static_cast<size_t>(blockIdx.z) * a.M + m) * a.N + n] = v;
                    else if (EPI == EPI_PLAIN_F32)
                        static_cast<float*>(a.c)[static_cast<size_t>(m) * a.N + n] = v;
                    else
                        static_cast<bf16_t*>(a.c)[static_cast<size_t>(m) * a.N + n] = from_float<bf16_t>(v);
                }
            }
        }
    }
}

template <int WAVES, int MT, int NT, int EPI>
int launch_norm(hipStream_t s, dim3 grid, const FusedArgs& a, bool norm, bool half) {
    if constexpr (NT == 1 && MT == 1) {
        if (half) {
            if (norm)
                gemm_fused_kernel<WAVES, MT, NT, EPI, true, true><<<grid, WAVES * 64, 0, s>>>(a);
            else
                gemm_fused_kernel<WAVES, MT, NT, EPI, false, true><<<grid, WAVES * 64, 0, s>>>(a);
            return cie_after_launch();
        }
    }
    if (half) return CIE_BAD_ARGUMENT;
    if (norm)
        gemm_fused_kernel<WAVES, MT, NT, EPI, true, false><<<grid, WAVES * 64, 0, s>>>(a);
    else
        gemm_fused_kernel<WAVES, MT, NT, EPI, false, false><<<grid, WAVES * 64, 0, s>>>(a);
    return cie_after_launch();
}

// waves * row tiles <= 16 keeps the LDS of the final sum within bounds
template <int MT, int NT, int EPI>
int launch_waves(hipStream_t s, int waves, dim3 grid, const FusedArgs& a, bool norm, bool half) {
    if (waves == 1) return launch_norm<1, MT, NT, EPI>(s, grid, a, norm, half);
    if (waves == 2) return launch_norm<2, MT, NT, EPI>(s, grid, a, norm, half);
    if (waves == 4) return launch_norm<4, MT, NT, EPI>(s, grid, a, norm, half);
    if constexpr (MT <= 2)
        if (waves == 8) return launch_norm<8, MT, NT, EPI>(s, grid, a, norm, half);
    if constexpr (MT == 1)
        if (waves == 16) return launch_norm<16, MT, NT, EPI>(s, grid, a, norm, half);
    return CIE_BAD_ARGUMENT;
}

template <int NT, int EPI>
int launch_rows(hipStream_t s, int mt, int waves, dim3 grid, const FusedArgs& a, bool norm, bool half) {
    switch (mt) {
        case 1: return launch_waves<1, NT, EPI>(s, waves, grid, a, norm, half);
        case 2: return launch_waves<2, NT, EPI>(s, waves, grid, a, norm, half);
        case 4: return launch_waves<4, NT, EPI>(s, waves, grid, a, norm, half);
    }
    return CIE_BAD_ARGUMENT;
}

}  // namespace

// epilogue: 0 bf16 out, 1 float32 out, 2 SiLU-gate (W = [gate rows; up rows], N = 2 * outputs), 3 residual accumulate,
// 4 partial products of k_parts parts of K to c[k_parts, M, N] (float32).
// row_tiles: 16-row tiles per workgroup (1, 2 or 4); waves: waves per workgroup that share K (1, 2, 4, 8, 16).
// half_tiles: workgroups of 8 columns instead of 16 (row_tiles 1, not SiLU); sumsq_out is then [M, N/8].
CIE_API int cie_gemm_fused(void* stream, const void* a, int lda, const float* residual_in,
                           const float* sumsq_in, int parts_in, const void* norm_w, int norm_w_f32, float eps,
                           const void* w, const void* bias, void* c, float* residual_out, float* sumsq_out,
                           int M, int N, int K, int epilogue, int row_tiles, int waves, int half_tiles,
                           int k_parts) {
    const bool norm = residual_in != nullptr;
    if (M <= 0 || N <= 0 || K <= 0 || K % 8 || N % 16) return CIE_BAD_ARGUMENT;
    if (!norm && (!a || lda < K || lda % 8)) return CIE_BAD_ARGUMENT;
    if (norm && (!sumsq_in || parts_in < 1 || !norm_w || !(eps > 0.f))) return CIE_BAD_ARGUMENT;
    if (row_tiles != 1 && row_tiles != 2 && row_tiles != 4) return CIE_BAD_ARGUMENT;
    if (epilogue == EPI_SILU && (N % 32 || bias)) return CIE_BAD_ARGUMENT;
    if (epilogue == EPI_RESID && (!residual_out || !sumsq_out)) return CIE_BAD_ARGUMENT;
    if ((epilogue == EPI_PLAIN_BF16 || epilogue == EPI_PLAIN_F32 || epilogue == EPI_SILU || epilogue == EPI_PARTIAL) && !c)
        return CIE_BAD_ARGUMENT;
    if (k_parts < 1 || k_parts > 64 || (k_parts > 1 && epilogue != EPI_PARTIAL)) return CIE_BAD_ARGUMENT;
    const int m_blocks = (M + 16 * row_tiles - 1) / (16 * row_tiles);
    if (m_blocks > 65535) return CIE_BAD_ARGUMENT;
    FusedArgs f;
    f.a = static_cast<const bf16_t*>(a);
    f.lda = lda;
    f.residual_in = residual_in;
    f.sumsq_in = sumsq_in;
    f.parts_in = parts_in;
    f.norm_w = norm_w;
    f.norm_w_f32 = norm_w_f32;
    f.eps = eps;
    f.w = static_cast<const bf16_t*>(w);
    f.bias = static_cast<const bf16_t*>(bias);
    f.c = c;
    f.residual_out = residual_out;
    f.sumsq_out = sumsq_out;
    f.M = M;
    f.N = N;
    f.K = K;
    f.k_per_part = ((K + k_parts - 1) / k_parts + 127) / 128 * 128;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (epilogue == EPI_SILU) {
        f.second_tile_offset = N / 2;
        return launch_rows<2, EPI_SILU>(s, row_tiles, waves, dim3((N / 2) / 16, m_blocks), f, norm, half_tiles != 0);
    }
    f.second_tile_offset = 0;
    const bool half = half_tiles != 0;
    dim3 grid(N / (half ? 8 : 16), m_blocks, k_parts);
    switch (epilogue) {
        case EPI_PLAIN_BF16: return launch_rows<1, EPI_PLAIN_BF16>(s, row_tiles, waves, grid, f, norm, half);
        case EPI_PLAIN_F32: return launch_rows<1, EPI_PLAIN_F32>(s, row_tiles, waves, grid, f, norm, half);
        case EPI_RESID: return launch_rows<1, EPI_RESID>(s, row_tiles, waves, grid, f, norm, half);
        case EPI_PARTIAL: return launch_rows<1, EPI_PARTIAL>(s, row_tiles, waves, grid, f, norm, half);
    }
    return CIE_BAD_ARGUMENT;
}
