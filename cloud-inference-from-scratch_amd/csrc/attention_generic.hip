// Paged grouped-query attention, generic form: any head size that is a multiple
// of 8 up to 256, any group size, float32 or bfloat16 storage, optional window.
// It is the whole of the float32 path's attention and the fallback of the
// bfloat16 path for shapes the matrix-core kernels refuse.
//
// One workgroup (4 waves) per (query token, query head).  A token at position p
// sees keys [lo, p] with lo = max(0, p + 1 - window) (window <= 0: all keys).
// Each wave takes 64-key chunks round-robin, one key per lane for the scores,
// then one slice of the head per lane for the value sum; the four running
// (max, sum, accumulator) triples are merged through LDS at the end.
// Scores, softmax and the value sum are float32:
//   s = (q . k) * scale;  p = exp(s - max);  out = sum(p * v) / sum(p)
//
//   q    [tokens, q_heads, D] with row stride q_row_stride (elements)
//   keys   [pages, kv_heads, page_size, D]
//   values [pages, kv_heads, D, page_size]  (transposed)
//   out  [tokens, q_heads * D]
#include "common.h"

namespace {

constexpr int kMaxSlices = 4;  // head_dim <= 64 * kMaxSlices

__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
paged_attention_generic_kernel(const T* __restrict__ q, int q_row_stride,
                               const T* __restrict__ k_pool, const T* __restrict__ v_pool,
                               const int* __restrict__ block_table, int table_width,
                               const int* __restrict__ positions,
                               const int* __restrict__ seq_of_token,
                               const int* __restrict__ seq_slot, T* __restrict__ out, int q_heads,
                               int kv_heads, int head_dim, int page_size, int window, float scale) {
    extern __shared__ float lds[];
    float* q_s = lds;                 // [head_dim]
    float* acc_s = lds + head_dim;    // [4][head_dim]
    __shared__ float m_s[4];
    __shared__ float l_s[4];

    const int token = blockIdx.x;
    const int head = blockIdx.y;
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int kv_head = head / (q_heads / kv_heads);
    const int len = positions[token] + 1;
    const int lo = (window > 0 && len > window) ? len - window : 0;
    const int slot = seq_slot[seq_of_token[token]];
    const int* table = block_table + static_cast<size_t>(slot) * table_width;

    const T* q_row = q + static_cast<size_t>(token) * q_row_stride + static_cast<size_t>(head) * head_dim;
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) q_s[d] = to_float(q_row[d]);
    __syncthreads();

    float m = -INFINITY;
    float l = 0.f;
    float acc[kMaxSlices] = {0.f, 0.f, 0.f, 0.f};

    for (int base = lo + wave * kWave; base < len; base += 4 * kWave) {
        const int key = base + lane;
        const bool valid = key < len;
        float s = -INFINITY;
        uint32_t head_block = 0;  // index of the (page, kv head) block of page_size * head_dim elements
        uint32_t in_page = 0;
        if (valid) {
            const int page = table[key / page_size];
            head_block = static_cast<uint32_t>(page) * kv_heads + kv_head;
            in_page = key % page_size;
            const T* k_row = k_pool + (static_cast<size_t>(head_block) * page_size + in_page) * head_dim;
            float dot = 0.f;
            for (int d = 0; d < head_dim; d += 8) {
                float kk[8];
                load8(k_row + d, kk);
#pragma unroll
                for (int j = 0; j < 8; ++j) dot = fmaf(q_s[d + j], kk[j], dot);
            }
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));  // finite: lane 0 of every chunk is valid
        const float alpha = expf(m - m_new);
        const float p = valid ? expf(s - m_new) : 0.f;
        l = l * alpha + wave_sum(p);
#pragma unroll
        for (int i = 0; i < kMaxSlices; ++i) acc[i] *= alpha;
        const int count = min(kWave, len - base);
        for (int j = 0; j < count; ++j) {
            const float pj = __shfl(p, j, kWave);
            const uint32_t block_j = __shfl(head_block, j, kWave);
            const uint32_t in_page_j = __shfl(in_page, j, kWave);
            const T* v_column = v_pool + static_cast<size_t>(block_j) * page_size * head_dim + in_page_j;
#pragma unroll
            for (int i = 0; i < kMaxSlices; ++i) {
                const int d = lane + kWave * i;
                if (d < head_dim) acc[i] = fmaf(pj, to_float(v_column[static_cast<size_t>(d) * page_size]), acc[i]);
            }
        }
        m = m_new;
    }

    if (lane == 0) {
        m_s[wave] = m;
        l_s[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < kMaxSlices; ++i) {
        const int d = lane + kWave * i;
        if (d < head_dim) acc_s[wave * head_dim + d] = acc[i];
    }
    __syncthreads();
    float m_all = m_s[0];
    for (int w = 1; w < 4; ++w) m_all = fmaxf(m_all, m_s[w]);
    T* out_row = out + static_cast<size_t>(token) * q_heads * head_dim + static_cast<size_t>(head) * head_dim;
    for (int d = threadIdx.x; d < head_dim; d += blockDim.x) {
        float num = 0.f;
        float den = 0.f;
        for (int w = 0; w < 4; ++w) {
            const float e = expf(m_s[w] - m_all);  // a wave that saw no key has m = -inf: weight 0
            num += acc_s[w * head_dim + d] * e;
            den += l_s[w] * e;
        }
        out_row[d] = from_float<T>(num / den);
    }
}

}  // namespace

CIE_API int cie_paged_attention_generic(void* stream, int dtype, const void* q, int q_row_stride,
                                        const void* k_pool, const void* v_pool,
                                        const int* block_table, int table_width,
                                        const int* positions, const int* seq_of_token,
                                        const int* seq_slot, void* out, int tokens, int q_heads,
                                        int kv_heads, int head_dim, int page_size, int window,
                                        float scale) {
    if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads || head_dim <= 0 ||
        head_dim % 8 || head_dim > kWave * kMaxSlices || page_size <= 0 || table_width <= 0 ||
        q_heads > 65535 || q_row_stride < q_heads * head_dim || q_row_stride % 8)
        return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(tokens, q_heads);
    const size_t lds = static_cast<size_t>(5) * head_dim * sizeof(float);
    if (dtype == CIE_F32)
        paged_attention_generic_kernel<float><<<grid, 256, lds, s>>>(
            static_cast<const float*>(q), q_row_stride, static_cast<const float*>(k_pool),
            static_cast<const float*>(v_pool), block_table, table_width, positions, seq_of_token,
            seq_slot, static_cast<float*>(out), q_heads, kv_heads, head_dim, page_size, window, scale);
    else if (dtype == CIE_BF16)
        paged_attention_generic_kernel<bf16_t><<<grid, 256, lds, s>>>(
            static_cast<const bf16_t*>(q), q_row_stride, static_cast<const bf16_t*>(k_pool),
            static_cast<const bf16_t*>(v_pool), block_table, table_width, positions, seq_of_token,
            seq_slot, static_cast<bf16_t*>(out), q_heads, kv_heads, head_dim, page_size, window, scale);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
