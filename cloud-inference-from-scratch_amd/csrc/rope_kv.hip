// Fused rotary position encoding of q and k, and the write of rotated k and of v
// into the paged cache.  The first R = rotary_dim dimensions of a head rotate
// (half-split pairing: element i rotates with element i + R/2, i < R/2); those
// from R on pass through unchanged.  R = D is the reference's rotation.
//
//   qkv  [tokens, (Hq + 2*Hkv) * D]   q rotated in place
//   keys   [pages, Hkv, page_size, D]
//   values [pages, Hkv, D, page_size]  (transposed, as the attention kernels read them)
//   slot of token t: page = block_table[seq_slot[seq_of_token[t]], pos / P], row = pos % P
//
// Angles come from a float32 cos/sin table [max_position, R/2]; the rotation is
// computed in float32 and rounded once.  One workgroup per (token, head).
#include "common.h"

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const float* __restrict__ cos_table,
                                     const float* __restrict__ sin_table,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ seq_of_token,
                                     const int* __restrict__ seq_slot,
                                     const int* __restrict__ block_table, int table_width,
                                     T* __restrict__ k_pool, T* __restrict__ v_pool, int q_heads,
                                     int kv_heads, int head_dim, int rotary_dim, int page_size, int rotate,
                                     int write_kv) {
    const int token = blockIdx.x;
    const int head = blockIdx.y;  // [0,Hq): q   [Hq,Hq+Hkv): k   [Hq+Hkv,Hq+2Hkv): v
    const int half = rotary_dim / 2;
    const int pos = positions[token];
    T* src = qkv + (static_cast<size_t>(token) * (q_heads + 2 * kv_heads) + head) * head_dim;

    const bool is_value = head >= q_heads + kv_heads;
    T* dst = nullptr;
    if (head >= q_heads) {
        if (!write_kv) return;
        const int kv_head = (head - q_heads) % kv_heads;
        const int slot = seq_slot[seq_of_token[token]];
        const int page = block_table[static_cast<size_t>(slot) * table_width + pos / page_size];
        if (page < 0) return;  // the host never schedules a token without a page
        const size_t head_base = (static_cast<size_t>(page) * kv_heads + kv_head) * page_size * head_dim;
        if (is_value) {  // value element d of the token goes to [d, pos % page_size]
            T* column = v_pool + head_base + pos % page_size;
            for (int i = threadIdx.x; i < head_dim; i += blockDim.x) column[static_cast<size_t>(i) * page_size] = src[i];
            return;
        }
        dst = k_pool + head_base + static_cast<size_t>(pos % page_size) * head_dim;
    }
    if (!rotate) {
        if (dst)
            for (int i = threadIdx.x; i < head_dim; i += blockDim.x) dst[i] = src[i];
        return;
    }
    const float* cos_row = cos_table + static_cast<size_t>(pos) * half;
    const float* sin_row = sin_table + static_cast<size_t>(pos) * half;
    T* target = dst ? dst : src;
    for (int i = threadIdx.x; i < half; i += blockDim.x) {
        const float x1 = to_float(src[i]);
        const float x2 = to_float(src[i + half]);
        const float c = cos_row[i];
        const float s = sin_row[i];
        target[i] = from_float<T>(x1 * c - x2 * s);
        target[i + half] = from_float<T>(x2 * c + x1 * s);
    }
    if (dst)  // what does not rotate goes to the cache as it is
        for (int i = rotary_dim + threadIdx.x; i < head_dim; i += blockDim.x) dst[i] = src[i];
}

// bf16, head_dim a multiple of 8 and rotary_dim of 16: one workgroup per token; a thread takes 8 rotation
// pairs (or 8 elements that pass through, or 8 value elements) at a time with 16-byte accesses.
__global__ void __launch_bounds__(256)
rope_kv_write_vec8_kernel(bf16_t* __restrict__ qkv, const float* __restrict__ cos_table,
                          const float* __restrict__ sin_table, const int* __restrict__ positions,
                          const int* __restrict__ seq_of_token, const int* __restrict__ seq_slot,
                          const int* __restrict__ block_table, int table_width, bf16_t* __restrict__ k_pool,
                          bf16_t* __restrict__ v_pool, int q_heads, int kv_heads, int head_dim, int rotary_dim,
                          int page_size, int rotate, int write_kv) {
    const int token = blockIdx.x;
    const int half = rotary_dim / 2;
    const int chunks = half / 8;  // 8-pair chunks per head
    const int pos = positions[token];
    bf16_t* row = qkv + static_cast<size_t>(token) * (q_heads + 2 * kv_heads) * head_dim;
    int page = -1;
    if (write_kv) page = block_table[static_cast<size_t>(seq_slot[seq_of_token[token]]) * table_width + pos / page_size];
    const int in_page = pos % page_size;
    const float* cos_row = cos_table + static_cast<size_t>(pos) * half;
    const float* sin_row = sin_table + static_cast<size_t>(pos) * half;
    const int rotating = (q_heads + kv_heads) * chunks;
    for (int item = threadIdx.x; item < rotating; item += blockDim.x) {
        const int head = item / chunks;
        const int i = (item - head * chunks) * 8;
        bf16_t* src = row + static_cast<size_t>(head) * head_dim;
        bf16_t* dst = src;
        if (head >= q_heads) {
            if (page < 0) continue;
            dst = k_pool + ((static_cast<size_t>(page) * kv_heads + (head - q_heads)) * page_size + in_page) * head_dim;
        }
        const uint4 lo = *reinterpret_cast<const uint4*>(src + i);
        const uint4 hi = *reinterpret_cast<const uint4*>(src + i + half);
        if (!rotate) {
            if (dst != src) {
                *reinterpret_cast<uint4*>(dst + i) = lo;
                *reinterpret_cast<uint4*>(dst + i + half) = hi;
            }
            continue;
        }
        const uint32_t lw[4] = {lo.x, lo.y, lo.z, lo.w};
        const uint32_t hw[4] = {hi.x, hi.y, hi.z, hi.w};
        const float4 c0 = *reinterpret_cast<const float4*>(cos_row + i), c1 = *reinterpret_cast<const float4*>(cos_row + i + 4);
        const float4 s0 = *reinterpret_cast<const float4*>(sin_row + i), s1 = *reinterpret_cast<const float4*>(sin_row + i + 4);
        const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        uint32_t out_lo[4], out_hi[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float a0 = __uint_as_float(lw[q] << 16), a1 = __uint_as_float(lw[q] & 0xffff0000u);
            const float b0 = __uint_as_float(hw[q] << 16), b1 = __uint_as_float(hw[q] & 0xffff0000u);
            out_lo[q] = pack_bf16(a0 * c[2 * q] - b0 * sn[2 * q], a1 * c[2 * q + 1] - b1 * sn[2 * q + 1]);
            out_hi[q] = pack_bf16(b0 * c[2 * q] + a0 * sn[2 * q], b1 * c[2 * q + 1] + a1 * sn[2 * q + 1]);
        }
        *reinterpret_cast<uint4*>(dst + i) = uint4{out_lo[0], out_lo[1], out_lo[2], out_lo[3]};
        *reinterpret_cast<uint4*>(dst + i + half) = uint4{out_hi[0], out_hi[1], out_hi[2], out_hi[3]};
    }
    if (page < 0) return;
    // key dimensions that do not rotate go to the cache as they are
    const int passing = (head_dim - rotary_dim) / 8;
    for (int item = threadIdx.x; item < kv_heads * passing; item += blockDim.x) {
        const int head = item / passing;
        const int d = rotary_dim + (item - head * passing) * 8;
        bf16_t* dst = k_pool + ((static_cast<size_t>(page) * kv_heads + head) * page_size + in_page) * head_dim;
        *reinterpret_cast<uint4*>(dst + d) =
            *reinterpret_cast<const uint4*>(row + static_cast<size_t>(q_heads + head) * head_dim + d);
    }
    // values: element d of the token goes to [d, pos % page_size] of the transposed page
    const int value_items = kv_heads * (head_dim / 8);
    for (int item = threadIdx.x; item < value_items; item += blockDim.x) {
        const int head = item / (head_dim / 8);
        const int d = (item - head * (head_dim / 8)) * 8;
        const uint4 raw = *reinterpret_cast<const uint4*>(row + static_cast<size_t>(q_heads + kv_heads + head) * head_dim + d);
        bf16_t* column = v_pool + (static_cast<size_t>(page) * kv_heads + head) * page_size * head_dim + in_page;
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            column[static_cast<size_t>(d + 2 * q) * page_size].bits = static_cast<uint16_t>(w[q] & 0xffffu);
            column[static_cast<size_t>(d + 2 * q + 1) * page_size].bits = static_cast<uint16_t>(w[q] >> 16);
        }
    }
}

CIE_API int cie_rope_kv_write(void* stream, int dtype, void* qkv, const float* cos_table,
                              const float* sin_table, const int* positions, const int* seq_of_token,
                              const int* seq_slot, const int* block_table, int table_width,
                              void* k_pool, void* v_pool, int tokens, int q_heads, int kv_heads,
                              int head_dim, int rotary_dim, int page_size, int rotate, int write_kv) {
    if (tokens < 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || page_size <= 0 || table_width <= 0 ||
        rotary_dim < 0 || rotary_dim % 2 || rotary_dim > head_dim)
        return CIE_BAD_ARGUMENT;
    if (!rotate) rotary_dim = 0;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_BF16 && head_dim % 8 == 0 && rotary_dim % 16 == 0) {
        rope_kv_write_vec8_kernel<<<tokens, 256, 0, s>>>(
            static_cast<bf16_t*>(qkv), cos_table, sin_table, positions, seq_of_token, seq_slot, block_table, table_width,
            static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), q_heads, kv_heads, head_dim, rotary_dim, page_size,
            rotate, write_kv);
        return cie_after_launch();
    }
    dim3 grid(tokens, q_heads + 2 * kv_heads);
    if (dtype == CIE_F32)
        rope_kv_write_kernel<float><<<grid, 64, 0, s>>>(
            static_cast<float*>(qkv), cos_table, sin_table, positions, seq_of_token, seq_slot, block_table,
            table_width, static_cast<float*>(k_pool), static_cast<float*>(v_pool), q_heads, kv_heads,
            head_dim, rotary_dim, page_size, rotate, write_kv);
    else if (dtype == CIE_BF16)
        rope_kv_write_kernel<bf16_t><<<grid, 64, 0, s>>>(
            static_cast<bf16_t*>(qkv), cos_table, sin_table, positions, seq_of_token, seq_slot, block_table,
            table_width, static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), q_heads, kv_heads,
            head_dim, rotary_dim, page_size, rotate, write_kv);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
