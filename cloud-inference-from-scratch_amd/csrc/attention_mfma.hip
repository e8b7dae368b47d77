// Paged grouped-query attention on the matrix cores (bfloat16), for decode
// tokens (with the context split over many waves) and for prompt portions.
//
// Cache layout: keys   [pages, kv_heads, page_size, D]   (a key row is contiguous)
//               values [pages, kv_heads, D, page_size]   (transposed: a head
//               dimension's page_size values are contiguous), so that both the
//               K operand of Q.K^T and the V operand of P.V are plain vector loads.
//
// Work unit = one wave = (tile, kv head, split):
//   tile   up to `tokens_per_tile` consecutive query tokens of one sequence; the
//          rows of the tile are (token, head of the group): row = token * G + head,
//          at most 16 * RT rows.  All rows share the KV head's keys and values.
//   split  a contiguous part of the tile's key range; partial results of the
//          splits are merged by `attention_merge_kernel`.
//
// Per block of 32 keys:
//   S^T[key, row] = K[key, :] . Q[row, :]      v_mfma_f32_16x16x32_bf16, A = K, B = Q
//   lane (r = lane % 16, g = lane / 16) then holds, for row r, the scores of keys
//   g*4 .. g*4+3 of each 16-key tile: exactly the A-operand layout of P for
//   O[row, d] += P[row, key] * V[key, d]       A = P (bf16), B = V^T rows
//   The spread of a block's keys (and of a head's dimensions) over the lanes is
//   the same for both operands of a product, which is all a dot product needs.
// Scores, running maximum, sums and the output accumulator are float32.  The softmax runs in base 2:
// scores are scaled by scale * log2(e) once, so that each probability is one v_exp_f32; the
// accumulator is rescaled only in blocks where some row's running maximum moved.
#include "attention_args.h"
#include "common.h"

using namespace cie_attention;

namespace {

template <int D, int RT>
__global__ void __launch_bounds__(64) paged_attention_mfma_kernel(AttentionArgs a) {
    constexpr int NK = D / 32;   // matrix products per 16-key tile of Q.K^T
    constexpr int ND = D / 16;   // 16-wide output tiles of the head dimension
    constexpr int ROWS = 16 * RT;
    const int lane = threadIdx.x;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int tile = blockIdx.x;
    const int kv_head = blockIdx.y;
    const int split = blockIdx.z;
    const int group = a.q_heads / a.kv_heads;
    const int seq = a.tile_seq ? a.tile_seq[tile] : tile;  // (no lists: tile i is the first tile of sequence i)
    const int q0 = a.tile_seq ? a.tile_q0[tile] : 0;
    const int start = a.seq_start[seq];
    const int n_tok = min(a.tokens_per_tile, a.seq_q_len[seq] - q0);
    const int n_rows = n_tok * group;
    const int first_row_token = a.q_start_loc[seq] + q0;
    const int page_size = 1 << a.page_shift;
    const int page_mask = page_size - 1;
    const int* table = a.block_table + static_cast<size_t>(a.seq_slot[seq]) * a.table_width;
    const float scale_log2 = a.scale * 1.44269504088896341f;

    // keys this tile can see at all, and this split's share of them
    const int hi = start + q0 + n_tok;
    const int lo = (a.window > 0) ? max(0, start + q0 + 1 - a.window) : 0;
    int range_begin = lo & ~(kKeysPerBlock - 1);
    int range_end = hi;
    if (a.n_splits > 1) {
        int per_split = a.keys_per_split;
        if (a.max_context_dev) {
            int most = *a.max_context_dev;
            if (a.window > 0) most = min(most, a.window + 2 * kKeysPerBlock);
            per_split = ((most + a.n_splits - 1) / a.n_splits + kKeysPerBlock - 1) & ~(kKeysPerBlock - 1);
        }
        range_begin += split * per_split;
        range_end = min(hi, range_begin + per_split);
        if (range_begin >= range_end) {  // no keys in this share: its statistics say so, its sums are never read
            float* pml = a.part_ml + ((static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + split) * ROWS * 2;
            if (lane < ROWS) {
                pml[lane * 2] = -INFINITY;
                pml[lane * 2 + 1] = 0.f;
            }
            return;
        }
    }

    // Q fragments (B operand) and each lane's row facts
    uint4 qf[RT][NK];
    int row_pos[RT];   // position of the lane's row r of tile rt; -1 for a row that does not exist
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = rt * 16 + r;
        const bool valid = row < n_rows;
        const int tok = row / group;
        const int head = row - tok * group;
        row_pos[rt] = valid ? start + q0 + tok : -1;
        const bf16_t* q_row = a.q + static_cast<size_t>(first_row_token + tok) * a.q_row_stride +
                              static_cast<size_t>(kv_head * group + head) * D + g * (D / 4);
#pragma unroll
        for (int j = 0; j < NK; ++j)
            qf[rt][j] = valid ? *reinterpret_cast<const uint4*>(q_row + j * 8) : uint4{0, 0, 0, 0};
    }

    float m_run[RT], l_run[RT];
    floatx4 o[RT][ND];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m_run[rt] = -INFINITY;
        l_run[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) o[rt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }

    for (int kb = range_begin; kb < range_end; kb += kKeysPerBlock) {
        // ---- S^T = K . Q^T for two 16-key tiles
        floatx4 s[RT][2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const int key = min(kb + kt * 16 + r, hi - 1);  // rows past the end are masked below
            const int page = table[key >> a.page_shift];
            const bf16_t* k_row = a.k_pool +
                (((static_cast<size_t>(page) * a.kv_heads + kv_head) << a.page_shift) + (key & page_mask)) * D +
                g * (D / 4);
            uint4 kf[NK];
#pragma unroll
            for (int j = 0; j < NK; ++j) kf[j] = *reinterpret_cast<const uint4*>(k_row + j * 8);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < NK; ++j)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[j]),
                                                                  __builtin_bit_cast(bf16x8, qf[rt][j]), acc, 0, 0, 0);
                s[rt][kt] = acc;
            }
        }
        // ---- V^T fragments of the block (B operand): for each 16-wide d tile, 4 keys of each 16-key tile
        uint2 vf[ND][2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const int key = min(kb + kt * 16 + g * 4, (hi - 1) & ~3);
            const int page = table[key >> a.page_shift];
            const bf16_t* v_base = a.v_pool +
                ((static_cast<size_t>(page) * a.kv_heads + kv_head) * D << a.page_shift) + (key & page_mask);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
                vf[dt][kt] = *reinterpret_cast<const uint2*>(v_base + (static_cast<size_t>(dt * 16 + r) << a.page_shift));
        }
        // ---- mask, running softmax, P as A operand, O += P . V
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int pos = row_pos[rt];
            const int row_lo = (a.window > 0) ? pos + 1 - a.window : 0;
            float block_max = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = kb + kt * 16 + g * 4 + i;
                    const bool seen = key <= pos && key >= row_lo && key < range_end;
                    const float v = seen ? s[rt][kt][i] * scale_log2 : -INFINITY;
                    s[rt][kt][i] = v;
                    block_max = fmaxf(block_max, v);
                }
            }
            block_max = fmaxf(block_max, __shfl_xor(block_max, 16, kWave));
            block_max = fmaxf(block_max, __shfl_xor(block_max, 32, kWave));
            const float m_new = fmaxf(m_run[rt], block_max);
            const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[rt] - m_safe);  // m_run = -inf: 0, and l, O are 0 anyway
            const bool moved = m_new != m_run[rt];
            m_run[rt] = m_new;
            float p_sum = 0.f;
            uint32_t pw[4];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                const float p0 = __builtin_amdgcn_exp2f(s[rt][kt][0] - m_safe);
                const float p1 = __builtin_amdgcn_exp2f(s[rt][kt][1] - m_safe);
                const float p2 = __builtin_amdgcn_exp2f(s[rt][kt][2] - m_safe);
                const float p3 = __builtin_amdgcn_exp2f(s[rt][kt][3] - m_safe);
                p_sum += (p0 + p1) + (p2 + p3);
                pw[kt * 2] = pack_bf16(p0, p1);
                pw[kt * 2 + 1] = pack_bf16(p2, p3);
            }
            l_run[rt] = l_run[rt] * alpha + p_sum;
            // with one row tile (decode) the straight-line form schedules better than the branch
            if (RT == 1 || __any(moved)) {
                // the accumulator's rows are g*4+i, the statistics' row is r: fetch alpha of those rows
                float alpha_o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) alpha_o[i] = __shfl(alpha, g * 4 + i, kWave);
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[rt][dt][i] *= alpha_o[i];
            }
            const bf16x8 p_frag = __builtin_bit_cast(bf16x8, (uint4{pw[0], pw[1], pw[2], pw[3]}));
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const uint4 v = uint4{vf[dt][0].x, vf[dt][0].y, vf[dt][1].x, vf[dt][1].y};
                o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag, __builtin_bit_cast(bf16x8, v), o[rt][dt], 0, 0, 0);
            }
        }
    }

    // ---- finish: sums over the four lane groups, then normalise or hand the partial to the merge
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float l = l_run[rt];
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        if (a.n_splits == 1) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = rt * 16 + g * 4 + i;
                const float l_row = __shfl(l, g * 4 + i, kWave);
                if (row < n_rows) {
                    const int tok = row / group;
                    const int head = row - tok * group;
                    bf16_t* dst = a.out + static_cast<size_t>(first_row_token + tok) * a.q_heads * D +
                                  static_cast<size_t>(kv_head * group + head) * D;
                    const float inv = 1.0f / l_row;
#pragma unroll
                    for (int dt = 0; dt < ND; ++dt) dst[dt * 16 + r] = from_float<bf16_t>(o[rt][dt][i] * inv);
                }
            }
        } else {
            const size_t unit = (static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + split;
            float* po = a.part_o + unit * ROWS * D;
            float* pml = a.part_ml + unit * ROWS * 2;
            if (g == 0) {
                pml[(rt * 16 + r) * 2] = m_run[rt];
                pml[(rt * 16 + r) * 2 + 1] = l;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = rt * 16 + g * 4 + i;
                if (row >= n_rows) continue;  // (the merge reads the tile's own rows only)
#pragma unroll
                for (int dt = 0; dt < ND; ++dt) po[static_cast<size_t>(row) * D + dt * 16 + r] = o[rt][dt][i];
            }
        }
    }
}

template <int D>
struct KeyBlock {
    uint4 k[2][D / 32];   // A operand of K.Q^T: key kt*16 + r, dimensions (j*4 + g)*8 .. +7
    uint2 v[D / 16][2];   // B operand of P.V: dimension dt*16 + r, keys kt*16 + g*4 .. +3
};

// The prompt form: a workgroup of WAVES waves per (tile, kv head).  Every wave holds all rows of the tile
// and takes every WAVES-th block of 32 keys, so each key and value is read once per workgroup, straight
// from memory into the operand registers; the waves' partial results meet in LDS at the end.
//  * Pages hold at least 16 keys here, so the 16 keys of a product lie in one page: page numbers and
//    base addresses are wave-uniform (scalar loads and scalar arithmetic), and a lane's part of every
//    address is the same for all blocks.
//  * Loads run one block ahead of the products that use them (the key registers are free once the scores
//    are made, the value registers once the output is updated), page numbers two blocks ahead.
//  * Masks are applied only in blocks that reach the causal edge or the window's edge of some row.
//  * The output accumulators stay in the accumulation registers for the whole loop; the vector ALU
//    cannot multiply there, so the rescaling after a moved maximum (rare once the first blocks have set
//    every row's scale) goes through a temporary, register by register.
//  * Tiles are taken from the last to the first: in a prompt the last tiles see the most keys, and
//    starting them first evens out the finish.
__device__ __forceinline__ void scale_accumulator(float& acc, float factor) {
    float t;
    asm volatile(
        "v_accvgpr_read_b32 %1, %0\n\t"
        "v_mul_f32 %1, %1, %2\n\t"
        "v_accvgpr_write_b32 %0, %1"
        : "+a"(acc), "=&v"(t)
        : "v"(factor));
}

template <int D, int RT, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) paged_attention_tile_kernel(AttentionArgs a) {
    constexpr int NK = D / 32;
    constexpr int ND = D / 16;
    constexpr int ROWS = 16 * RT;
    constexpr int STEP = kKeysPerBlock * WAVES;
    __shared__ float lds_ml[WAVES][ROWS][2];
    __shared__ float lds_o[(WAVES > 1 ? WAVES - 1 : 1) * ND * 4 * kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int r = lane & 15;
    const int g = lane >> 4;
    // Workgroups go to the 8 XCDs in turn (workgroup b to XCD b % 8), and each XCD has an L2 of its own.
    // All tiles of a kv head read the same keys and values, so where the heads divide the XCDs a head's
    // tiles are given to its own XCDs: that L2 then holds one head's cache instead of every head's.
    int tile_index, kv_head;
    if (a.xcds_per_head > 0) {
        const int xcd = blockIdx.x % kXcds;
        kv_head = xcd % a.kv_heads;
        tile_index = (blockIdx.x / kXcds) * a.xcds_per_head + xcd / a.kv_heads;
    } else {
        kv_head = blockIdx.x % a.kv_heads;
        tile_index = blockIdx.x / a.kv_heads;
    }
    if (tile_index >= a.n_tiles) return;  // padding of the grid; the whole workgroup leaves
    const int tile = a.n_tiles - 1 - tile_index;
    const int group = a.q_heads / a.kv_heads;
    const int seq = a.tile_seq ? a.tile_seq[tile] : tile;  // (no lists: tile i is the first tile of sequence i)
    const int q0 = a.tile_seq ? a.tile_q0[tile] : 0;
    const int start = a.seq_start[seq];
    const int n_tok = min(a.tokens_per_tile, a.seq_q_len[seq] - q0);
    const int n_rows = n_tok * group;
    const int rt_used = (n_rows + 15) / 16;  // row tiles that hold a row at all (a single token beside portions: one)
    const int first_row_token = a.q_start_loc[seq] + q0;
    const int page_mask = (1 << a.page_shift) - 1;
    const int* table = a.block_table + static_cast<size_t>(a.seq_slot[seq]) * a.table_width;
    const float scale_log2 = a.scale * 1.44269504088896341f;
    const int hi = start + q0 + n_tok;
    const int lo = (a.window > 0) ? max(0, start + q0 + 1 - a.window) : 0;
    int range_begin = lo & ~(kKeysPerBlock - 1);
    int range_end = hi;
    if (a.n_splits > 1) {  // this workgroup's share of the keys (blockIdx.y); the merge kernel joins the shares
        int per_split = a.keys_per_split;
        if (a.max_context_dev) {
            int most = *a.max_context_dev;
            if (a.window > 0) most = min(most, a.window + 2 * kKeysPerBlock);
            per_split = ((most + a.n_splits - 1) / a.n_splits + kKeysPerBlock - 1) & ~(kKeysPerBlock - 1);
        }
        range_begin += blockIdx.y * per_split;
        range_end = min(hi, range_begin + per_split);
        if (range_begin >= range_end) {  // no keys in this share: its statistics say so, its sums are never read
            float* pml = a.part_ml + ((static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + blockIdx.y) * ROWS * 2;
            if (threadIdx.x < ROWS) {
                pml[threadIdx.x * 2] = -INFINITY;
                pml[threadIdx.x * 2 + 1] = 0.f;
            }
            return;  // (the whole workgroup: the range is the same for all its waves)
        }
    }
    const int first_pos = start + q0;              // position of the tile's first token
    const int last_pos = start + q0 + n_tok - 1;   // and of its last
    const int last_group = (hi - 1) & ~15;         // the last 16 keys that have a page

    uint4 qf[RT][NK];
    int row_pos[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = rt * 16 + r;
        const bool valid = row < n_rows;
        const int tok = row / group;
        const int head = row - tok * group;
        row_pos[rt] = valid ? start + q0 + tok : -1;
        const bf16_t* q_row = a.q + static_cast<size_t>(first_row_token + tok) * a.q_row_stride +
                              static_cast<size_t>(kv_head * group + head) * D + g * 8;
#pragma unroll
        for (int j = 0; j < NK; ++j)  // product j takes dimensions (j*4 + g)*8 .. +7 of both operands
            qf[rt][j] = valid ? *reinterpret_cast<const uint4*>(q_row + j * 32) : uint4{0, 0, 0, 0};
    }
    float m_run[RT], l_run[RT];
    float o[RT][ND][4];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m_run[rt] = -INFINITY;
        l_run[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[rt][dt][i] = 0.f;
    }

    // a lane's share of the addresses, in bytes from the start of a (page, kv head)'s keys or values
    const uint32_t k_lane = static_cast<uint32_t>(r * D + g * 8) * 2u;
    uint32_t v_lane[ND];
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) v_lane[dt] = static_cast<uint32_t>(((dt * 16 + r) << a.page_shift) + g * 4) * 2u;

    // the wave-uniform rest: the 16 keys from `first` on (clamped to keys that have a page; what lies past
    // the end is masked where it is used)
    auto group_of = [&](int first) { return min(first, last_group); };
    // block tables do not change while a kernel runs: read them through the constant address space, with a
    // wave-uniform index, so that they come through the scalar cache and do not queue behind the key loads
    typedef const __attribute__((address_space(4))) int* const_int_ptr;
    const const_int_ptr table_c = (const_int_ptr)(uintptr_t)table;
    auto page_of = [&](int first) {
        return table_c[__builtin_amdgcn_readfirstlane(group_of(first) >> a.page_shift)];
    };
    auto load_keys = [&](int kb, const int (&page)[2], KeyBlock<D>& b) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const int in_page = group_of(kb + kt * 16) & page_mask;
            const char* base = reinterpret_cast<const char*>(
                a.k_pool + (((static_cast<size_t>(page[kt]) * a.kv_heads + kv_head) << a.page_shift) + in_page) * D);
#pragma unroll
            for (int j = 0; j < NK; ++j) b.k[kt][j] = *reinterpret_cast<const uint4*>(base + k_lane + j * 64);
        }
    };
    auto load_values = [&](int kb, const int (&page)[2], KeyBlock<D>& b) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            const int in_page = group_of(kb + kt * 16) & page_mask;
            const char* base = reinterpret_cast<const char*>(
                a.v_pool + ((static_cast<size_t>(page[kt]) * a.kv_heads + kv_head) * D << a.page_shift) + in_page);
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) b.v[dt][kt] = *reinterpret_cast<const uint2*>(base + v_lane[dt]);
        }
    };

    KeyBlock<D> blk;
    int page[2], page_next[2];
    int kb = range_begin + wave * kKeysPerBlock;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
        page[kt] = page_of(kb + kt * 16);
        page_next[kt] = page_of(kb + STEP + kt * 16);
    }
    load_keys(kb, page, blk);
    load_values(kb, page, blk);
    for (; kb < range_end; kb += STEP) {
        floatx4 s[RT][2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                // (Every row tile is multiplied, also one without rows: a way out of this loop would be a short cut
                // from a product to the first read of its result, and the compiler counts the wait between the two
                // along the straight path only.  With that short cut a tile of one token read scores that were not
                // finished, now and then.)
                floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < NK; ++j)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, blk.k[kt][j]),
                                                                  __builtin_bit_cast(bf16x8, qf[rt][j]), acc, 0, 0, 0);
                s[rt][kt] = acc;
            }
        load_keys(kb + STEP, page_next, blk);  // the next block's keys travel while this block's softmax runs
        int page_after[2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) page_after[kt] = page_of(kb + 2 * STEP + kt * 16);

        // ---- running maxima of all row tiles first; masks only in blocks that reach a row's edge
        const bool edge = kb + kKeysPerBlock - 1 > first_pos || (a.window > 0 && kb < last_pos + 1 - a.window);
        // The reference of a row moves only when a score passes it by more than kLazyRescale: until then
        // probabilities may reach 2^kLazyRescale, which float32 sums and bfloat16 products hold as well.  Each of
        // a row's four lanes can tell that of its own eight scores, so the common block needs no maximum across lanes.
        float own_max[RT], m_use[RT];
        bool moved = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (rt >= rt_used) break;
            if (edge) {
                const int pos = row_pos[rt];
                const int row_lo = (a.window > 0) ? pos + 1 - a.window : 0;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int key = kb + kt * 16 + g * 4 + i;
                        if (!(key <= pos && key >= row_lo)) s[rt][kt][i] = -INFINITY;
                    }
            }
            own_max[rt] = fmaxf(fmaxf(fmaxf(s[rt][0][0], s[rt][0][1]), fmaxf(s[rt][0][2], s[rt][0][3])),
                                fmaxf(fmaxf(s[rt][1][0], s[rt][1][1]), fmaxf(s[rt][1][2], s[rt][1][3])));
            moved = moved || own_max[rt] * scale_log2 > m_run[rt] + kLazyRescale;  // (the scale is positive)
        }
        if (__any(moved)) {
            // the products that wrote these accumulators were issued a whole score phase ago
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                if (rt >= rt_used) break;
                const float block_max = rows_max(own_max[rt]) * scale_log2;  // maxima are kept in scaled base-2 units
                const float m_new = (block_max > m_run[rt] + kLazyRescale) ? block_max : m_run[rt];
                const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = __builtin_amdgcn_exp2f(m_run[rt] - m_safe);  // m_run = -inf: 0, and l, O are 0 anyway
                m_run[rt] = m_new;
                l_run[rt] *= alpha;
                float alpha_o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) alpha_o[i] = __shfl(alpha, g * 4 + i, kWave);
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) scale_accumulator(o[rt][dt][i], alpha_o[i]);
            }
            asm volatile("s_nop 7");  // before a product reads what was just written
        }
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) m_use[rt] = (m_run[rt] == -INFINITY) ? 0.f : m_run[rt];
        // ---- probabilities (one fused multiply-add and one exp2 each) and O += P . V, row tile by row tile
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (rt >= rt_used) break;
            float p_sum = 0.f;
            uint32_t pw[4];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][0], scale_log2, -m_use[rt]));
                const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][1], scale_log2, -m_use[rt]));
                const float p2 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][2], scale_log2, -m_use[rt]));
                const float p3 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][3], scale_log2, -m_use[rt]));
                p_sum += (p0 + p1) + (p2 + p3);
                pw[kt * 2] = pack_bf16(p0, p1);
                pw[kt * 2 + 1] = pack_bf16(p2, p3);
            }
            l_run[rt] += p_sum;
            const bf16x8 p_frag = __builtin_bit_cast(bf16x8, (uint4{pw[0], pw[1], pw[2], pw[3]}));
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const uint4 v = uint4{blk.v[dt][0].x, blk.v[dt][0].y, blk.v[dt][1].x, blk.v[dt][1].y};
                floatx4 acc = {o[rt][dt][0], o[rt][dt][1], o[rt][dt][2], o[rt][dt][3]};
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag, __builtin_bit_cast(bf16x8, v), acc, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; ++i) o[rt][dt][i] = acc[i];
            }
        }
        load_values(kb + STEP, page_next, blk);  // and its values while the next scores are made
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) page_next[kt] = page_after[kt];
    }

    // ---- the waves' partial results meet: statistics first, then one row tile at a time through LDS
    float l_all[RT], m_all[RT], own_weight[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const float l = rows_sum(l_run[rt]);
        l_all[rt] = l;
        m_all[rt] = m_run[rt];
        own_weight[rt] = 1.f;
        if (WAVES > 1 && g == 0) {
            lds_ml[wave][rt * 16 + r][0] = m_run[rt];
            lds_ml[wave][rt * 16 + r][1] = l;
        }
    }
    if (WAVES > 1) {
        __syncthreads();
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            float m_max = -INFINITY;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) m_max = fmaxf(m_max, lds_ml[w][rt * 16 + r][0]);
            m_all[rt] = m_max;
            const float m_safe = (m_max == -INFINITY) ? 0.f : m_max;
            float l = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w)
                l += lds_ml[w][rt * 16 + r][1] * __builtin_amdgcn_exp2f(lds_ml[w][rt * 16 + r][0] - m_safe);
            l_all[rt] = l;
            own_weight[rt] = __builtin_amdgcn_exp2f(m_run[rt] - m_safe);
        }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (rt >= rt_used) break;  // (no row of it exists: nothing to sum, nothing to store)
        const int owner = rt % WAVES;
        if (WAVES > 1) {
            float w_o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) w_o[i] = __shfl(own_weight[rt], g * 4 + i, kWave);
            if (rt > 0) __syncthreads();  // the tile before has been read
            if (wave != owner) {
                float* slot = lds_o + (wave < owner ? wave : wave - 1) * (ND * 4 * kWave);
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) slot[(dt * 4 + i) * kWave + lane] = o[rt][dt][i] * w_o[i];
            } else {
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[rt][dt][i] *= w_o[i];
            }
            __syncthreads();
            if (wave == owner) {
#pragma unroll
                for (int w = 0; w < WAVES - 1; ++w)
#pragma unroll
                    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) o[rt][dt][i] += lds_o[w * (ND * 4 * kWave) + (dt * 4 + i) * kWave + lane];
            }
        }
        if (wave != owner) continue;
        if (a.n_splits > 1) {  // this share's sums and statistics for the merge kernel
            const size_t unit = (static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + blockIdx.y;
            float* po = a.part_o + unit * ROWS * D;
            float* pml = a.part_ml + unit * ROWS * 2;
            if (g == 0) {
                pml[(rt * 16 + r) * 2] = m_all[rt];
                pml[(rt * 16 + r) * 2 + 1] = l_all[rt];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = rt * 16 + g * 4 + i;
                if (row >= n_rows) continue;  // (the merge reads the tile's own rows only)
#pragma unroll
                for (int dt = 0; dt < ND; ++dt) po[static_cast<size_t>(row) * D + dt * 16 + r] = o[rt][dt][i];
            }
            continue;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = rt * 16 + g * 4 + i;
            const float l_row = __shfl(l_all[rt], g * 4 + i, kWave);
            if (row < n_rows) {
                const int tok = row / group;
                const int head = row - tok * group;
                bf16_t* dst = a.out + static_cast<size_t>(first_row_token + tok) * a.q_heads * D +
                              static_cast<size_t>(kv_head * group + head) * D;
                const float inv = 1.0f / l_row;
#pragma unroll
                for (int dt = 0; dt < ND; ++dt) dst[dt * 16 + r] = from_float<bf16_t>(o[rt][dt][i] * inv);
            }
        }
    }
}

// Merge the splits of every (tile, kv head): out = sum_s O_s e^(m_s - M) / sum_s l_s e^(m_s - M).
// One workgroup per (tile, kv head, row).  The parts' weights are made once in LDS; the threads are
// laid out as (group, four head dimensions): group g sums parts g, g + groups, ... with independent
// 16-byte loads, and the groups' sums meet in LDS.
constexpr int kMergeMaxSplits = 1024;
constexpr int kMergeThreads = 256;

__global__ void __launch_bounds__(kMergeThreads)
attention_merge_kernel(AttentionArgs a, int head_dim, int rows_per_tile) {
    __shared__ float weight[kMergeMaxSplits];
    __shared__ float scratch[16];
    __shared__ floatx4 group_sum[kMergeThreads];
    const int tile = blockIdx.x;
    const int kv_head = blockIdx.y;
    const int row = blockIdx.z;
    const int group = a.q_heads / a.kv_heads;
    const int seq = a.tile_seq ? a.tile_seq[tile] : tile;  // (no lists: tile i is the first tile of sequence i)
    const int q0 = a.tile_seq ? a.tile_q0[tile] : 0;
    const int n_tok = min(a.tokens_per_tile, a.seq_q_len[seq] - q0);
    if (row >= n_tok * group) return;
    if (a.whole_in_first_share) {  // a tile with all its keys in the first share has written its result itself
        const int hi = a.seq_start[seq] + q0 + n_tok;
        const int lo = (a.window > 0) ? max(0, a.seq_start[seq] + q0 + 1 - a.window) : 0;
        int per_split = a.keys_per_split;
        if (a.max_context_dev) {
            int most = *a.max_context_dev;
            if (a.window > 0) most = min(most, a.window + 2 * kKeysPerBlock);
            per_split = ((most + a.n_splits - 1) / a.n_splits + kKeysPerBlock - 1) & ~(kKeysPerBlock - 1);
        }
        if (all_in_first_share(lo & ~(kKeysPerBlock - 1), hi, per_split)) return;
    }
    const size_t unit0 = (static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits;
    const int per_row = head_dim / 4;            // threads that cover a row of sums
    const int groups = kMergeThreads / per_row;  // parts summed side by side
    const int mine = threadIdx.x / per_row;
    const int chunk = threadIdx.x - mine * per_row;
    const bool active = mine < groups;
    // The thread's share of its first parts' sums is fetched before the weights are known: these loads
    // depend on nothing and travel while the statistics are read and reduced.
    constexpr int kEarly = 4;
    const size_t stride = static_cast<size_t>(rows_per_tile) * per_row;
    const floatx4* po_row =
        reinterpret_cast<const floatx4*>(a.part_o + (unit0 * rows_per_tile + row) * head_dim) + chunk;
    floatx4 early[kEarly];
#pragma unroll
    for (int u = 0; u < kEarly; ++u) {
        const int s = mine + u * groups;
        early[u] = (active && s < a.n_splits) ? po_row[s * stride] : floatx4{0.f, 0.f, 0.f, 0.f};
    }
    // (a thread's first share: its maximum and its sum come together and are kept for the second pass)
    const bool has_first = threadIdx.x < a.n_splits;
    const float2 first_ml = has_first ? *reinterpret_cast<const float2*>(
                                            a.part_ml + ((unit0 + threadIdx.x) * rows_per_tile + row) * 2)
                                      : float2{-INFINITY, 0.f};
    float m_local = first_ml.x;
    for (int s = threadIdx.x + blockDim.x; s < a.n_splits; s += blockDim.x)
        m_local = fmaxf(m_local, a.part_ml[((unit0 + s) * rows_per_tile + row) * 2]);
    const float m_all = block_max(m_local, scratch);
    float den_local = 0.f;
    if (has_first) {
        const float w = (first_ml.x == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(first_ml.x - m_all);  // maxima are kept in base 2
        weight[threadIdx.x] = w;
        den_local = first_ml.y * w;
    }
    for (int s = threadIdx.x + blockDim.x; s < a.n_splits; s += blockDim.x) {
        const float* ml = a.part_ml + ((unit0 + s) * rows_per_tile + row) * 2;
        const float w = (ml[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ml[0] - m_all);
        weight[s] = w;
        den_local += ml[1] * w;
    }
    const float den = block_sum(den_local, scratch);  // its barriers also publish weight[]
    floatx4 num = {0.f, 0.f, 0.f, 0.f};
    if (active) {
#pragma unroll
        for (int u = 0; u < kEarly; ++u) {
            const int s = mine + u * groups;
            if (s < a.n_splits && weight[s] != 0.f) num += early[u] * weight[s];  // (a share without keys wrote no sums)
        }
        // the rest eight at a time, their loads all under way before the first is used: no branch stands between
        // them (behind one the compiler waits for each load in turn; a sequence over 4,096 keys in 128 shares
        // has twelve of them per thread).  A share past the last reads the last again, and what a share without
        // keys left in its place is read too: a select drops both.
        for (int s0 = mine + kEarly * groups; s0 < a.n_splits; s0 += 8 * groups) {
            floatx4 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = po_row[min(s0 + j * groups, a.n_splits - 1) * stride];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int s = s0 + j * groups;
                const float w = weight[min(s, a.n_splits - 1)];
                const bool real = s < a.n_splits && w != 0.f;
#pragma unroll
                for (int i = 0; i < 4; ++i) num[i] += real ? v[j][i] * w : 0.f;
            }
        }
    }
    group_sum[threadIdx.x] = num;
    __syncthreads();
    if (threadIdx.x >= per_row) return;
    for (int g = 1; g < groups; ++g) num += group_sum[g * per_row + chunk];
    const int tok = row / group;
    const int head = row - tok * group;
    bf16_t* dst = a.out + static_cast<size_t>(a.q_start_loc[seq] + q0 + tok) * a.q_heads * head_dim +
                  static_cast<size_t>(kv_head * group + head) * head_dim + 4 * chunk;
    const float inv = 1.0f / den;
    uint2 packed;
    packed.x = from_float<bf16_t>(num[0] * inv).bits | (static_cast<uint32_t>(from_float<bf16_t>(num[1] * inv).bits) << 16);
    packed.y = from_float<bf16_t>(num[2] * inv).bits | (static_cast<uint32_t>(from_float<bf16_t>(num[3] * inv).bits) << 16);
    *reinterpret_cast<uint2*>(dst) = packed;
}

// The same merge for tiles of many rows and few shares (prompt portions whose keys are cut): a workgroup
// takes 16 rows of a (tile, kv head), a thread four head dimensions at a time of one row; every thread
// of a row makes the shares' weights for itself from the few statistics.  (With one workgroup for each row,
// as above, a step of 2,048 tokens would start 32,768 workgroups.)
constexpr int kMergeFewShares = 16;

__global__ void __launch_bounds__(256)
attention_merge_rows_kernel(AttentionArgs a, int head_dim, int rows_per_tile) {
    const int tile = blockIdx.x;
    const int kv_head = blockIdx.y;
    const int row = blockIdx.z * 16 + threadIdx.x / 16;
    const int lane16 = threadIdx.x % 16;
    const int group = a.q_heads / a.kv_heads;
    const int seq = a.tile_seq ? a.tile_seq[tile] : tile;
    const int q0 = a.tile_seq ? a.tile_q0[tile] : 0;
    const int n_tok = min(a.tokens_per_tile, a.seq_q_len[seq] - q0);
    if (row >= n_tok * group) return;
    if (a.whole_in_first_share) {  // a tile with all its keys in the first share has written its result itself
        const int hi = a.seq_start[seq] + q0 + n_tok;
        const int lo = (a.window > 0) ? max(0, a.seq_start[seq] + q0 + 1 - a.window) : 0;
        int per_split = a.keys_per_split;
        if (a.max_context_dev) {
            int most = *a.max_context_dev;
            if (a.window > 0) most = min(most, a.window + 2 * kKeysPerBlock);
            per_split = ((most + a.n_splits - 1) / a.n_splits + kKeysPerBlock - 1) & ~(kKeysPerBlock - 1);
        }
        if (all_in_first_share(lo & ~(kKeysPerBlock - 1), hi, per_split)) return;
    }
    const size_t unit0 = (static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits;
    float weight[kMergeFewShares];
    float m_all = -INFINITY;
#pragma unroll
    for (int s = 0; s < kMergeFewShares; ++s) {
        weight[s] = (s < a.n_splits) ? a.part_ml[((unit0 + s) * rows_per_tile + row) * 2] : -INFINITY;
        m_all = fmaxf(m_all, weight[s]);
    }
    float den = 0.f;
#pragma unroll
    for (int s = 0; s < kMergeFewShares; ++s) {
        const float w = (weight[s] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(weight[s] - m_all);  // maxima are kept in base 2
        weight[s] = w;
        if (s < a.n_splits) den += a.part_ml[((unit0 + s) * rows_per_tile + row) * 2 + 1] * w;
    }
    const float inv = 1.0f / den;
    const int tok = row / group;
    const int head = row - tok * group;
    bf16_t* dst = a.out + static_cast<size_t>(a.q_start_loc[seq] + q0 + tok) * a.q_heads * head_dim +
                  static_cast<size_t>(kv_head * group + head) * head_dim;
    for (int d = lane16 * 4; d < head_dim; d += 64) {
        floatx4 num = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < kMergeFewShares; ++s)
            if (s < a.n_splits && weight[s] != 0.f)  // (a share without keys wrote no sums)
                num += *reinterpret_cast<const floatx4*>(a.part_o + ((unit0 + s) * rows_per_tile + row) * head_dim + d) * weight[s];
        uint2 packed;
        packed.x = from_float<bf16_t>(num[0] * inv).bits | (static_cast<uint32_t>(from_float<bf16_t>(num[1] * inv).bits) << 16);
        packed.y = from_float<bf16_t>(num[2] * inv).bits | (static_cast<uint32_t>(from_float<bf16_t>(num[3] * inv).bits) << 16);
        *reinterpret_cast<uint2*>(dst + d) = packed;
    }
}

// Which of the two merges a step's shape takes.
int launch_merge(hipStream_t s, const AttentionArgs& a, int n_tiles, int head_dim, int rows_per_tile) {
    const int rows = a.tokens_per_tile * (a.q_heads / a.kv_heads);
    if (rows_per_tile >= kPromptTileRows && a.n_splits <= kMergeFewShares)  // (with fewer rows a tile the first is the faster one)
        attention_merge_rows_kernel<<<dim3(n_tiles, a.kv_heads, (rows + 15) / 16), 256, 0, s>>>(a, head_dim, rows_per_tile);
    else
        attention_merge_kernel<<<dim3(n_tiles, a.kv_heads, rows), kMergeThreads, 0, s>>>(a, head_dim, rows_per_tile);
    return cie_after_launch();
}

template <int D>
int launch_for_dim(hipStream_t s, const AttentionArgs& a, int n_tiles, int row_tiles, int tile_waves) {
    dim3 grid(n_tiles, a.kv_heads, a.n_splits);
    if (tile_waves == kTileWaves) {
        grid = a.xcds_per_head > 0 ? dim3(kXcds * ((n_tiles + a.xcds_per_head - 1) / a.xcds_per_head), a.n_splits)
                                   : dim3(static_cast<unsigned>(n_tiles) * a.kv_heads, a.n_splits);
        if (row_tiles == 1)
            paged_attention_tile_kernel<D, 1, kTileWaves><<<grid, 64 * kTileWaves, 0, s>>>(a);
        else if constexpr (D <= 128) {  // wider heads hold one row tile of accumulators without spilling
            if (row_tiles == 2)
                paged_attention_tile_kernel<D, 2, kTileWaves><<<grid, 64 * kTileWaves, 0, s>>>(a);
            else if (row_tiles == 4)
                paged_attention_tile_kernel<D, 4, kTileWaves><<<grid, 64 * kTileWaves, 0, s>>>(a);
            else
                return CIE_BAD_ARGUMENT;
        } else
            return CIE_BAD_ARGUMENT;
        return cie_after_launch();
    }
    if (row_tiles == 1)
        paged_attention_mfma_kernel<D, 1><<<grid, 64, 0, s>>>(a);
    else if (row_tiles == 2)
        paged_attention_mfma_kernel<D, 2><<<grid, 64, 0, s>>>(a);
    else if (row_tiles == 4)
        paged_attention_mfma_kernel<D, 4><<<grid, 64, 0, s>>>(a);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}

}  // namespace

// tile_waves: 1 (one wave per tile and part), 4 (four waves take a tile's key blocks in turn; row_tiles 1, 2 or 4)
// or 8 (csrc/attention_prompt.hip: tiles of 128 rows, row_tiles = 8, keys and values shared through LDS).
// Workspace sizes (floats) the caller provides when n_splits > 1:
//   part_o  n_tiles * kv_heads * n_splits * 16*row_tiles * head_dim
//   part_ml n_tiles * kv_heads * n_splits * 16*row_tiles * 2
CIE_API int cie_paged_attention_mfma(void* stream, const void* q, int q_row_stride, const void* k_pool,
                                     const void* v_pool, const int* block_table, int table_width,
                                     const int* tile_seq, const int* tile_q0, const int* seq_slot,
                                     const int* seq_start, const int* seq_q_len, const int* q_start_loc,
                                     void* out, float* part_o, float* part_ml, int n_tiles, int q_heads,
                                     int kv_heads, int head_dim, int page_size, int window, float scale,
                                     int n_splits, int tokens_per_tile, int row_tiles, int keys_per_split,
                                     const int* max_context_dev, int tile_waves) {
    if (n_tiles < 0 || q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads || page_size < 4 ||
        (page_size & (page_size - 1)) || table_width <= 0 || n_splits < 1 || n_splits > 65535 ||
        kv_heads > 65535 || tokens_per_tile < 1 || q_row_stride % 8)
        return CIE_BAD_ARGUMENT;
    const int group = q_heads / kv_heads;
    if (tokens_per_tile * group > 16 * row_tiles) return CIE_BAD_ARGUMENT;
    if (n_splits > kMergeMaxSplits) return CIE_BAD_ARGUMENT;
    // the prompt form takes maxima before scaling, which needs a positive scale, and keeps the 16 keys of a
    // product in one page
    if (tile_waves != 1 && ((tile_waves != kTileWaves && tile_waves != kPromptWaves) || !(scale > 0.f) || page_size < 16))
        return CIE_BAD_ARGUMENT;
    // the form that shares keys and values through LDS has tiles of 128 rows (eight waves) or of 64 (four), and
    // heads of up to 128 dimensions
    if (tile_waves == kPromptWaves && ((row_tiles != 8 && row_tiles != 4) || head_dim > 128)) return CIE_BAD_ARGUMENT;
    if (n_splits > 1 && (!part_o || !part_ml ||
                         (!max_context_dev && (keys_per_split <= 0 || keys_per_split % kKeysPerBlock))))
        return CIE_BAD_ARGUMENT;
    if (n_tiles == 0) return CIE_OK;
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    AttentionArgs a;
    a.q = static_cast<const bf16_t*>(q);
    a.q_row_stride = q_row_stride;
    a.k_pool = static_cast<const bf16_t*>(k_pool);
    a.v_pool = static_cast<const bf16_t*>(v_pool);
    a.block_table = block_table;
    a.table_width = table_width;
    a.tile_seq = tile_seq;
    a.tile_q0 = tile_q0;
    a.seq_slot = seq_slot;
    a.seq_start = seq_start;
    a.seq_q_len = seq_q_len;
    a.q_start_loc = q_start_loc;
    a.out = static_cast<bf16_t*>(out);
    a.part_o = part_o;
    a.part_ml = part_ml;
    a.q_heads = q_heads;
    a.kv_heads = kv_heads;
    a.page_shift = page_shift;
    a.window = window;
    a.scale = scale;
    a.n_splits = n_splits;
    a.tokens_per_tile = tokens_per_tile;
    a.keys_per_split = n_splits > 1 ? keys_per_split : 0;
    a.max_context_dev = n_splits > 1 ? max_context_dev : nullptr;
    a.n_tiles = n_tiles;
    a.whole_in_first_share = (tile_waves == kPromptWaves && n_splits > 1) ? 1 : 0;
    a.xcds_per_head = (kv_heads <= kXcds && kXcds % kv_heads == 0) ? kXcds / kv_heads : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int rc;
    if (tile_waves == kPromptWaves) {
        rc = launch_prompt_form(s, a, head_dim, row_tiles);
        if (rc != CIE_OK || n_splits == 1) return rc;
        return launch_merge(s, a, n_tiles, head_dim, 16 * row_tiles);
    }
    switch (head_dim) {
        case 32: rc = launch_for_dim<32>(s, a, n_tiles, row_tiles, tile_waves); break;
        case 64: rc = launch_for_dim<64>(s, a, n_tiles, row_tiles, tile_waves); break;
        case 96: rc = launch_for_dim<96>(s, a, n_tiles, row_tiles, tile_waves); break;
        case 128: rc = launch_for_dim<128>(s, a, n_tiles, row_tiles, tile_waves); break;
        case 256: rc = launch_for_dim<256>(s, a, n_tiles, row_tiles, tile_waves); break;
        default: return CIE_BAD_ARGUMENT;
    }
    if (rc != CIE_OK || n_splits == 1) return rc;
    return launch_merge(s, a, n_tiles, head_dim, 16 * row_tiles);
}
