// Paged grouped-query attention for prompt portions: eight waves per tile of 128 (token, head) rows.
//
// A workgroup takes one tile (up to 128 rows = tokens_per_tile tokens x the heads of one kv head's group)
// and walks the tile's keys 64 at a time.  The keys and values of those 64 positions are read from the
// cache once per workgroup, in 16-byte pieces that follow one another in memory, and laid into LDS in the
// order the matrix instructions take their operands; every wave then reads them from there.  Two stages
// of LDS take turns, so that the loads of the keys after next are under way while a block is worked on.
//
// Wave w owns rows 32 * (w % 4) .. + 31 of the tile and, of each 64 keys, the half w / 4: four waves
// cover the rows, two such sets the keys.  A wave holds 32 rows of the output (64 accumulator registers
// where the head has 128 dimensions), so that two waves fit on a SIMD and the softmax arithmetic of one
// overlaps the matrix products of the other.  The two halves of the keys meet in LDS at the end.
//
// Per block of 32 keys a wave computes, as the other forms do (csrc/attention_mfma.hip):
//   S^T[key, row] = K[key, :] . Q[row, :]     v_mfma_f32_16x16x32_bf16, A = K (from LDS), B = Q (registers)
//   P = 2^(S * scale * log2 e - m)            float32; the reference m of a row moves lazily
//   O[row, d] += P[row, key] * V[key, d]      A = P (registers), B = V^T (from LDS)
//
// LDS layout of one stage (D = head size, C = D / 8 sixteen-byte chunks of a key):
//   keys    64 rows of CS chunk slots (CS = C rounded up to a power of two); chunk c of key k lies in slot
//           c ^ swizzle(k), so that the 16 lanes that read the same chunk of 16 different keys hit 16
//           different groups of banks
//   values  two blocks (one per half) of D rows of 64 bytes: row d holds, for each lane group g, the
//           values of keys g*4 .. g*4+3 of the block's first 16 keys and of its second 16 keys (16 bytes,
//           one read per product); the four 16-byte chunks of a row are swizzled by (d / 4) % 4
#include "attention_args.h"
#include "common.h"

using namespace cie_attention;

namespace {

constexpr int kKeysPerStage = 2 * kKeysPerBlock;  // 64: one block for each half of the waves

// The largest of three or two numbers in one instruction each, and the largest over the four 16-lane rows of a
// wave, written as instructions: the compiler's own maxima first copy every operand onto itself (to quiet
// signalling NaNs, which the hardware's maximum does anyway), three instructions where one does.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float out;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(out) : "v"(a), "v"(b), "v"(c));
    return out;
}

__device__ __forceinline__ float max2(float a, float b) {
    float out;
    asm("v_max_f32 %0, %1, %2" : "=v"(out) : "v"(a), "v"(b));
    return out;
}

__device__ __forceinline__ float rows_max_lean(float v) {
    swap_pair_t a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = max2(__uint_as_float(a[0]), __uint_as_float(a[1]));
    swap_pair_t b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

template <int D>
struct PromptLayout {
    static constexpr int C = D / 8;
    static constexpr int CS = C <= 4 ? 4 : C <= 8 ? 8 : C <= 16 ? 16 : 32;
    static constexpr int kKeyBytes = kKeysPerStage * CS * 16;
    static constexpr int kValueBlockBytes = D * 64;
    static constexpr int kStageBytes = kKeyBytes + 2 * kValueBlockBytes;
    // the swizzle of a key's chunk slots: over 16 consecutive keys, the same chunk lands in 16 different
    // sixteen-byte columns of the 256 bytes that the banks span
    __device__ static __forceinline__ int key_swizzle(int k) {
        if (CS >= 16) return k & 15;
        if (CS == 8) return (k >> 1) & 7;
        return (k >> 2) & 3;
    }
};

// WAVES = 8: tiles of 128 rows; WAVES = 4: the same with tiles of 64 rows, two such workgroups to a compute unit,
// which then walk their keys independently of each other (one's matrix products beside the other's softmax).
template <int D, int WAVES>
__global__ void __launch_bounds__(64 * WAVES, WAVES == 4 ? 2 : 1) paged_attention_prompt_kernel(AttentionArgs a) {
    using L = PromptLayout<D>;
    constexpr int NK = D / 32;
    constexpr int ND = D / 16;
    constexpr int RT = 2;  // 16-row tiles of a wave
    constexpr int QUARTERS = WAVES / 2;        // sets of 32 rows of the tile
    constexpr int kTileRows = 32 * QUARTERS;
    constexpr int kLoaderThreads = 64 * QUARTERS;  // threads that fetch one group of 16 keys
    extern __shared__ __align__(16) unsigned char lds[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int quarter = wave % QUARTERS;   // which 32 rows of the tile
    const int half = wave / QUARTERS;      // which 32 of each 64 keys
    const int r = lane & 15;
    const int g = lane >> 4;

    // tiles of a kv head go to that head's XCDs where the heads divide the 8 XCDs (see attention_mfma.hip)
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
    // The last tiles of a prompt see the most keys: they start first.  Where two workgroups share a compute
    // unit (WAVES = 4) the first half of the launch are the longest tiles in falling order and the second half
    // the shortest in rising order: the hardware fills the units' second places in the order of the first, so
    // that a unit gets a long tile and a short one, every unit about as many keys.
    int tile = a.n_tiles - 1 - tile_index;
    if (WAVES == 4 && tile_index >= (a.n_tiles + 1) / 2) tile = tile_index - (a.n_tiles + 1) / 2;
    const int group = a.q_heads / a.kv_heads;
    const int seq = a.tile_seq ? a.tile_seq[tile] : tile;
    const int q0 = a.tile_seq ? a.tile_q0[tile] : 0;
    const int start = a.seq_start[seq];
    const int n_tok = min(a.tokens_per_tile, a.seq_q_len[seq] - q0);
    const int n_rows = n_tok * group;
    const int first_row_token = a.q_start_loc[seq] + q0;
    const int page_mask = (1 << a.page_shift) - 1;
    const int* table = a.block_table + static_cast<size_t>(a.seq_slot[seq]) * a.table_width;
    const float scale_log2 = a.scale * 1.44269504088896341f;
    const int hi = start + q0 + n_tok;
    const int lo = (a.window > 0) ? max(0, start + q0 + 1 - a.window) : 0;
    int range_begin = lo & ~(kKeysPerBlock - 1);
    int range_end = hi;
    bool whole = a.n_splits == 1;  // this workgroup sees all the tile's keys and writes its result itself
    if (a.n_splits > 1) {
        int per_split = a.keys_per_split;
        if (a.max_context_dev) {
            int most = *a.max_context_dev;
            if (a.window > 0) most = min(most, a.window + 2 * kKeysPerBlock);
            per_split = ((most + a.n_splits - 1) / a.n_splits + kKeysPerBlock - 1) & ~(kKeysPerBlock - 1);
        }
        if (a.whole_in_first_share && all_in_first_share(range_begin, hi, per_split)) {
            if (blockIdx.y > 0) return;  // (the merge leaves such a tile alone too)
            whole = true;
        } else {
            range_begin += blockIdx.y * per_split;
            range_end = min(hi, range_begin + per_split);
            if (range_begin >= range_end) {  // no keys in this share: its statistics say so, its sums are never read
                float* pml = a.part_ml + ((static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + blockIdx.y) * kTileRows * 2;
                if (threadIdx.x < kTileRows) {
                    pml[threadIdx.x * 2] = -INFINITY;
                    pml[threadIdx.x * 2 + 1] = 0.f;
                }
                return;
            }
        }
    }
    const int last_group = (hi - 1) & ~15;  // the last 16 keys that have a page

    // ---- this wave's rows
    const int wave_row0 = quarter * 32;
    const int wave_rows = min(32, n_rows - wave_row0);  // <= 0: the wave has no rows, it only helps to load
    const int wave_first_pos = start + q0 + wave_row0 / group;
    const int wave_last_pos = start + q0 + (wave_row0 + max(wave_rows, 1) - 1) / group;
    uint4 qf[RT][NK];
    int row_pos[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = wave_row0 + rt * 16 + r;
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
    // The sums of a row's probabilities come from the matrix cores too: one more product of P with a column
    // of ones.  They are then the sums of the very (rounded) probabilities that weigh the values, they lie in
    // the accumulators' layout (lane group g holds rows g*4 .. +3), and the vector unit, which is the busy
    // one here, adds nothing.
    float m_run[RT];
    floatx4 o[RT][ND], l_acc[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m_run[rt] = -INFINITY;
        l_acc[rt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) o[rt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const bf16x8 ones = __builtin_bit_cast(bf16x8, (uint4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u}));

    // ---- this thread's share of the loads.  A stage is four groups of 16 keys (each within one page).  The
    // lower four waves fetch groups 0 and 2, the upper four groups 1 and 3, so that which page a load reads
    // is one number per wave; within its group a thread always takes the same 16-byte piece of the keys
    // and the same piece of the values, and puts them at the same places of the stage.
    // (Where a group has fewer pieces than the 256 threads that share it, the threads left over fetch and
    // store a piece a second time: the same bytes to the same place.)
    const int loader = half;  // (the same split of the waves, used here for something else)
    // (with four waves a loader's 128 threads take two pieces of each kind in a group: kPasses)
    constexpr int kKeyPieces = 16 * L::C, kValuePieces = 2 * D;
    constexpr int kPasses = (kKeyPieces > kValuePieces ? kKeyPieces : kValuePieces) > kLoaderThreads ? 2 : 1;
    static_assert(kKeyPieces <= kPasses * kLoaderThreads && kValuePieces <= kPasses * kLoaderThreads,
                  "at most two pieces of each kind per thread and group");
    const int loader_thread = threadIdx.x % kLoaderThreads;
    int key_from[kPasses], key_to[kPasses], value_from[kPasses], value_to_a[kPasses], value_to_b[kPasses];
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass) {
        const int key_piece = (loader_thread + pass * kLoaderThreads) % kKeyPieces;
        const int piece_key = key_piece / L::C;           // which of the group's 16 keys
        const int piece_chunk = key_piece - piece_key * L::C;
        key_from[pass] = (piece_key * D + piece_chunk * 8) * 2;  // bytes from the group's first key
        key_to[pass] = ((loader * 16 + piece_key) * L::CS + (piece_chunk ^ L::key_swizzle(piece_key))) * 16;  // + pair * 32 keys
        const int value_piece = (loader_thread + pass * kLoaderThreads) % kValuePieces;
        const int piece_d = value_piece >> 1;         // which dimension's row of values
        const int piece_h = value_piece & 1;          // which 8 of the group's 16 keys
        value_from[pass] = ((piece_d << a.page_shift) + piece_h * 8) * 2;  // bytes from the group's first key in row 0
        // row d of the block (pair); the group's keys are the block's first 16 (loader 0) or second 16 (loader 1):
        // the first or second 8 bytes of a chunk; keys h*8 .. +3 belong to lane group 2h, keys h*8+4 .. +7 to 2h+1
        const int value_row = L::kKeyBytes + piece_d * 64 + loader * 8;  // + pair * kValueBlockBytes
        const int value_sw = (piece_d >> 2) & 3;
        value_to_a[pass] = value_row + (((2 * piece_h) ^ value_sw) << 4);
        value_to_b[pass] = value_row + (((2 * piece_h + 1) ^ value_sw) << 4);
    }

    typedef const __attribute__((address_space(4))) int* const_int_ptr;
    const const_int_ptr table_c = (const_int_ptr)(uintptr_t)table;
    // the page of the 16 keys from `first` on (clamped to keys that have a page; what lies past the end is
    // masked where it is used)
    auto page_of = [&](int first) {
        return table_c[__builtin_amdgcn_readfirstlane(min(first, last_group) >> a.page_shift)];
    };
    // the pages of this wave's two groups of the stage that starts at key kb
    auto pages_of = [&](int kb, int (&page)[2]) {
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) page[pair] = page_of(kb + (2 * pair + loader) * 16);
    };
    uint4 key_regs[2][kPasses], value_regs[2][kPasses];
#pragma unroll
    for (int pair = 0; pair < 2; ++pair)
#pragma unroll
        for (int pass = 0; pass < kPasses; ++pass) key_regs[pair][pass] = value_regs[pair][pass] = uint4{0, 0, 0, 0};
    auto fetch = [&](int kb, const int (&page)[2]) {
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) {
            const int first = min(kb + (2 * pair + loader) * 16, last_group);
            const size_t page_head = static_cast<size_t>(page[pair]) * a.kv_heads + kv_head;
            const char* key_base = reinterpret_cast<const char*>(
                a.k_pool + ((page_head << a.page_shift) + (first & page_mask)) * D);
            const char* value_base = reinterpret_cast<const char*>(
                a.v_pool + (page_head * D << a.page_shift) + (first & page_mask));
#pragma unroll
            for (int pass = 0; pass < kPasses; ++pass) {
                key_regs[pair][pass] = *reinterpret_cast<const uint4*>(key_base + key_from[pass]);
                value_regs[pair][pass] = *reinterpret_cast<const uint4*>(value_base + value_from[pass]);
            }
        }
    };
    auto stash = [&](int stage) {
        unsigned char* base = lds + stage * L::kStageBytes;
#pragma unroll
        for (int pair = 0; pair < 2; ++pair) {
            unsigned char* block = base + pair * L::kValueBlockBytes;
#pragma unroll
            for (int pass = 0; pass < kPasses; ++pass) {
                *reinterpret_cast<uint4*>(base + key_to[pass] + pair * (32 * L::CS * 16)) = key_regs[pair][pass];
                const uint4 values = value_regs[pair][pass];
                *reinterpret_cast<uint2*>(block + value_to_a[pass]) = uint2{values.x, values.y};
                *reinterpret_cast<uint2*>(block + value_to_b[pass]) = uint2{values.z, values.w};
            }
        }
    };

    // ---- a lane's constant parts of its operand addresses in a stage
    const int k_read = ((half * 32 + r) * L::CS) * 16;       // + kt * 16 * CS * 16, + swizzled chunk
    const int k_sw = L::key_swizzle(r);
    const int v_read = L::kKeyBytes + half * L::kValueBlockBytes + r * 64 + ((g ^ ((r >> 2) & 3)) << 4);  // + dt * 1024

    const int n_iter = (range_end - range_begin + kKeysPerStage - 1) / kKeysPerStage;
    int page[2], page_next[2];
    if (n_iter > 0) {
        pages_of(range_begin, page);
        pages_of(range_begin + kKeysPerStage, page_next);
        fetch(range_begin, page);
        stash(0);
        __syncthreads();
        if (n_iter > 1) fetch(range_begin + kKeysPerStage, page_next);
    }

    for (int it = 0; it < n_iter; ++it) {
        const int kb = range_begin + it * kKeysPerStage + half * kKeysPerBlock;  // this wave's 32 keys
        const unsigned char* stage = lds + (it & 1) * L::kStageBytes;
        // pages of the stage after next, asked for early: the loads that need them come a whole block later
        int page_after[2] = {0, 0};
        if (it + 2 < n_iter) pages_of(range_begin + (it + 2) * kKeysPerStage, page_after);
        if (wave_rows > 0 && kb < range_end && kb <= wave_last_pos) {
            // ---- S^T = K . Q^T for two 16-key tiles
            floatx4 s[RT][2];
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                uint4 kf[NK];
#pragma unroll
                for (int j = 0; j < NK; ++j)
                    kf[j] = *reinterpret_cast<const uint4*>(stage + k_read + kt * (16 * L::CS * 16) +
                                                            (((j * 4 + g) ^ k_sw) << 4));
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
            // ---- the block's values: asked for now, used after the softmax arithmetic
            uint4 vf[ND];
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) vf[dt] = *reinterpret_cast<const uint4*>(stage + v_read + dt * 1024);
            // ---- running maxima; masks only in blocks that reach a row's edge
            const bool edge = kb + kKeysPerBlock - 1 > wave_first_pos || kb + kKeysPerBlock > range_end ||
                              (a.window > 0 && kb < wave_last_pos + 1 - a.window);
            // A row's reference moves only if one of its scores passes it by the margin, and each of the row's four
            // lanes can tell that of its own eight scores: the common block needs no maximum across lanes at all.
            float own_max[RT];
            bool moved = false;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                if (edge) {
                    const int pos = min(row_pos[rt], range_end - 1);  // (a row that does not exist has -1: nothing seen)
                    const int row_lo = (a.window > 0) ? row_pos[rt] + 1 - a.window : 0;
                    const int first_key = kb + g * 4;
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int key = first_key + kt * 16 + i;
                            if (!(key <= pos && key >= row_lo)) s[rt][kt][i] = -INFINITY;
                        }
                }
                own_max[rt] = max3(max3(s[rt][0][0], s[rt][0][1], s[rt][0][2]),
                                   max3(s[rt][0][3], s[rt][1][0], s[rt][1][1]),
                                   max3(s[rt][1][2], s[rt][1][3], s[rt][1][3]));
                moved = moved || own_max[rt] * scale_log2 > m_run[rt] + kLazyRescale;  // (the scale is positive)
            }
            if (__any(moved)) {
                // some row's reference moves (rare once the first blocks have set every row's scale): what the
                // row has summed so far is scaled down to the new reference
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    const float block_max = rows_max_lean(own_max[rt]) * scale_log2;  // maxima are kept in scaled base-2 units
                    const float m_new = (block_max > m_run[rt] + kLazyRescale) ? block_max : m_run[rt];
                    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
                    const float alpha = __builtin_amdgcn_exp2f(m_run[rt] - m_safe);  // m_run = -inf: 0, and the sums are 0 anyway
                    m_run[rt] = m_new;
                    float alpha_o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) alpha_o[i] = __shfl(alpha, g * 4 + i, kWave);
#pragma unroll
                    for (int i = 0; i < 4; ++i) l_acc[rt][i] *= alpha_o[i];
#pragma unroll
                    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) o[rt][dt][i] *= alpha_o[i];
                }
            }
            // ---- probabilities (one fused multiply-add and one exp2 each), then O += P . V and l += P . 1
            bf16x8 p_frag[RT];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float m_ref = (m_run[rt] == -INFINITY) ? 0.f : m_run[rt];
                uint32_t pw[4];
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][0], scale_log2, -m_ref));
                    const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][1], scale_log2, -m_ref));
                    const float p2 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][2], scale_log2, -m_ref));
                    const float p3 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rt][kt][3], scale_log2, -m_ref));
                    pw[kt * 2] = pack_bf16(p0, p1);
                    pw[kt * 2 + 1] = pack_bf16(p2, p3);
                }
                p_frag[rt] = __builtin_bit_cast(bf16x8, (uint4{pw[0], pw[1], pw[2], pw[3]}));
                l_acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag[rt], ones, l_acc[rt], 0, 0, 0);
            }
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int rt = 0; rt < RT; ++rt)
                    o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_frag[rt], __builtin_bit_cast(bf16x8, vf[dt]),
                                                                        o[rt][dt], 0, 0, 0);
        }
        // ---- the next stage's keys and values have arrived by now: into LDS; then ask for the ones after
        if (it + 1 < n_iter) stash((it + 1) & 1);
        __syncthreads();
        if (it + 2 < n_iter) {
            fetch(range_begin + (it + 2) * kKeysPerStage, page_after);
        }
    }

    // ---- the two halves of the keys meet: the upper waves hand their sums to the lower ones through LDS,
    // one 16-row tile at a time (the references of the rows, then ND tiles of the output and one of the
    // probabilities' sums, each as the 4 x 64 numbers the lanes hold)
    float* lds_m = reinterpret_cast<float*>(lds);                    // [quarters][16 rows]
    float* lds_o = reinterpret_cast<float*>(lds) + QUARTERS * 16;    // [quarters][(ND + 1) * 4][64 lanes]
    constexpr int kMeetTile = (ND + 1) * 4;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (rt > 0) __syncthreads();  // the tile before has been read
        if (half == 1) {
            if (g == 0) lds_m[quarter * 16 + r] = m_run[rt];
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) lds_o[(quarter * kMeetTile + dt * 4 + i) * kWave + lane] = o[rt][dt][i];
#pragma unroll
            for (int i = 0; i < 4; ++i) lds_o[(quarter * kMeetTile + ND * 4 + i) * kWave + lane] = l_acc[rt][i];
        }
        __syncthreads();
        if (half == 1 || wave_rows <= 0) continue;
        const float m_other = lds_m[quarter * 16 + r];
        const float m_all = fmaxf(m_run[rt], m_other);
        const float m_safe = (m_all == -INFINITY) ? 0.f : m_all;
        const float w_own = __builtin_amdgcn_exp2f(m_run[rt] - m_safe);
        const float w_other = __builtin_amdgcn_exp2f(m_other - m_safe);
        float w_own_o[4], w_other_o[4], l[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // from the lane of row r to the lanes that hold row g*4 + i
            w_own_o[i] = __shfl(w_own, g * 4 + i, kWave);
            w_other_o[i] = __shfl(w_other, g * 4 + i, kWave);
            l[i] = l_acc[rt][i] * w_own_o[i] + lds_o[(quarter * kMeetTile + ND * 4 + i) * kWave + lane] * w_other_o[i];
        }
#pragma unroll
        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                o[rt][dt][i] = o[rt][dt][i] * w_own_o[i] +
                               lds_o[(quarter * kMeetTile + dt * 4 + i) * kWave + lane] * w_other_o[i];
        if (!whole) {  // this share's sums and statistics for the merge kernel
            const size_t unit = (static_cast<size_t>(tile) * a.kv_heads + kv_head) * a.n_splits + blockIdx.y;
            float* po = a.part_o + unit * kTileRows * D;
            float* pml = a.part_ml + unit * kTileRows * 2;
            if (g == 0) pml[(wave_row0 + rt * 16 + r) * 2] = m_all;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = wave_row0 + rt * 16 + g * 4 + i;
                if (r == 0) pml[row * 2 + 1] = l[i];
#pragma unroll
                for (int dt = 0; dt < ND; ++dt) po[static_cast<size_t>(row) * D + dt * 16 + r] = o[rt][dt][i];
            }
            continue;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = wave_row0 + rt * 16 + g * 4 + i;
            if (row < n_rows) {
                const int tok = row / group;
                const int head = row - tok * group;
                bf16_t* dst = a.out + static_cast<size_t>(first_row_token + tok) * a.q_heads * D +
                              static_cast<size_t>(kv_head * group + head) * D;
                const float inv = 1.0f / l[i];
#pragma unroll
                for (int dt = 0; dt < ND; ++dt) dst[dt * 16 + r] = from_float<bf16_t>(o[rt][dt][i] * inv);
            }
        }
    }
}

template <int D, int WAVES>
int launch(hipStream_t s, const AttentionArgs& a) {
    using L = PromptLayout<D>;
    // the stages, or the meeting place of the two halves at the end, whichever is larger
    constexpr int kMeetBytes = ((WAVES / 2) * 16 + (WAVES / 2) * ((D / 16 + 1) * 4) * kWave) * 4;
    constexpr int kLdsBytes = 2 * L::kStageBytes > kMeetBytes ? 2 * L::kStageBytes : kMeetBytes;
    static_assert(kLdsBytes <= 64 * 1024, "a workgroup's LDS without asking for more");
    const dim3 grid = a.xcds_per_head > 0
                          ? dim3(kXcds * ((a.n_tiles + a.xcds_per_head - 1) / a.xcds_per_head), a.n_splits)
                          : dim3(static_cast<unsigned>(a.n_tiles) * a.kv_heads, a.n_splits);
    paged_attention_prompt_kernel<D, WAVES><<<grid, 64 * WAVES, kLdsBytes, s>>>(a);
    return cie_after_launch();
}

}  // namespace

namespace cie_attention {

int launch_prompt_form(hipStream_t stream, const AttentionArgs& a, int head_dim, int waves) {
    if (waves == 4) {
        switch (head_dim) {
            case 32: return launch<32, 4>(stream, a);
            case 64: return launch<64, 4>(stream, a);
            case 96: return launch<96, 4>(stream, a);
            case 128: return launch<128, 4>(stream, a);
            default: return CIE_BAD_ARGUMENT;
        }
    }
    switch (head_dim) {
        case 32: return launch<32, 8>(stream, a);
        case 64: return launch<64, 8>(stream, a);
        case 96: return launch<96, 8>(stream, a);
        case 128: return launch<128, 8>(stream, a);
        default: return CIE_BAD_ARGUMENT;  // wider heads: a wave's 32 rows of accumulators would not fit
    }
}

}  // namespace cie_attention
