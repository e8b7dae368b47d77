// What the matrix-core attention kernels share: operand types, the block size of the key loop, and the
// argument record that the entry point fills for every form (decode parts, tiled prompt forms, merge).
#pragma once

#include "common.h"

namespace cie_attention {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kKeysPerBlock = 32;
constexpr int kXcds = 8;  // an MI355X has 8 XCDs of 32 compute units, each with an L2 of its own; the
                          // hardware hands workgroup b of a launch to XCD b % 8
constexpr int kTileWaves = 4;  // waves of a workgroup in the prompt form
constexpr float kLazyRescale = 8.f;  // base-2 units a score may pass a row's reference before it moves

struct AttentionArgs {
    const bf16_t* q;
    int q_row_stride;
    const bf16_t* k_pool;
    const bf16_t* v_pool;
    const int* block_table;
    int table_width;
    const int* tile_seq;
    const int* tile_q0;
    const int* seq_slot;
    const int* seq_start;
    const int* seq_q_len;
    const int* q_start_loc;
    bf16_t* out;
    float* part_o;   // [tiles, kv_heads, splits, rows, D]
    float* part_ml;  // [tiles, kv_heads, splits, rows, 2]
    int q_heads;
    int kv_heads;
    int page_shift;
    int window;
    float scale;
    int n_splits;
    int tokens_per_tile;
    int keys_per_split;  // multiple of kKeysPerBlock; 0 with one split
    int n_tiles;
    int xcds_per_head;  // prompt forms: > 0 if every kv head has that many of the kXcds XCDs (and their L2) to itself
    const int* max_context_dev;  // if set (a captured graph replays with other lengths): keys per split are
                                 // derived from this device value, the longest context of the step
    int whole_in_first_share;    // with splits: a tile whose keys all lie in the first share writes its result
                                 // itself and takes no part in the merge (the form of eight waves)
};

// Whether a tile that sees the keys [first_begin, hi) has them all in the first of its shares of per_split keys.
__host__ __device__ inline bool all_in_first_share(int first_begin, int hi, int per_split) {
    return hi <= first_begin + per_split;
}

// The prompt form whose waves share a tile's keys and values through LDS (csrc/attention_prompt.hip): eight waves
// per tile of 128 rows, or four per tile of 64; returns a CIE_* code.
int launch_prompt_form(hipStream_t stream, const AttentionArgs& a, int head_dim, int waves);

constexpr int kPromptWaves = 8;       // waves of a workgroup in that form
constexpr int kPromptTileRows = 128;  // (token, head) rows of its tiles

}  // namespace cie_attention
