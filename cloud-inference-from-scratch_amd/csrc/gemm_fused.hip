// Matrix products for steps with few rows (decode steps, the output head), on the
// matrix cores, fused with the small operations around them.
//
//   C = A * W^T     A [M, K] bf16 with few rows, W [N, K] bf16 (a Linear's weight), float32 sums
//
// Such a product is bound by streaming W once and by the number of kernel launches
// (no kernel on this GPU finishes in under about 5 microseconds), so the epilogue
// takes over the neighbour's work:
//   BF16 / F32  C[m,n] = acc + bias[n]
//   SILU        W stacks gate rows over up rows: C[m,n] = silu(acc_gate) * acc_up, bf16
//   RESID       residual[m,n] += acc + bias[n] (float32, in place), and the partial sums of
//               squares of the new residual row (one per 16 columns) are written, so that the
//               RMSNorm that follows needs no reduction over the row
//   PARTIAL     K is cut into grid.z parts; part p writes acc to C[p, m, n] (float32, bias in
//               part 0).  The add + norm kernel sums the parts.  For few columns and long K.
//               (Only in the second form, further down.)
//   ROPE        W stacks the rows of q, k and v heads: a workgroup takes 16 dimensions of a head's
//               first half and the 16 they rotate with (half-split pairing), adds the bias, rounds
//               to bf16 as the plain epilogue would, rotates q and k by the row's position and
//               writes q to C[m, n], k and v into the paged cache (v transposed).
//   ROPE8       the same with one tile per workgroup: 8 dimensions of a head's first half and the 8 they
//               rotate with share the tile, so that a weight of few columns gives twice the workgroups
//               (up to 16 rows).
//
// One kernel: a workgroup owns one or two tiles of 16 columns (SILU: a gate tile and its up tile)
// and 16, 32 or 64 rows; its WAVES waves cut K into slices of 128 and take them round-robin.
// A wave fetches a 16 x 128 piece of W with loads that read whole 256-byte row segments and turns
// it into the MFMA operand layout through a small staging area in LDS (with more than 16 rows the
// rows of A too; with 16 the lanes load A as the MFMA wants it, from the cache); the waves' partial
// tiles are summed through LDS in wave order, by wave 0 or, with more than one row tile, by one
// wave per row tile.  v_mfma_f32_16x16x32_bf16 with A = activations (16 rows), B = weight rows
// (the order of k inside a product is free as long as both operands agree).
// No workgroup ever waits for another: a device-wide fence between workgroups costs more on
// this GPU than the whole product.
#include <type_traits>

#include "common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));  // 16 bytes as one value (a struct is copied as memory)

enum { EPI_BF16 = 0, EPI_F32 = 1, EPI_SILU = 2, EPI_RESID = 3, EPI_PARTIAL = 4, EPI_ROPE = 5, EPI_ROPE8 = 6, EPI_ATOMIC = 7 };

// What the ROPE epilogue needs beside the product: where each row's token sits, and the cache.
struct RopeArgs {
    const float* cos_table;  // [max_position, D/2]
    const float* sin_table;
    const int* positions;     // [M]
    const int* seq_of_token;  // [M]
    const int* seq_slot;      // [sequences]
    const int* block_table;   // [slots, table_width]
    int table_width;
    bf16_t* k_pool;           // [pages, Hkv, page_size, D]
    bf16_t* v_pool;           // [pages, Hkv, D, page_size]
    int q_heads, kv_heads, head_dim, page_size;
    int rotate, write_kv;
};

struct FusedArgs {
    const bf16_t* a;       // [M, K], row stride lda
    int lda;
    const bf16_t* w;       // [N, K]
    const bf16_t* bias;    // [N] or null
    void* c;               // BF16/F32: [M, N]; SILU: [M, N/2]; PARTIAL: [parts, M, N] float32
    float* residual;       // RESID: [M, N] float32, accumulated in place
    float* sumsq;          // RESID: [M, ceil(N/16)]
    int M, N, K;
    int up_offset;         // SILU: rows of W between a gate row and its up row (N/2)
    int k_per_part;        // k values per grid.z part (a multiple of 128); K with one part
    // An RMSNorm that follows the RESID product, folded into its neighbours: the RESID epilogue also
    // writes scaled_out[m, n] = bf16(residual[m, n] * norm_weight[n]) (the norm's output short of the
    // row's 1/rms), and a SILU product that reads such rows gets the sums of squares of the residual's
    // rows (row_sumsq [M, sumsq_parts] partial sums) and multiplies its sums by 1/rms before the SiLU.
    const float* norm_weight;  // RESID: [N] or null
    bf16_t* scaled_out;        // RESID: [M, N] or null
    const float* row_sumsq;    // SILU: [M, sumsq_parts] or null
    int sumsq_parts;
    float eps;
    // ROPE with the norm in front of it folded in (up to 16 rows): the rows of A are not read but made here, as
    // bf16(fold_residual * fold_weight), a lane making the very values its matrix operand holds, and the
    // product is multiplied by each row's 1/rms, whose sums of squares the lanes gather on the way.
    const float* fold_residual;  // [M, K] float32 or null
    const float* fold_weight;    // [K] float32
    RopeArgs rope;         // ROPE only
};

// One 16x16 tile of results in its MFMA layout: lane (r, g) holds rows g*4+i of column r.
// `n` is the lane's column (of C, or of the SILU output), `m_base` the tile's first row.
template <int EPI>
__device__ __forceinline__ void store_tile(const FusedArgs& a, const floatx4& acc, const floatx4& acc_up,
                                           int m_base, int n, int n_tile, int lane,
                                           const float (&row_scale)[4] = {1.f, 1.f, 1.f, 1.f}) {
    const int r = lane & 15;
    const int g = lane >> 4;
    const int cols = (EPI == EPI_SILU) ? a.up_offset : a.N;
    const bool col_ok = n < cols;
    const float add = (EPI != EPI_SILU && col_ok && a.bias && blockIdx.z == 0) ? to_float(a.bias[n]) : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m_base + g * 4 + i;
        const bool ok = col_ok && m < a.M;
        if (EPI == EPI_SILU) {
            if (ok) {
                const float gate = acc[i] * row_scale[i];
                static_cast<bf16_t*>(a.c)[static_cast<size_t>(m) * cols + n] =
                    from_float<bf16_t>((gate / (1.0f + __expf(-gate))) * (acc_up[i] * row_scale[i]));
            }
        } else if (EPI == EPI_RESID) {
            float v = 0.f;
            if (ok) {
                float* dst = a.residual + static_cast<size_t>(m) * a.N + n;
                v = *dst + acc[i] + add;
                *dst = v;
            }
            float sq = v * v;  // sum over the tile's 16 columns: the lanes that share g
            sq += __shfl_xor(sq, 1, kWave);
            sq += __shfl_xor(sq, 2, kWave);
            sq += __shfl_xor(sq, 4, kWave);
            sq += __shfl_xor(sq, 8, kWave);
            if (r == 0 && m < a.M) a.sumsq[static_cast<size_t>(m) * ((a.N + 15) / 16) + n_tile] = sq;
        } else if (ok) {
            const float v = acc[i] + add;
            if (EPI == EPI_PARTIAL)
                static_cast<float*>(a.c)[(static_cast<size_t>(blockIdx.z) * a.M + m) * a.N + n] = v;
            else if (EPI == EPI_ATOMIC)  // every part of K adds its share into the stream (the hardware's own float add)
                unsafeAtomicAdd(a.residual + static_cast<size_t>(m) * a.N + n, v);
            else if (EPI == EPI_F32)
                static_cast<float*>(a.c)[static_cast<size_t>(m) * a.N + n] = v;
            else
                static_cast<bf16_t*>(a.c)[static_cast<size_t>(m) * a.N + n] = from_float<bf16_t>(v);
        }
    }
}

// The RESID epilogue for one 16 x 16 tile.  What it needs beside the product (the old values of the
// residual, the bias, the weight of the norm that rides along) is fetched before the product starts, by
// the wave that will store the tile, so that these loads travel while the weights stream instead of
// standing between the product and its store.
struct ResidRows {
    float old[4];
    float add, weight;
};

__device__ __forceinline__ ResidRows resid_prefetch(const FusedArgs& a, int m_base, int n, int lane) {
    const int g = lane >> 4;
    const bool col_ok = n < a.N;
    ResidRows rows;
    rows.add = (col_ok && a.bias) ? to_float(a.bias[n]) : 0.f;
    rows.weight = (col_ok && a.scaled_out) ? a.norm_weight[n] : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m_base + g * 4 + i;
        rows.old[i] = (col_ok && m < a.M) ? a.residual[static_cast<size_t>(m) * a.N + n] : 0.f;
    }
    return rows;
}

__device__ __forceinline__ void store_resid(const FusedArgs& a, const floatx4& acc, const ResidRows& rows, int m_base,
                                            int n, int n_tile, int lane) {
    const int r = lane & 15;
    const int g = lane >> 4;
    const bool col_ok = n < a.N;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m_base + g * 4 + i;
        const bool ok = col_ok && m < a.M;
        const float v = ok ? rows.old[i] + acc[i] + rows.add : 0.f;
        if (ok) a.residual[static_cast<size_t>(m) * a.N + n] = v;
        if (ok && a.scaled_out) a.scaled_out[static_cast<size_t>(m) * a.N + n] = from_float<bf16_t>(v * rows.weight);
        float sq = v * v;  // sum over the tile's 16 columns: the lanes that share g
        sq += __shfl_xor(sq, 1, kWave);
        sq += __shfl_xor(sq, 2, kWave);
        sq += __shfl_xor(sq, 4, kWave);
        sq += __shfl_xor(sq, 8, kWave);
        if (r == 0 && m < a.M) a.sumsq[static_cast<size_t>(m) * ((a.N + 15) / 16) + n_tile] = sq;
    }
}

// The ROPE epilogue for one pair of tiles: `lo` holds dimensions j*16 + r of head `head`, `hi` those
// plus D/2.  Values are rounded to bf16 before the rotation, so that the results equal those of the
// plain epilogue followed by the rotation kernel.  What the epilogue needs of each of the lane's four
// rows (position, angle, cache page) is fetched before the product starts, so that these dependent
// loads travel while the weights stream.
struct RopeRows {
    int pos[4];
    int page[4];    // -1: nothing to write for this row
    float c[4], s[4];
    float bias_lo, bias_hi;
};

// In two steps, because the second reads where the first points: positions and sequences of the rows
// (and the bias) before the product starts; angles, slots and pages behind the wave's first loads of W.
__device__ __forceinline__ RopeRows rope_prefetch(const FusedArgs& a, int head, int j, int lane, int m_base) {
    const RopeArgs& p = a.rope;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int half = p.head_dim / 2;
    const int d = j * 16 + r;
    const bool is_query = head < p.q_heads;
    RopeRows rows;
    rows.bias_lo = a.bias ? to_float(a.bias[head * p.head_dim + d]) : 0.f;
    rows.bias_hi = a.bias ? to_float(a.bias[head * p.head_dim + d + half]) : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m_base + g * 4 + i;
        rows.pos[i] = -1;   // no such row
        rows.page[i] = -1;  // until the second step: the row's sequence, if its key or value is to be written
        rows.c[i] = 1.f;
        rows.s[i] = 0.f;
        if (m >= a.M) continue;
        rows.pos[i] = p.positions[m];
        if (!is_query && p.write_kv) rows.page[i] = p.seq_of_token[m];
    }
    return rows;
}

__device__ __forceinline__ void rope_prefetch_rest(const FusedArgs& a, int head, int j, int lane, RopeRows& rows) {
    const RopeArgs& p = a.rope;
    const int half = p.head_dim / 2;
    const int d = j * 16 + (lane & 15);
    const bool is_value = head >= p.q_heads + p.kv_heads;
    int slot[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int pos = rows.pos[i];
        if (pos >= 0 && !is_value && p.rotate) {
            rows.c[i] = p.cos_table[static_cast<size_t>(pos) * half + d];
            rows.s[i] = p.sin_table[static_cast<size_t>(pos) * half + d];
        }
        slot[i] = rows.page[i] >= 0 ? p.seq_slot[rows.page[i]] : -1;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (slot[i] >= 0)
            rows.page[i] = p.block_table[static_cast<size_t>(slot[i]) * p.table_width + rows.pos[i] / p.page_size];
        if (rows.pos[i] < 0) rows.pos[i] = 0;
    }
}

__device__ __forceinline__ void store_rope(const FusedArgs& a, const floatx4& lo, const floatx4& hi, int head,
                                           int j, int lane, const RopeRows& rows, int m_base) {
    const RopeArgs& p = a.rope;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int D = p.head_dim;
    const int half = D / 2;
    const int d = j * 16 + r;
    const bool is_query = head < p.q_heads;
    const bool is_value = head >= p.q_heads + p.kv_heads;
    const int kv_head = is_query ? 0 : (head - p.q_heads) % p.kv_heads;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m_base + g * 4 + i;
        if (m >= a.M) continue;
        const float x_lo = to_float(from_float<bf16_t>(lo[i] + rows.bias_lo));
        const float x_hi = to_float(from_float<bf16_t>(hi[i] + rows.bias_hi));
        // values and unrotated heads have c = 1, s = 0: the products are exact and the sums unchanged
        const bf16_t y_lo = from_float<bf16_t>(x_lo * rows.c[i] - x_hi * rows.s[i]);
        const bf16_t y_hi = from_float<bf16_t>(x_hi * rows.c[i] + x_lo * rows.s[i]);
        if (is_query) {
            bf16_t* dst = static_cast<bf16_t*>(a.c) + static_cast<size_t>(m) * a.N + head * D + d;
            dst[0] = y_lo;
            dst[half] = y_hi;
            continue;
        }
        const int page = rows.page[i];
        if (page < 0) continue;  // no cache write wanted (the host never schedules a token without a page)
        const int in_page = rows.pos[i] % p.page_size;
        const size_t head_base = (static_cast<size_t>(page) * p.kv_heads + kv_head) * p.page_size * D;
        if (is_value) {  // element d of the token goes to [d, in_page] of the transposed page
            bf16_t* column = p.v_pool + head_base + in_page;
            column[static_cast<size_t>(d) * p.page_size] = y_lo;
            column[static_cast<size_t>(d + half) * p.page_size] = y_hi;
        } else {
            bf16_t* dst = p.k_pool + head_base + static_cast<size_t>(in_page) * D + d;
            dst[0] = y_lo;
            dst[half] = y_hi;
        }
    }
}

// The same epilogue where one tile holds both halves: lane (r, g) has dimension j*8 + (r & 7) of the first
// half (r < 8) or of the second (r >= 8), and its partner sits eight lanes away.
__device__ __forceinline__ RopeRows rope8_prefetch(const FusedArgs& a, int head, int j, int lane, int m_base) {
    const RopeArgs& p = a.rope;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int d = j * 8 + (r & 7) + (r >> 3) * (p.head_dim / 2);
    const bool is_query = head < p.q_heads;
    RopeRows rows;
    rows.bias_lo = a.bias ? to_float(a.bias[head * p.head_dim + d]) : 0.f;  // (the lane's own column)
    rows.bias_hi = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m_base + g * 4 + i;
        rows.pos[i] = -1;
        rows.page[i] = -1;
        rows.c[i] = 1.f;
        rows.s[i] = 0.f;
        if (m >= a.M) continue;
        rows.pos[i] = p.positions[m];
        if (!is_query && p.write_kv) rows.page[i] = p.seq_of_token[m];
    }
    return rows;
}

__device__ __forceinline__ void rope8_prefetch_rest(const FusedArgs& a, int head, int j, int lane, RopeRows& rows) {
    const RopeArgs& p = a.rope;
    const int half = p.head_dim / 2;
    const int d = j * 8 + (lane & 7);  // the angle's index: the same for a dimension and its partner
    const bool is_value = head >= p.q_heads + p.kv_heads;
    int slot[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int pos = rows.pos[i];
        if (pos >= 0 && !is_value && p.rotate) {
            rows.c[i] = p.cos_table[static_cast<size_t>(pos) * half + d];
            rows.s[i] = p.sin_table[static_cast<size_t>(pos) * half + d];
        }
        slot[i] = rows.page[i] >= 0 ? p.seq_slot[rows.page[i]] : -1;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (slot[i] >= 0)
            rows.page[i] = p.block_table[static_cast<size_t>(slot[i]) * p.table_width + rows.pos[i] / p.page_size];
        if (rows.pos[i] < 0) rows.pos[i] = 0;
    }
}

__device__ __forceinline__ void store_rope8(const FusedArgs& a, const floatx4& acc, int head, int j, int lane,
                                            const RopeRows& rows, int m_base) {
    const RopeArgs& p = a.rope;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int D = p.head_dim;
    const bool second = r >= 8;
    const int d = j * 8 + (r & 7) + (second ? D / 2 : 0);
    const bool is_query = head < p.q_heads;
    const bool is_value = head >= p.q_heads + p.kv_heads;
    const int kv_head = is_query ? 0 : (head - p.q_heads) % p.kv_heads;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m_base + g * 4 + i;
        const float x = to_float(from_float<bf16_t>(acc[i] + rows.bias_lo));
        const float partner = __shfl_xor(x, 8, kWave);  // (every lane takes part, also those of rows that do not exist)
        if (m >= a.M) continue;
        // first half: x cos - partner sin; second half: x cos + partner sin (values, unrotated heads: c = 1, s = 0)
        const bf16_t y = from_float<bf16_t>(second ? x * rows.c[i] + partner * rows.s[i] : x * rows.c[i] - partner * rows.s[i]);
        if (is_query) {
            static_cast<bf16_t*>(a.c)[static_cast<size_t>(m) * a.N + head * D + d] = y;
            continue;
        }
        const int page = rows.page[i];
        if (page < 0) continue;
        const int in_page = rows.pos[i] % p.page_size;
        const size_t head_base = (static_cast<size_t>(page) * p.kv_heads + kv_head) * p.page_size * D;
        if (is_value)
            p.v_pool[head_base + in_page + static_cast<size_t>(d) * p.page_size] = y;
        else
            p.k_pool[head_base + static_cast<size_t>(in_page) * D + d] = y;
    }
}

// ---------------------------------------------------------------------------------------------
// MT row tiles (M <= 16*MT per workgroup row; more rows: more workgroup rows) and NT column tiles
// per workgroup: with SILU the gate tile and its up tile, else NT adjacent tiles.  Every weight
// value a wave loads meets all MT row tiles; every activation value meets the NT column tiles.
constexpr int kStageRow = 256 + 16;           // bytes of a row in a staging area: the padding spreads the rows over the banks
constexpr int kStageTile = 16 * kStageRow;    // a wave's staging area

constexpr int kFoldRows = 16;      // the most rows whose norm the q/k/v product makes itself: one row tile

// FOLD: 0, or the groups of four rows (2 or 4) of the float32 stream from which the rows of A are made (see FusedArgs).
template <int WAVES, int EPI, int MT, int NT, int FOLD = 0>
__global__ void __launch_bounds__(WAVES * 64) gemm_rows_kernel(FusedArgs a) {
    static_assert(FOLD == 0 || ((FOLD == 2 || FOLD == 4) && MT == 1 && (EPI == EPI_ROPE || EPI == EPI_ROPE8)),
                  "the folded norm: q/k/v of one row tile");
    static_assert(EPI != EPI_SILU || NT == 2, "the SiLU epilogue pairs a gate tile with its up tile");
    static_assert(EPI != EPI_ROPE || NT == 2, "the ROPE epilogue pairs the two halves of a head");
    static_assert(EPI != EPI_ROPE8 || NT == 1, "the one-tile ROPE epilogue: one column tile a workgroup");
    static_assert(MT <= WAVES || WAVES == 1, "a wave ends at most one row tile");
    // slices of 128 k values whose weight loads are in flight together
    constexpr int U = (MT == 1 && NT == 1) ? 4 : (MT == 4) ? 1 : 2;
    // During the product every wave has a staging area of its own for one 16 x 128 piece of W (below);
    // afterwards the same memory takes the waves' partial tiles.
    constexpr int kReduceBytes = WAVES > 1 ? (WAVES - 1) * MT * NT * 64 * 4 * 4 : 16;
    constexpr int kStageBytes = WAVES * kStageTile;
    constexpr int kSharedBytes = kReduceBytes > kStageBytes ? kReduceBytes : kStageBytes;
    __shared__ __attribute__((aligned(16))) char shared[kSharedBytes + 16 * sizeof(float)];  // + the rows' scales
    float* reduce = reinterpret_cast<float*>(shared);
    char* stage = shared + (threadIdx.x / kWave) * kStageTile;
    __shared__ float fold_sq[FOLD > 0 ? WAVES * kFoldRows : 1];  // the waves' shares of the rows' sums of squares

    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    const int m0 = blockIdx.y * (16 * MT);
    const int cols = (EPI == EPI_SILU) ? a.up_offset : a.N;
    const int tile_first = (EPI == EPI_SILU || EPI == EPI_ROPE) ? blockIdx.x : blockIdx.x * NT;
    // ROPE: workgroup b takes tile b % (D/32) of the first half of head b / (D/32), and its partner
    // (ROPE8: 8 dimensions b % (D/16) of the first half and their 8 partners)
    const int rope_tiles = (EPI == EPI_ROPE) ? a.rope.head_dim / 32 : (EPI == EPI_ROPE8) ? a.rope.head_dim / 16 : 1;
    const int rope_head = blockIdx.x / rope_tiles;
    const int rope_tile = blockIdx.x - rope_head * rope_tiles;

    // A 16 x 128 piece of W (16 rows of 256 bytes) is fetched by four loads of four rows each: sixteen
    // neighbouring lanes read one row's 256 bytes, which the memory pipeline takes as whole cache lines
    // (a load in which every lane reads another row costs it four times the cycles, and with as many
    // loads of A as of W that, not the memory, bounded the kernel).  The piece then passes through the
    // wave's staging area in LDS into the MFMA layout: lane (r, g) gets row r, k values j*32 + g*8 .. +7.
    // A column past the end computes a copy that is not stored.
    const int load_row = lane >> 4;        // of the four rows of a load
    const int load_col = (lane & 15) * 8;  // k offset inside the 128
    const bf16_t* w_rows[NT][4];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = i * 4 + load_row;
            int n;
            if (EPI == EPI_ROPE8)
                n = rope_head * a.rope.head_dim + rope_tile * 8 + (row & 7) + (row >> 3) * (a.rope.head_dim / 2);
            else if (EPI == EPI_ROPE)
                n = rope_head * a.rope.head_dim + rope_tile * 16 + row + t * (a.rope.head_dim / 2);
            else if (EPI == EPI_SILU)
                n = min(tile_first * 16 + row, cols - 1) + t * a.up_offset;
            else
                n = min((tile_first + t) * 16 + row, cols - 1);
            w_rows[t][i] = a.w + static_cast<size_t>(n) * a.K + load_col;
        }
    // With more than 16 rows the rows of A travel the same way (they come from the cache, but cost the
    // memory pipeline the same); with one row tile the extra step only adds to each slice's latency
    // and the lanes load A as the MFMA wants it: lane (r, g) row r, k values j*32 + g*8 .. +7.
    constexpr bool kStageA = MT > 1;
    const bf16_t* a_rows[MT][4];
    bool row_ok[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + mt * 16 + (kStageA ? i * 4 + load_row : r);
            row_ok[mt][i] = m < a.M;
            a_rows[mt][i] = FOLD ? nullptr
                                 : a.a + static_cast<size_t>(min(m, a.M - 1)) * a.lda + (kStageA ? load_col : i * 32 + g * 8);
        }

    floatx4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    RopeRows rope_rows;
    // (the wave that will store row tile `wave`, below)
    bool rope_pending = (EPI == EPI_ROPE || EPI == EPI_ROPE8) && wave < MT;
    if (rope_pending)
        rope_rows = (EPI == EPI_ROPE8) ? rope8_prefetch(a, rope_head, rope_tile, lane, m0 + wave * 16)
                                       : rope_prefetch(a, rope_head, rope_tile, lane, m0 + wave * 16);
    ResidRows resid_rows[NT];
    if (EPI == EPI_RESID && wave < MT) {
#pragma unroll
        for (int t = 0; t < NT; ++t) resid_rows[t] = resid_prefetch(a, m0 + wave * 16, (tile_first + t) * 16 + r, lane);
    }
    // Rows that still lack their 1/rms (one row tile only): the waves share the 16 rows, 4 * WAVES lanes
    // sum the partial sums of a row, and the scales meet in LDS for the wave that stores.  The loads are
    // issued behind the wave's first loads of W, so that they add nothing to its start.
    constexpr int kScaleLanes = 4 * WAVES;         // lanes per row
    constexpr int kScaleRows = 16 / WAVES;         // rows per wave
    float* scale_lds = reinterpret_cast<float*>(shared + kSharedBytes);
    float row_scale[4] = {1.f, 1.f, 1.f, 1.f};
    float sq_part = 0.f;
    const bool scaled_rows = EPI == EPI_SILU && MT == 1 && a.row_sumsq != nullptr;
    bool scale_pending = scaled_rows;
    const int scale_row = wave * kScaleRows + lane / kScaleLanes;  // of the tile
    auto sum_row_parts = [&]() {
        if (m0 + scale_row >= a.M) return;
        const float* row = a.row_sumsq + static_cast<size_t>(m0 + scale_row) * a.sumsq_parts;
        const int sub = lane % kScaleLanes;
        if (a.sumsq_parts % 4 == 0) {
            for (int p = sub * 4; p < a.sumsq_parts; p += kScaleLanes * 4) {
                const float4 v = *reinterpret_cast<const float4*>(row + p);
                sq_part += (v.x + v.y) + (v.z + v.w);
            }
        } else {
            for (int p = sub; p < a.sumsq_parts; p += kScaleLanes) sq_part += row[p];
        }
    };

    const int k_begin = blockIdx.z * a.k_per_part;
    const int k_end = min(a.K, k_begin + a.k_per_part);
    float fold_sq_lane[FOLD > 0 ? FOLD : 1] = {};  // FOLD: this lane's share of the sums of squares of rows i * 4 + load_row
    {
#pragma unroll 1
    for (int kbase = k_begin + wave * 128; kbase < k_end; kbase += U * WAVES * 128) {
        uint4 b[U][NT][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = kbase + u * WAVES * 128;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    b[u][t][i] = (k0 + load_col < k_end) ? *reinterpret_cast<const uint4*>(w_rows[t][i] + k0) : uint4{0, 0, 0, 0};
        }
        if (scale_pending) {  // once, behind the wave's first loads of W
            sum_row_parts();
            scale_pending = false;
        }
        if (rope_pending) {  // likewise
            if (EPI == EPI_ROPE8)
                rope8_prefetch_rest(a, rope_head, rope_tile, lane, rope_rows);
            else
                rope_prefetch_rest(a, rope_head, rope_tile, lane, rope_rows);
            rope_pending = false;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // the few rows of A come from the cache; their loads are issued slice by slice
            const int ka = kbase + u * WAVES * 128;
            uint4 av[MT][4];
            if constexpr (FOLD > 0) {
                // The piece of A (16 x 128) made from the float32 stream: sixteen neighbouring lanes read 256 bytes
                // (64 values) of a row, four rows a load, FOLD such loads for each half of the slice (rows past
                // the last are not read); times the norm's weight, as bf16 through the wave's staging area into
                // the operand layout.  Every load stands unconditionally; what lies past an end is dropped by a select.
                const int lc = lane & 15;
                float4 x[2][FOLD], nw[2];
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) {
                    const int k_col = min(ka + cb * 64 + lc * 4, a.K - 4);
                    nw[cb] = *reinterpret_cast<const float4*>(a.fold_weight + k_col);
#pragma unroll
                    for (int i = 0; i < FOLD; ++i)
                        x[cb][i] = *reinterpret_cast<const float4*>(
                            a.fold_residual + static_cast<size_t>(min(m0 + i * 4 + load_row, a.M - 1)) * a.K + k_col);
                }
#pragma unroll
                for (int cb = 0; cb < 2; ++cb)
#pragma unroll
                    for (int i = 0; i < FOLD; ++i) {
                        const bool inside = m0 + i * 4 + load_row < a.M && ka + cb * 64 + lc * 4 < k_end;
                        const float4 v = x[cb][i];
                        fold_sq_lane[i] += inside ? (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w) : 0.f;
                        uint2 packed;
                        packed.x = pack_bf16(v.x * nw[cb].x, v.y * nw[cb].y);
                        packed.y = pack_bf16(v.z * nw[cb].z, v.w * nw[cb].w);
                        *reinterpret_cast<uint2*>(stage + (i * 4 + load_row) * kStageRow + (cb * 64 + lc * 4) * 2) =
                            inside ? packed : uint2{0u, 0u};
                    }
#pragma unroll
                for (int j = 0; j < 4; ++j)  // (rows the loads left out hold what the piece before left: not used)
                    av[0][j] = r < 4 * FOLD ? *reinterpret_cast<const uint4*>(stage + r * kStageRow + j * 64 + g * 16)
                                            : uint4{0, 0, 0, 0};
            } else {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int k_lane = ka + (kStageA ? load_col : i * 32 + g * 8);
                    av[mt][i] = (row_ok[mt][i] && k_lane < k_end) ? *reinterpret_cast<const uint4*>(a_rows[mt][i] + ka)
                                                                  : uint4{0, 0, 0, 0};
                }
            }
            if (kStageA) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        *reinterpret_cast<uint4*>(stage + (i * 4 + load_row) * kStageRow + load_col * 2) = av[mt][i];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        av[mt][j] = *reinterpret_cast<const uint4*>(stage + r * kStageRow + j * 64 + g * 16);
                }
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                // through the staging area (a wave's LDS operations keep their order: no barrier)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    *reinterpret_cast<uint4*>(stage + (i * 4 + load_row) * kStageRow + load_col * 2) = b[u][t][i];
                uint4 bt[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) bt[j] = *reinterpret_cast<const uint4*>(stage + r * kStageRow + j * 64 + g * 16);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            __builtin_bit_cast(bf16x8, av[mt][j]), __builtin_bit_cast(bf16x8, bt[j]), acc[mt][t], 0, 0, 0);
            }
        }
    }
    }

    if (rope_pending) {  // (a K so short that this wave had no slice)
        if (EPI == EPI_ROPE8)
            rope8_prefetch_rest(a, rope_head, rope_tile, lane, rope_rows);
        else
            rope_prefetch_rest(a, rope_head, rope_tile, lane, rope_rows);
    }
    if (scaled_rows) {
        if (scale_pending) sum_row_parts();  // (likewise)
#pragma unroll
        for (int offset = kScaleLanes / 2; offset > 0; offset >>= 1) sq_part += __shfl_xor(sq_part, offset, kWave);
        if (lane % kScaleLanes == 0) scale_lds[scale_row] = 1.0f / sqrtf(sq_part / static_cast<float>(a.K) + a.eps);
        if (WAVES == 1) {  // (with more waves the barrier below stands between the write and the read)
#pragma unroll
            for (int i = 0; i < 4; ++i) row_scale[i] = scale_lds[g * 4 + i];
        }
    }
    if constexpr (FOLD > 0) {  // the rows' sums of squares over this wave's slices: sixteen lanes hold a row's
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = i < FOLD ? fold_sq_lane[i < FOLD ? i : 0] : 0.f;
            v += __shfl_xor(v, 1, kWave);
            v += __shfl_xor(v, 2, kWave);
            v += __shfl_xor(v, 4, kWave);
            v += __shfl_xor(v, 8, kWave);
            if ((lane & 15) == 0) fold_sq[wave * kFoldRows + i * 4 + load_row] = v;
        }
    }
    // With more than one row tile the waves share the end of the work: row tile mt belongs to wave
    // mt % WAVES, which sums the other waves' partial tiles of that row tile and stores it (one wave
    // doing all of it would take as long again as the product).
    constexpr bool kSharedEnd = WAVES > 1 && MT > 1;
    if constexpr (kSharedEnd) {
        __syncthreads();  // every wave is done with its staging area
        // slot of wave w for row tile mt: the waves other than the owner, in wave order
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int owner = mt % WAVES;
            if (wave != owner) {
                const int slot = wave < owner ? wave : wave - 1;
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        reduce[(((mt * (WAVES - 1) + slot) * NT + t) * 4 + i) * 64 + lane] = acc[mt][t][i];
            }
        }
        __syncthreads();
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (wave != mt % WAVES) continue;  // wave-uniform
#pragma unroll 1
            for (int slot = 0; slot < WAVES - 1; ++slot)
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[mt][t][i] += reduce[(((mt * (WAVES - 1) + slot) * NT + t) * 4 + i) * 64 + lane];
            if constexpr (EPI == EPI_RESID) {
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    if ((tile_first + t) * 16 < cols)  // wave-uniform
                        store_resid(a, acc[mt][t], resid_rows[t], m0 + mt * 16, (tile_first + t) * 16 + r, tile_first + t, lane);
            } else if (EPI == EPI_ROPE) {
                store_rope(a, acc[mt][0], acc[mt][NT - 1], rope_head, rope_tile, lane, rope_rows, m0 + mt * 16);
            } else if (EPI == EPI_ROPE8) {
                store_rope8(a, acc[mt][0], rope_head, rope_tile, lane, rope_rows, m0 + mt * 16);
            } else if (EPI == EPI_SILU) {
                store_tile<EPI>(a, acc[mt][0], acc[mt][NT - 1], m0 + mt * 16, tile_first * 16 + r, tile_first, lane);
            } else {
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    if ((tile_first + t) * 16 < cols)  // wave-uniform
                        store_tile<EPI>(a, acc[mt][t], acc[mt][t], m0 + mt * 16, (tile_first + t) * 16 + r, tile_first + t, lane);
            }
        }
        return;
    }
    if (WAVES > 1) {  // one row tile: sum the waves' partial tiles in wave order; wave 0 keeps the result
        __syncthreads();  // every wave is done with its staging area
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
        if (scaled_rows) {
#pragma unroll
            for (int i = 0; i < 4; ++i) row_scale[i] = scale_lds[g * 4 + i];
        }
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[mt][t][i] += reduce[((((w - 1) * MT + mt) * NT + t) * 4 + i) * 64 + lane];
    }
    if constexpr (EPI == EPI_RESID) {  // (one row tile, or one wave: this wave fetched the tiles' old values)
#pragma unroll
        for (int t = 0; t < NT; ++t)
            if ((tile_first + t) * 16 < cols)  // wave-uniform
                store_resid(a, acc[0][t], resid_rows[t], m0, (tile_first + t) * 16 + r, tile_first + t, lane);
        return;
    }
    if constexpr (FOLD > 0) {  // the rows' 1/rms, which the rows of A were made without
        // (wave 0, behind the barrier above if there are more; with one wave its LDS operations keep their order)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float total = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) total += fold_sq[w * kFoldRows + g * 4 + i];
            const float scale = 1.0f / sqrtf(total / static_cast<float>(a.K) + a.eps);
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[0][t][i] *= scale;
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (EPI == EPI_ROPE8) {
            store_rope8(a, acc[mt][0], rope_head, rope_tile, lane, rope_rows, m0 + mt * 16);
        } else if (EPI == EPI_ROPE) {
            store_rope(a, acc[mt][0], acc[mt][NT - 1], rope_head, rope_tile, lane, rope_rows, m0 + mt * 16);
        } else if (EPI == EPI_SILU) {
            store_tile<EPI>(a, acc[mt][0], acc[mt][NT - 1], m0 + mt * 16, tile_first * 16 + r, tile_first, lane, row_scale);
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t)
                if ((tile_first + t) * 16 < cols)  // wave-uniform
                    store_tile<EPI>(a, acc[mt][t], acc[mt][t], m0 + mt * 16, (tile_first + t) * 16 + r, tile_first + t, lane);
        }
    }
}

template <int EPI, int MT, int NT, int FOLD = 0>
int launch_waves(hipStream_t s, int waves, dim3 grid, const FusedArgs& a) {
    if constexpr (MT == 1) {
        switch (waves) {
            case 1: gemm_rows_kernel<1, EPI, MT, NT, FOLD><<<grid, 64, 0, s>>>(a); break;
            case 2: gemm_rows_kernel<2, EPI, MT, NT, FOLD><<<grid, 128, 0, s>>>(a); break;
            case 4: gemm_rows_kernel<4, EPI, MT, NT, FOLD><<<grid, 256, 0, s>>>(a); break;
            case 8: gemm_rows_kernel<8, EPI, MT, NT, FOLD><<<grid, 512, 0, s>>>(a); break;
            default: return CIE_BAD_ARGUMENT;
        }
    } else {  // more row tiles: four or eight waves (waves that find no slice of K add zeros)
        switch (waves) {
            case 4: gemm_rows_kernel<4, EPI, MT, NT><<<grid, 256, 0, s>>>(a); break;
            case 8: gemm_rows_kernel<8, EPI, MT, NT><<<grid, 512, 0, s>>>(a); break;
            default: return CIE_BAD_ARGUMENT;
        }
    }
    return cie_after_launch();
}

template <int EPI>
int launch(hipStream_t s, int row_tiles, int waves, int column_tiles, const FusedArgs& a) {
    const int cols = (EPI == EPI_SILU) ? a.up_offset : a.N;
    const int tiles = (cols + 15) / 16;
    const int m_blocks = (a.M + 16 * row_tiles - 1) / (16 * row_tiles);
    if (m_blocks > 65535) return CIE_BAD_ARGUMENT;
    constexpr int NT1 = (EPI == EPI_SILU) ? 2 : 1;  // the SiLU epilogue always pairs a gate tile with its up tile
    if (row_tiles == 1) {
        if (column_tiles != 1) return CIE_BAD_ARGUMENT;
        return launch_waves<EPI, 1, NT1>(s, waves, dim3(tiles, m_blocks, 1), a);
    }
    if (EPI == EPI_SILU || column_tiles == 2) {
        const int groups = (EPI == EPI_SILU) ? tiles : (tiles + 1) / 2;
        if (row_tiles == 2) return launch_waves<EPI, 2, 2>(s, waves, dim3(groups, m_blocks, 1), a);
        if (row_tiles == 4) return launch_waves<EPI, 4, 2>(s, waves, dim3(groups, m_blocks, 1), a);
    } else if constexpr (EPI != EPI_SILU) {
        if (column_tiles != 1) return CIE_BAD_ARGUMENT;
        if (row_tiles == 2) return launch_waves<EPI, 2, 1>(s, waves, dim3(tiles, m_blocks, 1), a);
        if (row_tiles == 4) return launch_waves<EPI, 4, 1>(s, waves, dim3(tiles, m_blocks, 1), a);
    }
    return CIE_BAD_ARGUMENT;
}

// ---------------------------------------------------------------------------------------------
// 17 to 128 rows: waves that own columns and share the rows of A.
//
// With more than 16 rows the kernel above spends more of the memory pipeline on the rows of A (which
// every wave fetches for its own slices of K) than on W.  Here the two to four waves of a workgroup take the
// same slice of 128 k values together: the workgroup's threads fetch the slice of A once (whole
// 256-byte row segments) into LDS, every wave streams its own NT tiles of 16 columns of W over all of
// K (or a grid.z part of it) and reads the rows of A from LDS in the MFMA layout.  A wave's loads run
// one slice ahead of its products, in two sets of registers that the loop, unrolled by two, addresses by
// constants (a copy from a set whose load is still under way would wait for it; two slices ahead, with
// three sets, were 1 to 3 us slower at every size).
// Its LDS: one or two stages of the rows' slice, a staging area per wave, the rows' scales.  Two stages where
// they fit the 160 KB of a workgroup (128 rows and four waves: 86 KB, more than a kernel gets without asking).
template <int MT, int WAVES>
struct SharedRowsLds {
    static constexpr int kStageBytesA = MT * 16 * kStageRow;
    static constexpr int kRest = WAVES * kStageTile + MT * 16 * static_cast<int>(sizeof(float));
    static constexpr int kStagesA = 2 * kStageBytesA + kRest <= 160 * 1024 ? 2 : 1;
    static constexpr int kBytes = kStagesA * kStageBytesA + kRest;
};

template <int EPI, int MT, int NT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) gemm_shared_rows_kernel(FusedArgs a) {
    static_assert(EPI == EPI_SILU || EPI == EPI_PARTIAL || EPI == EPI_BF16 || EPI == EPI_F32 || EPI == EPI_ATOMIC,
                  "epilogues of this form");
    static_assert(EPI != EPI_SILU || NT == 2, "the SiLU epilogue pairs a gate tile with its up tile");
    constexpr int kWaves = WAVES;
    constexpr int kThreads = WAVES * 64;
    constexpr int kRows = MT * 16;
    constexpr int kStageBytesA = kRows * kStageRow;
    constexpr int kStagesA = SharedRowsLds<MT, WAVES>::kStagesA;
    extern __shared__ __attribute__((aligned(16))) char shared[];  // SharedRowsLds<MT, WAVES>::kBytes of them
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    const int r = lane & 15;
    const int g = lane >> 4;
    char* stage_w = shared + kStagesA * kStageBytesA + wave * kStageTile;
    float* scale_lds = reinterpret_cast<float*>(shared + kStagesA * kStageBytesA + kWaves * kStageTile);
    const int cols = (EPI == EPI_SILU) ? a.up_offset : a.N;
    // SILU: the wave's gate tile and its up tile; else NT adjacent tiles
    const int tile_first = (EPI == EPI_SILU) ? blockIdx.x * kWaves + wave : (blockIdx.x * kWaves + wave) * NT;

    const int load_row = lane >> 4;        // of the four rows of a load of W
    const int load_col = (lane & 15) * 8;  // k offset inside the 128
    const bf16_t* w_rows[NT][4];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = i * 4 + load_row;
            const int n = (EPI == EPI_SILU) ? min(tile_first * 16 + row, cols - 1) + t * a.up_offset
                                            : min((tile_first + t) * 16 + row, cols - 1);
            w_rows[t][i] = a.w + static_cast<size_t>(n) * a.K;
        }
    // the slice of A: thread t takes the piece (t % 16) of rows t / 16 + (threads / 16) i (a row past the
    // last one computes a copy that is not stored; past the last row tile, a thread repeats the last row)
    constexpr int kRowsPerPass = kThreads / 16;
    constexpr int kPasses = (kRows + kRowsPerPass - 1) / kRowsPerPass;
    const int a_row = threadIdx.x >> 4;
    const bf16_t* a_rows[kPasses];
    int a_stage_row[kPasses];
#pragma unroll
    for (int i = 0; i < kPasses; ++i) {
        a_stage_row[i] = min(i * kRowsPerPass + a_row, kRows - 1);
        a_rows[i] = a.a + static_cast<size_t>(min(a_stage_row[i], a.M - 1)) * a.lda;
    }
    const int k_begin = blockIdx.z * a.k_per_part;
    const int k_end = min(a.K, k_begin + a.k_per_part);
    const int slices = (k_end - k_begin + 127) / 128;

    // Every load is unconditional and stands in straight-line code, so that the compiler can wait for a
    // slice by counting the loads behind it (after a load under a condition it waits for all): a piece
    // past the end of the part reads the part's last piece again, and the piece of A is zeroed when used.
    struct Slot {
        u32x4 w[NT][4];
        u32x4 a[kPasses];
    };
    Slot ring0, ring1;
    auto fetch = [&](Slot& into, int slice) __attribute__((always_inline)) {
        const int k = min(k_begin + slice * 128 + load_col, k_end - 8);
#pragma unroll
        for (int i = 0; i < kPasses; ++i) into.a[i] = *reinterpret_cast<const u32x4*>(a_rows[i] + k);
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) into.w[t][i] = *reinterpret_cast<const u32x4*>(w_rows[t][i] + k);
    };

    floatx4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[mt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    const int row_tiles_used = (a.M + 15) / 16;  // (row tiles past the last row are not multiplied)

    auto step = [&](const Slot& now, Slot& ahead, int slice) __attribute__((always_inline)) {
        char* stage_a = shared + (kStagesA == 2 ? (slice & 1) * kStageBytesA : 0);
        if (kStagesA == 1) __syncthreads();  // every wave has read the slice before
        const bool inside = k_begin + slice * 128 + load_col < k_end;
#pragma unroll
        for (int i = 0; i < kPasses; ++i)
            *reinterpret_cast<u32x4*>(stage_a + a_stage_row[i] * kStageRow + load_col * 2) =
                inside ? now.a[i] : u32x4{0u, 0u, 0u, 0u};
        fetch(ahead, slice + 1);
        u32x4 bt[NT][4];
#pragma unroll
        for (int t = 0; t < NT; ++t) {  // through the wave's staging area (its LDS operations keep their order)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<u32x4*>(stage_w + (i * 4 + load_row) * kStageRow + load_col * 2) = now.w[t][i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bt[t][j] = *reinterpret_cast<const u32x4*>(stage_w + r * kStageRow + j * 64 + g * 16);
        }
        __syncthreads();  // the slice of A is in LDS
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (mt >= row_tiles_used) break;  // uniform
            u32x4 av[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                av[j] = *reinterpret_cast<const u32x4*>(stage_a + (mt * 16 + r) * kStageRow + j * 64 + g * 16);
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, av[j]), __builtin_bit_cast(bf16x8, bt[t][j]), acc[mt][t], 0, 0, 0);
        }
    };

    // Rows that still lack their 1/rms: a few lanes sum a row's partial sums.  Their loads are issued
    // before the first loads of the product and summed behind them, so that the wait is for them alone
    // (a loop of load and add here would stand a row's whole latency chain before the first slice).
    const bool scaled_rows = EPI == EPI_SILU && a.row_sumsq != nullptr;
    constexpr int kPerRowAny = kThreads / kRows;
    constexpr int kPerRow = kPerRowAny >= 8 ? 8 : kPerRowAny >= 4 ? 4 : kPerRowAny >= 2 ? 2 : 1;  // lanes per row
    constexpr int kHeld = 16;  // float4 loads a lane has under way at once
    const int scale_row = threadIdx.x / kPerRow, scale_sub = threadIdx.x % kPerRow;
    const bool scale_lane = scaled_rows && scale_row < kRows;
    const bool scale_by_four = scaled_rows && a.sumsq_parts % 4 == 0 && a.sumsq_parts >= 4;
    const float* scale_from = scaled_rows ? a.row_sumsq + static_cast<size_t>(min(scale_row, a.M - 1)) * a.sumsq_parts : nullptr;
    float4 held[kHeld];
    if (scale_by_four) {
#pragma unroll
        for (int i = 0; i < kHeld; ++i)  // (past the end: the last four again, not added below)
            held[i] = *reinterpret_cast<const float4*>(scale_from + min((scale_sub + i * kPerRow) * 4, a.sumsq_parts - 4));
    }
    fetch(ring0, 0);
    if (scaled_rows) {
        float sq = 0.f;
        if (scale_by_four) {
#pragma unroll
            for (int i = 0; i < kHeld; ++i)
                if ((scale_sub + i * kPerRow) * 4 < a.sumsq_parts) sq += (held[i].x + held[i].y) + (held[i].z + held[i].w);
            for (int p = (scale_sub + kHeld * kPerRow) * 4; p < a.sumsq_parts; p += kPerRow * 4) {  // (a very wide model)
                const float4 v = *reinterpret_cast<const float4*>(scale_from + p);
                sq += (v.x + v.y) + (v.z + v.w);
            }
        } else {
            for (int p = scale_sub; p < a.sumsq_parts; p += kPerRow) sq += scale_from[p];
        }
#pragma unroll
        for (int offset = kPerRow / 2; offset > 0; offset >>= 1) sq += __shfl_xor(sq, offset, kWave);
        if (scale_lane && scale_sub == 0) scale_lds[scale_row] = 1.0f / sqrtf(sq / static_cast<float>(a.K) + a.eps);
    }
    // (whole turns of the ring: a step past the last slice multiplies zeros)
#pragma unroll 1
    for (int base = 0; base < slices; base += 2) {
        step(ring0, ring1, base);
        step(ring1, ring0, base + 1);
    }
    if (scaled_rows && slices == 0) __syncthreads();  // (the scales, if no step stood between)

#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (mt >= row_tiles_used) break;
        if (EPI == EPI_SILU) {
            float row_scale[4] = {1.f, 1.f, 1.f, 1.f};
            if (scaled_rows) {
#pragma unroll
                for (int i = 0; i < 4; ++i) row_scale[i] = scale_lds[mt * 16 + g * 4 + i];
            }
            if (tile_first * 16 < cols)  // wave-uniform
                store_tile<EPI>(a, acc[mt][0], acc[mt][NT - 1], mt * 16, tile_first * 16 + r, tile_first, lane, row_scale);
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t)
                if ((tile_first + t) * 16 < cols)  // wave-uniform
                    store_tile<EPI>(a, acc[mt][t], acc[mt][t], mt * 16, (tile_first + t) * 16 + r, tile_first + t, lane);
        }
    }
}

template <int EPI, int MT, int NT, int WAVES>
int launch_shared_rows_tiles(hipStream_t s, dim3 grid, const FusedArgs& a) {
    constexpr int kBytes = SharedRowsLds<MT, WAVES>::kBytes;
    if (kBytes > 64 * 1024) {  // more than a kernel gets without asking: once per kernel (and again is harmless)
        static bool asked = false;
        if (!asked) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_shared_rows_kernel<EPI, MT, NT, WAVES>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, kBytes) != hipSuccess) {
                (void)hipGetLastError();
                return CIE_LAUNCH_FAILED;
            }
            asked = true;
        }
    }
    gemm_shared_rows_kernel<EPI, MT, NT, WAVES><<<grid, WAVES * 64, kBytes, s>>>(a);
    return cie_after_launch();
}

template <int EPI, int NT, int WAVES>
int launch_shared_rows_waves(hipStream_t s, int k_parts, const FusedArgs& a) {
    const int cols = (EPI == EPI_SILU) ? a.up_offset : a.N;
    const int tiles = (cols + 15) / 16;
    const int per_workgroup = WAVES * ((EPI == EPI_SILU) ? 1 : NT);
    const dim3 grid((tiles + per_workgroup - 1) / per_workgroup, 1, k_parts);
    if (a.M <= 16) return launch_shared_rows_tiles<EPI, 1, NT, WAVES>(s, grid, a);
    if (a.M <= 32) return launch_shared_rows_tiles<EPI, 2, NT, WAVES>(s, grid, a);
    if (a.M <= 64) return launch_shared_rows_tiles<EPI, 4, NT, WAVES>(s, grid, a);
    // 65 to 96 rows (single tokens beside a prompt portion of 64): six row tiles instead of eight for the epilogues
    // that the engine's steps meet there (a thread fetches and stores six pieces of the rows a slice instead of eight)
    if constexpr (EPI == EPI_ATOMIC || EPI == EPI_SILU || EPI == EPI_F32)
        if (a.M <= 96) return launch_shared_rows_tiles<EPI, 6, NT, WAVES>(s, grid, a);
    return launch_shared_rows_tiles<EPI, 8, NT, WAVES>(s, grid, a);
}

template <int EPI, int NT>
int launch_shared_rows(hipStream_t s, int waves, int k_parts, const FusedArgs& a) {
    switch (waves) {
        case 2: return launch_shared_rows_waves<EPI, NT, 2>(s, k_parts, a);
        case 3: return launch_shared_rows_waves<EPI, NT, 3>(s, k_parts, a);
        case 4: return launch_shared_rows_waves<EPI, NT, 4>(s, k_parts, a);
    }
    return CIE_BAD_ARGUMENT;
}

}  // namespace

// epilogue: 0 bf16, 1 float32, 2 SiLU-gate (W = [gate rows; up rows], N = 2 * outputs), 3 residual
// accumulate (+ sums of squares).  (Products whose K is cut into parts take the other form, below.)
// row_tiles 1, 2, 4: 16, 32, 64 rows per workgroup (more rows: more workgroups, each streaming W again);
// `waves` waves per workgroup share K (1, 2, 4, 8; with more than one row tile 4 or 8);
// column_tiles 1 or 2 tiles of 16 columns per workgroup (2 only with more than one row tile: the rows of
// A that a wave loads then meet two tiles of W; the SiLU epilogue always takes a gate tile and its up tile).
// K and lda must be multiples of 8 (16-byte loads); N is free.
// norm_weight [N] float32 and scaled_out [M, N] bf16 (both or neither; RESID only): the epilogue also writes
// the new residual times the weight.  row_sumsq [M, sumsq_parts] and eps (SILU with one row tile only): the
// rows of `a` lack the factor rsqrt(sum of the row's partial sums / K + eps), applied before the SiLU.
CIE_API int cie_gemm_fused(void* stream, const void* a, int lda, const void* w, const void* bias, void* c,
                           float* residual, float* sumsq, int M, int N, int K, int epilogue, int row_tiles,
                           int waves, int column_tiles, const float* norm_weight, void* scaled_out,
                           const float* row_sumsq, int sumsq_parts, float eps) {
    if (M <= 0 || N <= 0 || K <= 0 || K % 8 || !a || !w || lda < K || lda % 8) return CIE_BAD_ARGUMENT;
    if (row_tiles != 1 && row_tiles != 2 && row_tiles != 4) return CIE_BAD_ARGUMENT;
    if (waves != 1 && waves != 2 && waves != 4 && waves != 8) return CIE_BAD_ARGUMENT;
    if (epilogue == EPI_SILU && (N % 2 || bias)) return CIE_BAD_ARGUMENT;
    if (epilogue == EPI_RESID && (!residual || !sumsq)) return CIE_BAD_ARGUMENT;
    if (epilogue != EPI_RESID && !c) return CIE_BAD_ARGUMENT;
    // the folded norm: a scaled copy needs the weight and the RESID epilogue; rows that lack their scale
    // are taken by the SILU epilogue of one row tile
    if ((scaled_out != nullptr) != (norm_weight != nullptr) || (scaled_out && epilogue != EPI_RESID)) return CIE_BAD_ARGUMENT;
    if (row_sumsq && (epilogue != EPI_SILU || row_tiles != 1 || M > 16 || sumsq_parts < 1 || !(eps > 0.f)))
        return CIE_BAD_ARGUMENT;
    FusedArgs f;
    f.a = static_cast<const bf16_t*>(a);
    f.lda = lda;
    f.w = static_cast<const bf16_t*>(w);
    f.bias = static_cast<const bf16_t*>(bias);
    f.c = c;
    f.residual = residual;
    f.sumsq = sumsq;
    f.M = M;
    f.N = N;
    f.K = K;
    f.up_offset = (epilogue == EPI_SILU) ? N / 2 : 0;
    f.k_per_part = (K + 127) / 128 * 128;
    f.norm_weight = norm_weight;
    f.scaled_out = static_cast<bf16_t*>(scaled_out);
    f.row_sumsq = row_sumsq;
    f.sumsq_parts = sumsq_parts;
    f.eps = eps;
    f.fold_residual = nullptr;
    f.fold_weight = nullptr;
    f.rope = RopeArgs{};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (epilogue) {
        case EPI_BF16: return launch<EPI_BF16>(s, row_tiles, waves, column_tiles, f);
        case EPI_F32: return launch<EPI_F32>(s, row_tiles, waves, column_tiles, f);
        case EPI_SILU: return launch<EPI_SILU>(s, row_tiles, waves, column_tiles, f);
        case EPI_RESID: return launch<EPI_RESID>(s, row_tiles, waves, column_tiles, f);
    }
    return CIE_BAD_ARGUMENT;
}

// q/k/v product with the ROPE epilogue (64 rows per workgroup; more rows run as more workgroup rows, each
// streaming the weight again): `w` [N, K] stacks the rows of q_heads query
// heads, kv_heads key heads and kv_heads value heads of head_dim dimensions each (a multiple of 32);
// `c` [M, N] receives the rotated queries (its key and value columns are left alone); rotated keys and
// values go to the cache page of each row's position.  `waves` waves per workgroup share K (1, 2, 4, 8;
// with more than 16 rows 4 or 8).
// (Below this many pairs of tiles a product of up to 64 rows takes one tile a workgroup: the 3B shape's 80 pairs
// leave two thirds of the compute units without a workgroup; 64 rows 12.1 -> 10.9 us.)
constexpr unsigned kSplitPairsBelow = 128;

namespace {
struct FoldedNorm {  // the norm in front of the q/k/v product, made by the product itself (see FusedArgs)
    const float* residual = nullptr;
    const float* weight = nullptr;
    float eps = 0.f;
};

int qkv_rope(void* stream, const void* a, int lda, const void* w, const void* bias, void* c,
             int M, int N, int K, int waves, const float* cos_table, const float* sin_table,
             const int* positions, const int* seq_of_token, const int* seq_slot,
             const int* block_table, int table_width, void* k_pool, void* v_pool, int q_heads,
             int kv_heads, int head_dim, int page_size, int rotate, int write_kv, const FoldedNorm* fold) {
    if (fold) {
        if (M <= 0 || M > kFoldRows || K < 8 || K % 8 || !w || !c) return CIE_BAD_ARGUMENT;
        if (!fold->residual || !fold->weight || !(fold->eps > 0.f)) return CIE_BAD_ARGUMENT;
        a = nullptr;
        lda = K;
    } else if (M <= 0 || (M + 63) / 64 > 65535 || K <= 0 || K % 8 || !a || !w || !c || lda < K || lda % 8) {
        return CIE_BAD_ARGUMENT;
    }
    if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim % 32 || page_size <= 0 || table_width <= 0 ||
        N != (q_heads + 2 * kv_heads) * head_dim)
        return CIE_BAD_ARGUMENT;
    if (!positions || (rotate && (!cos_table || !sin_table)) ||
        (write_kv && (!seq_of_token || !seq_slot || !block_table || !k_pool || !v_pool)))
        return CIE_BAD_ARGUMENT;
    FusedArgs f;
    f.a = static_cast<const bf16_t*>(a);
    f.lda = lda;
    f.w = static_cast<const bf16_t*>(w);
    f.bias = static_cast<const bf16_t*>(bias);
    f.c = c;
    f.residual = nullptr;
    f.sumsq = nullptr;
    f.M = M;
    f.N = N;
    f.K = K;
    f.up_offset = 0;
    f.k_per_part = (K + 127) / 128 * 128;
    f.norm_weight = nullptr;
    f.scaled_out = nullptr;
    f.row_sumsq = nullptr;
    f.sumsq_parts = 0;
    f.eps = 0.f;
    f.fold_residual = nullptr;
    f.fold_weight = nullptr;
    f.rope = RopeArgs{cos_table, sin_table, positions, seq_of_token, seq_slot, block_table, table_width,
                      static_cast<bf16_t*>(k_pool), static_cast<bf16_t*>(v_pool), q_heads, kv_heads, head_dim,
                      page_size, rotate, write_kv};
    const dim3 grid((q_heads + 2 * kv_heads) * (head_dim / 32), M <= 64 ? 1 : (M + 63) / 64, 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 twice((q_heads + 2 * kv_heads) * (head_dim / 16), 1, 1);
    const bool one_tile = M <= 16 && grid.x < kSplitPairsBelow;  // few columns: one tile a workgroup, twice the workgroups
    if (fold) {
        f.fold_residual = fold->residual;
        f.fold_weight = fold->weight;
        f.eps = fold->eps;
        if (M <= 8) {
            if (one_tile) return launch_waves<EPI_ROPE8, 1, 1, 2>(s, waves, twice, f);
            return launch_waves<EPI_ROPE, 1, 2, 2>(s, waves, grid, f);
        }
        if (one_tile) return launch_waves<EPI_ROPE8, 1, 1, 4>(s, waves, twice, f);
        return launch_waves<EPI_ROPE, 1, 2, 4>(s, waves, grid, f);
    }
    if (one_tile) return launch_waves<EPI_ROPE8, 1, 1>(s, waves, twice, f);
    if (M <= 64 && grid.x < kSplitPairsBelow) {  // the same with more row tiles
        if (M <= 32) return launch_waves<EPI_ROPE8, 2, 1>(s, waves, twice, f);
        return launch_waves<EPI_ROPE8, 4, 1>(s, waves, twice, f);
    }
    if (M <= 16) return launch_waves<EPI_ROPE, 1, 2>(s, waves, grid, f);
    if (M <= 32) return launch_waves<EPI_ROPE, 2, 2>(s, waves, grid, f);
    return launch_waves<EPI_ROPE, 4, 2>(s, waves, grid, f);
}
}  // namespace

CIE_API int cie_gemm_qkv_rope(void* stream, const void* a, int lda, const void* w, const void* bias, void* c,
                              int M, int N, int K, int waves, const float* cos_table, const float* sin_table,
                              const int* positions, const int* seq_of_token, const int* seq_slot,
                              const int* block_table, int table_width, void* k_pool, void* v_pool, int q_heads,
                              int kv_heads, int head_dim, int page_size, int rotate, int write_kv) {
    return qkv_rope(stream, a, lda, w, bias, c, M, N, K, waves, cos_table, sin_table, positions, seq_of_token, seq_slot,
                    block_table, table_width, k_pool, v_pool, q_heads, kv_heads, head_dim, page_size, rotate, write_kv,
                    nullptr);
}

// The same for up to 16 rows whose RMSNorm the product makes itself: the rows are residual [M, K] (float32) *
// norm_weight * 1/rms.  A decode step of a few sequences saves the norm's kernel.
CIE_API int cie_gemm_qkv_rope_folded_norm(void* stream, const float* residual,
                                          const float* norm_weight, float eps, const void* w,
                                          const void* bias, void* c, int M, int N, int K, int waves,
                                          const float* cos_table, const float* sin_table, const int* positions,
                                          const int* seq_of_token, const int* seq_slot, const int* block_table,
                                          int table_width, void* k_pool, void* v_pool, int q_heads, int kv_heads,
                                          int head_dim, int page_size, int rotate, int write_kv) {
    FoldedNorm fold;
    fold.residual = residual;
    fold.weight = norm_weight;
    fold.eps = eps;
    return qkv_rope(stream, nullptr, K, w, bias, c, M, N, K, waves, cos_table, sin_table, positions, seq_of_token,
                    seq_slot, block_table, table_width, k_pool, v_pool, q_heads, kv_heads, head_dim, page_size, rotate,
                    write_kv, &fold);
}

// The form for 17 to 128 rows in which a workgroup's waves own columns and share the rows of A
// through LDS (one workgroup row: M <= 128).  epilogue 0 (bf16, + bias), 1 (float32, + bias; two tiles a wave),
// 2 (SiLU-gate; row_sumsq as in
// cie_gemm_fused, for any number of rows here), 4 (k_parts partial products) or 7 (k_parts parts of K, each of
// which adds its products into `c`, float32 [M, N], with atomic adds: the order of the sums is not fixed).  column_tiles 1 or 2 tiles of
// 16 columns per wave (SiLU: the gate tile and its up tile), 2 to 4 waves per workgroup.
CIE_API int cie_gemm_shared_rows(void* stream, const void* a, int lda, const void* w, const void* bias, void* c, int M,
                                 int N, int K, int epilogue, int column_tiles, int waves, int k_parts,
                                 const float* row_sumsq, int sumsq_parts, float eps) {
    if (M <= 0 || M > 128 || N <= 0 || K <= 0 || K % 8 || !a || !w || !c || lda < K || lda % 8) return CIE_BAD_ARGUMENT;
    if (epilogue != EPI_BF16 && epilogue != EPI_F32 && epilogue != EPI_SILU && epilogue != EPI_PARTIAL && epilogue != EPI_ATOMIC)
        return CIE_BAD_ARGUMENT;
    if (epilogue == EPI_SILU && (N % 2 || bias || column_tiles != 2)) return CIE_BAD_ARGUMENT;
    if (column_tiles != 1 && column_tiles != 2) return CIE_BAD_ARGUMENT;
    if (k_parts < 1 || k_parts > 64 || (k_parts > 1 && epilogue != EPI_PARTIAL && epilogue != EPI_ATOMIC)) return CIE_BAD_ARGUMENT;
    if (row_sumsq && (epilogue != EPI_SILU || sumsq_parts < 1 || !(eps > 0.f))) return CIE_BAD_ARGUMENT;
    FusedArgs f;
    f.a = static_cast<const bf16_t*>(a);
    f.lda = lda;
    f.w = static_cast<const bf16_t*>(w);
    f.bias = static_cast<const bf16_t*>(bias);
    f.c = c;
    f.residual = (epilogue == EPI_ATOMIC) ? static_cast<float*>(c) : nullptr;
    f.sumsq = nullptr;
    f.M = M;
    f.N = N;
    f.K = K;
    f.up_offset = (epilogue == EPI_SILU) ? N / 2 : 0;
    f.k_per_part = ((K + k_parts - 1) / k_parts + 127) / 128 * 128;
    f.norm_weight = nullptr;
    f.scaled_out = nullptr;
    f.row_sumsq = row_sumsq;
    f.sumsq_parts = sumsq_parts;
    f.eps = eps;
    f.fold_residual = nullptr;
    f.fold_weight = nullptr;
    f.rope = RopeArgs{};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (epilogue) {
        case EPI_SILU: return launch_shared_rows<EPI_SILU, 2>(s, waves, 1, f);
        case EPI_BF16:
            return column_tiles == 2 ? launch_shared_rows<EPI_BF16, 2>(s, waves, 1, f) : launch_shared_rows<EPI_BF16, 1>(s, waves, 1, f);
        case EPI_F32:  // (the logits: two tiles a wave)
            if (column_tiles != 2) return CIE_BAD_ARGUMENT;
            return launch_shared_rows<EPI_F32, 2>(s, waves, 1, f);
        case EPI_PARTIAL:
            return column_tiles == 2 ? launch_shared_rows<EPI_PARTIAL, 2>(s, waves, k_parts, f)
                                     : launch_shared_rows<EPI_PARTIAL, 1>(s, waves, k_parts, f);
        case EPI_ATOMIC:
            return column_tiles == 2 ? launch_shared_rows<EPI_ATOMIC, 2>(s, waves, k_parts, f)
                                     : launch_shared_rows<EPI_ATOMIC, 1>(s, waves, k_parts, f);
    }
    return CIE_BAD_ARGUMENT;
}
