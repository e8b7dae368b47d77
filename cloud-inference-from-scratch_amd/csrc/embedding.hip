// Embedding gather: residual[t, :] = table[ids[t], :] widened to float32.
// The residual stream is float32 in both engine dtypes.
// With `feed` (int32 [tokens]) and `pool`: row t takes its token from pool[feed[t]] where feed[t] >= 0, so
// that a decode step can start from the tokens the step before it sampled, before the host has seen them.
#include "common.h"

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             const int* __restrict__ feed, const int* __restrict__ pool,
                             float* __restrict__ out, int hidden, int vocab) {
    const int token = blockIdx.x;
    int id = ids[token];
    if (feed != nullptr && feed[token] >= 0) id = pool[feed[token]];
    // Ids are validated on the host; clamp so that a stale padding row can never read outside.
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* row = table + static_cast<size_t>(id) * hidden;
    float* dst = out + static_cast<size_t>(token) * hidden;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) dst[h] = to_float(row[h]);
}

CIE_API int cie_embed(void* stream, int dtype, const void* table, const int* ids, const int* feed,
                      const int* pool, float* out, int tokens, int hidden, int vocab) {
    if (tokens < 0 || hidden <= 0 || vocab <= 0 || (feed && !pool)) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32)
        embed_kernel<float><<<tokens, 256, 0, s>>>(static_cast<const float*>(table), ids, feed, pool, out, hidden, vocab);
    else if (dtype == CIE_BF16)
        embed_kernel<bf16_t><<<tokens, 256, 0, s>>>(static_cast<const bf16_t*>(table), ids, feed, pool, out, hidden, vocab);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
