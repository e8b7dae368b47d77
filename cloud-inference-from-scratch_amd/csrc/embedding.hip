// Embedding gather: residual[t, :] = table[ids[t], :] widened to float32.
// The residual stream is float32 in both engine dtypes.
#include "common.h"

template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int hidden, int vocab) {
    const int token = blockIdx.x;
    int id = ids[token];
    // Ids are validated on the host; clamp so that a stale padding row can never read outside.
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const T* row = table + static_cast<size_t>(id) * hidden;
    float* dst = out + static_cast<size_t>(token) * hidden;
    for (int h = threadIdx.x; h < hidden; h += blockDim.x) dst[h] = to_float(row[h]);
}

CIE_API int cie_embed(void* stream, int dtype, const void* table, const int* ids, float* out,
                      int tokens, int hidden, int vocab) {
    if (tokens < 0 || hidden <= 0 || vocab <= 0) return CIE_BAD_ARGUMENT;
    if (tokens == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == CIE_F32)
        embed_kernel<float><<<tokens, 256, 0, s>>>(static_cast<const float*>(table), ids, out, hidden, vocab);
    else if (dtype == CIE_BF16)
        embed_kernel<bf16_t><<<tokens, 256, 0, s>>>(static_cast<const bf16_t*>(table), ids, out, hidden, vocab);
    else
        return CIE_BAD_ARGUMENT;
    return cie_after_launch();
}
