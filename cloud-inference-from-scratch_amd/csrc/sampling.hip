// Sampling over float32 logits [rows, vocab]; one workgroup per row.
//
// Greedy: the first index of the maximum (ties go to the lower index).
// Temperature: p_i = exp((l_i - max) / T); with the row's uniform number u in
// [0, 1) the token is the first i whose running sum of p exceeds u * sum(p).
// u is made on the host from (seed, request, step), so a draw depends neither
// on the batch nor on the thread layout.  T <= 0 means greedy.
#include <mutex>

#include "cie_no_alloc.h"
#include "common.h"

// Partial results of cie_argmax_static's first stage: CIE_ARGMAX_STATIC_MAX_ENTRIES best values (float),
// then as many indices (int).  Host code never passes this name to a kernel: in host code it is a stand-in,
// not a device address.  It asks for the array's address on the current device once (static_scratch) and
// uses that pointer.
static __device__ __align__(256) unsigned char scratch[CIE_ARGMAX_STATIC_MAX_ENTRIES * (sizeof(float) + sizeof(int))];

namespace {

constexpr int kThreads = 256;
constexpr int kMaxDevices = 64;

std::mutex scratch_lock;
void* scratch_on_device[kMaxDevices];  // the array's address on each device, once it has been asked for

// The address of `scratch` on the current device (every GPU holds its own copy at its own address).
int static_scratch(unsigned char** out) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return CIE_SETUP_FAILED;
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (scratch_on_device[device] == nullptr) {
        void* found = nullptr;
        if (hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)) != hipSuccess || found == nullptr) {
            (void)hipGetLastError();  // (so that the next launch check does not report this one)
            return CIE_SETUP_FAILED;
        }
        scratch_on_device[device] = found;
    }
    *out = static_cast<unsigned char*>(scratch_on_device[device]);
    return CIE_OK;
}

__device__ __forceinline__ void argmax_block(const float* row, int vocab, float* s_val, int* s_idx,
                                             float& best_out, int& idx_out) {
    float best = -INFINITY;
    int best_idx = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += kThreads) {
        const float v = row[i];
        if (v > best || (v == best && i < best_idx)) {
            best = v;
            best_idx = i;
        }
    }
    s_val[threadIdx.x] = best;
    s_idx[threadIdx.x] = best_idx;
    __syncthreads();
    for (int stride = kThreads / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) {
            const float v = s_val[threadIdx.x + stride];
            const int i = s_idx[threadIdx.x + stride];
            if (v > s_val[threadIdx.x] || (v == s_val[threadIdx.x] && i < s_idx[threadIdx.x])) {
                s_val[threadIdx.x] = v;
                s_idx[threadIdx.x] = i;
            }
        }
        __syncthreads();
    }
    best_out = s_val[0];
    idx_out = s_idx[0] == 0x7fffffff ? 0 : s_idx[0];
    __syncthreads();
}

// Temperature sampling walks the row in chunks of kChunk numbers, a thread's four neighbours at a time, so that
// a wave's loads are whole cache lines.  The running sum has a fixed order all the same: a chunk's sum is
// made by one fixed tree, the chunks are added one after the other, and inside the chunk that holds the
// target the numbers are added in the order of their indices.
constexpr int kChunk = kThreads * 4;
constexpr int kMaxChunks = 2048;  // of a row: vocabularies up to 2,097,152

__device__ __forceinline__ float4 exp_of_four(const float* row, int first, int vocab, float best, float inv_t) {
    float4 e = {0.f, 0.f, 0.f, 0.f};
    if (first + 3 < vocab && (reinterpret_cast<uintptr_t>(row + first) & 15) == 0) {
        const float4 v = *reinterpret_cast<const float4*>(row + first);
        e.x = expf((v.x - best) * inv_t);
        e.y = expf((v.y - best) * inv_t);
        e.z = expf((v.z - best) * inv_t);
        e.w = expf((v.w - best) * inv_t);
    } else {
        if (first < vocab) e.x = expf((row[first] - best) * inv_t);
        if (first + 1 < vocab) e.y = expf((row[first + 1] - best) * inv_t);
        if (first + 2 < vocab) e.z = expf((row[first + 2] - best) * inv_t);
        if (first + 3 < vocab) e.w = expf((row[first + 3] - best) * inv_t);
    }
    return e;
}

// Sum over the workgroup's threads in one fixed order; every thread gets the result (contains barriers).
__device__ __forceinline__ float fixed_block_sum(float v, float* s_val) {
    s_val[threadIdx.x] = v;
    __syncthreads();
    for (int stride = kThreads / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) s_val[threadIdx.x] += s_val[threadIdx.x + stride];
        __syncthreads();
    }
    const float total = s_val[0];
    __syncthreads();
    return total;
}

// The first index in [begin, end) of `row` whose running sum of exp((l - best) * inv_t), counted from `begin`,
// passes the target; the target is `fraction` of the span's whole sum if `of_whole`, else `fraction` itself.
// Every thread of the workgroup calls it and gets the result (it contains barriers).  s_chunk holds the sums of
// the span's chunks of kChunk numbers: the span has at most kMaxChunks of them.
__device__ int pick_in_span(const float* row, int begin, int end, float best, float inv_t, float fraction, bool of_whole,
                            float* s_val, int* s_idx, float* s_chunk, float* s_target, int* s_pick) {
    const int chunks = (end - begin + kChunk - 1) / kChunk;
    for (int c = 0; c < chunks; ++c) {
        const float4 e = exp_of_four(row, begin + c * kChunk + threadIdx.x * 4, end, best, inv_t);
        const float sum = fixed_block_sum((e.x + e.y) + (e.z + e.w), s_val);
        if (threadIdx.x == 0) s_chunk[c] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float target = fraction;
        if (of_whole) {
            float total = 0.f;
            for (int c = 0; c < chunks; ++c) total += s_chunk[c];
            target = fraction * total;
        }
        // If rounding leaves the target unreached (the sums here and the running sums below are made in
        // different orders), the token is the last one that has any probability at all: the last chunk whose
        // sum is not zero, and in it the last index whose own term is not zero.
        float running = 0.f, before_owner = 0.f;
        int owner = chunks - 1;
        for (int c = 0; c < chunks; ++c) {
            if (running + s_chunk[c] > target) {
                owner = c;
                before_owner = running;
                break;
            }
            if (s_chunk[c] > 0.f) {
                owner = c;
                before_owner = running;
            }
            running += s_chunk[c];
        }
        *s_target = target - before_owner;  // what is left to reach inside the chunk
        s_idx[0] = owner;
        s_idx[1] = -1;  // the last index of the chunk whose own term is not zero
        *s_pick = 0x7fffffff;
    }
    __syncthreads();
    const int owner = s_idx[0];
    const float target = *s_target;
    __syncthreads();
    // inside the chunk: the sums of the threads before this one (in index order), then the thread's own four
    const int first = begin + owner * kChunk + threadIdx.x * 4;
    const float4 e = exp_of_four(row, first, end, best, inv_t);
    s_val[threadIdx.x] = (e.x + e.y) + (e.z + e.w);
    __syncthreads();
    for (int offset = 1; offset < kThreads; offset <<= 1) {  // running sums over the threads, in place
        const float below = threadIdx.x >= offset ? s_val[threadIdx.x - offset] : 0.f;
        __syncthreads();
        s_val[threadIdx.x] += below;
        __syncthreads();
    }
    float running = threadIdx.x > 0 ? s_val[threadIdx.x - 1] : 0.f;
    int mine = 0x7fffffff;
    const float four[4] = {e.x, e.y, e.z, e.w};
    int last = -1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        running += four[i];
        // (a token whose own term is zero is never the one: the sums of the threads before are made in
        // another order than this running sum and may pass the target a hair earlier or later)
        if (mine == 0x7fffffff && first + i < end && four[i] > 0.f && running > target) mine = first + i;
        if (first + i < end && four[i] > 0.f) last = first + i;
    }
    if (mine != 0x7fffffff) atomicMin(s_pick, mine);  // the first index whose running sum passes the target
    if (last >= 0) atomicMax(&s_idx[1], last);
    __syncthreads();
    int picked = *s_pick;
    if (picked == 0x7fffffff)  // unreached: the last token with a probability, or (none has one) the span's last
        picked = s_idx[1] >= 0 ? s_idx[1] : min(end, begin + (owner + 1) * kChunk) - 1;
    __syncthreads();
    return picked;
}

__global__ void __launch_bounds__(kThreads)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
              const float* __restrict__ uniform, int* __restrict__ out, int vocab, int ld) {
    __shared__ float s_val[kThreads];
    __shared__ int s_idx[kThreads];
    __shared__ float s_chunk[kMaxChunks];
    __shared__ float s_target;
    __shared__ int s_pick;
    const int r = blockIdx.x;
    const float* row = logits + static_cast<size_t>(r) * ld;
    float best;
    int best_idx;
    argmax_block(row, vocab, s_val, s_idx, best, best_idx);
    const float temp = temperature ? temperature[r] : 0.f;
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) out[r] = best_idx;
        return;
    }
    const int picked = pick_in_span(row, 0, vocab, best, 1.0f / temp, uniform[r], true, s_val, s_idx, s_chunk, &s_target,
                                    &s_pick);
    if (threadIdx.x == 0) out[r] = picked;
}

// Over a large vocabulary a row is taken by many workgroups.  Stage 1: each scans one part of one row and leaves
// the part's largest logit, its first index and, where the row has a temperature, the part's sum of
// exp((l - the part's largest) / T), summed in a fixed order.  Stage 2 (one workgroup per row): the row's
// largest logit (greedy rows are done), the parts' sums brought to that scale and added in index order, the part
// in which the running sum passes u times the whole, and the index inside that part as above.
constexpr int kMaxParts = 1024;

__global__ void __launch_bounds__(kThreads)
sample_parts_kernel(const float* __restrict__ logits, const float* __restrict__ temperature, float* __restrict__ part_val,
                    int* __restrict__ part_idx, float* __restrict__ part_sum, int vocab, int ld, int part) {
    __shared__ float s_val[kThreads];
    __shared__ int s_idx[kThreads];
    const int r = blockIdx.y;
    const int begin = blockIdx.x * part;
    const int end = min(vocab, begin + part);
    const float* row = logits + static_cast<size_t>(r) * ld;
    float best;
    int best_idx;
    argmax_block(row + begin, end - begin, s_val, s_idx, best, best_idx);
    const float temp = temperature[r];
    float sum = 0.f;
    if (temp > 0.f) {
        const float inv_t = 1.0f / temp;
        for (int first = begin; first < end; first += kChunk) {  // chunk by chunk, each by the fixed tree
            const float4 e = exp_of_four(row, first + threadIdx.x * 4, end, best, inv_t);
            sum += fixed_block_sum((e.x + e.y) + (e.z + e.w), s_val);
        }
    }
    if (threadIdx.x == 0) {
        part_val[r * gridDim.x + blockIdx.x] = best;
        part_idx[r * gridDim.x + blockIdx.x] = begin + best_idx;
        part_sum[r * gridDim.x + blockIdx.x] = sum;
    }
}

__global__ void __launch_bounds__(kThreads)
sample_final_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                    const float* __restrict__ uniform, const float* __restrict__ part_val,
                    const int* __restrict__ part_idx, const float* __restrict__ part_sum, int* __restrict__ out, int vocab,
                    int ld, int part, int parts) {
    __shared__ float s_val[kThreads];
    __shared__ int s_idx[kThreads];
    __shared__ float s_chunk[kMaxParts];
    __shared__ float s_target;
    __shared__ int s_pick;
    const int r = blockIdx.x;
    float best = -INFINITY;
    int best_idx = 0x7fffffff;
    for (int c = threadIdx.x; c < parts; c += kThreads) {  // parts are in index order: ties keep the lower index
        const float v = part_val[r * parts + c];
        const int i = part_idx[r * parts + c];
        if (v > best || (v == best && i < best_idx)) {
            best = v;
            best_idx = i;
        }
    }
    s_val[threadIdx.x] = best;
    s_idx[threadIdx.x] = best_idx;
    __syncthreads();
    for (int stride = kThreads / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) {
            const float v = s_val[threadIdx.x + stride];
            const int i = s_idx[threadIdx.x + stride];
            if (v > s_val[threadIdx.x] || (v == s_val[threadIdx.x] && i < s_idx[threadIdx.x])) {
                s_val[threadIdx.x] = v;
                s_idx[threadIdx.x] = i;
            }
        }
        __syncthreads();
    }
    best = s_val[0];
    best_idx = s_idx[0] == 0x7fffffff ? 0 : s_idx[0];
    __syncthreads();
    const float temp = temperature[r];
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) out[r] = best_idx;
        return;
    }
    const float inv_t = 1.0f / temp;
    for (int c = threadIdx.x; c < parts; c += kThreads)
        s_chunk[c] = part_sum[r * parts + c] * expf((part_val[r * parts + c] - best) * inv_t);
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int c = 0; c < parts; ++c) total += s_chunk[c];
        const float target = uniform[r] * total;
        // (unreached through rounding: the last part that has any probability, as inside a part)
        float running = 0.f, before_owner = 0.f;
        int owner = parts - 1;
        for (int c = 0; c < parts; ++c) {
            if (running + s_chunk[c] > target) {
                owner = c;
                before_owner = running;
                break;
            }
            if (s_chunk[c] > 0.f) {
                owner = c;
                before_owner = running;
            }
            running += s_chunk[c];
        }
        s_target = target - before_owner;
        s_idx[0] = owner;
    }
    __syncthreads();
    const int owner = s_idx[0];
    const float left = s_target;
    __syncthreads();
    const float* row = logits + static_cast<size_t>(r) * ld;
    const int picked = pick_in_span(row, owner * part, min(vocab, (owner + 1) * part), best, inv_t, left, false, s_val, s_idx,
                                    s_chunk, &s_target, &s_pick);
    if (threadIdx.x == 0) out[r] = picked;
}

// Greedy over a large vocabulary, stage 1: each workgroup scans one chunk of one row and leaves its
// best (value, first index); stage 2 (one workgroup per row) picks among the chunks.
__global__ void __launch_bounds__(kThreads)
argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ chunk_val, int* __restrict__ chunk_idx,
                     int vocab, int ld, int chunk) {
    __shared__ float s_val[kThreads];
    __shared__ int s_idx[kThreads];
    const int r = blockIdx.y;
    const int begin = blockIdx.x * chunk;
    const int count = min(chunk, vocab - begin);
    float best;
    int best_idx;
    argmax_block(logits + static_cast<size_t>(r) * ld + begin, count, s_val, s_idx, best, best_idx);
    if (threadIdx.x == 0) {
        chunk_val[r * gridDim.x + blockIdx.x] = best;
        chunk_idx[r * gridDim.x + blockIdx.x] = begin + best_idx;
    }
}

__global__ void __launch_bounds__(kThreads)
argmax_final_kernel(const float* __restrict__ chunk_val, const int* __restrict__ chunk_idx, int* __restrict__ out,
                    int chunks) {
    __shared__ float s_val[kThreads];
    __shared__ int s_idx[kThreads];
    const int r = blockIdx.x;
    float best = -INFINITY;
    int best_idx = 0x7fffffff;
    for (int c = threadIdx.x; c < chunks; c += kThreads) {  // chunks are in index order: ties keep the lower index
        const float v = chunk_val[r * chunks + c];
        const int i = chunk_idx[r * chunks + c];
        if (v > best || (v == best && i < best_idx)) {
            best = v;
            best_idx = i;
        }
    }
    s_val[threadIdx.x] = best;
    s_idx[threadIdx.x] = best_idx;
    __syncthreads();
    for (int stride = kThreads / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) {
            const float v = s_val[threadIdx.x + stride];
            const int i = s_idx[threadIdx.x + stride];
            if (v > s_val[threadIdx.x] || (v == s_val[threadIdx.x] && i < s_idx[threadIdx.x])) {
                s_val[threadIdx.x] = v;
                s_idx[threadIdx.x] = i;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[r] = s_idx[0] == 0x7fffffff ? 0 : s_idx[0];
}

}  // namespace

// Greedy for every row in two stages; chunk_val / chunk_idx hold rows * chunks entries, chunks = ceil(vocab / chunk).
CIE_API int cie_argmax(void* stream, const float* logits, float* chunk_val, int* chunk_idx, int* out, int rows,
                       int vocab, int ld, int chunk) {
    if (rows < 0 || vocab <= 0 || ld < vocab || chunk <= 0 || rows > 65535 || !chunk_val || !chunk_idx)
        return CIE_BAD_ARGUMENT;
    if (rows == 0) return CIE_OK;
    const int chunks = (vocab + chunk - 1) / chunk;
    hipStream_t s = static_cast<hipStream_t>(stream);
    argmax_chunks_kernel<<<dim3(chunks, rows), kThreads, 0, s>>>(logits, chunk_val, chunk_idx, vocab, ld, chunk);
    if (cie_after_launch() != CIE_OK) return CIE_LAUNCH_FAILED;
    argmax_final_kernel<<<rows, kThreads, 0, s>>>(chunk_val, chunk_idx, out, chunks);
    return cie_after_launch();
}

// The same without a workspace from the caller and without any allocation: see cie_no_alloc.h.
CIE_API int cie_argmax_static(void* stream, const float* logits, int* out, int rows, int vocab, int ld, int chunk) {
    if (rows < 0 || vocab <= 0 || ld < vocab || chunk <= 0 || rows > 65535 || !logits || !out) return CIE_BAD_ARGUMENT;
    if (rows == 0) return CIE_OK;
    const long chunks = (static_cast<long>(vocab) + chunk - 1) / chunk;
    if (chunks * rows > CIE_ARGMAX_STATIC_MAX_ENTRIES) return CIE_TOO_LARGE;
    unsigned char* base = nullptr;
    const int found = static_scratch(&base);
    if (found != CIE_OK) return found;
    float* chunk_val = reinterpret_cast<float*>(base);
    int* chunk_idx = reinterpret_cast<int*>(base + CIE_ARGMAX_STATIC_MAX_ENTRIES * sizeof(float));
    hipStream_t s = static_cast<hipStream_t>(stream);
    argmax_chunks_kernel<<<dim3(static_cast<unsigned>(chunks), rows), kThreads, 0, s>>>(logits, chunk_val, chunk_idx,
                                                                                      vocab, ld, chunk);
    if (cie_after_launch() != CIE_OK) return CIE_LAUNCH_FAILED;
    argmax_final_kernel<<<rows, kThreads, 0, s>>>(chunk_val, chunk_idx, out, static_cast<int>(chunks));
    return cie_after_launch();
}

// Temperature sampling (and greedy where a row's temperature is 0) over a large vocabulary in two stages;
// part_val / part_idx / part_sum hold rows * parts entries, parts = ceil(vocab / part), part a multiple of 1,024.
CIE_API int cie_sample_parts(void* stream, const float* logits, const float* temperature, const float* uniform,
                             float* part_val, int* part_idx, float* part_sum, int* out, int rows, int vocab, int ld,
                             int part) {
    if (rows < 0 || vocab <= 0 || ld < vocab || part <= 0 || part % kChunk || part / kChunk > kMaxParts || rows > 65535 ||
        !temperature || !uniform || !part_val || !part_idx || !part_sum)
        return CIE_BAD_ARGUMENT;
    const int parts = (vocab + part - 1) / part;
    if (parts > kMaxParts) return CIE_BAD_ARGUMENT;
    if (rows == 0) return CIE_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    sample_parts_kernel<<<dim3(parts, rows), kThreads, 0, s>>>(logits, temperature, part_val, part_idx, part_sum, vocab, ld,
                                                              part);
    if (cie_after_launch() != CIE_OK) return CIE_LAUNCH_FAILED;
    sample_final_kernel<<<rows, kThreads, 0, s>>>(logits, temperature, uniform, part_val, part_idx, part_sum, out, vocab, ld,
                                                  part, parts);
    return cie_after_launch();
}

CIE_API int cie_sample(void* stream, const float* logits, const float* temperature,
                       const float* uniform, int* out, int rows, int vocab, int ld) {
    if (rows < 0 || vocab <= 0 || ld < vocab) return CIE_BAD_ARGUMENT;
    if (temperature && (!uniform || (vocab + kChunk - 1) / kChunk > kMaxChunks)) return CIE_BAD_ARGUMENT;
    if (rows == 0) return CIE_OK;
    sample_kernel<<<rows, kThreads, 0, static_cast<hipStream_t>(stream)>>>(logits, temperature, uniform,
                                                                           out, vocab, ld);
    return cie_after_launch();
}
