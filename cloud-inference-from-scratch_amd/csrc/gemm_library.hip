// Matrix products with many rows go to the vendor library (hipBLASLt), as the reference leaves its
// products to a library.  This is the thin host side of that: one handle, and for every shape the
// descriptors and the algorithm, kept after the first call, so that a step's few hundred products cost a
// table lookup and one launch each instead of a heuristic query.  The algorithm is the library's heuristic
// pick, the fastest of the heuristic's candidates, or the fastest of every algorithm the library has for
// the shape (a few hundred to two thousand for bf16, by the version of the library that the process has
// loaded; with 2,048 rows and a wide result the best of them is 14 to 18 % faster than the best the
// heuristic proposes, for up to a few seconds at the shape's first call).
//
//   C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]),  bf16 operands and bias, float32 sums, bf16 result
//   (or, without bias, a float32 result: the logits)
//
// In the library's column-major terms: D (N x M, ld N) = W^T (W stored K x N, ld K, transposed) *
// A (K x M, ld lda); the bias is added along D's rows (the N dimension).
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"

namespace {

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, a = nullptr, d = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
};

using Key = std::tuple<int, int, int, int, int, int>;  // M, N, K, lda, has bias, float32 result

hipblasLtHandle_t g_handle = nullptr;
std::map<Key, Plan> g_plans;
std::mutex g_mutex;

bool ok(hipblasStatus_t status) { return status == HIPBLAS_STATUS_SUCCESS; }

void destroy(Plan& plan) {
    if (plan.d) hipblasLtMatrixLayoutDestroy(plan.d);
    if (plan.a) hipblasLtMatrixLayoutDestroy(plan.a);
    if (plan.w) hipblasLtMatrixLayoutDestroy(plan.w);
    if (plan.desc) hipblasLtMatmulDescDestroy(plan.desc);
    plan = Plan{};
}

constexpr int kCandidates = 16;
using Found = std::vector<hipblasLtMatmulHeuristicResult_t>;

// Descriptors for a shape and the algorithms to choose from: those the library's heuristic proposes, best
// guess first, and after them, if `every`, all others the library says it can run on this shape.  Returns
// how many of the heuristic's fit the workspace (0: the library has none; `found` may then hold nothing).
int make_plan(Plan& plan, Found& found, int M, int N, int K, int lda, const void* bias, bool f32_out,
              size_t workspace_limit, bool every) {
    const bool has_bias = bias != nullptr;
    const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
    const hipDataType result_type = f32_out ? HIP_R_32F : HIP_R_16BF;
    bool good = ok(hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F)) &&
                ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed))) &&
                ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain))) &&
                ok(hipblasLtMatrixLayoutCreate(&plan.w, HIP_R_16BF, K, N, K)) &&
                ok(hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, K, M, lda)) &&
                ok(hipblasLtMatrixLayoutCreate(&plan.d, result_type, N, M, N));
    if (good && has_bias) {
        const hipblasLtEpilogue_t epilogue = HIPBLASLT_EPILOGUE_BIAS;
        const hipDataType bias_type = HIP_R_16BF;
        // (the pointer too: asked whether it can run an algorithm on a product with a bias and no pointer to it, the
        // library answers "invalid value", and a search over all its algorithms finds none; every call sets its
        // own pointer again)
        good = ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue))) &&
               ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type))) &&
               ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias)));
    }
    if (!good) return 0;
    hipblasLtMatmulPreference_t preference = nullptr;
    if (!ok(hipblasLtMatmulPreferenceCreate(&preference))) return 0;
    const uint64_t limit = workspace_limit;
    int count = 0;
    hipblasLtMatmulHeuristicResult_t proposed[kCandidates];
    good = ok(hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit))) &&
           ok(hipblasLtMatmulAlgoGetHeuristic(g_handle, plan.desc, plan.w, plan.a, plan.d, plan.d, preference, kCandidates,
                                              proposed, &count));
    hipblasLtMatmulPreferenceDestroy(preference);
    if (!good) return 0;
    found.clear();
    for (int i = 0; i < count; ++i)
        if (ok(proposed[i].state) && proposed[i].workspaceSize <= workspace_limit) found.push_back(proposed[i]);
    const int kept = static_cast<int>(found.size());
    if (kept == 0 || !every) return kept;
    Found all;
    if (!ok(hipblaslt_ext::getAllAlgos(g_handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, transposed, plain, HIP_R_16BF,
                                       HIP_R_16BF, result_type, result_type, HIPBLAS_COMPUTE_32F, all)))
        return kept;
    const float one = 1.f, zero = 0.f;
    for (auto& candidate : all) {
        size_t needs = 0;
        if (!ok(hipblaslt_ext::matmulIsAlgoSupported(g_handle, plan.desc, &one, plan.w, plan.a, &zero, plan.d, plan.d,
                                                     candidate.algo, needs)) ||
            needs > workspace_limit)
            continue;
        candidate.workspaceSize = needs;
        found.push_back(candidate);
    }
    return kept;
}

// Candidates are timed with the weight coming from memory, as it does inside a model's step: over copies
// of the weight that together exceed what the caches hold (the last-level cache is 256 MB), used in turn.
// Timed over one copy that stays in the caches, a short product picks an algorithm of few workgroups that
// is 2.5 times slower than another once its weight has to be streamed.
constexpr size_t kColdBytes = size_t(640) << 20;

// Two results compared element by element.  First the largest |x| (as the bits of a non-negative float, which
// order as unsigned integers do); then the number of elements with |x - y| > rel * |x| + abs_of_size * that
// largest |x|, a NaN on either side counting as one.
__device__ inline float as_float(float v) { return v; }
__device__ inline float as_float(unsigned short bf16_bits) { return __uint_as_float(unsigned(bf16_bits) << 16); }

template <typename T>
__global__ void results_size_kernel(const T* __restrict__ x, size_t count, unsigned* __restrict__ out) {
    float size = 0.f;
    for (size_t i = blockIdx.x * size_t(blockDim.x) + threadIdx.x; i < count; i += size_t(gridDim.x) * blockDim.x)
        size = fmaxf(size, fabsf(as_float(x[i])));
    atomicMax(out + 1, __float_as_uint(size));
}

template <typename T>
__global__ void results_differ_kernel(const T* __restrict__ x, const T* __restrict__ y, size_t count, float rel,
                                      float abs_of_size, unsigned* __restrict__ out) {
    const float floor = abs_of_size * __uint_as_float(out[1]);
    unsigned wrong = 0;
    for (size_t i = blockIdx.x * size_t(blockDim.x) + threadIdx.x; i < count; i += size_t(gridDim.x) * blockDim.x) {
        const float a = as_float(x[i]), b = as_float(y[i]);
        const float d = fabsf(a - b);
        if (!(d <= rel * fabsf(a) + floor)) ++wrong;  // (a NaN fails every comparison)
    }
    if (wrong) atomicAdd(out, wrong);
}

// Time the candidates on the call's own rows (the result is overwritten by the real call that follows)
// and return the index of the fastest; 0 if timing is not possible.  A candidate's time is the shortest of
// a few batches of runs; all candidates are timed once, then the best few again with more batches, taken in
// turn, so that a candidate is not chosen or dropped for what else happened while it ran (clocks that had
// not come up yet, a neighbour's work).  A winner that the heuristic did not propose is kept only if its
// result agrees with that of the heuristic's first choice.
struct Timing {
    const Plan& plan;
    const Found& found;
    hipStream_t stream;
    const void* a;
    const char* w;
    const char* cold;  // copies of w, or null
    size_t w_bytes;
    int copies;
    void* c;
    void* workspace;
    hipEvent_t begin, end;
    int turn = 0;

    bool run(int i, void* into = nullptr, bool first_copy = false) {
        const float one = 1.f, zero = 0.f;
        const void* weight = cold && !first_copy ? cold + w_bytes * (turn++ % copies) : w;
        void* result = into ? into : c;
        return ok(hipblasLtMatmul(g_handle, plan.desc, &one, weight, plan.w, a, plan.a, &zero, result, plan.d, result,
                                  plan.d, &found[i].algo, workspace, found[i].workspaceSize, stream));
    }
    // milliseconds of the fastest batch; negative if a call failed
    float time(int i, int batches, int runs, bool warm = true) {
        float best = -1.f;
        if (warm && !run(i)) return -1.f;
        for (int b = 0; b < batches; ++b) {
            bool good = hipEventRecord(begin, stream) == hipSuccess;
            for (int r = 0; r < runs && good; ++r) good = run(i);
            float ms = 0.f;
            good = good && hipEventRecord(end, stream) == hipSuccess && hipEventSynchronize(end) == hipSuccess &&
                   hipEventElapsedTime(&ms, begin, end) == hipSuccess;
            if (!good) {
                (void)hipGetLastError();
                return -1.f;
            }
            if (best < 0.f || ms < best) best = ms;
        }
        return best;
    }
};

// Does candidate `i` give what candidate 0 gives (to the rounding of the result type and of another order
// of sums)?  False also if that cannot be found out.
bool agrees_with_first(Timing& timing, int i, size_t elements, bool f32_out) {
    const size_t bytes = elements * (f32_out ? 4 : 2);
    char* other = nullptr;
    if (hipMalloc(reinterpret_cast<void**>(&other), bytes + 256) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    unsigned* outcome = reinterpret_cast<unsigned*>(other + (bytes + 7) / 8 * 8);
    bool good = hipMemsetAsync(outcome, 0, 8, timing.stream) == hipSuccess && timing.run(0, nullptr, true) &&
                timing.run(i, other, true);
    if (good) {
        // bf16 results: two roundings of the same sum lie an ulp (2^-8 of the value) apart, sums in another
        // order a little more where terms cancel; float32 results differ by the order of the sums only
        const int blocks = 1024, threads = 256;
        if (f32_out) {
            const float* mine = static_cast<const float*>(timing.c);
            results_size_kernel<float><<<blocks, threads, 0, timing.stream>>>(mine, elements, outcome);
            results_differ_kernel<float><<<blocks, threads, 0, timing.stream>>>(
                mine, reinterpret_cast<const float*>(other), elements, 1.f / 1024.f, 1.f / 4096.f, outcome);
        } else {
            const unsigned short* mine = static_cast<const unsigned short*>(timing.c);
            results_size_kernel<unsigned short><<<blocks, threads, 0, timing.stream>>>(mine, elements, outcome);
            results_differ_kernel<unsigned short><<<blocks, threads, 0, timing.stream>>>(
                mine, reinterpret_cast<const unsigned short*>(other), elements, 1.f / 64.f, 1.f / 256.f, outcome);
        }
        good = hipGetLastError() == hipSuccess;
    }
    unsigned bits[2] = {0, 0};
    good = good && hipMemcpyAsync(bits, outcome, 8, hipMemcpyDeviceToHost, timing.stream) == hipSuccess &&
           hipStreamSynchronize(timing.stream) == hipSuccess;
    hipStreamSynchronize(timing.stream);
    hipFree(other);
    if (!good) {
        (void)hipGetLastError();
        return false;
    }
    return bits[0] == 0;  // no element apart
}

int fastest(const Plan& plan, const Found& found, int proposed, hipStream_t stream, const void* a, const void* w,
            size_t w_bytes, void* c, void* workspace, bool many_rows, size_t elements, bool f32_out) {
    hipEvent_t begin = nullptr, end = nullptr;
    if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess) return 0;
    int copies = static_cast<int>((kColdBytes + w_bytes - 1) / w_bytes);
    copies = copies < 2 ? 2 : copies > 64 ? 64 : copies;
    char* cold = nullptr;
    if (hipMalloc(reinterpret_cast<void**>(&cold), w_bytes * copies) != hipSuccess) {
        (void)hipGetLastError();
        cold = nullptr;
    }
    for (int i = 0; cold && i < copies; ++i)
        if (hipMemcpyAsync(cold + w_bytes * i, w, w_bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess) {
            (void)hipGetLastError();
            hipStreamSynchronize(stream);
            hipFree(cold);
            cold = nullptr;
        }
    Timing timing{plan, found, stream, a, static_cast<const char*>(w), cold, w_bytes, copies, c, workspace, begin, end};
    // short products scatter more: more runs in a batch
    const int runs = many_rows ? 2 : 6;
    const int count = static_cast<int>(found.size());
    const bool every = count > proposed;
    // rounds: everything once; the best 32 of a long list twice more, in turn; the best eight five times; the
    // best three twelve times
    constexpr int kMost = 32;
    const int wanted = every ? kMost : 4;
    int finalist[kMost + 1];
    float finalist_ms[kMost + 1];
    int finalists = 0;
    for (int i = 0; i < count; ++i) {
        const float ms = timing.time(i, i < proposed ? 2 : 1, runs);
        if (ms < 0.f) continue;
        if (finalists == wanted && ms >= finalist_ms[finalists - 1]) continue;
        int at = finalists < wanted ? finalists++ : finalists - 1;
        for (; at > 0 && finalist_ms[at - 1] > ms; --at) {  // kept in order of time
            finalist[at] = finalist[at - 1];
            finalist_ms[at] = finalist_ms[at - 1];
        }
        finalist[at] = i;
        finalist_ms[at] = ms;
    }
    auto again = [&](int rounds) {
        for (int f = 0; f < finalists; ++f) finalist_ms[f] = -1.f;
        for (int round = 0; round < rounds; ++round)
            for (int f = 0; f < finalists; ++f) {
                const float ms = timing.time(finalist[f], 1, runs, round == 0);
                if (ms >= 0.f && (finalist_ms[f] < 0.f || ms < finalist_ms[f])) finalist_ms[f] = ms;
            }
        for (int f = 1; f < finalists; ++f) {  // in order of time again; failed ones last
            const int index = finalist[f];
            const float ms = finalist_ms[f];
            int at = f;
            for (; at > 0 && (finalist_ms[at - 1] < 0.f || (ms >= 0.f && finalist_ms[at - 1] > ms)); --at) {
                finalist[at] = finalist[at - 1];
                finalist_ms[at] = finalist_ms[at - 1];
            }
            finalist[at] = index;
            finalist_ms[at] = ms;
        }
    };
    if (finalists > 8) {
        again(2);
        finalists = 8;
    }
    again(5);
    if (finalists > 3) {  // the last few once more, longer: candidates within a few percent of each other change places
        finalists = 3;
        again(12);
    }
    int best = 0;
    for (;;) {
        int at = -1;
        for (int f = 0; f < finalists; ++f)
            if (finalist_ms[f] >= 0.f && (at < 0 || finalist_ms[f] < finalist_ms[at])) at = f;
        if (at < 0) break;  // none left: the heuristic's first choice
        if (finalist[at] < proposed || agrees_with_first(timing, finalist[at], elements, f32_out)) {
            best = finalist[at];
            break;
        }
        finalist_ms[at] = -1.f;
    }
    hipEventDestroy(begin);
    hipEventDestroy(end);
    if (cold) {
        hipStreamSynchronize(stream);
        hipFree(cold);
    }
    return best;
}

}  // namespace

// With `tune` 1, a shape's first call (outside graph capture) times the heuristic's candidates on the call's
// own rows and on copies of its weight (device memory of its own, freed again) and keeps the fastest; with
// `tune` 2 it times every algorithm the library can run on the shape (a few seconds); with 0 the heuristic's
// first choice is kept.
// Returns CIE_BAD_ARGUMENT for a shape the library has no algorithm for (the caller then takes another
// route) and CIE_LAUNCH_FAILED if the library's call itself fails.  `workspace` is device memory of
// `workspace_bytes` that stays valid while the product runs; calls on one stream may share it.
CIE_API int cie_gemm_library(void* stream, const void* a, int lda, const void* w, const void* bias, void* c, int M,
                             int N, int K, int f32_out, void* workspace, size_t workspace_bytes, int tune) {
    if (M <= 0 || N <= 0 || K <= 0 || lda < K || !a || !w || !c || (f32_out && bias)) return CIE_BAD_ARGUMENT;
    Plan* plan = nullptr;
    {
        std::lock_guard<std::mutex> guard(g_mutex);
        if (!g_handle && !ok(hipblasLtCreate(&g_handle))) return CIE_LAUNCH_FAILED;
        const Key key{M, N, K, lda, bias ? 1 : 0, f32_out ? 1 : 0};
        auto it = g_plans.find(key);
        if (it == g_plans.end()) {
            Plan fresh;
            Found found;
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            const bool may_time = tune && hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capturing) == hipSuccess &&
                                  capturing == hipStreamCaptureStatusNone;
            const int proposed = make_plan(fresh, found, M, N, K, lda, bias, f32_out != 0,
                                           workspace ? workspace_bytes : 0, may_time && tune >= 2);
            if (proposed == 0) {
                destroy(fresh);
                return CIE_BAD_ARGUMENT;
            }
            int chosen = 0;
            if (may_time && found.size() > 1) {
                // short products are timed over more runs: their times scatter more
                chosen = fastest(fresh, found, proposed, static_cast<hipStream_t>(stream), a, w, size_t(N) * K * 2, c,
                                 workspace, M >= 512, size_t(M) * N, f32_out != 0);
            }
            fresh.algo = found[chosen].algo;
            fresh.workspace = found[chosen].workspaceSize;
            if (getenv("CIE_LIBRARY_REPORT"))  // which algorithm a shape got, for whoever reads a profile
                fprintf(stderr, "[cie_amd library] %d x %d x %d: candidate %d of %zu (%d proposed): %s\n", M, N, K, chosen,
                        found.size(), proposed, hipblaslt_ext::getKernelNameFromAlgo(g_handle, fresh.algo).c_str());
            it = g_plans.emplace(key, fresh).first;
        }
        plan = &it->second;
    }
    if (bias &&
        !ok(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias))))
        return CIE_LAUNCH_FAILED;
    const float one = 1.f, zero = 0.f;
    const hipblasStatus_t status =
        hipblasLtMatmul(g_handle, plan->desc, &one, w, plan->w, a, plan->a, &zero, c, plan->d, c, plan->d, &plan->algo,
                        workspace, plan->workspace, static_cast<hipStream_t>(stream));
    return ok(status) ? CIE_OK : CIE_LAUNCH_FAILED;
}
