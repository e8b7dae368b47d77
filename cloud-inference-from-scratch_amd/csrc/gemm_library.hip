// Matrix products with many rows go to the vendor library (hipBLASLt), as the reference leaves its
// products to a library.  This is the thin host side of that: one handle, and for every shape the
// descriptors and the algorithm (the library's heuristic pick, or the fastest of its candidates), kept
// after the first call, so that a
// step's few hundred products cost a table lookup and one launch each instead of a heuristic query.
//
//   C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]),  bf16 operands and bias, float32 sums, bf16 result
//   (or, without bias, a float32 result: the logits)
//
// In the library's column-major terms: D (N x M, ld N) = W^T (W stored K x N, ld K, transposed) *
// A (K x M, ld lda); the bias is added along D's rows (the N dimension).
#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

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

// Descriptors for a shape and the algorithms the library's heuristic proposes, best guess first;
// returns how many fit the workspace (0: the library has none).
int make_plan(Plan& plan, hipblasLtMatmulHeuristicResult_t (&found)[kCandidates], int M, int N, int K, int lda,
              bool has_bias, bool f32_out, size_t workspace_limit) {
    const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
    bool good = ok(hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F)) &&
                ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed))) &&
                ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain))) &&
                ok(hipblasLtMatrixLayoutCreate(&plan.w, HIP_R_16BF, K, N, K)) &&
                ok(hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, K, M, lda)) &&
                ok(hipblasLtMatrixLayoutCreate(&plan.d, f32_out ? HIP_R_32F : HIP_R_16BF, N, M, N));
    if (good && has_bias) {
        const hipblasLtEpilogue_t epilogue = HIPBLASLT_EPILOGUE_BIAS;
        const hipDataType bias_type = HIP_R_16BF;
        good = ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue))) &&
               ok(hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)));
    }
    if (!good) return 0;
    hipblasLtMatmulPreference_t preference = nullptr;
    if (!ok(hipblasLtMatmulPreferenceCreate(&preference))) return 0;
    const uint64_t limit = workspace_limit;
    int count = 0;
    good = ok(hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &limit, sizeof(limit))) &&
           ok(hipblasLtMatmulAlgoGetHeuristic(g_handle, plan.desc, plan.w, plan.a, plan.d, plan.d, preference, kCandidates,
                                              found, &count));
    hipblasLtMatmulPreferenceDestroy(preference);
    if (!good) return 0;
    int kept = 0;
    for (int i = 0; i < count; ++i)
        if (ok(found[i].state) && found[i].workspaceSize <= workspace_limit) found[kept++] = found[i];
    return kept;
}

// Candidates are timed with the weight coming from memory, as it does inside a model's step: over copies
// of the weight that together exceed what the caches hold (the last-level cache is 256 MB), used in turn.
// Timed over one copy that stays in the caches, a short product picks an algorithm of few workgroups that
// is 2.5 times slower than another once its weight has to be streamed.
constexpr size_t kColdBytes = size_t(640) << 20;

// Time the candidates on the call's own rows (the result is overwritten by the real call that follows)
// and return the index of the fastest; 0 if timing is not possible.  A candidate's time is the shortest of
// a few batches of runs; all candidates are timed once, then the four best again with more batches, so
// that a candidate is not chosen or dropped for what else happened while it ran (clocks that had not come
// up yet, a neighbour's work).
struct Timing {
    const Plan& plan;
    const hipblasLtMatmulHeuristicResult_t* found;
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

    bool run(int i) {
        const float one = 1.f, zero = 0.f;
        const void* weight = cold ? cold + w_bytes * (turn++ % copies) : w;
        return ok(hipblasLtMatmul(g_handle, plan.desc, &one, weight, plan.w, a, plan.a, &zero, c, plan.d, c, plan.d,
                                  &found[i].algo, workspace, found[i].workspaceSize, stream));
    }
    // milliseconds of the fastest batch; negative if a call failed
    float time(int i, int batches, int runs) {
        float best = -1.f;
        if (!run(i)) return -1.f;  // warm-up
        for (int b = 0; b < batches; ++b) {
            bool good = hipEventRecord(begin, stream) == hipSuccess;
            for (int r = 0; r < runs && good; ++r) good = run(i);
            float ms = 0.f;
            good = good && hipEventRecord(end, stream) == hipSuccess && hipEventSynchronize(end) == hipSuccess &&
                   hipEventElapsedTime(&ms, begin, end) == hipSuccess;
            if (!good) return -1.f;
            if (best < 0.f || ms < best) best = ms;
        }
        return best;
    }
};

int fastest(const Plan& plan, const hipblasLtMatmulHeuristicResult_t* found, int count, hipStream_t stream,
            const void* a, const void* w, size_t w_bytes, void* c, void* workspace, bool many_rows) {
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
    constexpr int kFinalists = 4;
    int finalist[kCandidates];
    float finalist_ms[kCandidates];
    int finalists = 0;
    for (int i = 0; i < count && i < kCandidates; ++i) {
        const float ms = timing.time(i, 2, runs);
        if (ms < 0.f) continue;
        int at = finalists++;
        for (; at > 0 && finalist_ms[at - 1] > ms; --at) {  // kept in order of time
            finalist[at] = finalist[at - 1];
            finalist_ms[at] = finalist_ms[at - 1];
        }
        finalist[at] = i;
        finalist_ms[at] = ms;
    }
    if (finalists > kFinalists) finalists = kFinalists;
    int best = finalists ? finalist[0] : 0;
    float best_ms = -1.f;
    for (int f = 0; f < finalists; ++f) {
        const float ms = timing.time(finalist[f], 5, runs);
        if (ms >= 0.f && (best_ms < 0.f || ms < best_ms)) {
            best_ms = ms;
            best = finalist[f];
        }
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

// With `tune`, a shape's first call (outside graph capture) times the heuristic's candidates on the call's
// own rows and on copies of its weight (device memory of its own, freed again) and keeps the fastest;
// otherwise the heuristic's first choice is kept.
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
            hipblasLtMatmulHeuristicResult_t found[kCandidates];
            const int count = make_plan(fresh, found, M, N, K, lda, bias != nullptr, f32_out != 0, workspace ? workspace_bytes : 0);
            if (count == 0) {
                destroy(fresh);
                return CIE_BAD_ARGUMENT;
            }
            int chosen = 0;
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            if (tune && count > 1 && hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capturing) == hipSuccess &&
                capturing == hipStreamCaptureStatusNone) {
                if (bias) hipblasLtMatmulDescSetAttribute(fresh.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
                // short products are timed over more runs: their times scatter more
                chosen = fastest(fresh, found, count, static_cast<hipStream_t>(stream), a, w, size_t(N) * K * 2, c, workspace,
                                 M >= 512);
            }
            fresh.algo = found[chosen].algo;
            fresh.workspace = found[chosen].workspaceSize;
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
