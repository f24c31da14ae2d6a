// Matrix products of many rows through the vendor library (hipBLASLt): out = act(A W^T + bias), or
// out += A W^T + bias into an fp32 output, for bf16 A [M, K] and W [N, K].
//
// The kernels of this folder take every linear layer; this file hands those of a prompt (hundreds
// to thousands of rows) to the library where the library has a kernel for the case, because its
// kernels are faster there (measured at 2,048 rows of Moondream 2's four linears: 202 us against
// 249 us a layer). Bias, activation and the sum into the residual stay inside the product: they
// are the library's epilogues, not passes of their own.
//
// Row-major out [M, N] is the library's column-major D [N, M] = W (stored as column-major [K, N],
// transposed) x A (column-major [K, M]); the bias runs along D's rows.
//
// Plans. Asking the library's heuristic for an algorithm is the expensive part of a first call
// (hundreds of microseconds to milliseconds on the host), and under continuous batching the number
// of rows changes with almost every step. So the heuristic is asked once per bucket of rows (M
// rounded up to a multiple of 64, of 256 beyond 4,096 rows) at the bucket's upper edge, and that
// algorithm serves every row count of the bucket: a plan keeps the descriptors, whose row count is
// set per call, and the algorithm. Should the library refuse the bucket's algorithm for a row
// count, the heuristic is asked for exactly that count and the answer kept under its own key.
// The plans live in a map bounded at LT_MAX_PLANS; the one used longest ago makes room.
// The caller brings the workspace; nothing here allocates device memory.
#include "ka_common.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

namespace {

constexpr int LT_MAX_DEVICES = 64;
constexpr int LT_CANDIDATES = 8;
constexpr size_t LT_MAX_PLANS = 512;

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, a = nullptr, out = nullptr;
    hipblasLtMatmulAlgo_t algo;
    bool usable = false;
    bool every_count = true;       // false once the library has refused the algorithm for a row count of the bucket
    std::vector<hipblasLtMatmulAlgo_t> candidates;     // what the heuristic named, until the plan has been tuned
    int rows_set = 0;              // the row count the layouts of a and out stand at
    unsigned long used = 0;        // the call that used the plan last
};

// device, rows (a bucket's upper edge, or minus an exact count), N, K, lda, ldw, ldo, output type, activation,
// bias, accumulate, workspace
using Key = std::tuple<int, int, int, int, long, long, long, int, int, int, int, size_t>;

std::mutex g_lock;
hipblasLtHandle_t g_handle[LT_MAX_DEVICES];
std::map<Key, Plan> g_plans;
unsigned long g_calls = 0, g_heuristic_calls = 0, g_evicted = 0, g_tuned = 0, g_tuned_other = 0;
int g_tune_runs = 0;               // > 0: a new plan times the heuristic's candidates on its first call (ka_linear_library_set_tuning)

bool epilogue_of(int act, bool bias, hipblasLtEpilogue_t* epilogue) {
    switch (act) {
        case KA_ACT_NONE: *epilogue = bias ? HIPBLASLT_EPILOGUE_BIAS : HIPBLASLT_EPILOGUE_DEFAULT; return true;
        case KA_ACT_GELU_TANH: *epilogue = bias ? HIPBLASLT_EPILOGUE_GELU_BIAS : HIPBLASLT_EPILOGUE_GELU; return true;
        case KA_ACT_RELU: *epilogue = bias ? HIPBLASLT_EPILOGUE_RELU_BIAS : HIPBLASLT_EPILOGUE_RELU; return true;
        case KA_ACT_SILU: *epilogue = bias ? HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT : HIPBLASLT_EPILOGUE_SWISH_EXT; return true;
    }
    return false;
}

int rows_bucket(int M) {
    const int step = M > 4096 ? 256 : 64;
    return (M + step - 1) / step * step;
}

void destroy(Plan& plan) {
    if (plan.w) hipblasLtMatrixLayoutDestroy(plan.w);
    if (plan.a) hipblasLtMatrixLayoutDestroy(plan.a);
    if (plan.out) hipblasLtMatrixLayoutDestroy(plan.out);
    if (plan.desc) hipblasLtMatmulDescDestroy(plan.desc);
    plan = Plan{};
}

// Room for one more plan: the one used longest ago goes (a linear scan over at most LT_MAX_PLANS
// entries, once per new plan beyond the bound).
void make_room() {
    while (g_plans.size() >= LT_MAX_PLANS) {
        auto oldest = g_plans.begin();
        for (auto it = g_plans.begin(); it != g_plans.end(); ++it)
            if (it->second.used < oldest->second.used) oldest = it;
        destroy(oldest->second);
        g_plans.erase(oldest);
        ++g_evicted;
    }
}

// Descriptors for `rows` rows and the algorithm the library's heuristic names first for them.
// `usable` false: the library has no kernel for the case.
Plan make_plan(hipblasLtHandle_t handle, int rows, int N, int K, long lda, long ldw, long ldo, int out_dtype, int act,
               bool bias, size_t workspace_bytes) {
    Plan plan;
    hipblasLtEpilogue_t epilogue;
    const hipDataType out_type = out_dtype == KA_F32 ? HIP_R_32F : HIP_R_16BF;
    bool ok = epilogue_of(act, bias, &epilogue);
    ok = ok && hipblasLtMatmulDescCreate(&plan.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        const hipblasOperation_t transposed = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
        const hipDataType bias_type = HIP_R_32F;
        ok = hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &transposed, sizeof(transposed)) == HIPBLAS_STATUS_SUCCESS &&
             hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain)) == HIPBLAS_STATUS_SUCCESS &&
             hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue)) == HIPBLAS_STATUS_SUCCESS;
        if (ok && bias)
            ok = hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)) == HIPBLAS_STATUS_SUCCESS;
    }
    ok = ok && hipblasLtMatrixLayoutCreate(&plan.w, HIP_R_16BF, K, N, ldw) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, K, rows, lda) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatrixLayoutCreate(&plan.out, out_type, N, rows, ldo) == HIPBLAS_STATUS_SUCCESS;
    plan.rows_set = rows;
    if (ok) {
        hipblasLtMatmulPreference_t preference = nullptr;
        ok = hipblasLtMatmulPreferenceCreate(&preference) == HIPBLAS_STATUS_SUCCESS;
        if (ok) {
            const uint64_t cap = workspace_bytes;
            hipblasLtMatmulHeuristicResult_t candidates[LT_CANDIDATES];
            int n = 0;
            ++g_heuristic_calls;
            ok = hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &cap, sizeof(cap)) == HIPBLAS_STATUS_SUCCESS &&
                 hipblasLtMatmulAlgoGetHeuristic(handle, plan.desc, plan.w, plan.a, plan.out, plan.out, preference,
                                                 LT_CANDIDATES, candidates, &n) == HIPBLAS_STATUS_SUCCESS;
            if (ok) {
                for (int i = 0; i < n; ++i) {
                    if (candidates[i].state != HIPBLAS_STATUS_SUCCESS || candidates[i].workspaceSize > workspace_bytes) continue;
                    if (!plan.usable) plan.algo = candidates[i].algo;
                    plan.usable = true;
                    plan.candidates.push_back(candidates[i].algo);
                }
            }
            hipblasLtMatmulPreferenceDestroy(preference);
        }
    }
    return plan;
}

Plan* plan_for(hipblasLtHandle_t handle, const Key& key, int rows, int N, int K, long lda, long ldw, long ldo,
               int out_dtype, int act, bool bias, size_t workspace_bytes) {
    auto found = g_plans.find(key);
    if (found == g_plans.end()) {
        make_room();
        found = g_plans.emplace(key, make_plan(handle, rows, N, K, lda, ldw, ldo, out_dtype, act, bias, workspace_bytes)).first;
    }
    found->second.used = ++g_calls;
    return &found->second;
}

// Times every algorithm the heuristic named for this plan on the operands of the call at hand and keeps the
// fastest (the first named is the fastest at most sizes, but not at all: q|k|v of 2048 x 6144 at 1,318 rows
// 34.6 against 42.7 us). Only while tuning is switched on, which the engine does during its warm-up: the
// products are run several times over (a sum into the output is added several times), so the operands must
// be ones whose content nobody needs, and the stream must not be capturing. The stream is waited for.
void tune(hipblasLtHandle_t handle, Plan* plan, const float* alpha, const float* beta, const void* W, const void* A, void* out,
          void* workspace, size_t workspace_bytes, hipStream_t stream) {
    std::vector<hipblasLtMatmulAlgo_t> candidates;
    candidates.swap(plan->candidates);                  // (whatever happens, the plan is not tuned twice)
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (candidates.size() < 2 || hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) return;
    hipEvent_t start = nullptr, stop = nullptr;
    if (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess) {
        if (start) hipEventDestroy(start);
        return;
    }
    float best = 0.f;
    int best_index = -1;
    for (size_t i = 0; i < candidates.size(); ++i) {
        auto run = [&]() {
            return hipblasLtMatmul(handle, plan->desc, alpha, W, plan->w, A, plan->a, beta, out, plan->out, out, plan->out,
                                   &candidates[i], workspace, workspace_bytes, stream) == HIPBLAS_STATUS_SUCCESS;
        };
        if (!run()) continue;                           // (once untimed: the kernel's code is loaded)
        bool ok = hipEventRecord(start, stream) == hipSuccess;
        for (int r = 0; r < g_tune_runs && ok; ++r) ok = run();
        float ms = 0.f;
        ok = ok && hipEventRecord(stop, stream) == hipSuccess && hipEventSynchronize(stop) == hipSuccess &&
             hipEventElapsedTime(&ms, start, stop) == hipSuccess;
        if (ok && (best_index < 0 || ms < best)) {
            best = ms;
            best_index = (int)i;
        }
    }
    hipEventDestroy(start);
    hipEventDestroy(stop);
    if (best_index >= 0) {
        plan->algo = candidates[best_index];
        ++g_tuned;
        if (best_index > 0) ++g_tuned_other;
    }
}

// The layouts of a plan's A and out at M rows (they are made at the bucket's edge).
bool set_rows(Plan* plan, int M) {
    if (plan->rows_set == M) return true;
    const uint64_t cols = (uint64_t)M;
    if (hipblasLtMatrixLayoutSetAttribute(plan->a, HIPBLASLT_MATRIX_LAYOUT_COLS, &cols, sizeof(cols)) != HIPBLAS_STATUS_SUCCESS ||
        hipblasLtMatrixLayoutSetAttribute(plan->out, HIPBLASLT_MATRIX_LAYOUT_COLS, &cols, sizeof(cols)) != HIPBLAS_STATUS_SUCCESS)
        return false;
    plan->rows_set = M;
    return true;
}

}  // namespace

// 0: done. 1: the library has no kernel for the case (nothing was run; the caller takes its own).
// Negative: an error (ka_last_error). `workspace`: device memory of the caller's that calls on one
// device share; calls that overlap on a device must not share it.
KA_API int ka_linear_library_bf16(const void* A, long lda, const void* W, long ldw, const float* bias, void* out,
                                  int out_dtype, long ldo, int M, int N, int K, int act, int accumulate,
                                  void* workspace, long workspace_bytes, hipStream_t stream) {
    const char* who = "ka_linear_library_bf16";
    KA_CHECK(M > 0 && N > 0 && K > 0, "%s: M=%d N=%d K=%d", who, M, N, K);
    KA_CHECK(lda >= K && ldw >= K && ldo >= ka_act_outputs(act, N), "%s: a row stride is smaller than its row", who);
    KA_CHECK((uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0 && (uintptr_t)out % 16 == 0, "%s: operands must be 16-byte aligned", who);
    KA_CHECK(ka_act_known(act), "%s: unknown activation %d", who, act);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "%s: bad output type", who);
    KA_CHECK(!(accumulate && out_dtype != KA_F32), "%s: accumulate needs an fp32 output", who);
    KA_CHECK(workspace_bytes >= 0 && (workspace || workspace_bytes == 0), "%s: workspace missing", who);
    if (accumulate && act != KA_ACT_NONE) return 1;
    if (ka_act_gated(act)) return 1;              // (the library has no epilogue that multiplies neighbouring columns)
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    KA_CHECK(e == hipSuccess && device >= 0 && device < LT_MAX_DEVICES, "%s: no current device within the %d this library keeps a handle for", who, LT_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(g_lock);
    if (!g_handle[device]) {
        hipblasStatus_t s = hipblasLtCreate(&g_handle[device]);
        KA_CHECK(s == HIPBLAS_STATUS_SUCCESS, "%s: hipblasLtCreate failed with status %d", who, (int)s);
    }
    const float alpha = 1.0f, beta = accumulate ? 1.0f : 0.0f;
    // first the plan of the bucket of rows, then (if the library refuses its algorithm for this row
    // count) a plan for exactly these rows
    for (int attempt = 0; attempt < 2; ++attempt) {
        const int rows = attempt == 0 ? rows_bucket(M) : M;
        const Key key{device, attempt == 0 ? rows : -M, N, K, lda, ldw, ldo, out_dtype, act, bias != nullptr, accumulate != 0,
                      (size_t)workspace_bytes};
        Plan* plan = plan_for(g_handle[device], key, rows, N, K, lda, ldw, ldo, out_dtype, act, bias != nullptr,
                              (size_t)workspace_bytes);
        if (!plan->usable) {
            if (attempt == 0 && rows != M) continue;
            return 1;
        }
        if (rows != M && !plan->every_count) continue;
        if (!set_rows(plan, M)) continue;
        if (bias) {
            hipblasStatus_t s = hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
            KA_CHECK(s == HIPBLAS_STATUS_SUCCESS, "%s: cannot set the bias (status %d)", who, (int)s);
        }
        if (g_tune_runs > 0 && !plan->candidates.empty())
            tune(g_handle[device], plan, &alpha, &beta, W, A, out, workspace, (size_t)workspace_bytes, stream);
        hipblasStatus_t s = hipblasLtMatmul(g_handle[device], plan->desc, &alpha, W, plan->w, A, plan->a, &beta, out, plan->out,
                                            out, plan->out, &plan->algo, workspace, (size_t)workspace_bytes, stream);
        if (s == HIPBLAS_STATUS_SUCCESS) return 0;
        if (attempt == 0 && rows != M) {
            plan->every_count = false;
            continue;
        }
        KA_CHECK(false, "%s: hipblasLtMatmul failed with status %d (M=%d N=%d K=%d)", who, (int)s, M, N, K);
    }
    return 1;
}

// For measurements and tests: how many plans are kept, how often the heuristic was asked, how many
// plans had to make room, how many were tuned and how many of those took another algorithm than the first named.
KA_API void ka_linear_library_stats(long* plans, long* heuristic_calls, long* evicted, long* tuned, long* tuned_other) {
    std::lock_guard<std::mutex> hold(g_lock);
    if (plans) *plans = (long)g_plans.size();
    if (heuristic_calls) *heuristic_calls = (long)g_heuristic_calls;
    if (evicted) *evicted = (long)g_evicted;
    if (tuned) *tuned = (long)g_tuned;
    if (tuned_other) *tuned_other = (long)g_tuned_other;
}

// `runs` > 0: from now on a plan's first call times the algorithms the heuristic named, `runs` products each, on
// that call's operands and keeps the fastest (see `tune`: only for operands whose content nobody needs: a
// warm-up). 0: plans take the first algorithm named (the default).
KA_API void ka_linear_library_set_tuning(int runs) {
    std::lock_guard<std::mutex> hold(g_lock);
    g_tune_runs = runs > 0 ? runs : 0;
}
