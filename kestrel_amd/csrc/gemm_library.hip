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
// A plan (descriptors and the algorithm the library's heuristic names first) is made at the first
// call with a set of sizes and kept. The caller brings the workspace; nothing here allocates
// device memory.
#include "ka_common.h"

#include <hipblaslt/hipblaslt.h>

#include <map>
#include <mutex>
#include <tuple>

namespace {

constexpr int LT_MAX_DEVICES = 64;
constexpr int LT_CANDIDATES = 8;

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, a = nullptr, out = nullptr;
    hipblasLtMatmulAlgo_t algo;
    bool usable = false;
};

using Key = std::tuple<int, int, int, int, long, long, long, int, int, int, int, size_t>;

std::mutex g_lock;
hipblasLtHandle_t g_handle[LT_MAX_DEVICES];
std::map<Key, Plan> g_plans;

bool epilogue_of(int act, bool bias, hipblasLtEpilogue_t* epilogue) {
    switch (act) {
        case KA_ACT_NONE: *epilogue = bias ? HIPBLASLT_EPILOGUE_BIAS : HIPBLASLT_EPILOGUE_DEFAULT; return true;
        case KA_ACT_GELU_TANH: *epilogue = bias ? HIPBLASLT_EPILOGUE_GELU_BIAS : HIPBLASLT_EPILOGUE_GELU; return true;
        case KA_ACT_RELU: *epilogue = bias ? HIPBLASLT_EPILOGUE_RELU_BIAS : HIPBLASLT_EPILOGUE_RELU; return true;
        case KA_ACT_SILU: *epilogue = bias ? HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT : HIPBLASLT_EPILOGUE_SWISH_EXT; return true;
    }
    return false;
}

// The plan for these sizes on this device; made (and the library asked for an algorithm) at the
// first call. `usable` false: the library has no kernel for the case.
const Plan* plan_for(hipblasLtHandle_t handle, const Key& key, int M, int N, int K, long lda, long ldw, long ldo,
                     int out_dtype, int act, bool bias, bool accumulate, size_t workspace_bytes) {
    auto found = g_plans.find(key);
    if (found != g_plans.end()) return &found->second;
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
         hipblasLtMatrixLayoutCreate(&plan.a, HIP_R_16BF, K, M, lda) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatrixLayoutCreate(&plan.out, out_type, N, M, ldo) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        hipblasLtMatmulPreference_t preference = nullptr;
        ok = hipblasLtMatmulPreferenceCreate(&preference) == HIPBLAS_STATUS_SUCCESS;
        if (ok) {
            const uint64_t cap = workspace_bytes;
            hipblasLtMatmulHeuristicResult_t candidates[LT_CANDIDATES];
            int n = 0;
            ok = hipblasLtMatmulPreferenceSetAttribute(preference, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &cap, sizeof(cap)) == HIPBLAS_STATUS_SUCCESS &&
                 hipblasLtMatmulAlgoGetHeuristic(handle, plan.desc, plan.w, plan.a, plan.out, plan.out, preference,
                                                 LT_CANDIDATES, candidates, &n) == HIPBLAS_STATUS_SUCCESS;
            if (ok) {
                for (int i = 0; i < n && !plan.usable; ++i) {
                    if (candidates[i].state != HIPBLAS_STATUS_SUCCESS || candidates[i].workspaceSize > workspace_bytes) continue;
                    plan.algo = candidates[i].algo;
                    plan.usable = true;
                }
            }
            hipblasLtMatmulPreferenceDestroy(preference);
        }
    }
    (void)accumulate;
    return &g_plans.emplace(key, plan).first->second;
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
    KA_CHECK(lda >= K && ldw >= K && ldo >= N, "%s: a row stride is smaller than its row", who);
    KA_CHECK((uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0 && (uintptr_t)out % 16 == 0, "%s: operands must be 16-byte aligned", who);
    KA_CHECK(ka_act_known(act), "%s: unknown activation %d", who, act);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "%s: bad output type", who);
    KA_CHECK(!(accumulate && out_dtype != KA_F32), "%s: accumulate needs an fp32 output", who);
    KA_CHECK(workspace_bytes >= 0 && (workspace || workspace_bytes == 0), "%s: workspace missing", who);
    if (accumulate && act != KA_ACT_NONE) return 1;
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    KA_CHECK(e == hipSuccess && device >= 0 && device < LT_MAX_DEVICES, "%s: no current device within the %d this library keeps a handle for", who, LT_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(g_lock);
    if (!g_handle[device]) {
        hipblasStatus_t s = hipblasLtCreate(&g_handle[device]);
        KA_CHECK(s == HIPBLAS_STATUS_SUCCESS, "%s: hipblasLtCreate failed with status %d", who, (int)s);
    }
    const Key key{device, M, N, K, lda, ldw, ldo, out_dtype, act, bias != nullptr, accumulate != 0, (size_t)workspace_bytes};
    const Plan* plan = plan_for(g_handle[device], key, M, N, K, lda, ldw, ldo, out_dtype, act, bias != nullptr, accumulate != 0,
                                (size_t)workspace_bytes);
    if (!plan->usable) return 1;
    if (bias) {
        hipblasStatus_t s = hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
        KA_CHECK(s == HIPBLAS_STATUS_SUCCESS, "%s: cannot set the bias (status %d)", who, (int)s);
    }
    const float alpha = 1.0f, beta = accumulate ? 1.0f : 0.0f;
    hipblasStatus_t s = hipblasLtMatmul(g_handle[device], plan->desc, &alpha, W, plan->w, A, plan->a, &beta, out, plan->out, out,
                                        plan->out, &plan->algo, workspace, (size_t)workspace_bytes, stream);
    KA_CHECK(s == HIPBLAS_STATUS_SUCCESS, "%s: hipblasLtMatmul failed with status %d (M=%d N=%d K=%d)", who, (int)s, M, N, K);
    return 0;
}
