// bfloat16 products of many rows through hipBLASLt, as the reference sends them to cuBLASLt
// (crates/infer-backend-cuda/src/kernels/matmul/mod.rs:187-221).
//
//   C[M, N] = A[M, K] . W[N, K]^T      row-major, bfloat16 in, 32-bit accumulation, bfloat16 or float32 out
//
// In the library's column-major terms that is C^T[N, M] = W^T-stored[K, N]^T . A^T-stored[K, M]:
// transA = T on the weights, transB = N on the activations, m = N, n = M, k = K.
// What costs time on the host is asking the library which kernel to use; the answer (descriptor,
// layouts, algorithm) is kept per shape, so a repeated shape costs one hipblasLtMatmul call.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <mutex>
#include <unordered_map>

namespace {

struct Plan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
};

struct Key {
    int M, N, K, lda, ldw, ldc, out_f32;
    size_t ws;
    bool operator==(const Key& o) const {
        return M == o.M && N == o.N && K == o.K && lda == o.lda && ldw == o.ldw && ldc == o.ldc && out_f32 == o.out_f32 && ws == o.ws;
    }
};
struct KeyHash {
    size_t operator()(const Key& k) const {
        size_t h = 1469598103934665603ull;
        for (long long v : {(long long)k.M, (long long)k.N, (long long)k.K, (long long)k.lda, (long long)k.ldw,
                            (long long)k.ldc, (long long)k.out_f32, (long long)k.ws})
            h = (h ^ (size_t)v) * 1099511628211ull;
        return h;
    }
};

std::mutex g_mutex;
hipblasLtHandle_t g_handle = nullptr;
std::unordered_map<Key, Plan, KeyHash> g_plans;

#define RI_LT(call, what) do { hipblasStatus_t st_ = (call); \
    if (st_ != HIPBLAS_STATUS_SUCCESS) return ri_fail("ri_gemm_library: %s failed with status %d", what, (int)st_); } while (0)

int make_plan(const Key& k, Plan& p) {
    const hipblasOperation_t opT = HIPBLAS_OP_T, opN = HIPBLAS_OP_N;
    RI_LT(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
    RI_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opT, sizeof(opT)), "set transA");
    RI_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opN, sizeof(opN)), "set transB");
    // stored shapes (column-major): weights K x N, activations K x M, result N x M
    RI_LT(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, k.K, k.N, k.ldw), "layout of the weights");
    RI_LT(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, k.K, k.M, k.lda), "layout of the activations");
    RI_LT(hipblasLtMatrixLayoutCreate(&p.c, k.out_f32 ? HIP_R_32F : HIP_R_16BF, k.N, k.M, k.ldc), "layout of the result");
    hipblasLtMatmulPreference_t pref = nullptr;
    RI_LT(hipblasLtMatmulPreferenceCreate(&pref), "hipblasLtMatmulPreferenceCreate");
    hipblasStatus_t st = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &k.ws, sizeof(k.ws));
    hipblasLtMatmulHeuristicResult_t found;
    int n = 0;
    if (st == HIPBLAS_STATUS_SUCCESS)
        st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, p.b, p.c, p.c, pref, 1, &found, &n);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || n < 1)
        return ri_fail("ri_gemm_library: the library offers no kernel for M=%d N=%d K=%d (status %d)", k.M, k.N, k.K, (int)st);
    p.algo = found.algo;
    p.workspace = found.workspaceSize;
    return 0;
}

}  // namespace

// workspace: device memory the library may use (split products); the same size must be passed
// for a shape each time.  Returns 0, or non-zero with a message in ri_last_error().
// out_f32 != 0: C is float32 (logits), else bfloat16.
extern "C" int ri_gemm_library_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc,
                                    int M, int N, int K, int out_f32, void* workspace, size_t workspace_bytes,
                                    hipStream_t stream) {
    RI_REQUIRE(M > 0 && N > 0 && K > 0 && lda >= K && ldw >= K && ldc >= N, "ri_gemm_library: bad sizes M=%d N=%d K=%d", M, N, K);
    RI_REQUIRE(A && W && C && (workspace || workspace_bytes == 0), "ri_gemm_library: null pointer");
    const Plan* plan = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        if (!g_handle) RI_LT(hipblasLtCreate(&g_handle), "hipblasLtCreate");
        const Key key{M, N, K, lda, ldw, ldc, out_f32 ? 1 : 0, workspace_bytes};
        auto it = g_plans.find(key);
        if (it == g_plans.end()) {
            Plan p;
            if (int rc = make_plan(key, p)) return rc;
            it = g_plans.emplace(key, p).first;
        }
        plan = &it->second;                    // entries are never removed: the address stays good
    }
    const float one = 1.f, zero = 0.f;
    RI_LT(hipblasLtMatmul(g_handle, plan->desc, &one, W, plan->a, A, plan->b, &zero, C, plan->c, C, plan->c,
                          &plan->algo, workspace, workspace_bytes, stream), "hipblasLtMatmul");
    return 0;
}
