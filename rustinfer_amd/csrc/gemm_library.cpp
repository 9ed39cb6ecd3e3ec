// bfloat16 products of many rows through hipBLASLt, as the reference sends them to cuBLASLt
// (crates/infer-backend-cuda/src/kernels/matmul/mod.rs:187-221).
//
//   C[M, N] = A[M, K] . W[N, K]^T      row-major, bfloat16 in, 32-bit accumulation, bfloat16 or float32 out
//
// In the library's column-major terms that is C^T[N, M] = W^T-stored[K, N]^T . A^T-stored[K, M]:
// transA = T on the weights, transB = N on the activations, m = N, n = M, k = K.
// What costs time on the host is asking the library which kernel to use (milliseconds); the answer
// is kept per (row bucket, N, K): prompt portions of changing length ask once a bucket (row_bucket
// below), and a row count whose bucket has an answer only checks that the kernel
// takes it.  Descriptor and layouts are kept per exact shape, so a repeated shape costs one
// hipblasLtMatmul call; that table is emptied when it has grown to 1,024 shapes.
//
// The library's own choice of kernel is not always its fastest for the shapes of a prompt portion
// (2,048 rows at hidden 2,048..4,096: 3-8 % slower than the best of its kernels, measured with the
// step's own activations and weights; constant data runs cooler and misleads).  With tuning
// switched on (ri_gemm_library_set_tuning) the first product of a (row bucket, N, K) times every
// kernel of the library that takes the problem and keeps the fastest; the choice is also written
// to a file and read back by later processes.  Row counts share a bucket, so that a serving
// process tunes a handful of shapes, about a second each.
#include "common.h"
#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>
#include <algorithm>
#include <cstdio>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

enum { RI_NO_LIBRARY_KERNEL = 2 };

namespace {

// Row counts that share a kernel choice: up to the next multiple of 16 (to 256 rows), of 32 (to
// 512), of 128 (to 2,048) or of 512.  With the next power of two a count in the middle of its bucket ran the kernel
// chosen for twice its rows: 264 rows against 28,672 columns took 86 us where the kernel the
// library picks for 264 rows takes 63, 1,100 rows 288 us against 227.
int row_bucket(int M) {
    const int step = M <= 256 ? 16 : (M <= 512 ? 32 : (M <= 2048 ? 128 : 512));
    return (M + step - 1) / step * step;
}

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
constexpr size_t MAX_PLANS = 1024;
typedef std::tuple<int, int, int, int, int, size_t> BucketKey;     // row bucket, N, K, ldw, out_f32, workspace
std::map<BucketKey, hipblasLtMatmulAlgo_t> g_bucket_algo;          // the library's choice for the bucket's upper bound
int g_heuristic_calls = 0;

void destroy_plan(Plan& p) {
    if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
    if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
    if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
    if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
    p = Plan{};
}

// -- tuning ------------------------------------------------------------------------------
bool g_tune = false;
std::string g_tune_file;                                     // "" = choices are not kept on disk
typedef std::tuple<int, int, int, int> TuneKey;              // row bucket, N, K, out_f32
std::map<TuneKey, int> g_tuned;                              // -> the library's index of the kernel (-1: its own choice stays)
std::vector<hipblasLtMatmulHeuristicResult_t> g_all[2];      // every kernel of the library for bf16 in, [bf16 | f32] out

void read_tune_file() {
    FILE* f = g_tune_file.empty() ? nullptr : fopen(g_tune_file.c_str(), "r");
    if (!f) return;
    int b, n, k, o, idx;
    while (fscanf(f, "%d %d %d %d %d", &b, &n, &k, &o, &idx) == 5) g_tuned[TuneKey(b, n, k, o)] = idx;
    fclose(f);
}

void append_tune_file(const TuneKey& key, int idx) {
    FILE* f = g_tune_file.empty() ? nullptr : fopen(g_tune_file.c_str(), "a");
    if (!f) return;                                          // not writable: the choice lives as long as the process
    fprintf(f, "%d %d %d %d %d\n", std::get<0>(key), std::get<1>(key), std::get<2>(key), std::get<3>(key), idx);
    fclose(f);
}

// Times every kernel that takes the problem of `bucket` rows and returns the index of the
// fastest, or -1 if none beats the library's own choice.  A: activations of M rows (repeated to
// fill the bucket), W: the weight itself.  Allocates its operands and synchronises the device:
// never call it while a graph is being captured.
int tune_shape(const Key& k, int bucket, const void* A, const void* W, size_t ws_bytes, void* ws, hipblasLtMatmulAlgo_t library_choice) {
    const hipblasOperation_t opT = HIPBLAS_OP_T, opN = HIPBLAS_OP_N;
    const hipDataType out_t = k.out_f32 ? HIP_R_32F : HIP_R_16BF;
    std::vector<hipblasLtMatmulHeuristicResult_t>& all = g_all[k.out_f32 ? 1 : 0];
    if (all.empty() && hipblaslt_ext::getAllAlgos(g_handle, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, opT, opN, HIP_R_16BF, HIP_R_16BF,
                                                  out_t, out_t, HIPBLAS_COMPUTE_32F, all) != HIPBLAS_STATUS_SUCCESS)
        return -1;
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr;
    void *a_buf = nullptr, *c_buf = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int best = -1;
    const size_t a_row = (size_t)k.K * 2, c_bytes = (size_t)bucket * k.N * (k.out_f32 ? 4 : 2);
    bool ok = hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS
        && hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opT, sizeof(opT)) == HIPBLAS_STATUS_SUCCESS
        && hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opN, sizeof(opN)) == HIPBLAS_STATUS_SUCCESS
        && hipblasLtMatrixLayoutCreate(&la, HIP_R_16BF, k.K, k.N, k.ldw) == HIPBLAS_STATUS_SUCCESS
        && hipblasLtMatrixLayoutCreate(&lb, HIP_R_16BF, k.K, bucket, k.K) == HIPBLAS_STATUS_SUCCESS
        && hipblasLtMatrixLayoutCreate(&lc, out_t, k.N, bucket, k.N) == HIPBLAS_STATUS_SUCCESS
        && hipMalloc(&a_buf, (size_t)bucket * a_row) == hipSuccess && hipMalloc(&c_buf, c_bytes) == hipSuccess
        && hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
    ok = ok && hipDeviceSynchronize() == hipSuccess;           // the activations have been written
    if (ok) {
        for (int r = 0; r < bucket && ok; r += k.M) {          // the step's own activations, again and again
            const int n = std::min(k.M, bucket - r);
            ok = hipMemcpy2D((char*)a_buf + (size_t)r * a_row, a_row, A, (size_t)k.lda * 2, a_row, n, hipMemcpyDeviceToDevice) == hipSuccess;
        }
    }
    if (ok) {
        const float one = 1.f, zero = 0.f;
        auto time_of = [&](hipblasLtMatmulAlgo_t& algo, int reps) -> float {
            size_t need = 0;
            if (hipblaslt_ext::matmulIsAlgoSupported(g_handle, desc, &one, la, lb, &zero, lc, lc, algo, need) != HIPBLAS_STATUS_SUCCESS || need > ws_bytes)
                return -1.f;
            auto run = [&]() { return hipblasLtMatmul(g_handle, desc, &one, W, la, a_buf, lb, &zero, c_buf, lc, c_buf, lc, &algo, ws, ws_bytes, nullptr); };
            if (run() != HIPBLAS_STATUS_SUCCESS || hipDeviceSynchronize() != hipSuccess) return -1.f;
            (void)hipEventRecord(e0, nullptr);
            for (int i = 0; i < reps; ++i) run();
            (void)hipEventRecord(e1, nullptr);
            float ms = 0.f;
            if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) return -1.f;
            return ms / reps;
        };
        std::vector<std::pair<float, size_t>> timed;
        for (size_t i = 0; i < all.size(); ++i) {
            const float t = time_of(all[i].algo, 2);
            if (t > 0.f) timed.push_back({t, i});
        }
        std::sort(timed.begin(), timed.end());
        float best_t = 0.f;
        for (size_t j = 0; j < timed.size() && j < 8; ++j) {     // the first few once more, with more repetitions
            const float t = time_of(all[timed[j].second].algo, 10);
            if (t > 0.f && (best < 0 || t < best_t)) { best_t = t; best = hipblaslt_ext::getIndexFromAlgo(all[timed[j].second].algo); }
        }
        const float t_lib = time_of(library_choice, 10);
        if (best >= 0 && t_lib > 0.f && t_lib <= best_t) best = -1;     // nothing beats the library's own choice
        fprintf(stderr, "[rustinfer_amd] GEMM of up to %d rows, N=%d K=%d: %zu of the library's kernels timed, fastest %.1f us, its own choice %.1f us\n",
                bucket, k.N, k.K, timed.size(), (best >= 0 ? best_t : t_lib) * 1e3f, t_lib * 1e3f);
        fflush(stderr);
    }
    (void)hipGetLastError();                                   // a kernel that refused its launch leaves no error behind
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (a_buf) (void)hipFree(a_buf);
    if (c_buf) (void)hipFree(c_buf);
    if (la) hipblasLtMatrixLayoutDestroy(la);
    if (lb) hipblasLtMatrixLayoutDestroy(lb);
    if (lc) hipblasLtMatrixLayoutDestroy(lc);
    if (desc) hipblasLtMatmulDescDestroy(desc);
    return best;
}

#define RI_LT(call, what) do { hipblasStatus_t st_ = (call); \
    if (st_ != HIPBLAS_STATUS_SUCCESS) return ri_fail("ri_gemm_library: %s failed with status %d", what, (int)st_); } while (0)

int make_plan(const Key& k, Plan& p, const void* A, const void* W, void* ws, hipStream_t stream) {
    const hipblasOperation_t opT = HIPBLAS_OP_T, opN = HIPBLAS_OP_N;
    RI_LT(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
    RI_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &opT, sizeof(opT)), "set transA");
    RI_LT(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &opN, sizeof(opN)), "set transB");
    // stored shapes (column-major): weights K x N, activations K x M, result N x M
    RI_LT(hipblasLtMatrixLayoutCreate(&p.a, HIP_R_16BF, k.K, k.N, k.ldw), "layout of the weights");
    RI_LT(hipblasLtMatrixLayoutCreate(&p.b, HIP_R_16BF, k.K, k.M, k.lda), "layout of the activations");
    RI_LT(hipblasLtMatrixLayoutCreate(&p.c, k.out_f32 ? HIP_R_32F : HIP_R_16BF, k.N, k.M, k.ldc), "layout of the result");
    const float one_ = 1.f, zero_ = 0.f;
    const int bucket_rows = row_bucket(k.M);
    const BucketKey bk(bucket_rows, k.N, k.K, k.ldw, k.out_f32, k.ws);
    hipblasLtMatmulHeuristicResult_t found;
    // Which kernel a row count gets depends on its bucket and on itself alone, never on which
    // row counts were served before: the library is asked once a bucket, for the bucket's upper
    // bound, and a row count that this kernel does not take asks for itself.
    auto ask = [&](hipblasLtMatrixLayout_t b, hipblasLtMatrixLayout_t c, hipblasLtMatmulHeuristicResult_t& res) -> bool {
        hipblasLtMatmulPreference_t pref = nullptr;
        if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return false;
        hipblasStatus_t st = hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &k.ws, sizeof(k.ws));
        int n = 0;
        if (st == HIPBLAS_STATUS_SUCCESS)
            st = hipblasLtMatmulAlgoGetHeuristic(g_handle, p.desc, p.a, b, c, c, pref, 1, &res, &n);
        hipblasLtMatmulPreferenceDestroy(pref);
        ++g_heuristic_calls;
        return st == HIPBLAS_STATUS_SUCCESS && n >= 1;
    };
    auto known = g_bucket_algo.find(bk);
    if (known == g_bucket_algo.end() && bucket_rows != k.M) {
        hipblasLtMatrixLayout_t bb = nullptr, bc = nullptr;
        hipblasLtMatmulHeuristicResult_t res;
        if (hipblasLtMatrixLayoutCreate(&bb, HIP_R_16BF, k.K, bucket_rows, k.lda) == HIPBLAS_STATUS_SUCCESS
            && hipblasLtMatrixLayoutCreate(&bc, k.out_f32 ? HIP_R_32F : HIP_R_16BF, k.N, bucket_rows, k.ldc) == HIPBLAS_STATUS_SUCCESS
            && ask(bb, bc, res))
            known = g_bucket_algo.emplace(bk, res.algo).first;
        if (bb) hipblasLtMatrixLayoutDestroy(bb);
        if (bc) hipblasLtMatrixLayoutDestroy(bc);
    }
    size_t need_known = 0;
    if (known != g_bucket_algo.end()
        && hipblaslt_ext::matmulIsAlgoSupported(g_handle, p.desc, &one_, p.a, p.b, &zero_, p.c, p.c, known->second, need_known) == HIPBLAS_STATUS_SUCCESS
        && need_known <= k.ws) {
        found.algo = known->second;                            // the bucket's kernel takes this row count too
        found.workspaceSize = need_known;
    } else {
        if (!ask(p.b, p.c, found)) {
            ri_fail("ri_gemm_library: the library offers no kernel for M=%d N=%d K=%d", k.M, k.N, k.K);
            return RI_NO_LIBRARY_KERNEL;
        }
        if (bucket_rows == k.M && known == g_bucket_algo.end()) g_bucket_algo.emplace(bk, found.algo);
    }
    p.algo = found.algo;
    p.workspace = found.workspaceSize;
    if (g_tune && k.M > 64) {
        const int bucket = row_bucket(k.M);
        const TuneKey tk(bucket, k.N, k.K, k.out_f32);
        auto it = g_tuned.find(tk);
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (it == g_tuned.end() && hipStreamIsCapturing(stream, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone) {
            const int idx = tune_shape(k, bucket, A, W, k.ws, ws, found.algo);   // (never inside a capture: it synchronises)
            it = g_tuned.emplace(tk, idx).first;
            append_tune_file(tk, idx);
        }
        if (it != g_tuned.end() && it->second >= 0) {
            std::vector<int> index{it->second};
            std::vector<hipblasLtMatmulHeuristicResult_t> got;
            const float one = 1.f, zero = 0.f;
            size_t need = 0;
            if (hipblaslt_ext::getAlgosFromIndex(g_handle, index, got) == HIPBLAS_STATUS_SUCCESS && !got.empty()
                && hipblaslt_ext::matmulIsAlgoSupported(g_handle, p.desc, &one, p.a, p.b, &zero, p.c, p.c, got[0].algo, need) == HIPBLAS_STATUS_SUCCESS
                && need <= k.ws) {
                p.algo = got[0].algo;                          // takes this row count too; else the library's own choice stays
                p.workspace = need;
            }
        }
    }
    return 0;
}

}  // namespace

// workspace: device memory the library may use (split products); the same size must be passed
// for a shape each time.  Returns 0, or non-zero with a message in ri_last_error():
// RI_NO_LIBRARY_KERNEL (2) if the library has no kernel for the problem (nothing was launched; the
// caller may take a kernel of its own), 1 for every other failure.
// out_f32 != 0: C is float32 (logits), else bfloat16.
extern "C" int ri_gemm_library_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc,
                                    int M, int N, int K, int out_f32, void* workspace, size_t workspace_bytes,
                                    hipStream_t stream) {
    RI_REQUIRE(M > 0 && N > 0 && K > 0 && lda >= K && ldw >= K && ldc >= N, "ri_gemm_library: bad sizes M=%d N=%d K=%d", M, N, K);
    RI_REQUIRE(A && W && C && (workspace || workspace_bytes == 0), "ri_gemm_library: null pointer");
    // one caller at a time: the table of shapes may be emptied, and its descriptors with it
    std::lock_guard<std::mutex> lock(g_mutex);
    if (!g_handle) RI_LT(hipblasLtCreate(&g_handle), "hipblasLtCreate");
    const Key key{M, N, K, lda, ldw, ldc, out_f32 ? 1 : 0, workspace_bytes};
    auto it = g_plans.find(key);
    if (it == g_plans.end()) {
        if (g_plans.size() >= MAX_PLANS) {
            for (auto& kv : g_plans) destroy_plan(kv.second);
            g_plans.clear();
        }
        Plan p;
        if (int rc = make_plan(key, p, A, W, workspace, stream)) { destroy_plan(p); return rc; }
        it = g_plans.emplace(key, p).first;
    }
    const Plan* plan = &it->second;
    const float one = 1.f, zero = 0.f;
    const hipblasStatus_t st = hipblasLtMatmul(g_handle, plan->desc, &one, W, plan->a, A, plan->b, &zero, C, plan->c, C, plan->c,
                                               &plan->algo, workspace, workspace_bytes, stream);
    if (st == HIPBLAS_STATUS_NOT_SUPPORTED || st == HIPBLAS_STATUS_INVALID_VALUE) {
        // refused while the arguments were checked, before any launch (an alignment the chosen kernel does not take)
        ri_fail("ri_gemm_library: the library's kernel refuses M=%d N=%d K=%d (status %d)", M, N, K, (int)st);
        destroy_plan(it->second);
        g_plans.erase(it);
        return RI_NO_LIBRARY_KERNEL;
    }
    RI_LT(st, "hipblasLtMatmul");
    return 0;
}

// on != 0: products of more than 64 rows look for the library's fastest kernel the first time a
// (row bucket, N, K) is met (the device is synchronised and memory allocated, so the first product
// of a shape must not fall into a graph capture; inside one the library's own choice is taken).
// file: where choices are kept between processes, or null.  Shapes already planned keep their kernel.
extern "C" int ri_gemm_library_set_tuning(int on, const char* file) {
    std::lock_guard<std::mutex> lock(g_mutex);
    g_tune = on != 0;
    const std::string f = file ? file : "";
    if (g_tune && f != g_tune_file) {
        g_tune_file = f;
        read_tune_file();
    }
    return 0;
}

// Forget every kept descriptor and every kernel choice that was not tuned (tests: what a row count
// gets must not depend on what was served before).
extern "C" int ri_gemm_library_reset() {
    std::lock_guard<std::mutex> lock(g_mutex);
    for (auto& kv : g_plans) destroy_plan(kv.second);
    g_plans.clear();
    g_bucket_algo.clear();
    return 0;
}

// (shapes kept, questions put to the library's heuristic so far)
extern "C" int ri_gemm_library_stats(int* plans, int* heuristic_calls) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if (plans) *plans = (int)g_plans.size();
    if (heuristic_calls) *heuristic_calls = g_heuristic_calls;
    return 0;
}

// how many (row bucket, N, K) have been tuned or read from the file so far
extern "C" int ri_gemm_library_tuned_shapes() {
    std::lock_guard<std::mutex> lock(g_mutex);
    return (int)g_tuned.size();
}
