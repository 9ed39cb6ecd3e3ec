// Matrix products  C[M, N] = A[M, K] . W[N, K]^T  (weights stored [out, in] as in the
// checkpoint; reference contract: op_ports.rs:54-62).
//
//  * gemm_tiled: any M, N, K; float or bfloat16 inputs; 32-bit FMA accumulation in a fixed
//    order over K, so a row's result does not depend on the other rows of the batch.
//    This is the product of the exact 32-bit path (no reduced-precision matrix mode).
//  * gemv_bf16: M <= 8 rows against bfloat16 weights, one wave per output column, the
//    weight matrix streamed once with 16-byte loads (reference: hgemv_bf16_v3,
//    matmul.cu:870-929).
#include "common.h"

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(
        const TI* __restrict__ A, int lda, const TI* __restrict__ W, int ldw,
        TO* __restrict__ C, int ldc, int M, int N, int K) {
    constexpr int BM = 64, BN = 64, BK = 16;
    __shared__ float As[BK][BM + 1];
    __shared__ float Ws[BK][BN + 1];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int tx = tid & 15, ty = tid >> 4;          // 16 x 16 threads, 4 x 4 outputs each
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += BK) {
        // 64 x 16 elements of each operand, 4 per thread
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + i * 256;
            const int r = e >> 4, kk = e & 15;
            const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
            As[kk][r] = (gm < M && gk < K) ? ld_f32(A + (size_t)gm * lda + gk) : 0.f;
            Ws[kk][r] = (gn < N && gk < K) ? ld_f32(W + (size_t)gn * ldw + gk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; w[i] = Ws[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn < N) st_f32(C + (size_t)gm * ldc + gn, acc[i][j]);
        }
    }
}

extern "C" int ri_gemm_tiled(const void* A, int lda, const void* W, int ldw, void* C, int ldc,
                             int M, int N, int K, int in_dtype, int out_dtype, hipStream_t stream) {
    RI_REQUIRE(M >= 0 && N > 0 && K > 0, "ri_gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
    RI_REQUIRE(lda >= K && ldw >= K && ldc >= N, "ri_gemm_tiled: leading dimensions too small");
    if (M == 0) return 0;
    RI_REQUIRE(A && W && C, "ri_gemm_tiled: null pointer");
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    RI_REQUIRE(grid.y <= 65535, "ri_gemm_tiled: M=%d exceeds the grid limit", M);
    if (in_dtype == RI_F32 && out_dtype == RI_F32)
        gemm_tiled_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)A, lda, (const float*)W, ldw, (float*)C, ldc, M, N, K);
    else if (in_dtype == RI_BF16 && out_dtype == RI_BF16)
        gemm_tiled_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, ldw, (bf16_t*)C, ldc, M, N, K);
    else if (in_dtype == RI_BF16 && out_dtype == RI_F32)
        gemm_tiled_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)A, lda, (const bf16_t*)W, ldw, (float*)C, ldc, M, N, K);
    else
        return ri_fail("ri_gemm_tiled: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
    RI_LAUNCHED("ri_gemm_tiled");
    return 0;
}

// ---------------------------------------------------------------------------
// gemv_bf16: C[m, n] = sum_k A[m, k] W[n, k], m < MT <= 8.  One wave per n; each lane walks
// K in steps of 64 * 8 elements with 16-byte loads.  K % 8 == 0.
// ---------------------------------------------------------------------------
struct alignas(16) bf16x8 { bf16_t v[8]; };

template <int MT, typename TO>
__global__ __launch_bounds__(256) void gemv_bf16_kernel(
        const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
        TO* __restrict__ C, int ldc, int M, int N, int K) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + wave;
    if (n >= N) return;
    const bf16_t* wr = W + (size_t)n * ldw;
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.f;
    for (int k = lane * 8; k < K; k += 64 * 8) {
        const bf16x8 wv = *reinterpret_cast<const bf16x8*>(wr + k);
        float wf[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) wf[i] = bf16_to_f32(wv.v[i]);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m < M) {
                const bf16x8 av = *reinterpret_cast<const bf16x8*>(A + (size_t)m * lda + k);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[m] = fmaf(bf16_to_f32(av.v[i]), wf[i], acc[m]);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float s = wave_sum(acc[m]);
        if (lane == 0 && m < M) st_f32(C + (size_t)m * ldc + n, s);
    }
}

template <typename TO>
static int launch_gemv(const bf16_t* A, int lda, const bf16_t* W, int ldw, TO* C, int ldc,
                       int M, int N, int K, hipStream_t stream) {
    const int grid = (N + 3) / 4;
    if (M == 1) gemv_bf16_kernel<1, TO><<<grid, 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
    else if (M == 2) gemv_bf16_kernel<2, TO><<<grid, 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
    else if (M <= 4) gemv_bf16_kernel<4, TO><<<grid, 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
    else gemv_bf16_kernel<8, TO><<<grid, 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K);
    RI_LAUNCHED("ri_gemv_bf16");
    return 0;
}

extern "C" int ri_gemv_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc,
                            int M, int N, int K, int out_dtype, hipStream_t stream) {
    RI_REQUIRE(M >= 1 && M <= 8, "ri_gemv_bf16: M=%d not in [1, 8]", M);
    RI_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "ri_gemv_bf16: K=%d must be a positive multiple of 8 (N=%d)", K, N);
    RI_REQUIRE(lda >= K && ldw >= K && ldc >= N && lda % 8 == 0 && ldw % 8 == 0, "ri_gemv_bf16: leading dimensions must be >= K and multiples of 8");
    RI_REQUIRE(A && W && C, "ri_gemv_bf16: null pointer");
    RI_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "ri_gemv_bf16: operands must be 16-byte aligned");
    if (out_dtype == RI_BF16) return launch_gemv<bf16_t>((const bf16_t*)A, lda, (const bf16_t*)W, ldw, (bf16_t*)C, ldc, M, N, K, stream);
    if (out_dtype == RI_F32) return launch_gemv<float>((const bf16_t*)A, lda, (const bf16_t*)W, ldw, (float*)C, ldc, M, N, K, stream);
    return ri_fail("ri_gemv_bf16: unknown output dtype %d", out_dtype);
}
