// Matrix products  C[M, N] = A[M, K] . W[N, K]^T  (weights stored [out, in] as in the
// checkpoint; reference contract: op_ports.rs:54-62).
//
//  * gemm_tiled: any M, N, K; float or bfloat16 inputs; FMA accumulation in a fixed order over K,
//    so a row's result does not depend on the other rows of the batch.  This is the product of
//    the exact 32-bit path (no reduced-precision matrix mode): for float inputs the sum is kept
//    in 64-bit, as the reference's float path does on the CPU
//    (crates/infer-backend-cpu/src/lib.rs:403-418), so that a long K adds no rounding of its own.
//  * gemm_skinny_bf16: M <= 64 rows against bfloat16 weights on the matrix cores, the weight
//    matrix streamed once with 16-byte loads (reference: hgemv_bf16_v3 for one row,
//    matmul.cu:870-929, cuBLASLt otherwise).
#include "common.h"

template <typename TI> struct GemmAcc { typedef float type; };
template <> struct GemmAcc<float> { typedef double type; };
__device__ __forceinline__ float gemm_fma(float a, float w, float acc) { return fmaf(a, w, acc); }
__device__ __forceinline__ double gemm_fma(float a, float w, double acc) { return fma((double)a, (double)w, acc); }

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
    typedef typename GemmAcc<TI>::type TAcc;
    TAcc acc[4][4] = {};
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
                for (int j = 0; j < 4; ++j) acc[i][j] = gemm_fma(a[i], w[j], acc[i][j]);
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
            if (gn < N) st_f32(C + (size_t)gm * ldc + gn, (float)acc[i][j]);
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
// gemm_skinny_bf16: C[M, N] = A[M, K] . W[N, K]^T for M <= 64 on the matrix cores.
// The product is bound by the one pass over W, so the kernel is built around that stream:
// a block owns 16 rows of W (one MFMA tile); its waves take the 32-wide k-steps in turn
// (wave w takes steps w, w + WAVES, ...), so that at any moment the block reads a contiguous
// stretch of each row; every lane keeps several 16-byte loads in flight; partial tiles are
// summed through LDS.  W is the A operand (rows = n), the activations are the B operand
// (columns = m), read from L1/L2.  With SWIGLU the block also streams the 16 rows I further
// down (the "up" half of a stacked gate/up matrix) and writes silu(gate) * up.
// K % 8 == 0; any N.
// ---------------------------------------------------------------------------
typedef __bf16 gbf16x8_t __attribute__((ext_vector_type(8)));
typedef float gf32x4_t __attribute__((ext_vector_type(4)));

struct VecLoad4 {       // four consecutive outputs of a lane in one store
    static __device__ __forceinline__ void st(float* p, const float* v) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
    static __device__ __forceinline__ void st(bf16_t* p, const float* v) {
        uint2 t;
        t.x = (uint32_t)f32_to_bf16(v[0]) | ((uint32_t)f32_to_bf16(v[1]) << 16);
        t.y = (uint32_t)f32_to_bf16(v[2]) | ((uint32_t)f32_to_bf16(v[3]) << 16);
        *reinterpret_cast<uint2*>(p) = t;
    }
};

// TILED: W is a copy in tile order, [N/16][K/32][64 lanes][8]: the 16 x 32 block of an MFMA
// operand lies contiguous, each lane's 8 values where the lane reads them.  A wave then reads
// 1 KiB contiguous per instruction and a block one contiguous stretch of memory, which the
// memory system serves about a third faster than 64-byte pieces of 16 rows.  The copy is made
// once when the weights are loaded (N % 16 == 0 and K % 32 == 0).
//
// ROPE: the product is the fused q/k/v projection of single tokens and the kernel finishes what
// would otherwise be a kernel of its own: it rotates q and k by the token's position and writes
// k and v into the token's cache page; only q goes to C.  For that the rows of W are permuted
// within each head (qkv_rope_row_order below) so that a tile holds 8 features of the first half
// of a head and their 8 partners of the second half; the partner of a lane's value then sits in
// lane ^ 32.  Rotation in 32-bit on the unrounded sums, one rounding.
struct RopeEpilogue {
    const float* cos_t; const float* sin_t;        // [positions][hd / 2]
    const int* positions; const int* row_of_token; // per token (row of A)
    const int* table; int max_blocks;              // block table [rows][max_blocks]
    bf16_t* kc; bf16_t* vc;                        // k [pages][Hkv][page][hd], v [pages][Hkv][hd][page]
    int H, Hkv, hd, page;
};

// NORM: the activations are made in the kernel (at most four rows, no split over K between blocks):
// before it streams its weights every block puts row m of the operand, (x[m] + sum_p delta[p][m]) * w
// in 32-bit, rounded once to bfloat16, into LDS (dynamic, M * K * 2 bytes); the row's factor
// rsqrt(mean((x + delta)^2) + eps) multiplies the finished sums.  Block 0 also writes the sums x + delta to x_out, the residual
// stream after this layer half (x itself must stay as it is: the other blocks are reading it).
// With one or two rows this costs each block a few KB from L2 and saves the norm's own kernel,
// whose few microseconds are as long as the product's at that size.
struct NormPrologue {
    const float* x; const float* delta; int parts; size_t part_stride;   // delta: [parts][M][K] float, or null
    const float* w32; const bf16_t* w16;                                  // the norm's weight, one of the two
    float eps; float* x_out;
};

// NT: tiles of 16 rows of W a block owns.  With more than 16 activation rows (MT > 1) the
// activations are as much traffic through L1 as the weights; a wave that multiplies the same
// activation fragments with NT weight tiles needs them NT times less often.
template <int MT, int NT, int WAVES, typename TO, bool SWIGLU, bool TILED, bool ROPE = false, bool NORM = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_bf16_kernel(
        const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
        TO* __restrict__ C, int ldc, int M, int N, int K, int ks_per_block, size_t part_stride,
        RopeEpilogue ep = RopeEpilogue{}, NormPrologue np = NormPrologue{}) {
    static_assert(!NORM || MT == 1, "the norm is folded in for at most four rows");
    constexpr int NW = SWIGLU ? 2 * NT : NT;                 // weight tiles streamed: [gate tiles | up tiles]
    constexpr int U = (MT == 1 && NW == 1) ? 8 : ((MT + NW <= 3) ? 4 : 2);   // k-steps in flight per wave
    __shared__ float red[WAVES > 1 ? (WAVES - 1) * NW * 256 : 1];
    constexpr int NR = 4;                                    // NORM: the most rows
    __shared__ float red_ss[NORM ? WAVES * NR : 1];
    extern __shared__ __align__(16) unsigned char dyn_lds[];
    bf16_t* a_lds = reinterpret_cast<bf16_t*>(dyn_lds);      // NORM: the operand rows (x + delta) * w, [M][K]
    float rs = 1.f;                                          // NORM: rsqrt(mean((x + delta)^2) + eps) of this lane's row (col)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, grp = lane >> 4;
    const int ntiles = (N + 15) / 16;
    const int nks_all = (K + 31) / 32;
    const bf16_t* wp[NW];
#pragma unroll
    for (int a = 0; a < NW; ++a) {
        // tile index among the rows of W; rows beyond N are read (clamped) but never stored
        const int tile = min((int)blockIdx.x * NT + (a % NT), ntiles - 1);
        const int nrow = min(tile * 16 + col, N - 1) + (a >= NT ? N : 0);     // up half: N = I rows further down
        wp[a] = TILED ? W + ((size_t)(tile + (a >= NT ? N / 16 : 0)) * nks_all * 64 + lane) * 8
                      : W + (size_t)nrow * ldw + grp * 8;
    }
    gf32x4_t acc[NW][MT];
#pragma unroll
    for (int a = 0; a < NW; ++a)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[a][mt] = gf32x4_t{0.f, 0.f, 0.f, 0.f};
    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + col;
        xok[mt] = m < M;
        xrow[mt] = A + (size_t)min(m, M - 1) * lda + grp * 8;
    }
    // The waves of a block split the k range; at the end wave w sums up and stores the m-tile w
    // (the waves' partial tiles go through LDS), so that neither the sum nor the epilogue is left
    // to one wave while the others idle.
    static_assert(MT <= WAVES, "a wave owns at most one m-tile");
    // What the rotation and the cache write need beside the product (token's row, position and
    // page, cosines and sines) is asked for before the weights are streamed, so that the end of
    // the kernel does not wait for a chain of small loads.
    int rp_section = 0, rp_head = 0, rp_j = 0, rp_b = -1, rp_blk = -1, rp_slot = 0;
    float rp_c[NT][4], rp_s[NT][4];
#pragma unroll
    for (int a = 0; a < NT; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) { rp_c[a][i] = 1.f; rp_s[a][i] = 0.f; }
    if constexpr (ROPE) {
        // the NT tiles of a block lie within one head: (hd / 16) % NT == 0
        const int hd = ep.hd, half = hd >> 1;
        const int q_dim = ep.H * hd, kv_dim = ep.Hkv * hd;
        const int n0 = (int)blockIdx.x * NT * 16;
        rp_section = n0 < q_dim ? 0 : (n0 < q_dim + kv_dim ? 1 : 2);                     // q, k, v
        const int within = n0 - (rp_section == 0 ? 0 : (rp_section == 1 ? q_dim : q_dim + kv_dim));
        rp_head = within / hd;
        rp_j = (within % hd) >> 4;                                                       // the block's first tile is tile j of the head
        const int m = wave * 16 + col;                                                   // a token of this wave's m-tile
        if (wave < MT && m < M && n0 < N) {
            const int b = ep.row_of_token[m];
            const int pos = ep.positions[m];
            rp_b = b;
            rp_slot = pos % ep.page;
            if (b >= 0 && rp_section != 0) rp_blk = ep.table[(size_t)b * ep.max_blocks + pos / ep.page];
            if (b >= 0 && rp_section != 2) {
#pragma unroll
                for (int a = 0; a < NT; ++a)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int fi = 8 * (rp_j + a) + ((grp * 4 + i) & 7);
                        rp_c[a][i] = ep.cos_t[(size_t)pos * half + fi];
                        rp_s[a][i] = ep.sin_t[(size_t)pos * half + fi];
                    }
            }
        }
    }
    // blockIdx.y picks a range of k-steps; its partial product goes to its own slice of C
    const int ks_begin = blockIdx.y * ks_per_block;
    const int ks_end = min(nks_all, ks_begin + ks_per_block);
    C += (size_t)blockIdx.y * part_stride;
    const gbf16x8_t zero = {};
    // the weight fragments of the U k-steps from ks0 on
    auto load_weights = [&](int ks0, gbf16x8_t (&wf)[NW][U]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ks = ks0 + u * WAVES;
            const bool ok = ks < ks_end && ks * 32 + grp * 8 < K;   // K % 8 == 0: a lane's 8 values are in or out together
            const size_t wk = TILED ? (size_t)ks * 512 : (size_t)ks * 32;   // a tile of 16 x 32 has 512 values
#pragma unroll
            for (int a = 0; a < NW; ++a) wf[a][u] = ok ? *reinterpret_cast<const gbf16x8_t*>(wp[a] + wk) : zero;
        }
    };
    if constexpr (NORM) {
        // Every block makes the (at most four) operand rows itself, all its threads together, 8
        // values a thread and round, with every load asked for before the first is used.
        float ssr[NR] = {};
        const int nvec = M * K / 8;
        for (int i = threadIdx.x; i < nvec; i += WAVES * 64) {
            const size_t at = (size_t)i * 8;                   // x, delta and x_out have rows of K
            const int k = (int)(at % (size_t)K);
            float4 d[8][2];
#pragma unroll
            for (int p = 0; p < 8; ++p)
                if (p < np.parts) {
                    const float* dp = np.delta + (size_t)p * np.part_stride + at;
                    d[p][0] = *reinterpret_cast<const float4*>(dp);
                    d[p][1] = *reinterpret_cast<const float4*>(dp + 4);
                }
            const float4 x0 = *reinterpret_cast<const float4*>(np.x + at);
            const float4 x1 = *reinterpret_cast<const float4*>(np.x + at + 4);
            float v[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w}, wv[8];
            if (np.w16) {
                const gbf16x8_t w8 = *reinterpret_cast<const gbf16x8_t*>(np.w16 + k);
#pragma unroll
                for (int e = 0; e < 8; ++e) wv[e] = (float)w8[e];
            } else {
                const float4 w0 = *reinterpret_cast<const float4*>(np.w32 + k);
                const float4 w1 = *reinterpret_cast<const float4*>(np.w32 + k + 4);
                wv[0] = w0.x; wv[1] = w0.y; wv[2] = w0.z; wv[3] = w0.w; wv[4] = w1.x; wv[5] = w1.y; wv[6] = w1.z; wv[7] = w1.w;
            }
#pragma unroll
            for (int p = 0; p < 8; ++p)
                if (p < np.parts) {
                    v[0] += d[p][0].x; v[1] += d[p][0].y; v[2] += d[p][0].z; v[3] += d[p][0].w;
                    v[4] += d[p][1].x; v[5] += d[p][1].y; v[6] += d[p][1].z; v[7] += d[p][1].w;
                }
            if (blockIdx.x == 0) {
                *reinterpret_cast<float4*>(np.x_out + at) = make_float4(v[0], v[1], v[2], v[3]);
                *reinterpret_cast<float4*>(np.x_out + at + 4) = make_float4(v[4], v[5], v[6], v[7]);
            }
            float sq = 0.f;
            gbf16x8_t a8;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                sq = fmaf(v[e], v[e], sq);
                a8[e] = (__bf16)(v[e] * wv[e]);
            }
            *reinterpret_cast<gbf16x8_t*>(a_lds + at) = a8;
            const int r = (int)(at / (size_t)K);
#pragma unroll
            for (int q = 0; q < NR; ++q) ssr[q] += r == q ? sq : 0.f;
        }
#pragma unroll
        for (int r = 0; r < NR; ++r) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) ssr[r] += __shfl_xor(ssr[r], off, 64);
        }
        if ((threadIdx.x & 63) == 0) {
#pragma unroll
            for (int r = 0; r < NR; ++r) red_ss[(threadIdx.x >> 6) * NR + r] = ssr[r];
        }
        __syncthreads();                                       // the rows and the waves' sums are in LDS
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) total += red_ss[w * NR + (col & (NR - 1))];   // col < M <= NR
        rs = rsqrtf(total / (float)K + np.eps);
    }
    for (int ks0 = ks_begin + wave; ks0 < ks_end; ks0 += WAVES * U) {
        gbf16x8_t wf[NW][U], xf[MT][U];
        load_weights(ks0, wf);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ks = ks0 + u * WAVES;
            const int k = ks * 32;
            const bool ok = ks < ks_end && k + grp * 8 < K;
            if constexpr (NORM) {
                xf[0][u] = (ok && xok[0]) ? *reinterpret_cast<const gbf16x8_t*>(a_lds + (size_t)col * K + k + grp * 8) : zero;
            } else {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    xf[mt][u] = (ok && xok[mt]) ? *reinterpret_cast<const gbf16x8_t*>(xrow[mt] + k) : zero;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int a = 0; a < NW; ++a)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[a][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[a][u], xf[mt][u], acc[a][mt], 0, 0, 0);
    }
    if (WAVES > 1) {
        // One m-tile a round (that bounds the LDS to one tile's partial results): the other
        // waves put their partial tiles (a, mt) into slots, its owner adds them up.
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (mt > 0) __syncthreads();                   // the previous round's slots have been read
            if (wave != mt) {
                const int slot = wave < mt ? wave : wave - 1;
#pragma unroll
                for (int a = 0; a < NW; ++a)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        red[(slot * NW + a) * 256 + i * 64 + lane] = acc[a][mt][i];
            }
            __syncthreads();
            if (wave == mt) {
                for (int w = 0; w < WAVES - 1; ++w)
#pragma unroll
                    for (int a = 0; a < NW; ++a)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            acc[a][mt][i] += red[(w * NW + a) * 256 + i * 64 + lane];
            }
        }
        if (wave >= MT) return;
    }
    if constexpr (NORM) {
#pragma unroll
        for (int a = 0; a < NW; ++a)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[a][0][i] *= rs;
    }
    // acc[a][mt][i] = C[m = mt*16 + col][n = (blockIdx.x*NT + a)*16 + grp*4 + i]
#pragma unroll
    for (int a = 0; a < NT; ++a) {
        const int n0 = ((int)blockIdx.x * NT + a) * 16;
        if (n0 >= N) break;
        if constexpr (ROPE) {
            const int hd = ep.hd, half = hd >> 1;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (WAVES > 1 && wave != mt) continue;
                const int m = mt * 16 + col;
                const int b = rp_b, blk = rp_blk, slot = rp_slot;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int r = grp * 4 + i;                       // row of the tile: r < 8 first half, else partner
                    const float v = acc[a][mt][i];
                    const float other = __shfl_xor(v, 32, 64);       // row r ^ 8, same token
                    const int fi = 8 * (rp_j + a) + (r & 7);         // index within the half
                    const int d = r < 8 ? fi : half + fi;            // feature within the head
                    if (b < 0) continue;                             // padding token or beyond M
                    if (rp_section == 2) {
                        if (blk >= 0) ep.vc[((size_t)blk * ep.Hkv + rp_head) * ep.page * hd + (size_t)d * ep.page + slot] = f32_to_bf16(v);
                        continue;
                    }
                    const float c = rp_c[a][i], sn = rp_s[a][i];
                    const float res = r < 8 ? v * c - other * sn : other * sn + v * c;
                    if (rp_section == 0) st_f32(C + (size_t)m * ldc + rp_head * hd + d, res);
                    else if (blk >= 0) ep.kc[((size_t)blk * ep.Hkv + rp_head) * ep.page * hd + (size_t)slot * hd + d] = f32_to_bf16(res);
                }
            }
        } else {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (WAVES > 1 && wave != mt) continue;
                const int m = mt * 16 + col;
                if (m >= M) continue;
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    v[i] = acc[a][mt][i];
                    if (SWIGLU) v[i] = v[i] / (1.f + __expf(-v[i])) * acc[NT + a][mt][i];
                }
                const int n = n0 + grp * 4;                    // this lane's 4 consecutive columns
                TO* dst = C + (size_t)m * ldc + n;
                if (n + 3 < N && (ldc & 3) == 0 && ((uintptr_t)C & 15) == 0) {
                    VecLoad4::st(dst, v);                      // one 16-byte (float) or 8-byte (bfloat16) store
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (n + i < N) st_f32(dst + i, v[i]);
                }
            }
        }
    }
}

// Tiles of W a wave owns (NT) and slices of K given to separate blocks (parts).
//
// With few rows the activations cost as much as the weights once a wave asks for as many
// fragments of them: measured, a product takes about (weight bytes + activation bytes asked for
// by all waves) / 6-7 TB/s, whether the activations come from L2 or L1.  A wave that owns NT
// tiles of W uses each activation fragment NT times, so NT is taken as large as leaves blocks
// enough to fill the chip (counts below from sweeps over the 1B and 8B shapes at 8..64 rows).
// Products whose consumer adds up partial sums may also be split over K.
static int skinny_parts_for(int blocks, int nks) {
    int parts = 1;
    while (parts < 8 && blocks * parts < 512 && nks / (parts * 2) >= 8) parts *= 2;
    return parts;
}

// parts_given > 0: the caller has fixed the number of slices; 0: pick it too
static void skinny_plan(int M, int N, int K, bool swiglu, bool tiled, bool may_split, int parts_given,
                        int* nt_out, int* parts_out) {
    const int mt = (M + 15) / 16, tiles = (N + 15) / 16, nks = (K + 31) / 32;
    const int nt_fixed = swiglu ? (mt <= 2 ? 1 : 2) : (mt <= 2 ? mt : 4);
    int nt = 1, parts = 1;
    if (!tiled) {
        nt = nt_fixed;
        parts = parts_given > 0 ? parts_given : (may_split ? skinny_parts_for((tiles + nt - 1) / nt, nks) : 1);
    } else if (swiglu) {
        const int lim = mt == 1 ? 2 : 4, need = mt == 1 ? 448 : 224;
        while (nt * 2 <= lim && tiles / (nt * 2) >= need) nt *= 2;
    } else if (!may_split && parts_given <= 1) {
        nt = nt_fixed;
    } else {
        const int lim = M <= 8 ? 2 : 4, need = mt <= 2 ? 512 : 256;
        for (int cand = lim; cand >= 1; cand >>= 1) {
            const int blocks = (tiles + cand - 1) / cand;
            const int p = parts_given > 0 ? parts_given : skinny_parts_for(blocks, nks);
            nt = cand;
            parts = p;
            if (cand == 1 || (blocks * p >= need && nks / p >= (M <= 8 ? 64 : 32))) break;
        }
    }
    *nt_out = nt;
    *parts_out = parts_given > 0 ? parts_given : parts;
}

template <int MT, int NT, typename TO, bool SWIGLU, bool TILED>
static void launch_skinny_nt(const bf16_t* A, int lda, const bf16_t* W, int ldw, TO* C, int ldc,
                             int M, int N, int K, int parts, size_t part_stride, hipStream_t stream) {
    const int nks = (K + 31) / 32;
    const int ks_per_block = (nks + parts - 1) / parts;
    const int blocks = ((N + 15) / 16 + NT - 1) / NT;
    // enough waves to fill 256 CUs several times over, but no more waves than k-steps allow
    int waves = 4;
    if (MT <= 2 && blocks * parts * 4 < 4096 && ks_per_block >= 64) waves = 8;
    if (MT == 1 && NT == 1 && !SWIGLU && blocks * parts * 8 < 2048 && ks_per_block >= 128) waves = 16;
    dim3 grid(blocks, parts);
    if constexpr (MT == 1 && NT == 1 && !SWIGLU) {
        if (waves == 16) {
            gemm_skinny_bf16_kernel<1, 1, 16, TO, false, TILED><<<grid, 1024, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, ks_per_block, part_stride);
            return;
        }
    }
    if constexpr (MT <= 2) {
        if (waves == 8) {
            gemm_skinny_bf16_kernel<MT, NT, 8, TO, SWIGLU, TILED><<<grid, 512, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, ks_per_block, part_stride);
            return;
        }
    }
    gemm_skinny_bf16_kernel<MT, NT, 4, TO, SWIGLU, TILED><<<grid, 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, ks_per_block, part_stride);
}

template <int MT, typename TO, bool SWIGLU, bool TILED>
static int launch_skinny(const bf16_t* A, int lda, const bf16_t* W, int ldw, TO* C, int ldc,
                         int M, int N, int K, int parts, size_t part_stride, hipStream_t stream) {
    if (MT == 1 && !SWIGLU && (N + 15) / 16 >= 2048) {
        // a very wide product (the output head): four tiles per block even for few rows, so that
        // the activation fragments are fetched a quarter as often; blocks remain plentiful
        const int nks = (K + 31) / 32;
        const int wide_blocks = ((N + 15) / 16 + 3) / 4;
        gemm_skinny_bf16_kernel<1, 4, 4, TO, false, TILED><<<dim3(wide_blocks, parts), 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, (nks + parts - 1) / parts, part_stride);
        RI_LAUNCHED("ri_gemm_skinny_bf16");
        return 0;
    }
    int nt = 1, parts_same = 1;
    skinny_plan(M, N, K, SWIGLU, TILED, parts > 1, parts, &nt, &parts_same);
#define RI_SKINNY_NT(NT_) launch_skinny_nt<MT, NT_, TO, SWIGLU, TILED>(A, lda, W, ldw, C, ldc, M, N, K, parts, part_stride, stream)
    if (nt == 4) RI_SKINNY_NT(4);
    else if (nt == 2) RI_SKINNY_NT(2);
    else RI_SKINNY_NT(1);
#undef RI_SKINNY_NT
    RI_LAUNCHED("ri_gemm_skinny_bf16");
    return 0;
}

template <typename TO, bool SWIGLU>
static int dispatch_skinny(const bf16_t* A, int lda, const bf16_t* W, int ldw, TO* C, int ldc,
                           int M, int N, int K, int parts, size_t part_stride, int tiled, hipStream_t stream) {
#define RI_SKINNY(MT) (tiled ? launch_skinny<MT, TO, SWIGLU, true>(A, lda, W, ldw, C, ldc, M, N, K, parts, part_stride, stream) \
                             : launch_skinny<MT, TO, SWIGLU, false>(A, lda, W, ldw, C, ldc, M, N, K, parts, part_stride, stream))
    if (M <= 16) return RI_SKINNY(1);
    if (M <= 32) return RI_SKINNY(2);
    if (M <= 48) return RI_SKINNY(3);
    return RI_SKINNY(4);
#undef RI_SKINNY
}

template <int MT>
static int launch_skinny_rope(const bf16_t* A, int lda, const bf16_t* W, bf16_t* C, int ldc,
                              int M, int N, int K, const RopeEpilogue& ep, hipStream_t stream) {
    // The product cannot be split over K (the epilogue needs whole sums), so the number of blocks
    // is all the parallelism there is.  Two tiles (of one head) per wave halve what the waves ask
    // for of the activations; that pays where it leaves 128 blocks or more (measured: 384 tiles,
    // 8..64 rows: 13.6 -> 12.5 us .. 40 -> 27 us; with 192 tiles one tile per wave is faster).
    const int tiles = N / 16, nks = K / 32;
    const int nt = ((ep.hd / 16) % 2 == 0 && tiles / 2 >= 128) ? 2 : 1;
    const int blocks = tiles / nt;
    const bool w8 = blocks * 4 < 4096 && nks >= 64;
#define RI_ROPE(NT_) do { \
        if (w8) gemm_skinny_bf16_kernel<MT, NT_, 8, bf16_t, false, true, true><<<dim3(blocks, 1), 512, 0, stream>>>(A, lda, W, K, C, ldc, M, N, K, nks, 0, ep); \
        else gemm_skinny_bf16_kernel<MT, NT_, 4, bf16_t, false, true, true><<<dim3(blocks, 1), 256, 0, stream>>>(A, lda, W, K, C, ldc, M, N, K, nks, 0, ep); } while (0)
    if (nt == 2) RI_ROPE(2);
    else RI_ROPE(1);
#undef RI_ROPE
    RI_LAUNCHED("ri_gemm_qkv_rope");
    return 0;
}

// Row r of the permuted fused q/k/v weight (what ri_gemm_qkv_rope reads, in tile order) is row
// qkv_rope_row_order(r) of the checkpoint's [q; k; v] matrix.
extern "C" int ri_qkv_rope_row_order(int r, int hd) {
    const int head = r / hd, within = r % hd, j = within >> 4, rr = within & 15;
    return head * hd + (rr < 8 ? 8 * j + rr : hd / 2 + 8 * j + (rr - 8));
}

// q/k/v projection of M <= 64 single tokens with rotation and cache write fused (see RopeEpilogue).
// W: the row-permuted weight in tile order.  C [M, ldc]: receives rotated q in its first H*hd columns.
extern "C" int ri_gemm_qkv_rope(const void* A, int lda, const void* W, void* C, int ldc, int M, int K,
                                int H, int Hkv, int hd, const float* cos_t, const float* sin_t, int table_rows,
                                const int* positions, const int* row_of_token, void* kc, void* vc,
                                int num_pages, const int* table, int max_blocks, int page, hipStream_t stream) {
    const int N = (H + 2 * Hkv) * hd;
    RI_REQUIRE(M >= 1 && M <= 64, "ri_gemm_qkv_rope: M=%d not in [1, 64]", M);
    RI_REQUIRE(H > 0 && Hkv > 0 && hd > 0 && hd % 16 == 0 && K > 0 && K % 32 == 0, "ri_gemm_qkv_rope: needs head size %% 16 == 0 and K %% 32 == 0 (hd=%d K=%d)", hd, K);
    RI_REQUIRE(lda >= K && lda % 8 == 0 && ldc >= H * hd, "ri_gemm_qkv_rope: bad leading dimensions");
    RI_REQUIRE(page > 0 && max_blocks > 0 && num_pages > 0 && table_rows > 0, "ri_gemm_qkv_rope: bad cache sizes");
    RI_REQUIRE(A && W && C && cos_t && sin_t && positions && row_of_token && kc && vc && table, "ri_gemm_qkv_rope: null pointer");
    RI_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "ri_gemm_qkv_rope: operands must be 16-byte aligned");
    RopeEpilogue ep{cos_t, sin_t, positions, row_of_token, table, max_blocks, (bf16_t*)kc, (bf16_t*)vc, H, Hkv, hd, page};
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    if (M <= 16) return launch_skinny_rope<1>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, stream);
    if (M <= 32) return launch_skinny_rope<2>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, stream);
    if (M <= 48) return launch_skinny_rope<3>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, stream);
    return launch_skinny_rope<4>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, stream);
}

// The two products that follow a norm, for at most four single tokens, with the norm folded in
// (NormPrologue): x [M, K] and delta [parts][M][K] (part_stride elements apart; parts 0..8) are
// 32-bit, w_norm [K] is 32-bit or bfloat16, x_out [M, K] receives x + delta and must not be x.
static int norm_prologue(const float* x, const float* delta, int parts, long long part_stride, const void* w_norm,
                         int w_dtype, float eps, float* x_out, int M, int K, NormPrologue* np, const char* who) {
    RI_REQUIRE(M >= 1 && M <= 4, "%s: M=%d not in [1, 4]", who, M);
    RI_REQUIRE((long long)M * K * 2 <= 48 * 1024, "%s: M * K = %d * %d does not fit the 48 KB of LDS this form uses", who, M, K);
    RI_REQUIRE(K > 0 && K % 32 == 0, "%s: K=%d must be a positive multiple of 32", who, K);
    RI_REQUIRE(x && w_norm && x_out && x_out != x, "%s: null pointer, or x_out is x", who);
    RI_REQUIRE(parts >= 0 && parts <= 8 && (parts == 0 || (delta && part_stride >= (long long)M * K && part_stride % 4 == 0)),
               "%s: bad partial sums (parts=%d)", who, parts);
    RI_REQUIRE(eps > 0.f, "%s: eps must be > 0", who);
    RI_REQUIRE(w_dtype == RI_F32 || w_dtype == RI_BF16, "%s: the norm's weight must be float32 or bfloat16", who);
    RI_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)delta % 16 == 0 && (uintptr_t)w_norm % 16 == 0 && (uintptr_t)x_out % 16 == 0,
               "%s: operands must be 16-byte aligned", who);
    *np = NormPrologue{x, delta, parts, (size_t)part_stride, w_dtype == RI_F32 ? (const float*)w_norm : nullptr,
                       w_dtype == RI_BF16 ? (const bf16_t*)w_norm : nullptr, eps, x_out};
    return 0;
}

// ri_gemm_qkv_rope with the norm before it folded in.
extern "C" int ri_gemm_qkv_rope_norm(const float* x, const float* delta, int parts, long long part_stride,
                                     const void* w_norm, int w_dtype, float eps, float* x_out,
                                     const void* W, void* C, int ldc, int M, int K,
                                     int H, int Hkv, int hd, const float* cos_t, const float* sin_t, int table_rows,
                                     const int* positions, const int* row_of_token, void* kc, void* vc,
                                     int num_pages, const int* table, int max_blocks, int page, hipStream_t stream) {
    const int N = (H + 2 * Hkv) * hd;
    NormPrologue np;
    if (int rc = norm_prologue(x, delta, parts, part_stride, w_norm, w_dtype, eps, x_out, M, K, &np, "ri_gemm_qkv_rope_norm")) return rc;
    RI_REQUIRE(H > 0 && Hkv > 0 && hd > 0 && hd % 16 == 0, "ri_gemm_qkv_rope_norm: needs head size %% 16 == 0 (hd=%d)", hd);
    RI_REQUIRE(ldc >= H * hd, "ri_gemm_qkv_rope_norm: bad leading dimension");
    RI_REQUIRE(page > 0 && max_blocks > 0 && num_pages > 0 && table_rows > 0, "ri_gemm_qkv_rope_norm: bad cache sizes");
    RI_REQUIRE(W && C && cos_t && sin_t && positions && row_of_token && kc && vc && table, "ri_gemm_qkv_rope_norm: null pointer");
    RI_REQUIRE((uintptr_t)W % 16 == 0, "ri_gemm_qkv_rope_norm: operands must be 16-byte aligned");
    RopeEpilogue ep{cos_t, sin_t, positions, row_of_token, table, max_blocks, (bf16_t*)kc, (bf16_t*)vc, H, Hkv, hd, page};
    const bf16_t* w = (const bf16_t*)W;
    const int tiles = N / 16, nks = K / 32;
    const int nt = ((hd / 16) % 2 == 0 && tiles / 2 >= 128) ? 2 : 1;      // as launch_skinny_rope
    const int blocks = tiles / nt;
    const bool w8 = blocks * 4 < 4096 && nks >= 64;
#define RI_ROPE_NORM(NT_) do { \
        if (w8) gemm_skinny_bf16_kernel<1, NT_, 8, bf16_t, false, true, true, true><<<dim3(blocks, 1), 512, (size_t)M * K * 2, stream>>>((const bf16_t*)x, K, w, K, (bf16_t*)C, ldc, M, N, K, nks, 0, ep, np); \
        else gemm_skinny_bf16_kernel<1, NT_, 4, bf16_t, false, true, true, true><<<dim3(blocks, 1), 256, (size_t)M * K * 2, stream>>>((const bf16_t*)x, K, w, K, (bf16_t*)C, ldc, M, N, K, nks, 0, ep, np); } while (0)
    if (nt == 2) RI_ROPE_NORM(2);
    else RI_ROPE_NORM(1);
#undef RI_ROPE_NORM
    RI_LAUNCHED("ri_gemm_qkv_rope_norm");
    return 0;
}

// C[M, I] = silu(n . gate^T) * (n . up^T) with n = rmsnorm(x + delta) * w_norm made in the kernel;
// W: the stacked [2I, K] weight in tile order (I % 16 == 0).
extern "C" int ri_gemm_skinny_norm_swiglu(const float* x, const float* delta, int parts, long long part_stride,
                                          const void* w_norm, int w_dtype, float eps, float* x_out,
                                          const void* W, void* C, int ldc, int M, int I, int K, hipStream_t stream) {
    NormPrologue np;
    if (int rc = norm_prologue(x, delta, parts, part_stride, w_norm, w_dtype, eps, x_out, M, K, &np, "ri_gemm_skinny_norm_swiglu")) return rc;
    RI_REQUIRE(I > 0 && I % 16 == 0 && ldc >= I, "ri_gemm_skinny_norm_swiglu: I=%d must be a positive multiple of 16, ldc >= I", I);
    RI_REQUIRE(W && C && (uintptr_t)W % 16 == 0, "ri_gemm_skinny_norm_swiglu: null or unaligned pointer");
    int nt = 1, parts_same = 1;
    skinny_plan(M, I, K, true, true, false, 1, &nt, &parts_same);
    const int nks = K / 32;
    const int blocks = (I / 16 + nt - 1) / nt;
    const bool w8 = blocks * 4 < 4096 && nks >= 64;                        // as launch_skinny_nt
    const bf16_t* w = (const bf16_t*)W;
#define RI_SWIGLU_NORM(NT_) do { \
        if (w8) gemm_skinny_bf16_kernel<1, NT_, 8, bf16_t, true, true, false, true><<<dim3(blocks, 1), 512, (size_t)M * K * 2, stream>>>((const bf16_t*)x, K, w, K, (bf16_t*)C, ldc, M, I, K, nks, 0, RopeEpilogue{}, np); \
        else gemm_skinny_bf16_kernel<1, NT_, 4, bf16_t, true, true, false, true><<<dim3(blocks, 1), 256, (size_t)M * K * 2, stream>>>((const bf16_t*)x, K, w, K, (bf16_t*)C, ldc, M, I, K, nks, 0, RopeEpilogue{}, np); } while (0)
    if (nt == 2) RI_SWIGLU_NORM(2);
    else RI_SWIGLU_NORM(1);
#undef RI_SWIGLU_NORM
    RI_LAUNCHED("ri_gemm_skinny_norm_swiglu");
    return 0;
}

// How many slices of K to give to separate blocks so that a product with few output columns
// still fills the chip; the slices' partial sums are added by the consumer (add_rmsnorm).
extern "C" int ri_gemm_skinny_parts(int M, int N, int K) {
    int nt = 1, parts = 1;
    skinny_plan(M, N, K, false, N % 16 == 0 && K % 32 == 0, true, 0, &nt, &parts);
    return parts;
}

// swiglu != 0: W is [2N, K] (gate rows, then up rows) and C[M, N] = silu(A.gate^T) * (A.up^T)
// parts > 1: C is a float32 stack [parts][M][ldc] (part_stride elements apart) of partial sums
// tiled != 0: W points to the copy in tile order (ldw is ignored)
extern "C" int ri_gemm_skinny_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc,
                                   int M, int N, int K, int out_dtype, int swiglu, int parts,
                                   long long part_stride, int tiled, hipStream_t stream) {
    RI_REQUIRE(!tiled || (N % 16 == 0 && K % 32 == 0), "ri_gemm_skinny_bf16: the tiled layout needs N %% 16 == 0 and K %% 32 == 0");
    RI_REQUIRE(parts >= 1 && parts <= 64, "ri_gemm_skinny_bf16: parts=%d not in [1, 64]", parts);
    RI_REQUIRE(parts == 1 || (out_dtype == RI_F32 && !swiglu && part_stride >= (long long)M * ldc),
               "ri_gemm_skinny_bf16: partial sums need a float32 stack and no activation");
    const size_t ps = parts > 1 ? (size_t)part_stride : 0;
    RI_REQUIRE(M >= 1 && M <= 64, "ri_gemm_skinny_bf16: M=%d not in [1, 64]", M);
    RI_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "ri_gemm_skinny_bf16: K=%d must be a positive multiple of 8 (N=%d)", K, N);
    RI_REQUIRE(lda >= K && (tiled || ldw >= K) && ldc >= N && lda % 8 == 0 && (tiled || ldw % 8 == 0), "ri_gemm_skinny_bf16: leading dimensions must be >= K and multiples of 8");
    RI_REQUIRE(A && W && C, "ri_gemm_skinny_bf16: null pointer");
    RI_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "ri_gemm_skinny_bf16: operands must be 16-byte aligned");
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    if (swiglu) {
        RI_REQUIRE(out_dtype == RI_BF16, "ri_gemm_skinny_bf16: the fused SwiGLU form writes bfloat16");
        return dispatch_skinny<bf16_t, true>(a, lda, w, ldw, (bf16_t*)C, ldc, M, N, K, 1, 0, tiled, stream);
    }
    if (out_dtype == RI_BF16) return dispatch_skinny<bf16_t, false>(a, lda, w, ldw, (bf16_t*)C, ldc, M, N, K, 1, 0, tiled, stream);
    if (out_dtype == RI_F32) return dispatch_skinny<float, false>(a, lda, w, ldw, (float*)C, ldc, M, N, K, parts, ps, tiled, stream);
    return ri_fail("ri_gemm_skinny_bf16: unknown output dtype %d", out_dtype);
}
