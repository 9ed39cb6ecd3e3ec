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
// gemm_rows_f32: the exact path's product for few rows (decoding; 16 a pass), where the tiled kernel
// above would leave most of its 64 x 64 tile and of the chip idle.  The weights are streamed
// once, 16 bytes a lane and row; a block brings 512 values of every activation row into LDS and
// its four waves multiply them with four weight rows each.  Sums are kept in 64-bit as in the tiled
// kernel; a lane adds its share of K in a fixed order and the lanes are added in a fixed tree, so
// a row's result depends neither on the other rows nor on their number.  K % 4 == 0.
// ---------------------------------------------------------------------------
template <int MR, int NB>
__global__ __launch_bounds__(256) void gemm_rows_f32_kernel(
        const float* __restrict__ A, int lda, const float* __restrict__ W, int ldw,
        float* __restrict__ C, int ldc, int M, int N, int K) {
    constexpr int KC = 512;
    __shared__ __align__(16) float xs[MR][KC];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = ((int)blockIdx.x * 4 + wave) * NB;
    const float* wrow[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) wrow[j] = W + (size_t)min(n0 + j, N - 1) * ldw;
    double acc[MR][NB];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int j = 0; j < NB; ++j) acc[m][j] = 0.0;
    // The weights are read once (the streaming form of the load) and a stretch ahead: while the
    // sums of one stretch are made, the loads of the next are under way.
    auto ask = [&](int k0, float4 (&w)[KC / 256][NB]) {
#pragma unroll
        for (int i = 0; i < KC / 256; ++i) {
            const int k = k0 + i * 256 + lane * 4;
#pragma unroll
            for (int j = 0; j < NB; ++j)
                w[i][j] = k < K ? ld_stream16<float4>(wrow[j] + k) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto stretch = [&](int k0, const float4 (&w)[KC / 256][NB], float4 (&w_next)[KC / 256][NB]) {
        __syncthreads();                                        // the last stretch has been read
        for (int e = threadIdx.x * 4; e < MR * KC; e += 256 * 4) {
            const int m = e / KC, k = k0 + e % KC;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < M && k < K) v = *reinterpret_cast<const float4*>(A + (size_t)m * lda + k);
            *reinterpret_cast<float4*>(&xs[m][e % KC]) = v;
        }
        ask(k0 + KC, w_next);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < KC / 256; ++i) {
            const int kk = i * 256 + lane * 4;
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const float4 x = *reinterpret_cast<const float4*>(&xs[m][kk]);
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    double a = acc[m][j];
                    a = fma((double)x.x, (double)w[i][j].x, a);
                    a = fma((double)x.y, (double)w[i][j].y, a);
                    a = fma((double)x.z, (double)w[i][j].z, a);
                    a = fma((double)x.w, (double)w[i][j].w, a);
                    acc[m][j] = a;
                }
            }
        }
    };
    float4 wa[KC / 256][NB], wb[KC / 256][NB];
    ask(0, wa);
    for (int k0 = 0; k0 < K; k0 += 2 * KC) {
        stretch(k0, wa, wb);
        if (k0 + KC < K) stretch(k0 + KC, wb, wa);
    }
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            double a = acc[m][j];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) a += __shfl_xor(a, o, 64);
            if (lane == 0 && m < M && n0 + j < N) C[(size_t)m * ldc + n0 + j] = (float)a;
        }
}

extern "C" int ri_gemm_rows_f32(const float* A, int lda, const float* W, int ldw, float* C, int ldc,
                                int M, int N, int K, hipStream_t stream) {
    RI_REQUIRE(M >= 1 && M <= 64 && N > 0 && K > 0 && K % 4 == 0, "ri_gemm_rows_f32: needs 1..64 rows and K %% 4 == 0 (M=%d N=%d K=%d)", M, N, K);
    RI_REQUIRE(lda >= K && ldw >= K && ldc >= N && lda % 4 == 0 && ldw % 4 == 0, "ri_gemm_rows_f32: leading dimensions must be >= K and multiples of 4");
    RI_REQUIRE(A && W && C && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0, "ri_gemm_rows_f32: null or unaligned pointer");
    // 16 rows a pass: more rows stream the weights once more for every 16 (still ahead of the tiled kernel).
    // A wave owns four columns, or two where four would leave compute units without a block's worth
    // of loads in flight (a row's sums do not depend on that choice: a lane adds its share of K in
    // the same order either way).
    const bool narrow = (N + 15) / 16 < 1024;
    const int blocks = narrow ? (N + 7) / 8 : (N + 15) / 16;
    for (int m0 = 0; m0 < M; m0 += 16) {
        const int m = min(16, M - m0);
        const float* a = A + (size_t)m0 * lda;
        float* c = C + (size_t)m0 * ldc;
#define RI_ROWS_F32(MR_) do { \
        if (narrow) gemm_rows_f32_kernel<MR_, 2><<<blocks, 256, 0, stream>>>(a, lda, W, ldw, c, ldc, m, N, K); \
        else gemm_rows_f32_kernel<MR_, 4><<<blocks, 256, 0, stream>>>(a, lda, W, ldw, c, ldc, m, N, K); } while (0)
        if (m <= 4) RI_ROWS_F32(4);
        else if (m <= 8) RI_ROWS_F32(8);
        else RI_ROWS_F32(16);
#undef RI_ROWS_F32
    }
    RI_LAUNCHED("ri_gemm_rows_f32");
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

// A norm between two few-row products needs no kernel of its own.  rmsnorm(x) * w followed by a
// product is the product of (x * w) scaled row by row with rsqrt(mean(x^2) + eps), so:
//
// RESID (the product before the norm: o_proj, down_proj): no split over K between blocks, so a
// block holds whole sums for its 16 columns.  Its epilogue adds them to the 32-bit residual stream
// in place (x += sums), writes (x * w_norm) rounded once to bfloat16 as the next product's operand,
// and leaves the sum of x^2 over its columns in ssq[m][N / 16]: one slot for every 16 columns,
// the block's sum in the first of its slots.
struct ResidualEpilogue {
    float* x;                                      // [M][N] residual stream, updated in place; null: plain store to C
    const float* w32; const bf16_t* w16;           // the following norm's weight [N], one of the two
    bf16_t* a_out;                                 // [M][N]  (x * w)
    float* ssq;                                    // [M][N / 16] partial sums of x^2 ([M][N / 8] with halves)
    int halves;                                    // 1: a block owns 8 columns (half a tile: the rows of W its
                                                   // lanes do not own are not read), so that a product of few
                                                   // columns still has a block for every CU
};
// SCALE (the product after the norm: q/k/v, gate/up, the output head): the operand rows are
// (x * w_norm); the finished sums of row m are multiplied by rsqrt(sum_p ssq[m][p] / dim + eps)
// before rotation, activation or store.  The partial sums are asked for before the weights.
struct RowScale {
    const float* ssq; int parts; float eps; float inv_dim;    // ssq null: rows are used as they are
};

// NT: tiles of 16 rows of W a block owns.  With more than 16 activation rows (MT > 1) the
// activations are as much traffic through L1 as the weights; a wave that multiplies the same
// activation fragments with NT weight tiles needs them NT times less often.
template <int MT, int NT, int WAVES, typename TO, bool SWIGLU, bool TILED, bool ROPE = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_bf16_kernel(
        const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
        TO* __restrict__ C, int ldc, int M, int N, int K, int ks_per_block, size_t part_stride,
        RopeEpilogue ep = RopeEpilogue{}, RowScale sc = RowScale{}, ResidualEpilogue re = ResidualEpilogue{}) {
    constexpr int NW = SWIGLU ? 2 * NT : NT;                 // weight tiles streamed: [gate tiles | up tiles]
    constexpr int U = (MT == 1 && NW == 1) ? 8 : ((MT + NW <= 3) ? 4 : 2);   // k-steps in flight per wave
    __shared__ float red[WAVES > 1 ? (WAVES - 1) * NW * 256 : 1];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same in all lanes of a wave
    const int col = lane & 15, grp = lane >> 4;
    // SCALE: the rows' factors.  The partial sums are many (one for every 16 columns of the product
    // that made them) and the kernel's end waits for them, so all waves fetch them together at
    // the start, 16 bytes a lane, and leave the factors in LDS for the waves that finish the tiles.
    __shared__ float rs_lds[MT * 16];
    if (sc.ssq) {
        const bool vec = (sc.parts & 3) == 0 && ((uintptr_t)sc.ssq & 15) == 0;
        for (int r = wave; r < M; r += WAVES) {
            const float* row = sc.ssq + (size_t)r * sc.parts;
            float ss = 0.f;
            if (vec) {
                for (int p = lane * 4; p < sc.parts; p += 256) {
                    const float4 v = *reinterpret_cast<const float4*>(row + p);
                    ss += (v.x + v.y) + (v.z + v.w);
                }
            } else {
                for (int p = lane; p < sc.parts; p += 64) ss += row[p];
            }
            ss = wave_sum(ss);
            if (lane == 0) rs_lds[r] = rsqrtf(ss * sc.inv_dim + sc.eps);
        }
    }
    // RESID: what the epilogue adds to and multiplies with (this lane's four columns of the residual
    // stream and of the norm's weight) is asked for now: a chain of loads at the end of a kernel
    // of 10 us costs a tenth of it.
    float4 re_x[NT], re_w[NT];
    if constexpr (!SWIGLU && !ROPE && TILED && sizeof(TO) == 4) {
        if (re.x && wave < MT) {
            const int m = wave * 16 + col;
#pragma unroll
            for (int a = 0; a < NT; ++a) {
                const int n = (re.halves ? (int)blockIdx.x >> 1 : (int)blockIdx.x * NT + a) * 16 + grp * 4;
                re_x[a] = re_w[a] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (m < M && n < N && (!re.halves || (grp >> 1) == ((int)blockIdx.x & 1))) {
                    re_x[a] = *reinterpret_cast<const float4*>(re.x + (size_t)m * N + n);
                    if (re.w16) {
                        const uint2 w4 = *reinterpret_cast<const uint2*>(re.w16 + n);
                        re_w[a] = make_float4(bf16_to_f32((bf16_t)(w4.x & 0xffff)), bf16_to_f32((bf16_t)(w4.x >> 16)),
                                              bf16_to_f32((bf16_t)(w4.y & 0xffff)), bf16_to_f32((bf16_t)(w4.y >> 16)));
                    } else {
                        re_w[a] = *reinterpret_cast<const float4*>(re.w32 + n);
                    }
                }
            }
        }
    }
    const int ntiles = (N + 15) / 16;
    const int nks_all = (K + 31) / 32;
    const bf16_t* wp[NW];
#pragma unroll
    for (int a = 0; a < NW; ++a) {
        // tile index among the rows of W; rows beyond N are read (clamped) but never stored
        const int tile = min((re.halves ? (int)blockIdx.x >> 1 : (int)blockIdx.x * NT + (a % NT)), ntiles - 1);
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
            const bool ok = ks < ks_end && ks * 32 + grp * 8 < K    // K % 8 == 0: a lane's 8 values are in or out together
                && (!re.halves || (col >> 3) == ((int)blockIdx.x & 1));
            const size_t wk = TILED ? (size_t)ks * 512 : (size_t)ks * 32;   // a tile of 16 x 32 has 512 values
#pragma unroll
            for (int a = 0; a < NW; ++a) wf[a][u] = ok ? ld_stream16<gbf16x8_t>(wp[a] + wk) : zero;
        }
    };
    for (int ks0 = ks_begin + wave; ks0 < ks_end; ks0 += WAVES * U) {
        gbf16x8_t wf[NW][U], xf[MT][U];
        load_weights(ks0, wf);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ks = ks0 + u * WAVES;
            const int k = ks * 32;
            const bool ok = ks < ks_end && k + grp * 8 < K;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                xf[mt][u] = (ok && xok[mt]) ? *reinterpret_cast<const gbf16x8_t*>(xrow[mt] + k) : zero;
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
    if (sc.ssq) {
        if (WAVES == 1) __syncthreads();                   // else the sums' barrier above has published rs_lds
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            if (WAVES == 1 || wave == mt) {
                const float rs = rs_lds[min(mt * 16 + col, M - 1)];
#pragma unroll
                for (int a = 0; a < NW; ++a)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[a][mt][i] *= rs;
            }
    }
    if constexpr (!SWIGLU && !ROPE && TILED && sizeof(TO) == 4) {
        if (re.x) {
            // whole sums of 16 * NT columns (N % 16 == 0): finish the residual stream and prepare the next norm
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (WAVES > 1 && wave != mt) continue;
                const int m = mt * 16 + col;
                const bool live = m < M;
                float sq = 0.f;
#pragma unroll
                for (int a = 0; a < NT; ++a) {
                    const int n = (re.halves ? (int)blockIdx.x >> 1 : (int)blockIdx.x * NT + a) * 16 + grp * 4;
                    if (live && n < N && (!re.halves || (grp >> 1) == ((int)blockIdx.x & 1))) {
                        float* xp = re.x + (size_t)m * N + n;
                        const float4 xv = re_x[a];            // this wave's own tile (mt == wave): fetched at the start
                        float v[4] = {xv.x + acc[a][mt][0], xv.y + acc[a][mt][1], xv.z + acc[a][mt][2], xv.w + acc[a][mt][3]};
                        *reinterpret_cast<float4*>(xp) = make_float4(v[0], v[1], v[2], v[3]);
                        const float wv[4] = {re_w[a].x, re_w[a].y, re_w[a].z, re_w[a].w};
                        float aw[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) { sq = fmaf(v[i], v[i], sq); aw[i] = v[i] * wv[i]; }
                        VecLoad4::st(re.a_out + (size_t)m * N + n, aw);
                    }
                }
                sq += __shfl_xor(sq, 16, 64);               // the four column groups of a row
                sq += __shfl_xor(sq, 32, 64);
                if (live && grp == 0) {
                    // one slot for every 16 columns (8 with halves): the block's sum in its first, zeros in the others
                    float* slot = re.ssq + ((size_t)m * gridDim.x + blockIdx.x) * NT;
#pragma unroll
                    for (int a = 0; a < NT; ++a) slot[a] = a == 0 ? sq : 0.f;
                }
            }
            return;
        }
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
        // Tiles a wave owns of each half (it asks for the activations once for all of them), while
        // the blocks stay enough.  Measured, us, one / two tiles a wave at 1, 8, 16 rows: 896 tiles
        // (14336 x 4096) 40.0 41.7 46.2 / 40.8 40.9 42.4; 864 (13824 x 5120) 48.4 50.9 58.2 / 46.9
        // 48.5 51.8; 688 (11008 x 4096) 30.8 32.6 37.1 / 36.9 38.0 39.1; 1792 (28672 x 8192) 142
        // 144 161 / 149 152 157.  17..32 rows, two / four tiles at 17, 24, 32 rows: 688 tiles 41.0
        // 42.5 45.2 / 39.5 40.4 42.5; 864: 53.8 58.4 63.2 / 51.4 52.8 54.8.
        if (mt == 1) {
            if (tiles / 2 >= 416 && (tiles / 2 <= 512 || M > 8)) nt = 2;
        } else {
            const int need = mt == 2 ? 160 : 224;
            while (nt * 2 <= 4 && tiles / (nt * 2) >= need) nt *= 2;
        }
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
                             int M, int N, int K, int parts, size_t part_stride, const RowScale& sc, hipStream_t stream) {
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
            gemm_skinny_bf16_kernel<1, 1, 16, TO, false, TILED><<<grid, 1024, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, ks_per_block, part_stride, RopeEpilogue{}, sc);
            return;
        }
    }
    if constexpr (MT <= 2) {
        if (waves == 8) {
            gemm_skinny_bf16_kernel<MT, NT, 8, TO, SWIGLU, TILED><<<grid, 512, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, ks_per_block, part_stride, RopeEpilogue{}, sc);
            return;
        }
    }
    gemm_skinny_bf16_kernel<MT, NT, 4, TO, SWIGLU, TILED><<<grid, 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, ks_per_block, part_stride, RopeEpilogue{}, sc);
}

template <int MT, typename TO, bool SWIGLU, bool TILED>
static int launch_skinny(const bf16_t* A, int lda, const bf16_t* W, int ldw, TO* C, int ldc,
                         int M, int N, int K, int parts, size_t part_stride, const RowScale& sc, hipStream_t stream) {
    if (MT == 1 && !SWIGLU && (N + 15) / 16 >= 2048) {
        // a very wide product (the output head): four tiles per block even for few rows, so that
        // the activation fragments are fetched a quarter as often; blocks remain plentiful
        const int nks = (K + 31) / 32;
        const int wide_blocks = ((N + 15) / 16 + 3) / 4;
        gemm_skinny_bf16_kernel<1, 4, 4, TO, false, TILED><<<dim3(wide_blocks, parts), 256, 0, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, (nks + parts - 1) / parts, part_stride, RopeEpilogue{}, sc);
        RI_LAUNCHED("ri_gemm_skinny_bf16");
        return 0;
    }
    int nt = 1, parts_same = 1;
    skinny_plan(M, N, K, SWIGLU, TILED, parts > 1, parts, &nt, &parts_same);
#define RI_SKINNY_NT(NT_) launch_skinny_nt<MT, NT_, TO, SWIGLU, TILED>(A, lda, W, ldw, C, ldc, M, N, K, parts, part_stride, sc, stream)
    if (nt == 4) RI_SKINNY_NT(4);
    else if (nt == 2) RI_SKINNY_NT(2);
    else RI_SKINNY_NT(1);
#undef RI_SKINNY_NT
    RI_LAUNCHED("ri_gemm_skinny_bf16");
    return 0;
}

template <typename TO, bool SWIGLU>
static int dispatch_skinny(const bf16_t* A, int lda, const bf16_t* W, int ldw, TO* C, int ldc,
                           int M, int N, int K, int parts, size_t part_stride, int tiled, const RowScale& sc, hipStream_t stream) {
#define RI_SKINNY(MT) (tiled ? launch_skinny<MT, TO, SWIGLU, true>(A, lda, W, ldw, C, ldc, M, N, K, parts, part_stride, sc, stream) \
                             : launch_skinny<MT, TO, SWIGLU, false>(A, lda, W, ldw, C, ldc, M, N, K, parts, part_stride, sc, stream))
    if (M <= 16) return RI_SKINNY(1);
    if (M <= 32) return RI_SKINNY(2);
    if (M <= 48) return RI_SKINNY(3);
    return RI_SKINNY(4);
#undef RI_SKINNY
}

template <int MT>
static int launch_skinny_rope(const bf16_t* A, int lda, const bf16_t* W, bf16_t* C, int ldc,
                              int M, int N, int K, const RopeEpilogue& ep, const RowScale& sc, hipStream_t stream) {
    // The product cannot be split over K (the epilogue needs whole sums), so the number of blocks
    // is all the parallelism there is.  Two tiles (of one head) per wave halve what the waves ask
    // for of the activations; that pays where it leaves 128 blocks or more (measured: 384 tiles,
    // 8..64 rows: 13.6 -> 12.5 us .. 40 -> 27 us; with 192 tiles one tile per wave is faster).
    const int tiles = N / 16, nks = K / 32;
    // (four tiles per wave at 49..64 rows: 2.5 % slower at 384 tiles, 1 % faster at 192)
    // (160 or 192 blocks of two tiles leave compute units idle: with up to four rows one tile a wave
    // makes a decode step 2.5 % faster at 320 tiles and 4.5 % at 384; with eight rows 1.4 % slower)
    // (256..415 blocks of two tiles, up to eight rows, us at 1, 4, 8 rows, one / two tiles a wave:
    // 768 tiles (12288 x 4096) 20.4 19.7 21.4 / 21.8 23.2 24.0; 640 (10240 x 8192) 32.7 33.3 37.7 /
    // 35.7 36.7 39.1; but 960 (15360 x 5120) 28.1 29.5 32.9 / 27.8 28.1 30.0)
    const int pairs = tiles / 2;
    const int nt = ((ep.hd / 16) % 2 == 0 && pairs >= 128 && (pairs >= 416 || M > (pairs >= 256 ? 8 : 4))) ? 2 : 1;
    const int blocks = tiles / nt;
    const bool w8 = blocks * 4 < 4096 && nks >= 64;
#define RI_ROPE(NT_) do { \
        if (w8) gemm_skinny_bf16_kernel<MT, NT_, 8, bf16_t, false, true, true><<<dim3(blocks, 1), 512, 0, stream>>>(A, lda, W, K, C, ldc, M, N, K, nks, 0, ep, sc); \
        else gemm_skinny_bf16_kernel<MT, NT_, 4, bf16_t, false, true, true><<<dim3(blocks, 1), 256, 0, stream>>>(A, lda, W, K, C, ldc, M, N, K, nks, 0, ep, sc); } while (0)
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

// ssq null: no row factors.  Else ssq [M][ssq_parts] float32 and the rows of A are (x * w_norm) of
// a norm over K elements with this eps (see RowScale).
static int row_scale(const float* ssq, int ssq_parts, float eps, int K, RowScale* sc, const char* who) {
    *sc = RowScale{nullptr, 0, 0.f, 0.f};
    if (!ssq) return 0;
    RI_REQUIRE(ssq_parts >= 1 && ssq_parts <= 65536 && eps > 0.f, "%s: bad row factors (parts=%d eps=%g)", who, ssq_parts, (double)eps);
    *sc = RowScale{ssq, ssq_parts, eps, 1.f / (float)K};
    return 0;
}

// q/k/v projection of M <= 64 single tokens with rotation and cache write fused (see RopeEpilogue).
// W: the row-permuted weight in tile order.  C [M, ldc]: receives rotated q in its first H*hd columns.
extern "C" int ri_gemm_qkv_rope(const void* A, int lda, const void* W, void* C, int ldc, int M, int K,
                                int H, int Hkv, int hd, const float* cos_t, const float* sin_t, int table_rows,
                                const int* positions, const int* row_of_token, void* kc, void* vc,
                                int num_pages, const int* table, int max_blocks, int page,
                                const float* ssq, int ssq_parts, float eps, hipStream_t stream) {
    RowScale sc;
    if (int rc = row_scale(ssq, ssq_parts, eps, K, &sc, "ri_gemm_qkv_rope")) return rc;
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
    if (M <= 16) return launch_skinny_rope<1>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, sc, stream);
    if (M <= 32) return launch_skinny_rope<2>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, sc, stream);
    if (M <= 48) return launch_skinny_rope<3>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, sc, stream);
    return launch_skinny_rope<4>(a, lda, w, (bf16_t*)C, ldc, M, N, K, ep, sc, stream);
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
// ssq: row factors of a norm folded into this product (see RowScale), or null
extern "C" int ri_gemm_skinny_bf16(const void* A, int lda, const void* W, int ldw, void* C, int ldc,
                                   int M, int N, int K, int out_dtype, int swiglu, int parts,
                                   long long part_stride, int tiled, const float* ssq, int ssq_parts, float eps,
                                   hipStream_t stream) {
    RowScale sc;
    if (int rc = row_scale(ssq, ssq_parts, eps, K, &sc, "ri_gemm_skinny_bf16")) return rc;
    RI_REQUIRE(!ssq || parts == 1, "ri_gemm_skinny_bf16: row factors go with whole sums, not with slices of K");
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
        return dispatch_skinny<bf16_t, true>(a, lda, w, ldw, (bf16_t*)C, ldc, M, N, K, 1, 0, tiled, sc, stream);
    }
    if (out_dtype == RI_BF16) return dispatch_skinny<bf16_t, false>(a, lda, w, ldw, (bf16_t*)C, ldc, M, N, K, 1, 0, tiled, sc, stream);
    if (out_dtype == RI_F32) return dispatch_skinny<float, false>(a, lda, w, ldw, (float*)C, ldc, M, N, K, parts, ps, tiled, sc, stream);
    return ri_fail("ri_gemm_skinny_bf16: unknown output dtype %d", out_dtype);
}

// The product before a norm, for M <= 16 rows (see ResidualEpilogue):
//   x[M, N] += A[M, K] . W[N, K]^T;  a_out[M, N] = x * w_norm (bfloat16);  ssq[M][N / 16] = partial sums of x^2
// W in tile order (N % 16 == 0, K % 32 == 0).  No split over K between blocks: the eight waves of a
// block share K.  One weight tile a block: with two the activations are asked for half as often, but
// products of 4,096 columns then leave half the chip idle (measured, 8 rows, us: 4096 x 14336: 25.2
// against 31.4; 4096 x 4096: 9.1 against 10.4; the split product and the norm's kernel it replaces:
// 27.7 and 13.1).
extern "C" int ri_gemm_skinny_residual_max_rows() { return 16; }
// Half a tile a block where the tiles are at most half as many as the CUs (2,048 columns: decode
// at batch 8 of the 1B shape 2 % faster; 3,072 columns: 9 % slower).
// (with up to four rows half tiles at 4,096 columns too: 7 % of a decode step slower)
static int residual_halves(int N) { return N / 16 <= 128 ? 1 : 0; }
// slots of partial sums a row: one for every 16 columns, or for every 8 where blocks own half tiles
extern "C" int ri_gemm_skinny_residual_parts(int N) { return residual_halves(N) ? N / 8 : N / 16; }

extern "C" int ri_gemm_skinny_residual(const void* A, int lda, const void* W, int M, int N, int K,
                                       float* x, const void* w_norm, int w_dtype, void* a_out, float* ssq,
                                       hipStream_t stream) {
    RI_REQUIRE(M >= 1 && M <= 16, "ri_gemm_skinny_residual: M=%d not in [1, 16]", M);
    RI_REQUIRE(N > 0 && N % 16 == 0 && K > 0 && K % 32 == 0, "ri_gemm_skinny_residual: needs N %% 16 == 0 and K %% 32 == 0 (N=%d K=%d)", N, K);
    RI_REQUIRE(lda >= K && lda % 8 == 0, "ri_gemm_skinny_residual: bad leading dimension");
    RI_REQUIRE(A && W && x && w_norm && a_out && ssq, "ri_gemm_skinny_residual: null pointer");
    RI_REQUIRE(w_dtype == RI_F32 || w_dtype == RI_BF16, "ri_gemm_skinny_residual: the norm's weight must be float32 or bfloat16");
    RI_REQUIRE((uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w_norm % 16 == 0
               && (uintptr_t)a_out % 8 == 0, "ri_gemm_skinny_residual: operands must be 16-byte aligned");
    const int halves = residual_halves(N);
    ResidualEpilogue re{x, w_dtype == RI_F32 ? (const float*)w_norm : nullptr, w_dtype == RI_BF16 ? (const bf16_t*)w_norm : nullptr,
                        (bf16_t*)a_out, ssq, halves};
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    const int nks = K / 32, blocks = (N / 16) * (halves ? 2 : 1);
    if (nks >= 16)
        gemm_skinny_bf16_kernel<1, 1, 8, float, false, true><<<dim3(blocks, 1), 512, 0, stream>>>(
            a, lda, w, K, (float*)nullptr, N, M, N, K, nks, 0, RopeEpilogue{}, RowScale{}, re);
    else
        gemm_skinny_bf16_kernel<1, 1, 4, float, false, true><<<dim3(blocks, 1), 256, 0, stream>>>(
            a, lda, w, K, (float*)nullptr, N, M, N, K, nks, 0, RopeEpilogue{}, RowScale{}, re);
    RI_LAUNCHED("ri_gemm_skinny_residual");
    return 0;
}
