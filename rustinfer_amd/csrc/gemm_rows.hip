// C[M, N] = A[M, K] . W[N, K]^T for 17..64 rows of bfloat16 against weights in tile order
// ([N/16][K/32][64 lanes][8], see gemm.hip), with the activations shared through LDS.
//
// With that many rows a wave of the few-row kernel (gemm.hip) asks for as many bytes of
// activations as of weights, and the product takes as long as if both came from memory.  Here
// the four waves of a block work on the same 256 values of K at a time: the block brings that
// stretch of all (up to 64) rows into LDS once, in the order the matrix instructions read them,
// and every wave multiplies it with weight tiles of its own, which it streams from memory
// straight into registers, a whole stretch (8 k-steps) ahead.  What is asked of memory is then
// the weights, once, and one copy of the activations a block.
//
// A block owns 4 * NT tiles of 16 columns (SWIGLU: as many of the gate half and of the up half of
// a stacked [2N, K] matrix, and writes silu(gate) * up).  Products with few columns are also
// split over K between blocks (blockIdx.y), each leaving 32-bit partial sums in its own slice of
// C, which the norm that follows adds up.  N % 16 == 0, K % 32 == 0.
//
// At 64 rows the two stretch buffers of a block take 64 KB, two blocks of four waves a compute
// unit; where the columns give too few blocks for that, a block holds two or four groups of waves
// instead, which split its share of K between them through buffers of their own (128 KB).
#include "common.h"
#include <mutex>

typedef __bf16 rbf16x8_t __attribute__((ext_vector_type(8)));
typedef float rf32x4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int KS_LONG = 8;                // k-steps of 32 in a stretch; 4 where four groups share a block

struct Store4 {
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

// LDS holds a stretch as [k-step][m-tile][k-group][row of the tile] in units of 8 values (16
// bytes), the order in which a wave's lanes read an operand; the row index is xor-ed with
// (4 * k-step + k-group) % 16 so that the threads that bring a row in (32 of them write the
// 32 units of one row) spread over the banks, while a read still takes 64 different units.
template <int MT>
__device__ __forceinline__ int lds_unit(int ks, int mt, int g, int c) {
    return ((ks * MT + mt) * 4 + g) * 16 + (c ^ ((4 * ks + g) & 15));
}

// ROPE: the product is the fused q/k/v projection of single tokens, with the weight's rows permuted
// within each head as for the few-row kernel (gemm.hip, ri_qkv_rope_row_order): a tile holds 8
// features of the first half of a head and their 8 partners, the partner of a lane's value sits in
// lane ^ 32.  The epilogue rotates q and k by the token's position (32-bit, one rounding), writes
// k and v into the token's cache page and only q to C.
struct RowsRope {
    const float* cos_t; const float* sin_t;        // [positions][hd / 2]
    const int* positions; const int* row_of_token; // per token (row of A)
    const int* table; int max_blocks;              // block table [rows][max_blocks]
    bf16_t* kc; bf16_t* vc;                        // k [pages][Hkv][page][hd], v [pages][Hkv][hd][page]
    int H, Hkv, hd, page;
};

// KG groups of WAVES waves share a block: each group takes its own half of the block's stretches,
// through LDS buffers of its own, and the groups' sums meet in LDS at the end.  That doubles the
// waves and the bytes under way on a compute unit where the columns make too few blocks for two a unit.
template <int MT, int NT, bool SWIGLU, typename TO, int WAVES, int KG, int KS, bool ROPE = false>
__global__ __launch_bounds__(WAVES * KG * 64) void gemm_rows_lds_kernel(
        const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W,
        TO* __restrict__ C, int ldc, int M, int N, int K, int stretches_per_block, size_t part_stride,
        RowsRope rp) {
    static_assert(!ROPE || (NT == 1 && !SWIGLU && sizeof(TO) == 2), "the rotation goes with one bfloat16 tile a wave");
    constexpr int NW = SWIGLU ? 2 * NT : NT;
    constexpr int THREADS = WAVES * 64;                     // of a group
    constexpr int XP = MT * KS / WAVES;                     // 16-byte pieces of a stretch a thread brings in
    constexpr int RU = KS * 4;                              // such pieces in a row of a stretch
    static_assert(MT * 16 * RU == XP * THREADS, "a stretch must divide evenly over the threads of a group");
    constexpr int STRETCH = KS * MT * 64;                   // units of a stretch in LDS
    extern __shared__ __align__(16) rbf16x8_t xs_all[];     // [KG][2][STRETCH]
    const int kg = threadIdx.x / THREADS, tid = threadIdx.x % THREADS;
    rbf16x8_t* xs = xs_all + kg * 2 * STRETCH;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), col = lane & 15, grp = lane >> 4;   // the same in all lanes of a wave
    const int ntiles = N / 16, nks_all = K / 32;
    const int s_all = (nks_all + KS - 1) / KS;
    const int b_begin = blockIdx.y * stretches_per_block;
    const int b_end = min(s_all, b_begin + stretches_per_block);
    const int span = (max(b_end - b_begin, 0) + KG - 1) / KG;      // stretches of a group; the same for all
    const int s_begin = b_begin + kg * span;
    const int s_end = min(b_end, s_begin + span);
    C += (size_t)blockIdx.y * part_stride;

    const bf16_t* wp[NW];
#pragma unroll
    for (int a = 0; a < NW; ++a) {
        // tiles beyond N are read (clamped) but never stored
        const int tile = min(((int)blockIdx.x * WAVES + wave) * NT + (a % NT), ntiles - 1) + (a >= NT ? ntiles : 0);
        wp[a] = W + ((size_t)tile * nks_all * 64 + lane) * 8;
    }
    rf32x4_t acc[NW][MT];
#pragma unroll
    for (int a = 0; a < NW; ++a)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[a][mt] = rf32x4_t{0.f, 0.f, 0.f, 0.f};
    const rbf16x8_t zero = {};

    // piece j of this thread: row m = p / RU, values k = 8 * (p % RU) .. + 7 of the stretch, p = tid + THREADS j
    auto load_x = [&](int s, rbf16x8_t (&xr)[XP]) {
#pragma unroll
        for (int j = 0; j < XP; ++j) {
            const int p = tid + THREADS * j;
            const int m = p / RU, k = s * (KS * 32) + (p % RU) * 8;
            xr[j] = (m < M && k < K) ? *reinterpret_cast<const rbf16x8_t*>(A + (size_t)m * lda + k) : zero;
        }
    };
    auto store_x = [&](int buf, const rbf16x8_t (&xr)[XP]) {
#pragma unroll
        for (int j = 0; j < XP; ++j) {
            const int p = tid + THREADS * j;
            const int m = p / RU, kp = p % RU;
            xs[buf * STRETCH + lds_unit<MT>(kp >> 2, m >> 4, kp & 3, m & 15)] = xr[j];
        }
    };
    auto load_w = [&](int s, rbf16x8_t (&wf)[NW][KS]) {
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            const int ks = s * KS + u;
#pragma unroll
            for (int a = 0; a < NW; ++a)
                wf[a][u] = ks < nks_all ? ld_stream16<rbf16x8_t>(wp[a] + (size_t)ks * 512) : zero;
        }
    };
    auto multiply = [&](int buf, const rbf16x8_t (&wf)[NW][KS]) {
#pragma unroll
        for (int u = 0; u < KS; ++u) {
            rbf16x8_t xf[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) xf[mt] = xs[buf * STRETCH + lds_unit<MT>(u, mt, grp, col)];
#pragma unroll
            for (int a = 0; a < NW; ++a)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[a][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[a][u], xf[mt], acc[a][mt], 0, 0, 0);
        }
    };

    // what the rotation needs of each token is asked for now: a chain of small loads at the end of
    // a short kernel would cost microseconds
    int rp_section = 0, rp_head = 0, rp_j = 0;
    int rp_b[ROPE ? MT : 1], rp_blk[ROPE ? MT : 1], rp_slot[ROPE ? MT : 1];
    float4 rp_c[ROPE ? MT : 1], rp_s[ROPE ? MT : 1];
    if constexpr (ROPE) {
        const int hd = rp.hd, half = hd >> 1, q_dim = rp.H * hd, kv_dim = rp.Hkv * hd;
        const int n0 = min(((int)blockIdx.x * WAVES + wave), ntiles - 1) * 16;
        rp_section = n0 < q_dim ? 0 : (n0 < q_dim + kv_dim ? 1 : 2);                     // q, k, v
        const int within = n0 - (rp_section == 0 ? 0 : (rp_section == 1 ? q_dim : q_dim + kv_dim));
        rp_head = within / hd;
        rp_j = (within % hd) >> 4;                                                       // the tile is tile j of its head
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + col;
            rp_b[mt] = -1; rp_blk[mt] = -1; rp_slot[mt] = 0;
            rp_c[mt] = make_float4(1.f, 1.f, 1.f, 1.f);
            rp_s[mt] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (kg == 0 && m < M) {
                const int b = rp.row_of_token[m], pos = rp.positions[m];
                rp_b[mt] = b;
                rp_slot[mt] = pos % rp.page;
                if (b >= 0) {
                    if (rp_section != 0) rp_blk[mt] = rp.table[(size_t)b * rp.max_blocks + pos / rp.page];
                    if (rp_section != 2) {
                        // this lane's four values are features 8 j + (grp & 1) 4 + i of a half
                        const size_t at = (size_t)pos * half + 8 * rp_j + (grp & 1) * 4;
                        rp_c[mt] = *reinterpret_cast<const float4*>(rp.cos_t + at);
                        rp_s[mt] = *reinterpret_cast<const float4*>(rp.sin_t + at);
                    }
                }
            }
        }
    }

    // two stretches an iteration, so that the weights' registers swap roles without being copied;
    // every wave of the block passes the same barriers, with or without a stretch of its own left
    rbf16x8_t w0[NW][KS], w1[NW][KS], xr[XP];
    if (s_begin < s_end) {
        load_x(s_begin, xr);
        load_w(s_begin, w0);
        store_x(0, xr);
    }
    __syncthreads();
    for (int i = 0; i < span; i += 2) {
        const int s = s_begin + i;
        const bool have0 = s < s_end, more1 = s + 1 < s_end, more2 = s + 2 < s_end;
        if (more1) { load_x(s + 1, xr); load_w(s + 1, w1); }
        if (have0) multiply(0, w0);
        if (more1) store_x(1, xr);
        __syncthreads();
        if (i + 1 >= span) break;
        if (more2) { load_x(s + 2, xr); load_w(s + 2, w0); }
        if (more1) multiply(1, w1);
        if (more2) store_x(0, xr);
        __syncthreads();
    }
    if (KG > 1) {
        // the other groups' sums, through the LDS the stretches have left: [group - 1][wave][a][mt][lane]
        rf32x4_t* red = reinterpret_cast<rf32x4_t*>(xs_all);
        if (kg > 0) {
#pragma unroll
            for (int a = 0; a < NW; ++a)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    red[((((kg - 1) * WAVES + wave) * NW + a) * MT + mt) * 64 + lane] = acc[a][mt];
        }
        __syncthreads();
        if (kg > 0) return;
#pragma unroll
        for (int g = 1; g < KG; ++g)
#pragma unroll
            for (int a = 0; a < NW; ++a)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const rf32x4_t o = red[((((g - 1) * WAVES + wave) * NW + a) * MT + mt) * 64 + lane];
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[a][mt][i] += o[i];
                }
    }

    // acc[a][mt][i] = C[m = mt * 16 + col][n = tile(a) * 16 + grp * 4 + i]
    if constexpr (ROPE) {
        if ((int)blockIdx.x * WAVES + wave >= ntiles) return;
        const int hd = rp.hd, half = hd >> 1;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + col;
            const int b = rp_b[mt], blk = rp_blk[mt], slot = rp_slot[mt];
            const float cs[4] = {rp_c[mt].x, rp_c[mt].y, rp_c[mt].z, rp_c[mt].w};
            const float sn[4] = {rp_s[mt].x, rp_s[mt].y, rp_s[mt].z, rp_s[mt].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = grp * 4 + i;                           // row of the tile: r < 8 first half, else partner
                const float v = acc[0][mt][i];
                const float other = __shfl_xor(v, 32, 64);           // row r ^ 8, same token
                const int fi = 8 * rp_j + (r & 7);                   // index within the half
                const int d = r < 8 ? fi : half + fi;                // feature within the head
                if (b < 0) continue;                                 // padding token or beyond M
                if (rp_section == 2) {
                    if (blk >= 0) rp.vc[((size_t)blk * rp.Hkv + rp_head) * rp.page * hd + (size_t)d * rp.page + slot] = f32_to_bf16(v);
                    continue;
                }
                const float res = r < 8 ? v * cs[i] - other * sn[i] : other * sn[i] + v * cs[i];
                if (rp_section == 0) st_f32(C + (size_t)m * ldc + rp_head * hd + d, res);
                else if (blk >= 0) rp.kc[((size_t)blk * rp.Hkv + rp_head) * rp.page * hd + (size_t)slot * hd + d] = f32_to_bf16(res);
            }
        }
        return;
    }
#pragma unroll
    for (int a = 0; a < NT; ++a) {
        const int tile = ((int)blockIdx.x * WAVES + wave) * NT + a;
        if (tile >= ntiles) break;
        const int n = tile * 16 + grp * 4;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + col;
            if (m >= M) continue;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i] = acc[a][mt][i];
                if (SWIGLU) v[i] = v[i] / (1.f + __expf(-v[i])) * acc[NT + a][mt][i];
            }
            TO* dst = C + (size_t)m * ldc + n;
            if ((ldc & 3) == 0 && ((uintptr_t)C & 15) == 0) {
                Store4::st(dst, v);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) st_f32(dst + i, v[i]);
            }
        }
    }
}

template <int MT, int NT, bool SWIGLU, typename TO, int KG>
int launch_rows_groups(const bf16_t* A, int lda, const bf16_t* W, TO* C, int ldc, int M, int N, int K,
                       int parts, size_t part_stride, hipStream_t stream) {
    // four waves a group (eight: twice the columns, half the blocks, slower throughout); four groups:
    // of two waves and half as long stretches, so that twice the blocks take the same LDS
    constexpr int waves = KG == 4 ? 2 : 4;
    constexpr int KS = KG == 4 ? KS_LONG / 2 : KS_LONG;
    constexpr size_t lds = (size_t)KG * 2 * KS * MT * 64 * sizeof(rbf16x8_t);
    auto kernel = gemm_rows_lds_kernel<MT, NT, SWIGLU, TO, waves, KG, KS>;
    if (lds > 64 * 1024) {          // beyond what a kernel may take unasked: ask once a device
        static std::mutex mu;
        static bool asked[64] = {};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        RI_REQUIRE(e == hipSuccess && dev >= 0 && dev < 64, "ri_gemm_rows_bf16: no current device: %s", hipGetErrorString(e));
        std::lock_guard<std::mutex> lock(mu);
        if (!asked[dev]) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            RI_REQUIRE(e == hipSuccess, "ri_gemm_rows_bf16: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
            asked[dev] = true;
        }
    }
    const int s_all = (K / 32 + KS - 1) / KS;
    const int per = (s_all + parts - 1) / parts;
    const int blocks = (N / 16 + waves * NT - 1) / (waves * NT);
    kernel<<<dim3(blocks, parts), waves * KG * 64, lds, stream>>>(A, lda, W, C, ldc, M, N, K, per, part_stride, RowsRope{});
    return 0;
}

template <int MT, int NT, bool SWIGLU, typename TO>
int launch_rows(const bf16_t* A, int lda, const bf16_t* W, TO* C, int ldc, int M, int N, int K,
                int parts, size_t part_stride, int groups, hipStream_t stream) {
    if (groups == 2) return launch_rows_groups<MT, NT, SWIGLU, TO, 2>(A, lda, W, C, ldc, M, N, K, parts, part_stride, stream);
    if (groups == 4) return launch_rows_groups<MT, NT, SWIGLU, TO, 4>(A, lda, W, C, ldc, M, N, K, parts, part_stride, stream);
    return launch_rows_groups<MT, NT, SWIGLU, TO, 1>(A, lda, W, C, ldc, M, N, K, parts, part_stride, stream);
}

template <int NT, bool SWIGLU, typename TO>
int dispatch_rows(const bf16_t* A, int lda, const bf16_t* W, TO* C, int ldc, int M, int N, int K,
                  int parts, size_t part_stride, int groups, hipStream_t stream) {
    if (M <= 32) return launch_rows<2, NT, SWIGLU, TO>(A, lda, W, C, ldc, M, N, K, parts, part_stride, groups, stream);
    if (M <= 48) return launch_rows<3, NT, SWIGLU, TO>(A, lda, W, C, ldc, M, N, K, parts, part_stride, groups, stream);
    return launch_rows<4, NT, SWIGLU, TO>(A, lda, W, C, ldc, M, N, K, parts, part_stride, groups, stream);
}

// The fused q/k/v projection with rotation: four groups of two waves a block (32 columns) or two
// groups of four (64 columns), see launch_rows_groups.
template <int MT, int KG>
int launch_rows_rope(const bf16_t* A, int lda, const bf16_t* W, bf16_t* C, int ldc, int M, int N, int K,
                     const RowsRope& rp, hipStream_t stream) {
    static_assert(KG == 2 || KG == 4, "two or four groups");
    constexpr int waves = KG == 4 ? 2 : 4, KS = KG == 4 ? KS_LONG / 2 : KS_LONG;
    constexpr size_t lds = (size_t)KG * 2 * KS * MT * 64 * sizeof(rbf16x8_t);
    auto kernel = gemm_rows_lds_kernel<MT, 1, false, bf16_t, waves, KG, KS, true>;
    if (lds > 64 * 1024) {
        static std::mutex mu;
        static bool asked[64] = {};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        RI_REQUIRE(e == hipSuccess && dev >= 0 && dev < 64, "ri_gemm_rows_qkv_rope: no current device: %s", hipGetErrorString(e));
        std::lock_guard<std::mutex> lock(mu);
        if (!asked[dev]) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            RI_REQUIRE(e == hipSuccess, "ri_gemm_rows_qkv_rope: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
            asked[dev] = true;
        }
    }
    const int s_all = (K / 32 + KS - 1) / KS;
    const int blocks = (N / 16 + waves - 1) / waves;
    kernel<<<dim3(blocks, 1), waves * KG * 64, lds, stream>>>(A, lda, W, C, ldc, M, N, K, s_all, 0, rp);
    return 0;
}

template <int MT>
int launch_rows_rope_groups(const bf16_t* A, int lda, const bf16_t* W, bf16_t* C, int ldc, int M, int N, int K,
                            int groups, const RowsRope& rp, hipStream_t stream) {
    if (groups == 2) return launch_rows_rope<MT, 2>(A, lda, W, C, ldc, M, N, K, rp, stream);
    return launch_rows_rope<MT, 4>(A, lda, W, C, ldc, M, N, K, rp, stream);
}

}  // namespace

// Slices of K, and wave groups a block, for a product of M rows, N columns and K inner values whose
// partial sums a norm adds up.  Blocks enough to fill the chip twice, at most 8 slices (measured
// at 64 rows, us: 4096 x 4096 with 2, 4, 8, 16 slices 16.5, 12.2, 11.3, 15.0; 4096 x 14336: 53,
// 35, 29, 32; 2048 x 8192: 26, 16, 11.8, 11.2, but the norm that adds 16 slices up loses more than
// that gains: 64 rows decode at 29,200 tokens a second with 8 slices at most and at 26,600 with
// 16).  With more than 32 rows a block of two groups takes 128 KB of LDS, one block a compute
// unit: then two groups pay where a block's share of K is short (half the slices do as well:
// 4096 x 4096, 8 slices of one group 12.1, 4 of two 12.1; 3072 x 3072: 9.7, 8.9) or where all
// blocks still fit the chip at once (2048 x 8192: 8 slices, 12.9 with one group, 11.6 with two);
// not for a long K over many columns (4096 x 14336: 8 of one 28.5, 4 of two 32.2, 8 of two 35.2).
extern "C" int ri_gemm_rows_plan(int M, int N, int K, int nt, int* parts_out, int* groups_out) {
    RI_REQUIRE(parts_out && groups_out && N > 0 && K > 0 && (nt == 1 || nt == 2), "ri_gemm_rows_plan: bad arguments");
    const int blocks = (N / 16 + 4 * nt - 1) / (4 * nt), stretches = (K / 32 + KS_LONG - 1) / KS_LONG;
    int parts = 1, groups = 1;
    while (parts < 8 && blocks * parts < 512 && stretches / (parts * 2) >= 1) parts *= 2;
    // with more than 32 rows two blocks fit a compute unit: no more blocks than the chip holds at once
    // (5120 x 5120 at 64 rows, 80 blocks of columns: 8 slices 19.9 us, 4 slices 18.2)
    if (M > 32 && parts > 1 && blocks * parts > 512) parts /= 2;
    if (M > 32 && parts == 8) {
        if (blocks * parts <= 256 && stretches / parts >= 4) groups = 2;
        else if (stretches / parts <= 2 && blocks * 4 <= 256) { parts = 4; groups = 2; }
    }
    *parts_out = parts;
    *groups_out = groups;
    return 0;
}

// W: the copy in tile order.  swiglu != 0: W is [2N, K] (gate rows, then up rows), C bfloat16.
// parts > 1: C is a float32 stack [parts][M][ldc] (part_stride elements apart) of partial sums.
// nt: tiles of 16 columns a wave owns (1 or 2).  groups: 1, or 2 for blocks of eight waves whose
// halves split the block's share of K between them, or 4 for blocks of four pairs of waves that do
// (half the columns a block, so twice the blocks).
extern "C" int ri_gemm_rows_bf16(const void* A, int lda, const void* W, void* C, int ldc, int M, int N, int K,
                                 int out_dtype, int swiglu, int parts, long long part_stride, int nt, int groups,
                                 hipStream_t stream) {
    RI_REQUIRE(groups == 1 || groups == 2 || groups == 4, "ri_gemm_rows_bf16: groups=%d not 1, 2 or 4", groups);
    RI_REQUIRE(M >= 1 && M <= 64, "ri_gemm_rows_bf16: M=%d not in [1, 64]", M);
    RI_REQUIRE(N > 0 && N % 16 == 0 && K > 0 && K % 32 == 0, "ri_gemm_rows_bf16: needs N %% 16 == 0 and K %% 32 == 0 (N=%d K=%d)", N, K);
    RI_REQUIRE(lda >= K && lda % 8 == 0 && ldc >= N, "ri_gemm_rows_bf16: bad leading dimensions");
    RI_REQUIRE(A && W && C && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0, "ri_gemm_rows_bf16: null or unaligned pointer");
    RI_REQUIRE(nt == 1 || nt == 2, "ri_gemm_rows_bf16: nt=%d not 1 or 2", nt);
    RI_REQUIRE(parts >= 1 && parts <= 64, "ri_gemm_rows_bf16: parts=%d not in [1, 64]", parts);
    RI_REQUIRE(parts == 1 || (out_dtype == RI_F32 && !swiglu && part_stride >= (long long)M * ldc),
               "ri_gemm_rows_bf16: partial sums need a float32 stack and no activation");
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    const size_t ps = parts > 1 ? (size_t)part_stride : 0;
    int rc = 0;
    if (swiglu) {
        RI_REQUIRE(out_dtype == RI_BF16, "ri_gemm_rows_bf16: the fused SwiGLU form writes bfloat16");
        RI_REQUIRE(nt == 1, "ri_gemm_rows_bf16: the SwiGLU form takes one gate and one up tile a wave");
        rc = dispatch_rows<1, true, bf16_t>(a, lda, w, (bf16_t*)C, ldc, M, N, K, 1, 0, groups, stream);
    } else if (out_dtype == RI_BF16) {
        if (nt == 2) rc = dispatch_rows<2, false, bf16_t>(a, lda, w, (bf16_t*)C, ldc, M, N, K, 1, 0, groups, stream);
        else rc = dispatch_rows<1, false, bf16_t>(a, lda, w, (bf16_t*)C, ldc, M, N, K, 1, 0, groups, stream);
    } else if (out_dtype == RI_F32) {
        if (nt == 2) rc = dispatch_rows<2, false, float>(a, lda, w, (float*)C, ldc, M, N, K, parts, ps, groups, stream);
        else rc = dispatch_rows<1, false, float>(a, lda, w, (float*)C, ldc, M, N, K, parts, ps, groups, stream);
    } else {
        return ri_fail("ri_gemm_rows_bf16: unknown output dtype %d", out_dtype);
    }
    if (rc) return rc;
    RI_LAUNCHED("ri_gemm_rows_bf16");
    return 0;
}

// The q/k/v projection of 17..64 single tokens with rotation and cache write in the epilogue, as
// ri_gemm_qkv_rope (gemm.hip) does it for fewer rows: W is the same row-permuted weight in tile
// order, C [M, ldc] receives rotated q in its first H * hd columns.  Measured at 64 rows against
// the few-row kernel (product alone, us): 6144 x 4096 25.9 -> 21.5, 5120 x 3072 21.1 -> 16.5,
// 3072 x 2048 16.4 -> 10.9 (but no gain left there once the epilogue is in); from 32 rows down the
// few-row kernel is as fast or faster at these sizes and slower at larger ones (24 rows: 12288 x
// 4096 27.3 -> 23.5, 15360 x 5120 35.9 -> 28.8, 10240 x 8192 49.0 -> 42.4): the caller chooses.
//
// Blocks of 32 columns (four pairs of waves) where all of them run at once: a block takes the LDS
// of a whole compute unit with more than 32 rows and half of it with fewer; else blocks of 64
// columns (two groups of four waves), half as many.  64 rows, 32 / 64 columns a block, us: 6144
// columns of K = 4096 22.7 / 28.1, 12288: 43.2 / 32.1; 15360 x 5120: 55.2 / 40.5; 10240 x 8192:
// 79.1 / 56.7; with 32 rows 12288 x 4096 24.6 / 27.1, 15360 x 5120 31.5 / 33.7.
extern "C" int ri_gemm_rows_qkv_rope(const void* A, int lda, const void* W, void* C, int ldc, int M, int K,
                                     int H, int Hkv, int hd, const float* cos_t, const float* sin_t, int table_rows,
                                     const int* positions, const int* row_of_token, void* kc, void* vc,
                                     int num_pages, const int* table, int max_blocks, int page, hipStream_t stream) {
    const int N = (H + 2 * Hkv) * hd;
    RI_REQUIRE(M >= 17 && M <= 64, "ri_gemm_rows_qkv_rope: M=%d not in [17, 64]", M);
    RI_REQUIRE(H > 0 && Hkv > 0 && hd > 0 && hd % 16 == 0 && K > 0 && K % 32 == 0, "ri_gemm_rows_qkv_rope: needs head size %% 16 == 0 and K %% 32 == 0 (hd=%d K=%d)", hd, K);
    RI_REQUIRE(lda >= K && lda % 8 == 0 && ldc >= H * hd, "ri_gemm_rows_qkv_rope: bad leading dimensions");
    RI_REQUIRE(page > 0 && max_blocks > 0 && num_pages > 0 && table_rows > 0, "ri_gemm_rows_qkv_rope: bad cache sizes");
    RI_REQUIRE(A && W && C && cos_t && sin_t && positions && row_of_token && kc && vc && table, "ri_gemm_rows_qkv_rope: null pointer");
    RI_REQUIRE((uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0 && (uintptr_t)cos_t % 16 == 0 && (uintptr_t)sin_t % 16 == 0,
               "ri_gemm_rows_qkv_rope: operands and tables must be 16-byte aligned");
    const RowsRope rp{cos_t, sin_t, positions, row_of_token, table, max_blocks, (bf16_t*)kc, (bf16_t*)vc, H, Hkv, hd, page};
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    const int at_once = M <= 32 ? 512 : 256;
    const int groups = (N / 16 + 1) / 2 <= at_once ? 4 : 2;
    int rc;
    if (M <= 32) rc = launch_rows_rope_groups<2>(a, lda, w, (bf16_t*)C, ldc, M, N, K, groups, rp, stream);
    else if (M <= 48) rc = launch_rows_rope_groups<3>(a, lda, w, (bf16_t*)C, ldc, M, N, K, groups, rp, stream);
    else rc = launch_rows_rope_groups<4>(a, lda, w, (bf16_t*)C, ldc, M, N, K, groups, rp, stream);
    if (rc) return rc;
    RI_LAUNCHED("ri_gemm_rows_qkv_rope");
    return 0;
}
