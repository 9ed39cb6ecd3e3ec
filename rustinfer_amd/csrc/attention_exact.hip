// Attention of prompt portions over the paged cache on the exact 32-bit path: the same formula
// as attention_generic.hip (reference: fused_ops.rs:430-535), tiled so that the keys and values a
// block needs are read once for a tile of query tokens and all query heads of a key/value head.
//
// A block of four waves owns up to 32 query rows: TQ = 32 / G consecutive tokens of one request
// (G = H / Hkv query heads each) on one key/value head.  Keys go by in blocks of 64 that are
// aligned to absolute key positions (block c holds keys 64 c .. 64 c + 63), so that what a query
// row adds up, and in which order, depends on its position alone and not on how the prompt was
// cut.  A block of keys and values is brought into LDS by all threads; a wave then works on
// four of its rows at a time with one key a lane: dot products of head-size terms in ascending
// order, the row's maximum and sum over the 64 lanes in a fixed tree, the probabilities to LDS,
// and then, one value feature a lane (two above 64), the weighted sum over the 64 keys in
// ascending order.  All arithmetic is 32-bit FMA; nothing is rounded below that.
// Cache layout: keys [pages][Hkv][page][hd], values [pages][Hkv][hd][page].  hd % 4 == 0, hd <= 128.
#include "common.h"
#include <math.h>

namespace {

constexpr int EX_ROWS = 32;      // query rows a block
constexpr int EX_KEYS = 64;      // keys a step: one a lane

template <int NC>                // 64-wide slices of the head size a lane holds: 1 or 2
__global__ __launch_bounds__(256) void attn_exact_f32_kernel(
        const float* __restrict__ q, int q_stride, float* __restrict__ out, int out_stride,
        const float* __restrict__ kc, const float* __restrict__ vc,
        const int* __restrict__ table, int max_blocks,
        const int* __restrict__ cu_q, const int* __restrict__ q_start, const int* __restrict__ kv_lens,
        int num_rows, int H, int Hkv, int hd, int page, float scale, int window, int TQ) {
    extern __shared__ __align__(16) float lds[];
    const int ks_stride = hd + 4, vs_stride = hd + 1;
    float* Qs = lds;                                   // [EX_ROWS][hd]
    float* Ks = Qs + EX_ROWS * hd;                     // [EX_KEYS][hd + 4]
    float* Vs = Ks + EX_KEYS * ks_stride;              // [EX_KEYS][hd + 1]
    float* Ps = Vs + EX_KEYS * vs_stride;              // [EX_ROWS][EX_KEYS]
    int* koff = reinterpret_cast<int*>(Ps + EX_ROWS * EX_KEYS);   // [EX_KEYS] key slot in the cache, -1: none

    // which request and which of its tokens: tiles are numbered request by request
    const int tile = blockIdx.x, g = blockIdx.y, G = H / Hkv;
    int b = -1, t0 = 0, nt = 0, before = 0;
    for (int r = 0; r < num_rows; ++r) {
        const int lo = cu_q[r], ql = cu_q[r + 1] - lo, tiles = (ql + TQ - 1) / TQ;
        if (tile < before + tiles) {
            b = r;
            t0 = lo + (tile - before) * TQ;
            nt = min(TQ, lo + ql - t0);
            break;
        }
        before += tiles;
    }
    if (b < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int R = nt * G;                              // rows in use: row r = token r / G, head g G + r % G
    const int p0 = q_start[b] + (t0 - cu_q[b]);        // position of the tile's first token
    const int kv_len = kv_lens[b];
    const int last_visible = min(kv_len, p0 + nt);     // of the tile's last token
    const int first_key = window > 0 ? max(0, p0 + 1 - window) : 0;   // of its first

    for (int e = tid; e < EX_ROWS * hd; e += 256) {
        const int r = e / hd, dd = e % hd;
        Qs[e] = r < R ? q[(size_t)(t0 + r / G) * q_stride + (g * G + r % G) * hd + dd] : 0.f;
    }

    // this wave's rows: wave, wave + 4, ...; four of them a batch
    const int batches = (R + 15) / 16;                 // the same for all waves: they share the barriers
    float m[8], l[8], acc[8][NC];
    int row_lo[8], row_hi[8];                          // keys [row_lo, row_hi) are the row's
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        m[i] = -INFINITY;
        l[i] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[i][c] = 0.f;
        const int r = wave + 4 * i, p = p0 + r / G;
        row_hi[i] = r < R ? min(kv_len, p + 1) : 0;
        row_lo[i] = window > 0 ? max(0, p + 1 - window) : 0;
    }

    for (int kb = first_key / EX_KEYS; kb * EX_KEYS < last_visible; ++kb) {
        const int j_base = kb * EX_KEYS;
        __syncthreads();                               // the last block of keys has been used (first pass: Qs is written)
        if (tid < EX_KEYS) {
            const int j = j_base + tid;
            int off = -1;
            if (j < last_visible) off = (table[(size_t)b * max_blocks + j / page] * Hkv + g) * page + j % page;
            koff[tid] = off;
        }
        __syncthreads();
        // keys: 16-byte pieces, hd / 4 a key
        const int pieces = hd / 4;
        for (int e = tid; e < EX_KEYS * pieces; e += 256) {
            const int jj = e / pieces, pc = e % pieces, off = koff[jj];
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (off >= 0) v = *reinterpret_cast<const float4*>(kc + (size_t)off * hd + pc * 4);
            *reinterpret_cast<float4*>(Ks + jj * ks_stride + pc * 4) = v;
        }
        // values: thread -> key tid % 64, features tid / 64, + 4, ...; zero where there is no key (0 * garbage)
        {
            const int jj = tid & 63, off = koff[jj];
            const size_t vbase = off >= 0 ? (size_t)(off / page) * page * hd + off % page : 0;
            for (int d = tid >> 6; d < hd; d += 4)
                Vs[jj * vs_stride + d] = off >= 0 ? vc[vbase + (size_t)d * page] : 0.f;
        }
        __syncthreads();
        // scores, running maximum and sum, probabilities
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {               // unrolled: the rows' registers are indexed by constants
            if (bi >= batches) break;
            float s[4] = {0.f, 0.f, 0.f, 0.f};
            const float* kr = Ks + lane * ks_stride;
#pragma unroll 2
            for (int dd = 0; dd < hd; dd += 4) {
                const float4 k4 = *reinterpret_cast<const float4*>(kr + dd);
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) {
                    const float4 q4 = *reinterpret_cast<const float4*>(Qs + (wave + 4 * (4 * bi + rb)) * hd + dd);
                    s[rb] = fmaf(q4.x, k4.x, s[rb]);
                    s[rb] = fmaf(q4.y, k4.y, s[rb]);
                    s[rb] = fmaf(q4.z, k4.z, s[rb]);
                    s[rb] = fmaf(q4.w, k4.w, s[rb]);
                }
            }
            const int j = j_base + lane;
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const int i = 4 * bi + rb;
                const bool mine = j >= row_lo[i] && j < row_hi[i];
                const float sc = mine ? s[rb] * scale : -INFINITY;
                const float m_new = fmaxf(m[i], wave_max(sc));
                float pj = 0.f, alpha = 1.f;
                if (m_new > -INFINITY) {               // else the row has seen no key yet
                    pj = mine ? expf(sc - m_new) : 0.f;
                    alpha = expf(m[i] - m_new);        // first keys: exp(-inf) = 0
                }
                l[i] = l[i] * alpha + wave_sum(pj);
                m[i] = m_new;
#pragma unroll
                for (int c = 0; c < NC; ++c) acc[i][c] *= alpha;
                Ps[(wave + 4 * i) * EX_KEYS + lane] = pj;
            }
        }
        __syncthreads();                               // probabilities written (each wave reads its own rows)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
            if (bi >= batches) break;
#pragma unroll 1
            for (int jj = 0; jj < EX_KEYS; jj += 4) {
                float4 p4[4];
#pragma unroll
                for (int rb = 0; rb < 4; ++rb)
                    p4[rb] = *reinterpret_cast<const float4*>(Ps + (wave + 4 * (4 * bi + rb)) * EX_KEYS + jj);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        const int d = lane + 64 * c;
                        const float v = d < hd ? Vs[(jj + u) * vs_stride + d] : 0.f;
#pragma unroll
                        for (int rb = 0; rb < 4; ++rb) {
                            const float pv = u == 0 ? p4[rb].x : u == 1 ? p4[rb].y : u == 2 ? p4[rb].z : p4[rb].w;
                            acc[4 * bi + rb][c] = fmaf(pv, v, acc[4 * bi + rb][c]);
                        }
                    }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = wave + 4 * i;
        if (r >= R) continue;
        float* o = out + (size_t)(t0 + r / G) * out_stride + (g * G + r % G) * hd;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int d = lane + 64 * c;
            if (d < hd) o[d] = l[i] > 0.f ? acc[i][c] / l[i] : 0.f;
        }
    }
}

size_t exact_lds_bytes(int hd) {
    return sizeof(float) * ((size_t)EX_ROWS * hd + (size_t)EX_KEYS * (hd + 4) + (size_t)EX_KEYS * (hd + 1) + (size_t)EX_ROWS * EX_KEYS)
           + sizeof(int) * EX_KEYS;
}

}  // namespace

// Whether ri_attention_exact_f32 takes these sizes (else: the generic kernel).
extern "C" int ri_attention_exact_supported(int H, int Hkv, int hd, int page) {
    return H > 0 && Hkv > 0 && H % Hkv == 0 && H / Hkv <= EX_ROWS && hd > 0 && hd % 4 == 0 && hd <= 128 && page > 0;
}

// Every token of the step belongs to a request row (cu_q covers all T tokens); rows of one token
// are taken as well, but a step of single tokens only is better served by the generic kernel,
// which spreads it over more blocks.
extern "C" int ri_attention_exact_f32(
        const float* q, int q_stride, float* out, int out_stride, const float* kc, const float* vc,
        int num_pages, int page, int H, int Hkv, int hd, const int* table, int max_blocks,
        const int* cu_q, const int* q_start, const int* kv_lens, int num_rows, int T,
        float scale, int window, hipStream_t stream) {
    RI_REQUIRE(ri_attention_exact_supported(H, Hkv, hd, page), "ri_attention_exact_f32: sizes not taken (H=%d Hkv=%d hd=%d page=%d)", H, Hkv, hd, page);
    RI_REQUIRE(T >= 0 && num_rows >= 0 && max_blocks > 0 && num_pages > 0 && window >= 0, "ri_attention_exact_f32: bad sizes");
    RI_REQUIRE(q_stride >= H * hd && out_stride >= H * hd, "ri_attention_exact_f32: row strides too small");
    if (T == 0 || num_rows == 0) return 0;
    RI_REQUIRE(q && out && kc && vc && table && cu_q && q_start && kv_lens, "ri_attention_exact_f32: null pointer");
    RI_REQUIRE((uintptr_t)kc % 16 == 0, "ri_attention_exact_f32: unaligned key cache");
    RI_REQUIRE(Hkv <= 65535, "ri_attention_exact_f32: too many key/value heads for the grid");
    const int G = H / Hkv, TQ = EX_ROWS / G;
    const int tiles = (T + TQ - 1) / TQ + num_rows;    // at most: every request may end in a short tile
    const size_t lds = exact_lds_bytes(hd);
    auto kernel = hd <= 64 ? attn_exact_f32_kernel<1> : attn_exact_f32_kernel<2>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        RI_REQUIRE(e == hipSuccess, "ri_attention_exact_f32: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
    }
    kernel<<<dim3(tiles, Hkv), 256, lds, stream>>>(q, q_stride, out, out_stride, kc, vc, table, max_blocks, cu_q, q_start,
                                                   kv_lens, num_rows, H, Hkv, hd, page, scale, window, TQ);
    RI_LAUNCHED("ri_attention_exact_f32");
    return 0;
}
