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
//
// What a query row adds up, and in which order, is the same in both kernels of this file (the
// tiled one for prompt portions and the split-key one for single tokens), so that a token's
// output has the same bits whether its step held prompt portions or not:
//   - a block of 64 keys gives the row a partial result of its own: the largest score m_b, the
//     probabilities exp(s - m_b), their sum l_b and the weighted values acc_b, each summed in
//     ascending order from zero (block_scores / the P.V loops);
//   - the partial results are merged in ascending order of the blocks (merge_block).
// Products and sums that must round the same way everywhere are written with fmaf, __fmul_rn and
// __fsub_rn, and contraction is switched off for the file.
#include "common.h"
#include <math.h>

#pragma clang fp contract(off)

namespace {

constexpr int EX_ROWS = 32;      // query rows a block
constexpr int EX_KEYS = 64;      // keys a step: one a lane

// One row's scores against the 64 keys of a block, one key a lane: s = q.k * scale (or -inf where
// the key is not the row's), the block's maximum, exp(s - maximum) and its sum over the lanes.
// Returns this lane's probability; m_b = -inf (and l_b = 0) if the row sees no key of the block.
__device__ __forceinline__ float block_scores(float dot, bool mine, float scale, float& m_b, float& l_b) {
    const float sc = mine ? __fmul_rn(dot, scale) : -INFINITY;
    m_b = wave_max(sc);
    float pj = 0.f;
    if (m_b > -INFINITY) pj = mine ? expf(__fsub_rn(sc, m_b)) : 0.f;
    l_b = wave_sum(pj);
    return pj;
}

// Merge a block's partial result (m_b, l_b, acc_b) into the running one (m, l, acc).
template <int NC>
__device__ __forceinline__ void merge_block(float& m, float& l, float (&acc)[NC], float m_b, float l_b, const float (&acc_b)[NC]) {
    if (!(m_b > -INFINITY)) return;                    // the row saw no key of this block
    const float M = fmaxf(m, m_b);
    const float alpha = expf(__fsub_rn(m, M));         // 0 while nothing has been seen (m = -inf)
    const float beta = expf(__fsub_rn(m_b, M));
    l = fmaf(l, alpha, __fmul_rn(l_b, beta));
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = fmaf(acc[c], alpha, __fmul_rn(acc_b[c], beta));
    m = M;
}

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
            if (j < last_visible) {
                const int pid = table[(size_t)b * max_blocks + j / page];
                if (pid >= 0) off = (pid * Hkv + g) * page + j % page;      // -1: a page the window has passed and given back
            }
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
        // scores and probabilities of the block, each row's relative to the block's own maximum
        float m_b[8], l_b[8], acc_b[8][NC];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            m_b[i] = -INFINITY;
            l_b[i] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) acc_b[i][c] = 0.f;
        }
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
                Ps[(wave + 4 * i) * EX_KEYS + lane] = block_scores(s[rb], mine, scale, m_b[i], l_b[i]);
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
                            acc_b[4 * bi + rb][c] = fmaf(pv, v, acc_b[4 * bi + rb][c]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) merge_block<NC>(m[i], l[i], acc[i], m_b[i], l_b[i], acc_b[i]);
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

// ---------------------------------------------------------------------------
// Single tokens: the key range is split over waves, one block of 64 keys each ("flash decoding";
// reference: crates/infer-backend-cuda/src/kernels/flash_attn_gqa/flash_attn_paged_decode.cu:75-337),
// so that a step of few tokens still fills the chip: the tiled kernel above would give a token
// one block of threads for all its keys.  A wave computes the partial result of its key block for
// all G query heads of one key/value head, with one key a lane for the scores (the key's row is
// read straight from the cache, 16 bytes at a time; the query rows are the same for all lanes) and
// one value feature a lane (two above 64) for the weighted values, the probabilities passing
// through LDS.  The arithmetic of a row is that of the tiled kernel, term for term.  A second
// kernel merges a row's partial results in ascending order of the blocks.
// Partial results: part_ml [T][H][slots][2] = (m_b, l_b), part_o [T][H][slots][hd]; slot s of a
// token is key block first_block + s, first_block = (first visible key) / 64.
// ---------------------------------------------------------------------------
template <int NC>
__global__ __launch_bounds__(256) void attn_exact_decode_kernel(
        const float* __restrict__ q, int q_stride, const float* __restrict__ kc, const float* __restrict__ vc,
        const int* __restrict__ table, int max_blocks, const int* __restrict__ row_of_token,
        const int* __restrict__ positions, const int* __restrict__ kv_lens,
        int H, int Hkv, int hd, int page, float scale, int window, int slots,
        float* __restrict__ part_ml, float* __restrict__ part_o) {
    extern __shared__ __align__(16) float lds[];       // [4 waves][G][64] probabilities
    const int t = blockIdx.z, g = blockIdx.y, G = H / Hkv;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = row_of_token[t];
    if (b < 0) return;                                  // a padding token
    const int p = positions[t];
    const int visible = min(kv_lens[b], p + 1);
    const int j0 = window > 0 ? max(0, p + 1 - window) : 0;
    if (visible <= j0) return;
    const int first_block = j0 / EX_KEYS;
    const int slot = (int)blockIdx.x * 4 + wave;
    const int kb = first_block + slot;
    if (kb * EX_KEYS >= visible) return;
    float* Ps = lds + (size_t)wave * G * EX_KEYS;

    // this lane's key
    const int j = kb * EX_KEYS + lane;
    long long off = -1;                                 // key slot in the cache; -1: none
    if (j < visible) {
        const int pid = table[(size_t)b * max_blocks + j / page];
        if (pid >= 0) off = ((long long)pid * Hkv + g) * page + j % page;
    }
    const bool mine = j >= j0 && j < visible;
    const float* kr = off >= 0 ? kc + (size_t)off * hd : nullptr;
    const float* qrow = q + (size_t)t * q_stride + (size_t)g * G * hd;
    float* ml = part_ml + (((size_t)t * H + (size_t)g * G) * slots + slot) * 2;
    // scores: four heads a pass over the key's row (which the next pass finds in the cache)
    for (int h0 = 0; h0 < G; h0 += 4) {
        float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
        for (int dd = 0; dd < hd; dd += 4) {
            float4 k4 = make_float4(0.f, 0.f, 0.f, 0.f);
            if (kr) k4 = *reinterpret_cast<const float4*>(kr + dd);
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const float4 q4 = *reinterpret_cast<const float4*>(qrow + (size_t)min(h0 + rb, G - 1) * hd + dd);
                s[rb] = fmaf(q4.x, k4.x, s[rb]);
                s[rb] = fmaf(q4.y, k4.y, s[rb]);
                s[rb] = fmaf(q4.z, k4.z, s[rb]);
                s[rb] = fmaf(q4.w, k4.w, s[rb]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            if (h0 + rb >= G) break;
            float m_b, l_b;
            Ps[(h0 + rb) * EX_KEYS + lane] = block_scores(s[rb], mine, scale, m_b, l_b);
            if (lane == 0) {
                float* dst = ml + (size_t)(h0 + rb) * slots * 2;
                dst[0] = m_b;
                dst[1] = l_b;
            }
        }
    }
    // weighted values: lane = feature; four keys a load where pages allow (the value cache keeps
    // the positions of a feature contiguous)
    const bool vec = (page & 3) == 0;
    for (int h0 = 0; h0 < G; h0 += 4) {
        float acc_b[4][NC];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int c = 0; c < NC; ++c) acc_b[rb][c] = 0.f;
#pragma unroll 4
        for (int jj = 0; jj < EX_KEYS; jj += 4) {
            const int key = kb * EX_KEYS + jj;         // four keys of one page if page % 4 == 0
            float v[4][NC];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int c = 0; c < NC; ++c) v[u][c] = 0.f;
            if (key < visible) {
                if (vec) {
                    const int pid = table[(size_t)b * max_blocks + key / page];
                    if (pid >= 0) {
#pragma unroll
                        for (int c = 0; c < NC; ++c) {
                            const int d = lane + 64 * c;
                            if (d < hd) {
                                const float4 v4 = *reinterpret_cast<const float4*>(
                                    vc + (((size_t)pid * Hkv + g) * hd + d) * page + key % page);
                                v[0][c] = v4.x;
                                v[1][c] = key + 1 < visible ? v4.y : 0.f;      // slots never written may hold anything
                                v[2][c] = key + 2 < visible ? v4.z : 0.f;
                                v[3][c] = key + 3 < visible ? v4.w : 0.f;
                            }
                        }
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (key + u >= visible) continue;
                        const int pid = table[(size_t)b * max_blocks + (key + u) / page];
                        if (pid < 0) continue;
#pragma unroll
                        for (int c = 0; c < NC; ++c) {
                            const int d = lane + 64 * c;
                            if (d < hd) v[u][c] = vc[(((size_t)pid * Hkv + g) * hd + d) * page + (key + u) % page];
                        }
                    }
                }
            }
            float4 p4[4];
#pragma unroll
            for (int rb = 0; rb < 4; ++rb)
                p4[rb] = *reinterpret_cast<const float4*>(Ps + min(h0 + rb, G - 1) * EX_KEYS + jj);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int c = 0; c < NC; ++c)
#pragma unroll
                    for (int rb = 0; rb < 4; ++rb) {
                        const float pv = u == 0 ? p4[rb].x : u == 1 ? p4[rb].y : u == 2 ? p4[rb].z : p4[rb].w;
                        acc_b[rb][c] = fmaf(pv, v[u][c], acc_b[rb][c]);
                    }
        }
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            if (h0 + rb >= G) break;
            float* dst = part_o + (((size_t)t * H + (size_t)g * G + h0 + rb) * slots + slot) * hd;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const int d = lane + 64 * c;
                if (d < hd) dst[d] = acc_b[rb][c];
            }
        }
    }
}

// One wave per (token, head): the partial results of its key blocks, merged in ascending order.
template <int NC>
__global__ __launch_bounds__(64) void attn_exact_combine_kernel(
        const float* __restrict__ part_ml, const float* __restrict__ part_o,
        const int* __restrict__ row_of_token, const int* __restrict__ positions, const int* __restrict__ kv_lens,
        int H, int hd, int window, int slots, float* __restrict__ out, int out_stride) {
    const int t = blockIdx.y, h = blockIdx.x, lane = threadIdx.x;
    const int b = row_of_token[t];
    int n = 0;                                          // a padding token, or nothing to see: zeros
    if (b >= 0) {
        const int p = positions[t];
        const int visible = min(kv_lens[b], p + 1);
        const int j0 = window > 0 ? max(0, p + 1 - window) : 0;
        if (visible > j0) n = (visible - 1) / EX_KEYS - j0 / EX_KEYS + 1;
    }
    const float* ml = part_ml + ((size_t)t * H + h) * slots * 2;
    const float* po = part_o + ((size_t)t * H + h) * slots * hd;
    float m = -INFINITY, l = 0.f, acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.f;
    // eight partial results are asked for at a time (the loads do not depend on the merging), then
    // merged one after the other
    for (int s0 = 0; s0 < n; s0 += 8) {
        float mb[8], lb[8], acc_b[8][NC];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int s = min(s0 + u, n - 1);
            mb[u] = s0 + u < n ? ml[2 * s] : -INFINITY;      // -inf: merge_block leaves everything as it is
            lb[u] = ml[2 * s + 1];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const int d = lane + 64 * c;
                acc_b[u][c] = d < hd ? po[(size_t)s * hd + d] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) merge_block<NC>(m, l, acc, mb[u], lb[u], acc_b[u]);
    }
    float* o = out + (size_t)t * out_stride + (size_t)h * hd;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int d = lane + 64 * c;
        if (d < hd) o[d] = l > 0.f ? acc[c] / l : 0.f;
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
        // more LDS than a kernel gets unasked: requested once a device
        static bool asked[64] = {};
        int dev = 0;
        RI_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64, "ri_attention_exact_f32: no current device");
        if (!asked[dev]) {
            const size_t most = exact_lds_bytes(128);           // the largest head this kernel takes
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attn_exact_f32_kernel<2>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)most);
            RI_REQUIRE(e == hipSuccess, "ri_attention_exact_f32: %zu bytes of LDS refused: %s", most, hipGetErrorString(e));
            asked[dev] = true;
        }
    }
    kernel<<<dim3(tiles, Hkv), 256, lds, stream>>>(q, q_stride, out, out_stride, kc, vc, table, max_blocks, cu_q, q_start,
                                                   kv_lens, num_rows, H, Hkv, hd, page, scale, window, TQ);
    RI_LAUNCHED("ri_attention_exact_f32");
    return 0;
}

// Floats of workspace ri_attention_exact_decode_f32 needs for T tokens whose longest request has
// max_kv_len keys.
extern "C" size_t ri_attention_exact_decode_workspace(int T, int H, int hd, int max_kv_len) {
    const size_t slots = (size_t)(max_kv_len + EX_KEYS - 1) / EX_KEYS + 1;
    return (size_t)T * H * slots * (hd + 2);
}

// A step of single tokens on the exact path (every row of the step has one token; padding tokens
// carry row -1).  Same sizes as ri_attention_exact_supported.  The output of a token has the bits
// that ri_attention_exact_f32 gives the same token as part of any step.
extern "C" int ri_attention_exact_decode_f32(
        const float* q, int q_stride, float* out, int out_stride, const float* kc, const float* vc,
        int num_pages, int page, int H, int Hkv, int hd, const int* table, int max_blocks,
        const int* row_of_token, const int* positions, const int* kv_lens, int T, int max_kv_len,
        float scale, int window, float* workspace, size_t workspace_floats, hipStream_t stream) {
    RI_REQUIRE(ri_attention_exact_supported(H, Hkv, hd, page), "ri_attention_exact_decode_f32: sizes not taken (H=%d Hkv=%d hd=%d page=%d)", H, Hkv, hd, page);
    RI_REQUIRE(T >= 0 && max_kv_len > 0 && max_blocks > 0 && num_pages > 0 && window >= 0, "ri_attention_exact_decode_f32: bad sizes");
    RI_REQUIRE(q_stride >= H * hd && out_stride >= H * hd && q_stride % 4 == 0, "ri_attention_exact_decode_f32: bad row strides");
    if (T == 0) return 0;
    RI_REQUIRE(q && out && kc && vc && table && row_of_token && positions && kv_lens && workspace, "ri_attention_exact_decode_f32: null pointer");
    RI_REQUIRE((uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0 && (uintptr_t)q % 16 == 0, "ri_attention_exact_decode_f32: unaligned operands");
    RI_REQUIRE(Hkv <= 65535 && T <= 65535 && H <= 65535, "ri_attention_exact_decode_f32: too many heads or tokens for the grid");
    RI_REQUIRE(workspace_floats >= ri_attention_exact_decode_workspace(T, H, hd, max_kv_len),
               "ri_attention_exact_decode_f32: workspace of %zu floats, %zu needed", workspace_floats,
               ri_attention_exact_decode_workspace(T, H, hd, max_kv_len));
    const int G = H / Hkv;
    const int slots = (max_kv_len + EX_KEYS - 1) / EX_KEYS + 1;       // a window may begin inside a block: one more
    float* part_ml = workspace;
    float* part_o = workspace + (size_t)T * H * slots * 2;
    const size_t lds = sizeof(float) * 4 * G * EX_KEYS;
    dim3 grid((slots + 3) / 4, Hkv, T);
    if (hd <= 64) {
        attn_exact_decode_kernel<1><<<grid, 256, lds, stream>>>(q, q_stride, kc, vc, table, max_blocks, row_of_token, positions,
                                                               kv_lens, H, Hkv, hd, page, scale, window, slots, part_ml, part_o);
        RI_LAUNCHED("ri_attention_exact_decode_f32");
        attn_exact_combine_kernel<1><<<dim3(H, T), 64, 0, stream>>>(part_ml, part_o, row_of_token, positions, kv_lens, H, hd, window,
                                                                     slots, out, out_stride);
    } else {
        attn_exact_decode_kernel<2><<<grid, 256, lds, stream>>>(q, q_stride, kc, vc, table, max_blocks, row_of_token, positions,
                                                               kv_lens, H, Hkv, hd, page, scale, window, slots, part_ml, part_o);
        RI_LAUNCHED("ri_attention_exact_decode_f32");
        attn_exact_combine_kernel<2><<<dim3(H, T), 64, 0, stream>>>(part_ml, part_o, row_of_token, positions, kv_lens, H, hd, window,
                                                                     slots, out, out_stride);
    }
    RI_LAUNCHED("ri_attention_exact_decode_f32(combine)");
    return 0;
}
