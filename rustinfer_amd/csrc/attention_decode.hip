// bfloat16 attention of single tokens over the paged cache on the matrix cores (gfx950),
// with the key range split over waves ("flash decoding"; reference:
// crates/infer-backend-cuda/src/kernels/flash_attn_gqa/flash_attn_paged_decode.cu:75-337).
//
// One wave per (chunk of 64 or 128 keys, kv head, token); for long contexts a wave takes several
// chunks, one after the other, with a running maximum and sum, so that the number of partial
// results stays bounded.  All query heads of the kv head share each key and value load (they are the 16 columns of the MFMA tiles, G = H/Hkv <= 16 used).
//   S^T[key, q]  = K_tile[16 keys, hd] . Q^T[hd, 16 q]        v_mfma_f32_16x16x32_bf16
//   P^T = exp(S^T * scale - max)                                 in registers, 32-bit
//   O[q, d]     += P[16 q, 32 keys] . V[32 keys, 16 d]           v_mfma_f32_16x16x32_bf16
// The accumulator layout of the first product (a lane holds 4 keys of one q in each of two
// tiles) is the operand layout of the second for a suitable order of the 32 keys, and values are
// cached position-contiguous ([hd][page]), so nothing passes through LDS.  The keys of a span of
// 32 are dealt to its two tiles so that those 8 keys of a lane are consecutive (tile 0 takes keys
// 0-3, 8-11, 16-19, 24-27 of the span, tile 1 the others): a lane then reads its 8 values of a
// feature with one 16-byte load.
// Each wave writes an unnormalised partial output with its maximum and sum; a second kernel
// combines the partial results of a token.
//
// Layout of an MFMA 16x16x32 operand: lane l holds, for row/column l % 16, the 8 k-values
// of group l / 16; the accumulator holds rows (l / 16) * 4 + i, column l % 16.
#include "common.h"
#include <math.h>
#include <algorithm>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// TILES: 16-key tiles per wave (chunk = TILES * 16 keys).  Smaller chunks give more waves to
// hide latency with when the batch is small; larger ones fewer partial results.
// LOOP: a wave may take several chunks (false: exactly one, and the loop below folds away).
// BW: waves of a block.  1: the waves of a (kv head, token) are blocks of their own (blockIdx.x)
// and leave partial results for the second kernel.  More: they are the waves of one block, take
// the chunks in turn and combine their results through LDS; a single such block per (kv head,
// token) writes the output itself (with enough pairs to fill the chip that saves the second
// kernel and the trip of the partial results through memory), several of them (gridDim.x; where
// one a pair would leave compute units idle) leave one partial result each.
template <int HD, int TILES, bool LOOP, int BW>
__global__ __launch_bounds__(BW * 64) void attn_decode_split_kernel(
        const bf16_t* __restrict__ q, int q_stride,
        const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
        const int* __restrict__ table, int max_blocks,
        const int* __restrict__ row_of_token, const int* __restrict__ positions,
        const int* __restrict__ kv_lens, const int* __restrict__ cu_q, int H, int Hkv, int page,
        float scale, int window, int splits, float* __restrict__ part_o, float* __restrict__ part_ml,
        bf16_t* __restrict__ out, int out_stride, int rows, const int* __restrict__ single_tokens) {
    static_assert(BW == 1 || LOOP, "the waves of a block take the chunks in turn");
    extern __shared__ float lds[];                        // BW > 1: [BW][G][HD] outputs, [BW][16] maxima, [BW][16] sums
    // single_tokens (beside prompt portions): the tokens of the rows of one token, then -1; the grid
    // then spans those instead of every token of the step, most of which would have nothing to do
    const int g = blockIdx.y, t = single_tokens ? single_tokens[blockIdx.z] : (int)blockIdx.z;
    if (t < 0) return;
    // the wave's index is the same in all its lanes: said so, what depends on it alone (the chunk,
    // its pages' ids) is computed and loaded once a wave, on the scalar unit
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), col = lane & 15, grp = lane >> 4;
    const int G = H / Hkv;
    // Q^T fragments: column = query head of this group, k = head dimension
    bf16x8_t qf[HD / 32];
#pragma unroll
    for (int kk = 0; kk < HD / 32; ++kk) {
        if (col < G)
            qf[kk] = *reinterpret_cast<const bf16x8_t*>(q + (size_t)t * q_stride + (size_t)(g * G + col) * HD + kk * 32 + grp * 8);
        else
            for (int e = 0; e < 8; ++e) qf[kk][e] = (__bf16)0.f;
    }

    // Rows of one token usually come in the order of their tokens (token t is row t).  The row's
    // length and the page ids of the first chunk are asked for on that guess, together with the
    // token's row and position and before it is known whether the chunk lies within the row, so
    // that the keys can be asked for after one round trip to memory instead of three.
    constexpr int CHUNK = TILES * 16;
    const int S = BW * (int)gridDim.x;                    // waves per (kv head, token)
    int c = (int)blockIdx.x * BW + wave;
    const bool whole = BW > 1 && gridDim.x == 1;          // this block sees all the chunks and writes the output itself
    const int b_guess = min(t, rows - 1);
    int blk_of[TILES];                                    // pages of the chunk's 16-key stretches
#pragma unroll
    for (int tile = 0; tile < TILES; ++tile)
        blk_of[tile] = table[(size_t)b_guess * max_blocks + min((c * CHUNK + tile * 16) / page, max_blocks - 1)];
    int kv_len = kv_lens[b_guess];
    const int p = positions[t];
    const int b = row_of_token[t];
    if (b >= 0 && cu_q && cu_q[b + 1] - cu_q[b] != 1) return;      // rows of several tokens belong to the tiled kernel
    if (b < 0) {                                          // a padding token
        if (whole) {
            bf16_t* o_row = out + (size_t)t * out_stride + (size_t)g * G * HD;
            for (int e = threadIdx.x; e < G * HD; e += BW * 64) o_row[e] = 0;
        }
        return;
    }
    if (b != b_guess) {                                   // the guess was wrong: ask again
#pragma unroll
        for (int tile = 0; tile < TILES; ++tile)
            blk_of[tile] = table[(size_t)b * max_blocks + min((c * CHUNK + tile * 16) / page, max_blocks - 1)];
        kv_len = kv_lens[b];
    }
    const int visible = min(kv_len, p + 1);
    const int j0 = window > 0 ? max(0, p + 1 - window) : 0;
    if (visible <= j0) {                                  // nothing to see (the same for the whole block)
        if (whole) {
            bf16_t* o_row = out + (size_t)t * out_stride + (size_t)g * G * HD;
            for (int e = threadIdx.x; e < G * HD; e += BW * 64) o_row[e] = 0;
        }
        return;
    }
    const int c_last = (visible - 1) / CHUNK;
    // the combine reads the slots of the blocks whose first chunk exists: [0, min(blocks, c_last / BW + 1))
    if (!whole && (int)blockIdx.x * BW > c_last) return;

    // A wave takes the chunks c, c + S, c + 2S, ... of its row and keeps a running maximum, sum
    // and output over them, so that a long context leaves S partial results, not one per chunk.
    f32x4_t o[HD / 16];
#pragma unroll
    for (int db = 0; db < HD / 16; ++db) o[db] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    for (bool first = true; (LOOP || first) && c <= c_last; c += S, first = false) {
        const int c_lo = c * CHUNK;
        if (LOOP && !first) {
#pragma unroll
            for (int tile = 0; tile < TILES; ++tile)
                blk_of[tile] = table[(size_t)b * max_blocks + min((c_lo + tile * 16) / page, max_blocks - 1)];
        }
        if (c_lo + CHUNK <= j0) continue;                 // the window has passed this chunk

        // All key and value fragments of the chunk are requested before anything is computed, so
        // a wave waits for memory once a chunk.
        // Span sp = keys c_lo + 32 sp .. + 31; its tile e holds, in row r, key 8 (r / 4) + 4 e + r % 4.
        bf16x8_t kf[TILES][HD / 32];
        bf16x8_t vf[TILES / 2][HD / 16];
        bool live[TILES / 2];
#pragma unroll
        for (int sp = 0; sp < TILES / 2; ++sp) {
            const int span0 = c_lo + sp * 32;
            live[sp] = span0 < visible && span0 + 32 > j0;
            // keys: this lane's row of either tile lies in the first 16 keys of the span (col < 8) or the second
            const int kblk = live[sp] ? (col < 8 ? blk_of[2 * sp] : blk_of[2 * sp + 1]) : -1;
            const int krow = span0 + (col >> 2) * 8 + (col & 3);                  // tile 0; tile 1: + 4
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                if (kblk >= 0 && krow + 4 * e < visible) {
                    const bf16_t* kt = kc + ((size_t)kblk * Hkv + g) * (size_t)page * HD + (size_t)((krow + 4 * e) % page) * HD + grp * 8;
#pragma unroll
                    for (int kk = 0; kk < HD / 32; ++kk) kf[2 * sp + e][kk] = ld_stream16<bf16x8_t>(kt + kk * 32);
                } else {                                  // a page the window has passed, or a key not written yet
#pragma unroll
                    for (int kk = 0; kk < HD / 32; ++kk) for (int x = 0; x < 8; ++x) kf[2 * sp + e][kk][x] = (__bf16)0.f;
                }
            }
            // values: this lane's 8 keys are span0 + 8 grp .. + 7, one 16-byte piece of a feature's row
            const int vblk = live[sp] ? (grp < 2 ? blk_of[2 * sp] : blk_of[2 * sp + 1]) : -1;
            const int vkey = span0 + grp * 8;
            if (vblk >= 0 && vkey < visible) {
                const bf16_t* vt = vc + ((size_t)vblk * Hkv + g) * (size_t)page * HD + (size_t)col * page + vkey % page;
#pragma unroll
                for (int db = 0; db < HD / 16; ++db) vf[sp][db] = ld_stream16<bf16x8_t>(vt + (size_t)db * 16 * page);
                // positions never written (the rest of the last page) may hold anything, NaN included
                if (vkey + 8 > visible) {
                    const int n = visible - vkey;
#pragma unroll
                    for (int db = 0; db < HD / 16; ++db)
#pragma unroll
                        for (int x = 0; x < 8; ++x)
                            if (x >= n) vf[sp][db][x] = (__bf16)0.f;
                }
            } else {
#pragma unroll
                for (int db = 0; db < HD / 16; ++db) for (int x = 0; x < 8; ++x) vf[sp][db][x] = (__bf16)0.f;
            }
        }
        // scores: st[tile][i] = S^T[key = c_lo + 32 (tile / 2) + 8 grp + 4 (tile % 2) + i][q = col]
        f32x4_t st[TILES];
#pragma unroll
        for (int tile = 0; tile < TILES; ++tile) {
            st[tile] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < HD / 32; ++kk)
                st[tile] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[tile][kk], qf[kk], st[tile], 0, 0, 0);
        }
        // mask, scale, maximum over the keys of each q (this chunk and those before)
        float m = m_run;
#pragma unroll
        for (int tile = 0; tile < TILES; ++tile) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = c_lo + (tile >> 1) * 32 + grp * 8 + (tile & 1) * 4 + i;
                const float sc = (key < visible && key >= j0) ? st[tile][i] * scale : -INFINITY;
                st[tile][i] = sc;
                m = fmaxf(m, sc);
            }
        }
        m = fmaxf(m, __shfl_xor(m, 16, 64));
        m = fmaxf(m, __shfl_xor(m, 32, 64));
        float lsum = 0.f;
#pragma unroll
        for (int tile = 0; tile < TILES; ++tile) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = __expf(st[tile][i] - m);        // exp(-inf) = 0 for masked keys
                st[tile][i] = e;
                lsum += e;
            }
        }
        lsum += __shfl_xor(lsum, 16, 64);
        lsum += __shfl_xor(lsum, 32, 64);
        if (LOOP && !first) {
            // what the earlier chunks left is brought to the new maximum; m and l belong to the
            // query in this lane's column, the output rows to the queries grp*4 + i
            const float alpha = __expf(m_run - m);              // 0 if nothing was seen so far
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float ai = __shfl(alpha, grp * 4 + i, 64);
#pragma unroll
                for (int db = 0; db < HD / 16; ++db) o[db][i] *= ai;
            }
        }
        l_run += lsum;
        m_run = m;

        // O[q, d] += P . V over the spans: this lane's 8 keys are span keys 8 grp .. + 7, for P
        // (4 from either tile) and for V alike
#pragma unroll
        for (int sp = 0; sp < TILES / 2; ++sp) {
            if (!live[sp]) continue;
            bf16x8_t pf;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                pf[i] = (__bf16)st[2 * sp][i];
                pf[4 + i] = (__bf16)st[2 * sp + 1][i];
            }
#pragma unroll
            for (int db = 0; db < HD / 16; ++db)
                o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf[sp][db], o[db], 0, 0, 0);
        }
    }
    if constexpr (BW > 1) {
        // the waves' results meet in LDS; then every thread finishes a few outputs
        float* so = lds;                                   // [BW][G][HD]
        float* sm = lds + (size_t)BW * G * HD;              // [BW][16]
        float* sl = sm + BW * 16;                          // [BW][16]
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int qi = grp * 4 + i;
            if (qi < G) {
#pragma unroll
                for (int db = 0; db < HD / 16; ++db) so[((size_t)wave * G + qi) * HD + db * 16 + col] = o[db][i];
            }
        }
        if (grp == 0) { sm[wave * 16 + col] = m_run; sl[wave * 16 + col] = l_run; }
        __syncthreads();
        bf16_t* o_row = out + (size_t)t * out_stride + (size_t)g * G * HD;
        for (int e = threadIdx.x; e < G * HD; e += BW * 64) {
            const int qi = e / HD, d = e - qi * HD;
            float m = -INFINITY;
#pragma unroll
            for (int w = 0; w < BW; ++w) m = fmaxf(m, sm[w * 16 + qi]);
            float acc = 0.f, l = 0.f;
#pragma unroll
            for (int w = 0; w < BW; ++w) {
                // 0 for a wave without chunks (and for all of them, if a window has passed every chunk of this block)
                const float wgt = sm[w * 16 + qi] == -INFINITY ? 0.f : __expf(sm[w * 16 + qi] - m);
                acc += wgt * so[((size_t)w * G + qi) * HD + d];
                l += wgt * sl[w * 16 + qi];
            }
            if (whole) {
                o_row[e] = f32_to_bf16(acc / l);
            } else {
                // one of several blocks of this (kv head, token): its sums go to slot blockIdx.x
                const size_t slot = ((size_t)b * H + g * G + qi) * splits + blockIdx.x;
                part_o[slot * HD + d] = acc;
                if (d == 0) { part_ml[slot * 2] = m; part_ml[slot * 2 + 1] = l; }
            }
        }
        return;
    }
    // partial results in slot blockIdx.x: o[db][i] = O[q = grp*4 + i][d = db*16 + col]
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int qi = grp * 4 + i;
        if (qi < G) {
            float* dst = part_o + (((size_t)b * H + g * G + qi) * splits + blockIdx.x) * HD;   // a row of one token: indexed by row
#pragma unroll
            for (int db = 0; db < HD / 16; ++db) dst[db * 16 + col] = o[db][i];
        }
    }
    if (grp == 0 && col < G) {
        float* dst = part_ml + (((size_t)b * H + g * G + col) * splits + blockIdx.x) * 2;
        dst[0] = m_run;
        dst[1] = l_run;
    }
}

// One block of CW waves per (token, head).  The partial results of the chunks are rows of HD
// floats; a wave reads them 16 bytes a lane, 64 / (HD / 4) rows per load instruction, several
// instructions in flight, and each wave takes its share of the rows, so that long contexts
// (hundreds of chunks) are combined by more than a trickle of 4-byte loads.
template <int HD, int CW>
__global__ __launch_bounds__(CW * 64) void attn_decode_combine_kernel(
        const float* __restrict__ part_o, const float* __restrict__ part_ml, int splits, int chunk,
        const int* __restrict__ row_of_token, const int* __restrict__ positions,
        const int* __restrict__ kv_lens, const int* __restrict__ cu_q, int H, int window,
        bf16_t* __restrict__ out, int out_stride, int rows, const int* __restrict__ single_tokens) {
    constexpr int LPP = HD / 4;               // lanes per row of partial results (a float4 each)
    constexpr int PPW = 64 / LPP;             // rows per load instruction of a wave
    constexpr int UNR = 4;                    // load instructions in flight
    __shared__ float red[16];
    __shared__ float4 accs[CW][LPP];
    __shared__ float ls[CW];
    const int t = single_tokens ? single_tokens[blockIdx.x] : (int)blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    if (t < 0) return;
    const int lane = tid & 63, wave = tid >> 6;
    bf16_t* o = out + (size_t)t * out_stride + (size_t)h * HD;
    // as in the first kernel, the row is guessed to be the token's index, and what depends on it
    // (the row's length, this thread's first maximum) is asked for together with the row itself
    const int b_guess = min(t, rows - 1);
    int kv_len = kv_lens[b_guess];
    float m_first = tid < splits ? part_ml[(((size_t)b_guess * H + h) * splits + tid) * 2] : -INFINITY;
    const int p = positions[t];
    const int b = row_of_token[t];
    if (b >= 0 && cu_q && cu_q[b + 1] - cu_q[b] != 1) return;
    if (b >= 0 && b != b_guess) {
        kv_len = kv_lens[b];
        m_first = tid < splits ? part_ml[(((size_t)b * H + h) * splits + tid) * 2] : -INFINITY;
    }
    int visible = 0, j0 = 0;
    if (b >= 0) {
        visible = min(kv_len, p + 1);
        j0 = window > 0 ? max(0, p + 1 - window) : 0;
    }
    if (visible <= j0) {                      // a padding token, or nothing to see: zeros
        for (int e = tid; e < HD; e += CW * 64) o[e] = 0;
        return;
    }
    // the waves of the first kernel left one slot each; those beyond the row's last chunk none
    const int n = min(splits, (visible - 1) / chunk + 1);
    const float2* ml = reinterpret_cast<const float2*>(part_ml) + ((size_t)b * H + h) * splits;
    const float4* po = reinterpret_cast<const float4*>(part_o + ((size_t)b * H + h) * splits * HD);
    float m = tid < n ? m_first : -INFINITY;             // slots beyond n hold nothing of this step
    for (int i = tid + CW * 64; i < n; i += CW * 64) m = fmaxf(m, ml[i].x);
    m = CW > 1 ? block_max(m, red) : wave_max(m);
    const int sub = lane / LPP, colv = lane % LPP;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float l = 0.f;
    for (int i0 = wave * PPW + sub; i0 < n; i0 += CW * PPW * UNR) {
        float4 pv[UNR];
        float2 mv[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int i = i0 + u * CW * PPW;
            const bool ok = i < n;
            pv[u] = ok ? po[(size_t)i * LPP + colv] : make_float4(0.f, 0.f, 0.f, 0.f);
            mv[u] = ok ? ml[i] : make_float2(-INFINITY, 0.f);
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const float wgt = __expf(mv[u].x - m);                // 0 for rows beyond the end
            acc.x += wgt * pv[u].x; acc.y += wgt * pv[u].y; acc.z += wgt * pv[u].z; acc.w += wgt * pv[u].w;
            if (colv == 0) l += wgt * mv[u].y;
        }
    }
    // rows that share a wave, then the waves
#pragma unroll
    for (int off = LPP; off < 64; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off, 64); acc.y += __shfl_xor(acc.y, off, 64);
        acc.z += __shfl_xor(acc.z, off, 64); acc.w += __shfl_xor(acc.w, off, 64);
    }
    l = wave_sum(l);
    if (CW > 1) {
        if (lane < LPP) accs[wave][lane] = acc;
        if (lane == 0) ls[wave] = l;
        __syncthreads();
        if (wave > 0) return;
        for (int w = 1; w < CW; ++w) {
            if (lane < LPP) { const float4 a = accs[w][lane]; acc.x += a.x; acc.y += a.y; acc.z += a.z; acc.w += a.w; }
            l += ls[w];
        }
    }
    if (lane < LPP) {
        const float inv = 1.f / l;
        uint2 r;
        r.x = (uint32_t)f32_to_bf16(acc.x * inv) | ((uint32_t)f32_to_bf16(acc.y * inv) << 16);
        r.y = (uint32_t)f32_to_bf16(acc.z * inv) | ((uint32_t)f32_to_bf16(acc.w * inv) << 16);
        *reinterpret_cast<uint2*>(o + lane * 4) = r;
    }
}

// keys per wave: 128 when there are waves enough anyway, else 64 (with 8 or fewer rows of 2,000
// keys, chunks of 32, 64 and 128 keys take the same time within 1 %: the kernel is not bound by
// the number of its waves or of its load instructions)
static int decode_chunk(int T, int Hkv, int hd, int max_kv_len) {
    if (hd == 128) return 64;
    const long long waves128 = (long long)T * Hkv * ((max_kv_len + 127) / 128);
    return waves128 >= 4096 ? 128 : 64;
}

extern "C" size_t ri_attention_decode_workspace(int rows, int H, int hd, int max_kv_len) {
    const size_t splits = (size_t)(max_kv_len + 63) / 64;        // the smaller chunk bounds both
    return (size_t)rows * H * splits * (hd + 2) * sizeof(float);
}

extern "C" int ri_attention_decode_supported(int H, int Hkv, int hd, int page) {
    return (hd == 64 || hd == 128) && page % 16 == 0 && Hkv > 0 && H % Hkv == 0 && H / Hkv <= 16;
}

extern "C" int ri_attention_decode(
        const void* q, int q_stride, void* out, int out_stride,
        const void* kc, const void* vc, int num_pages, int page, int H, int Hkv, int hd,
        const int* table, int max_blocks, const int* row_of_token, const int* positions,
        const int* kv_lens, const int* cu_q, int T, int rows, int max_kv_len, float scale, int window,
        void* workspace, size_t workspace_bytes, int singles, const int* single_tokens, int pair_blocks,
        hipStream_t stream) {
    // singles: how many of the T tokens are rows of one token, at most (the others belong to longer
    // portions and are left alone); <= 0: all of them.  It steers how the work is divided, and with
    // single_tokens (their `singles` flat token indices, -1 where there are fewer; may be null) the
    // grids span those tokens only: a step of a 256-token portion beside 8 single tokens otherwise
    // starts 8,448 blocks for the 256 that have work, 42 us instead of 16.
    RI_REQUIRE(ri_attention_decode_supported(H, Hkv, hd, page),
               "ri_attention_decode: needs head size 64 or 128, pages that are multiples of 16 and at most 16 "
               "query heads per kv head; got hd=%d page=%d H=%d Hkv=%d", hd, page, H, Hkv);
    RI_REQUIRE(T >= 0 && max_kv_len > 0 && max_blocks > 0 && num_pages > 0 && window >= 0, "ri_attention_decode: bad sizes");
    RI_REQUIRE(q_stride >= H * hd && out_stride >= H * hd && q_stride % 8 == 0 && out_stride % 4 == 0, "ri_attention_decode: bad row strides");
    RI_REQUIRE((long long)max_blocks * page >= max_kv_len, "ri_attention_decode: block table shorter than max_kv_len");
    if (T == 0) return 0;
    RI_REQUIRE(T <= 65535 && Hkv <= 65535, "ri_attention_decode: grid too large");
    RI_REQUIRE(q && out && kc && vc && table && row_of_token && positions && kv_lens && workspace, "ri_attention_decode: null pointer");
    RI_REQUIRE((uintptr_t)q % 16 == 0 && (uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0 && (uintptr_t)out % 8 == 0 && (uintptr_t)workspace % 16 == 0,
               "ri_attention_decode: operands must be 16-byte aligned (the output 8-byte)");
    RI_REQUIRE(rows >= 1, "ri_attention_decode: %d tokens but no rows", T);
    RI_REQUIRE(workspace_bytes >= ri_attention_decode_workspace(rows, H, hd, max_kv_len), "ri_attention_decode: workspace too small");
    const int busy = singles > 0 && singles < T ? singles : T;      // tokens that have work
    const int chunk = decode_chunk(busy, Hkv, hd, max_kv_len);
    // One wave per chunk while that keeps the number of waves and of partial results moderate;
    // beyond, about 2048 waves (two per SIMD) take several chunks each, the same number as
    // nearly as it divides, which bounds what the second kernel has to read.
    const int nchunks = (max_kv_len + chunk - 1) / chunk;
    const long long rows_heads = (long long)busy * Hkv;
    int splits = nchunks;
    if (nchunks > 64 || nchunks * rows_heads > 16384) {
        const long long cap = 2048 / rows_heads > 1 ? 2048 / rows_heads : 1;
        if (nchunks > cap) {
            const int per = (int)((nchunks + cap - 1) / cap);
            splits = (nchunks + per - 1) / per;
        }
    }
    // Blocks of several waves (as many as their registers allow) that take a pair's chunks in turn
    // and combine through LDS: one block a (kv head, token) pair that writes the output itself, or
    // several that leave a partial result each.  A compute unit holds one such block, and the time
    // is that of the fullest unit: the number of blocks a pair is the one (up to 8, and no more
    // than give every wave a chunk of the longest row) that fills whole rounds of the chip's 256
    // units best, where one a pair would leave a fifth of them idle or more; if that makes blocks
    // enough and leaves a wave at most 8 chunks (with 512 pairs or more any number); else the form
    // of one wave a chunk above.  Measured against what
    // ran before, head 128, us: 8 rows of 2,048 keys 20.3 -> 17.9 (4 blocks a pair), 16 rows
    // 43.1 -> 28.7 (2), 24 rows 45.9 -> 43.5 (4); 4,096 keys: 8 rows 34.6 -> 28.4, 16 rows 79.0 ->
    // 50.6, 4 rows 20.3 -> 18.0 (8); head 64: 16 rows of 2,048 keys 23.8 -> 18.1, 8 rows of 4,096
    // 20.7 -> 18.1.  pair_blocks: 0 lets the entry point choose, 1 forbids several blocks a pair,
    // more asks for that many.
    const int bw_ = hd == 64 ? 16 : 8;
    const int chunks64_ = (max_kv_len + 63) / 64;
    const bool lds_ok = (size_t)bw_ * ((size_t)(H / Hkv) * hd + 32) * sizeof(float) <= 64 * 1024;
    int nblk = 0;                                         // 0: one wave a chunk; 1: one block a pair; more: several
    if (pair_blocks > 1) {
        nblk = std::min(pair_blocks, std::max(chunks64_ / bw_, 1));
    } else if (lds_ok && rows_heads >= 32) {
        const int max_n = pair_blocks == 1 ? 1 : std::max(std::min(chunks64_ / bw_, 8), 1);
        auto fill = [&](int n) {
            const long long blocks = rows_heads * n;
            return (double)blocks / (256.0 * (double)((blocks + 255) / 256));
        };
        nblk = 1;
        if (fill(1) < 0.8) {                              // else one block a pair wastes little (56 rows: four a pair lose 10-25 %)
            double best = 0.0;
            for (int n = 1; n <= max_n; ++n)
                if (fill(n) > best + 1e-9) { best = fill(n); nblk = n; }
        }
        const bool few_chunks_a_wave = chunks64_ <= bw_ * 8 * nblk || rows_heads >= 512;
        // Blocks enough: 128 of one a pair (measured with caches larger than the last-level cache:
        // from 128 pairs on 6 % faster than one wave a chunk, 20 % at 256; at 96 pairs 10 % slower);
        // of several a pair 192, and 256 at head 64, where a block of 16 waves costs more to start
        // and to combine (8 rows of 3,072 keys: 3 blocks a pair lose 4 %)
        const long long min_blocks = nblk == 1 ? 128 : (hd == 64 ? 256 : 192);
        if (rows_heads * nblk < min_blocks || !few_chunks_a_wave) nblk = 0;
    }
    RI_REQUIRE(nblk == 0 || lds_ok, "ri_attention_decode: %d heads a kv head are too many for blocks of several waves", H / Hkv);
    if (nblk > 1) splits = nblk;
    const int* sel = (single_tokens && singles > 0 && singles < T) ? single_tokens : nullptr;
    const int TZ = sel ? singles : T;                     // tokens the grids span
    float* part_o = (float*)workspace;
    float* part_ml = part_o + (size_t)rows * H * splits * hd;
#define RI_DECODE_ARGS (const bf16_t*)q, q_stride, (const bf16_t*)kc, (const bf16_t*)vc, table, max_blocks, row_of_token, positions, kv_lens, cu_q, H, Hkv, page, scale, window, splits, part_o, part_ml, (bf16_t*)out, out_stride, rows, sel
    if (nblk > 0) {
        const int G = H / Hkv;
        const size_t lds_bytes = (size_t)bw_ * ((size_t)G * hd + 32) * sizeof(float);
        dim3 gridh(nblk, Hkv, TZ);
        if (hd == 64) attn_decode_split_kernel<64, 4, true, 16><<<gridh, 16 * 64, lds_bytes, stream>>>(RI_DECODE_ARGS);
        else attn_decode_split_kernel<128, 4, true, 8><<<gridh, 8 * 64, lds_bytes, stream>>>(RI_DECODE_ARGS);
        RI_LAUNCHED("ri_attention_decode(blocks)");
        if (nblk == 1) return 0;                          // the block has written the output itself
        dim3 grid2(TZ, H);
        const int block_keys = 64 * bw_;                  // a block's first chunk begins a multiple of this many keys in
        if (hd == 64) attn_decode_combine_kernel<64, 1><<<grid2, 64, 0, stream>>>(part_o, part_ml, splits, block_keys, row_of_token, positions, kv_lens, cu_q, H, window, (bf16_t*)out, out_stride, rows, sel);
        else attn_decode_combine_kernel<128, 1><<<grid2, 64, 0, stream>>>(part_o, part_ml, splits, block_keys, row_of_token, positions, kv_lens, cu_q, H, window, (bf16_t*)out, out_stride, rows, sel);
        RI_LAUNCHED("ri_attention_decode(combine)");
        return 0;
    }
    dim3 grid(splits, Hkv, TZ);
    dim3 grid2(TZ, H);
    const bool loop = splits < nchunks;
#define RI_DECODE_LAUNCH(HD_, TILES_) do { \
        if (loop) attn_decode_split_kernel<HD_, TILES_, true, 1><<<grid, 64, 0, stream>>>(RI_DECODE_ARGS); \
        else attn_decode_split_kernel<HD_, TILES_, false, 1><<<grid, 64, 0, stream>>>(RI_DECODE_ARGS); } while (0)
    if (hd == 64 && chunk == 128) RI_DECODE_LAUNCH(64, 8);
    else if (hd == 64) RI_DECODE_LAUNCH(64, 4);
    else RI_DECODE_LAUNCH(128, 4);
#undef RI_DECODE_LAUNCH
#undef RI_DECODE_ARGS
    RI_LAUNCHED("ri_attention_decode");
    // more waves per (token, head) where there are many chunks to combine
#define RI_COMBINE_ARGS part_o, part_ml, splits, chunk, row_of_token, positions, kv_lens, cu_q, H, window, (bf16_t*)out, out_stride, rows, sel
    if (hd == 64 && splits <= 64) attn_decode_combine_kernel<64, 1><<<grid2, 64, 0, stream>>>(RI_COMBINE_ARGS);
    else if (hd == 64) attn_decode_combine_kernel<64, 4><<<grid2, 256, 0, stream>>>(RI_COMBINE_ARGS);
    else if (splits <= 32) attn_decode_combine_kernel<128, 1><<<grid2, 64, 0, stream>>>(RI_COMBINE_ARGS);
    else attn_decode_combine_kernel<128, 4><<<grid2, 256, 0, stream>>>(RI_COMBINE_ARGS);
#undef RI_COMBINE_ARGS
    RI_LAUNCHED("ri_attention_decode(combine)");
    return 0;
}
