// bfloat16 attention of prompt portions over the paged cache on the matrix cores (gfx950):
// ragged rows, causal from the bottom right (a portion sees the cached prefix), optional
// window.  Reference: crates/infer-backend-cuda/src/kernels/flash_attn_gqa/flash_attn_paged_prefill.cu:316-540.
//
// A wave owns 16 consecutive queries of one request and NQ query heads of one kv head; the
// four waves of a block own a tile of 64 consecutive queries, so they read the same keys and
// values at about the same time.  Under the causal mask a late tile sees many keys and an
// early one few, so every block does two tiles one after the other, the i-th from the end and
// the i-th from the start: all waves of a launch then have the same amount of work, whatever
// order blocks are started in.  Blocks of one kv head are Hkv apart in the grid, which with 8
// kv heads puts each head's keys and values into one XCD's L2.  Per step of 32 keys:
//   S^T[key, q] = K_tile[16 keys, hd] . Q^T[hd, 16 q]      (two tiles)   v_mfma_f32_16x16x32_bf16
//   online softmax per query in 32-bit (running maximum and sum, exp2)
//   O[q, d]    += P[16 q, 32 keys] . V[32 keys, 16 d]                    v_mfma_f32_16x16x32_bf16
// As in the single-token kernel the accumulator of the first product is the operand of the
// second, and values are cached position-contiguous, so scores and probabilities never go
// through LDS; keys and values do in the SHARE form below, once per block instead of per wave.
// A wave issues at most one instruction every four cycles, scalar ones included, so the loop
// is bound by its instruction count: steps that lie wholly below the diagonal run a body without
// masks (raw v_exp_f32, one fused multiply-add per score, a softmax reference that moves only
// when it must), the page size is a compile-time 16 where it can be, and only the last one or
// two steps of a tile take the general body.
#include "common.h"
#include <math.h>
#include <algorithm>

typedef __bf16 pbf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 pbf16x4_t __attribute__((ext_vector_type(4)));
typedef float pf32x4_t __attribute__((ext_vector_type(4)));

// Max of three.  This file is compiled without IEEE mode and with NaNs assumed absent (the
// scores are finite or -inf by construction), so that fmaxf becomes a bare v_max3_f32 without
// the NaN-quieting moves it otherwise brings along.  It must stay a compiler-visible
// operation: inline assembly that reads the result registers of a matrix instruction gets
// none of the wait states such a read needs, and then reads stale values now and then.
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    return __builtin_fmaxf(__builtin_fmaxf(a, b), c);
}

template <int HD>
struct PrefillFrags {
    pbf16x8_t k0[HD / 32], k1[HD / 32];
    pbf16x8_t v[HD / 16];
    int blk0, blk1;                                               // pages of keys 0-15 and 16-31 of the step
};

// Which key sits in which row of the two 16-key MFMA tiles of a 32-key step is free, as long
// as P and V use the same order in the second product.  Rows are dealt so that the 8 scores a
// lane ends up with (4 rows of each tile) are 8 CONSECUTIVE keys: tile 0 holds keys
// {0-3, 8-11, 16-19, 24-27} of the step, tile 1 the others.  Then a lane's value operand is one
// 16-byte load from the position-contiguous value cache.
// FAST: pages of 16 and no window, the usual case, known when compiling; else the arguments count.
// SHARE (with FAST): the four waves of a block ask for the same keys and values; each fetches a
// quarter of a step's fragments and hands them to the others through LDS, in the order the
// matrix instructions read them (a fragment is 64 lanes x 16 bytes, contiguous).  The waves then
// walk the keys in step, up to the last key any of them sees; a quarter of the traffic between
// L2 and the CUs, which is what bounds the kernel once a prompt portion has waves enough.
// SPLIT (with SHARE): the keys are also divided between blocks, split_keys of them (a multiple of
// 128) to each value of the grid's third index; a block leaves what its range of keys gives a
// query (the sums, their softmax reference and the probabilities' total, in 32-bit) in part_o /
// part_ml, and attn_prefill_combine_kernel puts a query's ranges together.  For short portions
// behind a long cached prefix, whose few tiles would otherwise each walk all the keys one step
// after the other while most of the chip has nothing to do.
template <int HD, int NQ, bool FAST, bool SHARE = false, int WPE = 1, bool SPLIT = false>
__global__ __launch_bounds__(256, WPE) void attn_prefill_kernel(
        const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
        const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
        const int* __restrict__ table, int max_blocks,
        const int* __restrict__ cu_q, const int* __restrict__ q_start, const int* __restrict__ kv_lens,
        int H, int Hkv, int page_arg, float scale_log2e, int window_arg, int head_groups, int min_q_len,
        int split_keys, int nsplit, float* __restrict__ part_o, float* __restrict__ part_ml, int part_tokens,
        const int* __restrict__ row_list) {
    typedef PrefillFrags<HD> Frags;
    static_assert(!SHARE || FAST, "fragments are shared only with pages of 16 and no window");
    static_assert(!SPLIT || SHARE, "the keys are divided between blocks only in the shared form");
    // this block's range of keys [kb, ke)
    const int split = SPLIT ? (int)__builtin_amdgcn_workgroup_id_z() : 0;
    const int kb = SPLIT ? split * split_keys : 0;
    const int ke = SPLIT && split + 1 < nsplit ? kb + split_keys : 0x7fffffff;     // the last range takes what is left
    constexpr int NF = HD / 8;                                   // fragments of a step: 2 * HD/32 of keys, HD/16 of values
    __shared__ pbf16x8_t kv_lds[SHARE ? 4 * NF * 64 : 1];             // a ring of four steps' fragments
    const int page = FAST ? 16 : page_arg;
    const int window = FAST ? 0 : window_arg;
    // Block and thread ids are taken from the builtins: this file's floating-point flags keep
    // the device library's id functions from being inlined, and a call would hide from the
    // compiler that block ids are the same for all lanes.
    // row_list (may be null): the rows this kernel is for, then -1; the grid's second index then runs over those
    const int bx = __builtin_amdgcn_workgroup_id_x();
    const int b = row_list ? row_list[__builtin_amdgcn_workgroup_id_y()] : (int)__builtin_amdgcn_workgroup_id_y();
    if (b < 0) return;
    const int tx = __builtin_amdgcn_workitem_id_x();
    const int t_lo = cu_q[b], q_len = cu_q[b + 1] - t_lo;
    // the wave index is the same for all lanes; telling the compiler lets it keep the key loop
    // and the block-table reads on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(tx >> 6), lane = tx & 63;
    const int g = bx % Hkv, rest = bx / Hkv;
    const int hsub = rest % head_groups, pair = rest / head_groups;
    const int ntiles = (q_len + 63) / 64;                        // tiles of 64 queries of this row
    if (q_len < min_q_len || pair >= (ntiles + 1) / 2) return;
    const int G = H / Hkv;
    const int col = lane & 15, grp = lane >> 4;
    const int start = q_start[b];
    const int kv_len = kv_lens[b];
    const int* trow = table + (size_t)b * max_blocks;
    // this lane's key row in the tiles: rows 0-7 come from the first 16 keys of the step
    const int krow = ((col >> 2) & 1) * 8 + (col & 3);           // + 4 for tile 1
    const bool k_second_half = col >= 8;                         // keys 16-31 of the step
    const bool v_second_half = grp >= 2;
    const uint32_t slab = (uint32_t)page * HD;                   // one kv head of one page
    const uint32_t page_stride = (uint32_t)Hkv * slab;           // checked on the host to fit 32 bits
    const bf16_t* kbase = kc + (size_t)g * slab + (size_t)krow * HD + grp * 8;
    const bf16_t* vbase = vc + (size_t)g * slab + (size_t)col * page + (grp & 1) * 8;

#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
        const int tile = half == 0 ? ntiles - 1 - pair : pair;   // the late tile first
        if (half == 1 && tile == ntiles - 1 - pair) break;       // the middle tile of an odd number is done once
        if constexpr (SPLIT) {
            // no query of the tile sees a key of this block's range (the same for all waves)
            if (min(kv_len, start + min(q_len, tile * 64 + 64)) <= kb) continue;
        }
        const int tile0 = (tile * 4 + wave) * 16;                // first query of this wave within the row
        const bool active = tile0 < q_len;                       // a wave without queries still fetches its share
        if (!SHARE && !active) continue;
        const int n_valid = active ? min(16, q_len - tile0) : 0; // queries of this tile that exist
        const int p_first = start + tile0, p_last = p_first + n_valid - 1;
        const bool q_ok = col < n_valid;
        const int p = q_ok ? p_first + col : -1;                 // this lane's query position (as a column)
        const int j0 = (window > 0 && q_ok) ? max(0, p + 1 - window) : 0;

        // Q^T fragments of the NQ heads
        pbf16x8_t qf[NQ][HD / 32];
        int head[NQ];
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq) {
            const int hq = hsub * NQ + nq;                       // head within the group
            head[nq] = hq < G ? g * G + hq : -1;
            const bf16_t* src = q + (size_t)(t_lo + (active ? tile0 + min(col, n_valid - 1) : 0)) * q_stride + (size_t)max(head[nq], 0) * HD + grp * 8;
#pragma unroll
            for (int kk = 0; kk < HD / 32; ++kk) qf[nq][kk] = *reinterpret_cast<const pbf16x8_t*>(src + kk * 32);
        }
        pf32x4_t o[NQ][HD / 16];
        float m[NQ], l[NQ];
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq) {
            m[nq] = -INFINITY;
            l[nq] = 0.f;
#pragma unroll
            for (int db = 0; db < HD / 16; ++db) o[nq][db] = pf32x4_t{0.f, 0.f, 0.f, 0.f};
        }
        const int key_end = min(min(kv_len, p_last + 1), ke);
        const int key_begin = window > 0 ? (max(0, p_first + 1 - window) / 32) * 32 : 0;
        const int j0_last = window > 0 ? max(0, p_last + 1 - window) : 0;
        const int last_idx = max(key_end - 1, 0) / page;         // the last page this tile may read
        // steps before hot_end lie wholly below the diagonal and inside the cache: no masks
        const int hot_end = window > 0 ? key_begin : (min(p_first + 1, key_end) / 32) * 32;

        // Page ids of a step.  Without a window every page up to last_idx is held, and steps
        // asked for ahead of time past the end read the last page's id; with a window, pages
        // that are not held (beyond the end, or passed by the window) come back as -1.
        auto pages_of = [&](int key0, int& blk0, int& blk1) {
            if (window > 0) {
                blk0 = key0 < key_end ? trow[key0 / page] : -1;
                blk1 = key0 + 16 < key_end ? trow[(key0 + 16) / page] : -1;
            } else {
                blk0 = trow[min(key0 / page, last_idx)];
                blk1 = trow[min((key0 + 16) / page, last_idx)];
            }
        };
        // asks for the keys and values of the step at key0; pages that are not held are replaced
        // by a held one and masked when the step is computed
        auto request = [&](int key0, Frags& f) {
            int ba = f.blk0, bb = f.blk1;
            int sa = FAST ? 0 : key0 % page, sb = FAST ? 0 : (key0 + 16) % page;
            if (window > 0) {
                const int any = max(max(ba, bb), 0);
                if (ba < 0) { ba = any; sa = 0; }
                if (bb < 0) { bb = any; sb = 0; }
            }
            const bf16_t* kt = kbase + (uint64_t)(uint32_t)(k_second_half ? bb : ba) * page_stride + (uint32_t)((k_second_half ? sb : sa) * HD);
            const bf16_t* vt = vbase + (uint64_t)(uint32_t)(v_second_half ? bb : ba) * page_stride + (uint32_t)(v_second_half ? sb : sa);
#pragma unroll
            for (int kk = 0; kk < HD / 32; ++kk) {
                f.k0[kk] = *reinterpret_cast<const pbf16x8_t*>(kt + kk * 32);
                f.k1[kk] = *reinterpret_cast<const pbf16x8_t*>(kt + 4 * HD + kk * 32);
            }
#pragma unroll
            for (int db = 0; db < HD / 16; ++db) f.v[db] = *reinterpret_cast<const pbf16x8_t*>(vt + (size_t)db * 16 * page);
        };
        // mx[nq]: this lane's largest raw score of the keys about to be added.  Moves the softmax
        // reference of a head, and rescales its sums so far, if some lane's value lies more than
        // 2^24 above it (in the scaled log2 domain); rare after a query's first step.
        auto move_reference = [&](const float (&mx)[NQ]) {
            bool move = false;
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) move |= mx[nq] * scale_log2e > m[nq] + 24.f;
            if (__builtin_expect(__any(move), 0)) {
#pragma unroll
                for (int nq = 0; nq < NQ; ++nq) {
                    float v = mx[nq];
                    v = fmaxf(v, __shfl_xor(v, 16, 64));
                    v = fmaxf(v, __shfl_xor(v, 32, 64));
                    const float m_new = fmaxf(m[nq], v * scale_log2e);        // m lives in the scaled (log2) domain
                    const float alpha = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m[nq] - m_new);
                    l[nq] *= alpha;
                    float a[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) a[i] = __shfl(alpha, grp * 4 + i, 64);
#pragma unroll
                    for (int db = 0; db < HD / 16; ++db)
#pragma unroll
                        for (int i = 0; i < 4; ++i) o[nq][db][i] *= a[i];
                    m[nq] = m_new;
                }
            }
        };
        // one step; masked = false promises that every (key, query) pair of the step counts
        // shared: where the step's fragments lie in LDS (SHARE), else null and f holds them already
        auto compute = [&](int key0, Frags& f, const bool masked, const pbf16x8_t* shared = nullptr) {
            constexpr int NKF = HD / 32;
            if constexpr (SHARE) {
#pragma unroll
                for (int kk = 0; kk < NKF; ++kk) { f.k0[kk] = shared[kk * 64]; f.k1[kk] = shared[(NKF + kk) * 64]; }
            }
            bool mask = false;
            if (masked) {
                // does any (key, query) pair of this step need masking?
                mask = key0 + 31 > p_first || key0 + 32 > key_end || key0 < j0_last || n_valid < 16;
            }
            // The heads of the wave go through each stage together, so that the matrix
            // instructions of one overlap the vector arithmetic of another and a step has one
            // branch (the rare move of a softmax reference) instead of one per head.
            // sv[nq][e] = raw score of key key0 + grp*8 + e; the scale and log2(e) enter through
            // one fused multiply-add per value
            float sv[NQ][8];
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) {
                pf32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < HD / 32; ++kk) {
                    s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k0[kk], qf[nq][kk], s0, 0, 0, 0);
                    s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k1[kk], qf[nq][kk], s1, 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) { sv[nq][i] = s0[i]; sv[nq][4 + i] = s1[i]; }
            }
            if (mask) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = key0 + grp * 8 + e;
                    if (!(key <= p && key >= j0 && key < key_end)) {
#pragma unroll
                        for (int nq = 0; nq < NQ; ++nq) sv[nq][e] = -INFINITY;
                    }
                }
            }
            // The reference m[nq] that is subtracted before exp2 need not be the maximum: any
            // value that the scores do not exceed by much will do, and the final division removes
            // it.  It is the same in the four lanes of a query, and it is only moved (with a
            // rescale of the sums so far) when some score of the step lies more than 2^24 above
            // it, which after a query's first step is rare.  So the usual step has no cross-lane
            // traffic and no rescale.
            float mx[NQ];
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq)
                mx[nq] = max3_raw(max3_raw(sv[nq][0], sv[nq][1], sv[nq][2]), max3_raw(sv[nq][3], sv[nq][4], sv[nq][5]),
                                  max3_raw(sv[nq][6], sv[nq][7], sv[nq][7]));
            move_reference(mx);
            // the values are taken late, so that they and the keys need not be held at the same time
            if constexpr (SHARE) {
#pragma unroll
                for (int db = 0; db < HD / 16; ++db) f.v[db] = shared[(2 * NKF + db) * 64];
            }
            if (masked) {
                // Values of positions that were never written (the rest of the last page) or of a
                // page that is not held may be anything, NaN included; 0 * NaN must not reach the output.
                if (key0 + 32 > key_end || f.blk0 < 0 || f.blk1 < 0) {
                    const bool held = v_second_half ? f.blk1 >= 0 : f.blk0 >= 0;
                    const int n = held ? min(8, max(0, key_end - (key0 + grp * 8))) : 0;
#pragma unroll
                    for (int db = 0; db < HD / 16; ++db)
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (e >= n) f.v[db][e] = (__bf16)0.f;
                }
            }
            pbf16x8_t pf[NQ];
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) {
                const float m_ref = m[nq] == -INFINITY ? 0.f : m[nq];       // a query that sees nothing yet
                float e[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) e[i] = __builtin_amdgcn_exp2f(fmaf(sv[nq][i], scale_log2e, -m_ref));
                l[nq] += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
#pragma unroll
                for (int i = 0; i < 8; ++i) pf[nq][i] = (__bf16)e[i];
            }
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
                for (int db = 0; db < HD / 16; ++db)
                    o[nq][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[nq], f.v[db], o[nq][db], 0, 0, 0);
        };

        // Two steps without masks from LDS (SHARE): the scores of both are made first and the
        // softmax reference is looked at once for the 64 keys, at a point where no product into
        // the output is under way; then each step's probabilities and its product with the values.
        auto compute_pair = [&](const pbf16x8_t* sa, const pbf16x8_t* sb) {
            constexpr int NKF = HD / 32;
            float sv[NQ][16];
            {
                pbf16x8_t ka0[NKF], ka1[NKF], kb0[NKF], kb1[NKF];
#pragma unroll
                for (int kk = 0; kk < NKF; ++kk) { ka0[kk] = sa[kk * 64]; ka1[kk] = sa[(NKF + kk) * 64]; }
#pragma unroll
                for (int kk = 0; kk < NKF; ++kk) { kb0[kk] = sb[kk * 64]; kb1[kk] = sb[(NKF + kk) * 64]; }
#pragma unroll
                for (int nq = 0; nq < NQ; ++nq) {
                    pf32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0, s2 = s0, s3 = s0;
#pragma unroll
                    for (int kk = 0; kk < NKF; ++kk) {
                        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka0[kk], qf[nq][kk], s0, 0, 0, 0);
                        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka1[kk], qf[nq][kk], s1, 0, 0, 0);
                        s2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb0[kk], qf[nq][kk], s2, 0, 0, 0);
                        s3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb1[kk], qf[nq][kk], s3, 0, 0, 0);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) { sv[nq][i] = s0[i]; sv[nq][4 + i] = s1[i]; sv[nq][8 + i] = s2[i]; sv[nq][12 + i] = s3[i]; }
                }
            }
            float mx[NQ];
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) {
                const float lo = max3_raw(max3_raw(sv[nq][0], sv[nq][1], sv[nq][2]), max3_raw(sv[nq][3], sv[nq][4], sv[nq][5]),
                                          max3_raw(sv[nq][6], sv[nq][7], sv[nq][8]));
                mx[nq] = max3_raw(max3_raw(sv[nq][9], sv[nq][10], sv[nq][11]), max3_raw(sv[nq][12], sv[nq][13], sv[nq][14]),
                                  max3_raw(sv[nq][15], lo, lo));
            }
            move_reference(mx);
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                const pbf16x8_t* src = st == 0 ? sa : sb;
                pbf16x8_t vf[HD / 16];
#pragma unroll
                for (int db = 0; db < HD / 16; ++db) vf[db] = src[(2 * NKF + db) * 64];
                pbf16x8_t pf[NQ];
#pragma unroll
                for (int nq = 0; nq < NQ; ++nq) {
                    const float m_ref = m[nq] == -INFINITY ? 0.f : m[nq];
                    float e[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) e[i] = __builtin_amdgcn_exp2f(fmaf(sv[nq][st * 8 + i], scale_log2e, -m_ref));
                    l[nq] += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
#pragma unroll
                    for (int i = 0; i < 8; ++i) pf[nq][i] = (__bf16)e[i];
                }
#pragma unroll
                for (int nq = 0; nq < NQ; ++nq)
#pragma unroll
                    for (int db = 0; db < HD / 16; ++db)
                        o[nq][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[nq], vf[db], o[nq][db], 0, 0, 0);
            }
        };
        if constexpr (SHARE) {
            // the block's keys: up to the last one that its last query sees
            const int blk_key_end = min(min(kv_len, start + min(q_len, tile * 64 + 64)), ke);
            const int blk_last_idx = max(blk_key_end - 1, 0) / 16;
            constexpr int MINE = NF / 4;                         // fragments this wave fetches per step
            constexpr int NK = HD / 32;
            auto ids_of = [&](int key0, int& blk0, int& blk1) {
                blk0 = trow[min(key0 / 16, blk_last_idx)];
                blk1 = trow[min(key0 / 16 + 1, blk_last_idx)];
            };
            // fragment id (0..NK-1: first key tile, NK..2NK-1: second, then the value blocks) -> this lane's 16 bytes
            auto frag_src = [&](int id, int ba, int bb) -> const bf16_t* {
                if (id < 2 * NK) {
                    const int kk = id < NK ? id : id - NK;
                    return kbase + (uint64_t)(uint32_t)(k_second_half ? bb : ba) * page_stride + (id < NK ? 0 : 4 * HD) + kk * 32;
                }
                return vbase + (uint64_t)(uint32_t)(v_second_half ? bb : ba) * page_stride + (size_t)(id - 2 * NK) * 16 * 16;
            };
            // memory -> LDS without a stop in registers: lane i's 16 bytes land at the fragment's
            // start + 16 i, which is the order the fragments are read in
            auto fetch = [&](int ba, int bb, int buf) {
#pragma unroll
                for (int j = 0; j < MINE; ++j) {
                    const int id = wave * MINE + j;
                    __builtin_amdgcn_global_load_lds(
                        (const __attribute__((address_space(1))) void*)frag_src(id, ba, bb),
                        (__attribute__((address_space(3))) void*)(kv_lds + (buf * NF + id) * 64), 16, 0, 0);
                }
            };
            // what this wave has fetched is in LDS (0x0f70: vmcnt 0, the other counters left alone)
            auto fetched = [&]() { __builtin_amdgcn_s_waitcnt(0x0f70); };
            auto ring = [&](int key0) { return (key0 >> 5) & 3; };
            auto frags_of = [&](int key0) { return kv_lds + (size_t)ring(key0) * NF * 64 + lane; };
            // Steps that lie below the diagonal for all four waves (the first wave's queries are
            // the earliest) are taken two at a time in a loop without conditions on the wave: one
            // barrier, one wait and one round of loop control for 64 keys, and the two steps'
            // matrix and vector work can overlap.  The loop asks for the two steps after its own.
            const int q0 = tile * 64;
            const bool all_active = q0 + 48 < q_len;
            const int p_first0 = start + q0;
            const int pair_end = all_active ? (min(min(p_first0 + 1, min(kv_len, p_first0 + 16)), ke) / 64) * 64 : 0;
            int a0, a1, n0, n1;
            // kb is a multiple of 128, so the range's first step lies in buffer 0 of the ring
            ids_of(kb, a0, a1);
            if (half == 1) __syncthreads();                      // the first tile's last step has been read
            if (blk_key_end > kb) fetch(a0, a1, 0);
            ids_of(kb + 32, a0, a1);
            int key0 = kb;
            bool ahead = false;                                  // the step after key0 has been asked for already
            if (pair_end > kb) {
                int b0, b1, c0, c1, d0, d1;
                if (kb + 32 < blk_key_end) fetch(a0, a1, 1);
                ids_of(kb + 64, a0, a1);
                ids_of(kb + 96, b0, b1);
                fetched();
                __syncthreads();
                for (; key0 < pair_end; key0 += 64) {
                    ids_of(key0 + 128, c0, c1);
                    ids_of(key0 + 160, d0, d1);
                    if (key0 + 64 < blk_key_end) fetch(a0, a1, ring(key0 + 64));   // read two steps ago, before the last barrier
                    if (key0 + 96 < blk_key_end) fetch(b0, b1, ring(key0 + 96));
                    compute_pair(frags_of(key0), frags_of(key0 + 32));
                    a0 = c0; a1 = c1;
                    b0 = d0; b1 = d1;
                    fetched();
                    __syncthreads();
                }
                // the steps at key0 and key0 + 32 are in LDS; (a0, a1) are the pages of key0 + 64
                ahead = true;
            } else {
                fetched();
                __syncthreads();
            }
            for (; key0 < blk_key_end; key0 += 32) {
                const bool more = key0 + 32 < blk_key_end;
                ids_of(key0 + 64, n0, n1);
                if (more && !ahead) fetch(a0, a1, ring(key0 + 32)); // that buffer was read three steps ago
                if (active && key0 < key_end) {
                    Frags f;
                    f.blk0 = 0;
                    f.blk1 = 0;                                  // every page of the block's range is held
                    const pbf16x8_t* src = frags_of(key0);
                    if (key0 + 32 <= hot_end) compute(key0, f, false, src);
                    else compute(key0, f, true, src);
                }
                if (!ahead) { a0 = n0; a1 = n1; }
                ahead = false;
                fetched();
                __syncthreads();
            }
        } else {
        // Keys and values of the next step are requested before this step is computed, and the
        // page ids one step earlier still, so that no step waits for what it has just asked for.
        // Two sets of fragments take turns.
        Frags fa, fb;
        pages_of(key_begin, fa.blk0, fa.blk1);
        pages_of(key_begin + 32, fb.blk0, fb.blk1);
        if (key_begin < key_end) request(key_begin, fa);
        int key0 = key_begin;
        for (; key0 + 64 <= hot_end; key0 += 64) {               // two steps without masks
            int n0, n1;
            pages_of(key0 + 64, n0, n1);
            request(key0 + 32, fb);
            compute(key0, fa, false);
            fa.blk0 = n0; fa.blk1 = n1;
            pages_of(key0 + 96, n0, n1);
            if (__builtin_expect(key0 + 64 < key_end, 1)) request(key0 + 64, fa);
            compute(key0 + 32, fb, false);
            fb.blk0 = n0; fb.blk1 = n1;
        }
        for (; key0 < key_end; key0 += 64) {                     // the steps on the diagonal
            int n0, n1;
            pages_of(key0 + 64, n0, n1);
            if (key0 + 32 < key_end) request(key0 + 32, fb);
            compute(key0, fa, true);
            fa.blk0 = n0; fa.blk1 = n1;
            if (key0 + 32 >= key_end) break;
            pages_of(key0 + 96, n0, n1);
            if (key0 + 64 < key_end) request(key0 + 64, fa);
            compute(key0 + 32, fb, true);
            fb.blk0 = n0; fb.blk1 = n1;
        }
        }
        if (SHARE && !active) continue;
        if constexpr (SPLIT) {
            // what this range of keys gives each query, unnormalised: [split][token][head][HD] and
            // (reference, total) beside it; the reference is the same in the four lanes of a query
#pragma unroll
            for (int nq = 0; nq < NQ; ++nq) {
                if (head[nq] < 0) continue;
                float lt = l[nq];
                lt += __shfl_xor(lt, 16, 64);
                lt += __shfl_xor(lt, 32, 64);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int qi = grp * 4 + i;
                    const float li = __shfl(lt, qi, 64), mi = __shfl(m[nq], qi, 64);
                    if (qi < n_valid) {
                        const size_t row = ((size_t)split * part_tokens + (t_lo + tile0 + qi)) * H + head[nq];
                        float* dst = part_o + row * HD + col;
#pragma unroll
                        for (int db = 0; db < HD / 16; ++db) dst[db * 16] = o[nq][db][i];
                        if (col == 0) { part_ml[row * 2] = mi; part_ml[row * 2 + 1] = li; }
                    }
                }
            }
            continue;
        }
        // o[nq][db][i] = O[q = grp*4 + i][d = db*16 + col]; the sums of a query are spread over its 4 lanes
#pragma unroll
        for (int nq = 0; nq < NQ; ++nq) {
            if (head[nq] < 0) continue;
            float lt = l[nq];
            lt += __shfl_xor(lt, 16, 64);
            lt += __shfl_xor(lt, 32, 64);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int qi = grp * 4 + i;
                const float li = __shfl(lt, qi, 64);
                if (qi < n_valid) {
                    bf16_t* dst = out + (size_t)(t_lo + tile0 + qi) * out_stride + (size_t)head[nq] * HD + col;
                    const float inv = li > 0.f ? 1.f / li : 0.f;
#pragma unroll
                    for (int db = 0; db < HD / 16; ++db) dst[db * 16] = f32_to_bf16(o[nq][db][i] * inv);
                }
            }
        }
    }
}

// Puts together what the ranges of keys gave each query of the rows with min_q_len tokens or
// more (SPLIT above).  A thread owns four features of one (query, head); the ranges that hold a
// key the query sees are the first min(position, kv_len - 1) / split_keys + 1, and only those
// were written.
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_combine_kernel(
        const float* __restrict__ part_o, const float* __restrict__ part_ml, int part_tokens, int nsplit,
        int split_keys, bf16_t* __restrict__ out, int out_stride, const int* __restrict__ cu_q,
        const int* __restrict__ q_start, const int* __restrict__ kv_lens, int H, int min_q_len,
        const int* __restrict__ row_list) {
    constexpr int F4 = HD / 4;
    const int b = row_list ? row_list[blockIdx.y] : (int)blockIdx.y;
    if (b < 0) return;
    const int t_lo = cu_q[b], q_len = cu_q[b + 1] - t_lo;
    if (q_len < min_q_len) return;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const int f4 = (int)(idx % F4), head = (int)((idx / F4) % H);
    const long long i = idx / ((long long)F4 * H);
    if (i >= q_len) return;
    const int p = min(q_start[b] + (int)i, kv_lens[b] - 1);
    const int n = p < 0 ? 0 : min(nsplit, p / split_keys + 1);
    const size_t row = (size_t)(t_lo + i) * H + head, step = (size_t)part_tokens * H;
    float mx = -INFINITY;
    for (int s = 0; s < n; ++s) {
        const float l = part_ml[(row + s * step) * 2 + 1];
        if (l > 0.f) mx = fmaxf(mx, part_ml[(row + s * step) * 2]);
    }
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float total = 0.f;
    for (int s = 0; s < n; ++s) {
        const float m = part_ml[(row + s * step) * 2], l = part_ml[(row + s * step) * 2 + 1];
        if (!(l > 0.f)) continue;
        const float w = exp2f(m - mx);                           // the references are in the scaled log2 domain
        const float4 o = *reinterpret_cast<const float4*>(part_o + (row + s * step) * HD + f4 * 4);
        acc.x = fmaf(o.x, w, acc.x); acc.y = fmaf(o.y, w, acc.y); acc.z = fmaf(o.z, w, acc.z); acc.w = fmaf(o.w, w, acc.w);
        total = fmaf(l, w, total);
    }
    const float inv = total > 0.f ? 1.f / total : 0.f;
    bf16_t* dst = out + (size_t)(t_lo + i) * out_stride + (size_t)head * HD + f4 * 4;
    dst[0] = f32_to_bf16(acc.x * inv);
    dst[1] = f32_to_bf16(acc.y * inv);
    dst[2] = f32_to_bf16(acc.z * inv);
    dst[3] = f32_to_bf16(acc.w * inv);
}

// How a step's prompt portions are divided over ranges of keys: 1 (not at all) where the tiles of
// queries alone give the chip its waves or few keys lie before the portion, else as many ranges
// (multiples of 128 keys) as bring the waves to about two a SIMD, at most one for every 256 keys
// that were cached before the step.  Measured on 32 heads over 8 kv heads of 128, us, undivided ->
// divided: 16 tokens behind 2,048: 40 -> 20; 256 behind 2,048: 78 -> 40; 256 behind 8,192: 271 ->
// 73; 512 behind 1,536: 66 -> 43; 512 behind 7,680: 259 -> 110; 1,024 behind 3,072: 126 -> 99.  A
// portion that starts a prompt has its work balanced by the pairing of late and early tiles and
// only loses (1,024 tokens: 28 -> 40 in two ranges).
static void prefill_split_plan(int H, int Hkv, int hd, int page, int window, int total_q, int max_prefix,
                               int max_kv_len, int forced, int* nsplit, int* split_keys) {
    *nsplit = 1;
    *split_keys = 0;
    if (!(page == 16 && window == 0 && (hd == 64 || hd == 128)) || max_kv_len <= 0 || forced == 1) return;
    const long long tile_pairs = ((total_q + 63) / 64 + 1) / 2;
    const long long waves = tile_pairs * 4 * H;                  // of one head each
    int n = forced > 1 ? forced : (int)std::min<long long>(2048 / std::max<long long>(waves, 1), std::max(max_prefix, 0) / 256);
    n = std::min(n, 32);
    if (n < 2) return;
    const int keys = (((max_kv_len + n - 1) / n + 127) / 128) * 128;
    n = (max_kv_len + keys - 1) / keys;
    if (n < 2) return;
    *nsplit = n;
    *split_keys = keys;
}

// bytes of workspace ri_attention_prefill may use for a step of total_q tokens whose rows hold at
// most max_kv_len keys (0: it will not divide the keys)
extern "C" size_t ri_attention_prefill_workspace(int H, int Hkv, int hd, int page, int window, int total_q,
                                                 int max_prefix, int max_kv_len, int splits) {
    int n, keys;
    prefill_split_plan(H, Hkv, hd, page, window, total_q, max_prefix, max_kv_len, splits, &n, &keys);
    return n < 2 ? 0 : (size_t)n * total_q * H * (hd + 2) * sizeof(float);
}

extern "C" int ri_attention_prefill_supported(int H, int Hkv, int hd, int page) {
    return (hd == 64 || hd == 128) && page % 16 == 0 && Hkv > 0 && H % Hkv == 0;
}

// Rows with fewer than min_q_len tokens are left alone (they go to the single-token kernel).
// total_q: the tokens of all rows together (it steers how the work is divided, and sizes the workspace).
// max_prefix, max_kv_len: no row of min_q_len tokens or more had more tokens cached before the
// step, or holds more keys after it (0: unknown, the keys are not divided); splits: 0 lets the entry point choose into how
// many ranges the keys are divided between blocks, 1 forbids it, more asks for that many; the
// workspace (ri_attention_prefill_workspace bytes of it, may be null) holds the ranges' results.
// row_list (may be null): the num_listed rows of min_q_len tokens or more (-1 where there are
// fewer); the grids then span those instead of all B rows, most of which may be single tokens.
extern "C" int ri_attention_prefill(
        const void* q, int q_stride, void* out, int out_stride,
        const void* kc, const void* vc, int num_pages, int page, int H, int Hkv, int hd,
        const int* table, int max_blocks, const int* cu_q, const int* q_start, const int* kv_lens,
        int B, int max_q_len, int total_q, float scale, int window, int min_q_len,
        int max_prefix, int max_kv_len, int splits, void* workspace, size_t workspace_bytes,
        const int* row_list, int num_listed, hipStream_t stream) {
    RI_REQUIRE(ri_attention_prefill_supported(H, Hkv, hd, page),
               "ri_attention_prefill: needs head size 64 or 128 and pages that are multiples of 16; got hd=%d page=%d H=%d Hkv=%d", hd, page, H, Hkv);
    RI_REQUIRE(B >= 0 && max_q_len > 0 && total_q >= 0 && max_blocks > 0 && num_pages > 0 && window >= 0, "ri_attention_prefill: bad sizes");
    RI_REQUIRE(q_stride >= H * hd && out_stride >= H * hd && q_stride % 8 == 0, "ri_attention_prefill: bad row strides");
    RI_REQUIRE((long long)Hkv * page * hd <= 0x7fffffffLL, "ri_attention_prefill: a page of all kv heads exceeds 2^31 elements");
    if (B == 0) return 0;
    RI_REQUIRE(q && out && kc && vc && table && cu_q && q_start && kv_lens, "ri_attention_prefill: null pointer");
    RI_REQUIRE(!row_list || (num_listed >= 1 && num_listed <= B), "ri_attention_prefill: %d listed rows of %d", num_listed, B);
    const int BY = row_list ? num_listed : B;             // rows the grids span
    RI_REQUIRE((uintptr_t)q % 16 == 0 && (uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0, "ri_attention_prefill: operands must be 16-byte aligned");
    const int G = H / Hkv;
    const bool fast = page == 16 && window == 0;
    // Query heads per wave: more of them share each key and value load, fewer of them give more
    // waves.  Four (head size 64) or two as long as that leaves two waves for every SIMD of the chip.
    int NQ = G < 2 ? G : 2;
    for (int n = hd == 64 ? 4 : 2; n > 2; --n) {
        const long long waves = (long long)((total_q + 15) / 16) * Hkv * (G / n);
        if (G % n == 0 && waves >= 2048) { NQ = n; break; }
    }
    // Pages of 16, no window: the waves of a block may hand each other the keys and values
    // through LDS (SHARE).  Measured on 32 heads over 8 kv heads, times of the plain form = 1:
    //   head 128: one head per wave (twice the waves, and sharing takes away what that would
    //     cost in traffic) 0.77 at 2,048 tokens, 0.59 for 512 tokens behind 1,536; from 2,048
    //     waves of two heads on, two heads per wave with registers capped at 256 so that two
    //     waves share a SIMD: 0.68 at 4,096 tokens, 0.61 at 8,192, 0.56 behind 16,384.
    //   head 64: one head per wave up to 8,192 waves of one head (against the plain form with
    //     four heads per wave: 0.85 at 2,048 tokens, 0.86 at 4,096); beyond that four heads per
    //     wave, two waves per SIMD (0.84 at 8,192 tokens, 0.78 behind 16,384; one head per wave
    //     there: 1.0 and 1.05).
    const float sl2 = scale * 1.4426950408889634f;
    const long long pairs = ((max_q_len + 63) / 64 + 1) / 2;
    RI_REQUIRE(B <= 65535, "ri_attention_prefill: too many rows");
    int nsplit = 1, split_keys = 0;
    prefill_split_plan(H, Hkv, hd, page, window, total_q, max_prefix, max_kv_len, workspace ? splits : 1, &nsplit, &split_keys);
    if (nsplit > 1) {
        const size_t need = (size_t)nsplit * total_q * H * (hd + 2) * sizeof(float);
        RI_REQUIRE(workspace_bytes >= need && (uintptr_t)workspace % 16 == 0, "ri_attention_prefill: workspace of %zu bytes, %zu needed", workspace_bytes, need);
        RI_REQUIRE(pairs * Hkv * G <= 0x7fffffffLL && nsplit <= 65535, "ri_attention_prefill: grid too large");
        float* part_o = (float*)workspace;
        float* part_ml = part_o + (size_t)nsplit * total_q * H * hd;
        dim3 grid((unsigned)(pairs * Hkv * G), BY, nsplit);
#define RI_PREFILL_SPLIT_ARGS (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kc, (const bf16_t*)vc, table, max_blocks, cu_q, q_start, kv_lens, H, Hkv, page, sl2, window, G, min_q_len, split_keys, nsplit, part_o, part_ml, total_q, row_list
        const long long per_row = (long long)max_q_len * H * (hd / 4);
        dim3 cgrid((unsigned)((per_row + 255) / 256), BY);
        if (hd == 64) {
            attn_prefill_kernel<64, 1, true, true, 1, true><<<grid, 256, 0, stream>>>(RI_PREFILL_SPLIT_ARGS);
            RI_LAUNCHED("ri_attention_prefill(ranges)");
            attn_prefill_combine_kernel<64><<<cgrid, 256, 0, stream>>>(part_o, part_ml, total_q, nsplit, split_keys, (bf16_t*)out, out_stride, cu_q, q_start, kv_lens, H, min_q_len, row_list);
        } else {
            attn_prefill_kernel<128, 1, true, true, 1, true><<<grid, 256, 0, stream>>>(RI_PREFILL_SPLIT_ARGS);
            RI_LAUNCHED("ri_attention_prefill(ranges)");
            attn_prefill_combine_kernel<128><<<cgrid, 256, 0, stream>>>(part_o, part_ml, total_q, nsplit, split_keys, (bf16_t*)out, out_stride, cu_q, q_start, kv_lens, H, min_q_len, row_list);
        }
#undef RI_PREFILL_SPLIT_ARGS
        RI_LAUNCHED("ri_attention_prefill(combine)");
        return 0;
    }
    bool share = false, two_per_simd = false;
    const long long tile_pairs = ((total_q + 63) / 64 + 1) / 2;
    if (hd == 128 && fast) {
        const long long waves_two_heads = tile_pairs * 4 * Hkv * ((G + 1) / 2);
        share = true;
        two_per_simd = G >= 2 && waves_two_heads >= 2048;
        NQ = two_per_simd ? 2 : 1;
    } else if (hd == 64 && fast) {
        const long long waves_one_head = tile_pairs * 4 * Hkv * G;
        share = true;
        if (waves_one_head >= 8192 && G % 4 == 0) { two_per_simd = true; NQ = 4; }
        else NQ = 1;
    }
    const int head_groups = (G + NQ - 1) / NQ;
    RI_REQUIRE(pairs * Hkv * head_groups <= 0x7fffffffLL, "ri_attention_prefill: grid too large");
    dim3 grid((unsigned)(pairs * Hkv * head_groups), BY);
#define RI_PREFILL_ARGS (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kc, (const bf16_t*)vc, table, max_blocks, cu_q, q_start, kv_lens, H, Hkv, page, sl2, window, head_groups, min_q_len, 0, 1, nullptr, nullptr, 0, row_list
    // pages of 16 without a window always take a shared form; the plain form serves the rest
#define RI_PREFILL_LAUNCH(HD_, NQ_) attn_prefill_kernel<HD_, NQ_, false><<<grid, 256, 0, stream>>>(RI_PREFILL_ARGS)
    if (hd == 64 && share) {
        if (two_per_simd) attn_prefill_kernel<64, 4, true, true, 2><<<grid, 256, 0, stream>>>(RI_PREFILL_ARGS);
        else attn_prefill_kernel<64, 1, true, true><<<grid, 256, 0, stream>>>(RI_PREFILL_ARGS);
    } else if (hd == 64) {
        if (NQ == 1) RI_PREFILL_LAUNCH(64, 1);
        else if (NQ == 2) RI_PREFILL_LAUNCH(64, 2);
        else if (NQ == 3) RI_PREFILL_LAUNCH(64, 3);
        else RI_PREFILL_LAUNCH(64, 4);
    } else if (share) {
        if (two_per_simd) attn_prefill_kernel<128, 2, true, true, 2><<<grid, 256, 0, stream>>>(RI_PREFILL_ARGS);
        else attn_prefill_kernel<128, 1, true, true><<<grid, 256, 0, stream>>>(RI_PREFILL_ARGS);
    } else {
        if (NQ == 1) RI_PREFILL_LAUNCH(128, 1);
        else RI_PREFILL_LAUNCH(128, 2);
    }
#undef RI_PREFILL_LAUNCH
#undef RI_PREFILL_ARGS
    RI_LAUNCHED("ri_attention_prefill");
    return 0;
}
