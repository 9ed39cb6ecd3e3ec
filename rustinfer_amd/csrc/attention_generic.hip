// Attention over the paged cache for any head size up to 256, any number of heads and
// groups, 32-bit or bfloat16 storage, with all arithmetic in 32-bit.  It serves the exact
// 32-bit path and the sizes the tuned bfloat16 kernels do not take.
//
// For query token t of request row b at absolute position p, head h (kv head g = h / (H/Hkv)):
//   keys j in [max(0, p+1-window), min(kv_len_b, p+1)),  s_j = (q . K_j) * scale,
//   out = sum_j softmax(s)_j V_j                 (reference: fused_ops.rs:430-535)
// One block of 256 threads per (token, head); keys in chunks of 256 with a running
// maximum and sum.  Cache layout: keys [pages][Hkv][page][hd], values [pages][Hkv][hd][page].
#include "common.h"
#include <math.h>

template <typename T>
__global__ __launch_bounds__(256) void attn_generic_kernel(
        const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
        const T* __restrict__ kc, const T* __restrict__ vc,
        const int* __restrict__ table, int max_blocks,
        const int* __restrict__ row_of_token, const int* __restrict__ positions,
        const int* __restrict__ kv_lens, int H, int Hkv, int hd, int page,
        float scale, int window) {
    __shared__ float qs[256];
    __shared__ float ps[256];
    __shared__ float accs[256];
    __shared__ int koff[256];
    __shared__ float red[16];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int b = row_of_token[t];
    T* o = out + (size_t)t * out_stride + h * hd;
    if (b < 0) {                                   // padding token: defined output, no reads
        if (tid < hd) st_f32(o + tid, 0.f);
        return;
    }
    const int p = positions[t];
    const int visible = min(kv_lens[b], p + 1);
    const int j0 = window > 0 ? max(0, p + 1 - window) : 0;
    const int g = h / (H / Hkv);
    if (tid < hd) qs[tid] = ld_f32(q + (size_t)t * q_stride + h * hd + tid);
    const int nparts = 256 / hd;
    const bool active = tid < nparts * hd;
    const int d = tid % hd, part = tid / hd;
    float m = -INFINITY, l = 0.f, acc = 0.f;
    __syncthreads();
    for (int c0 = j0; c0 < visible; c0 += 256) {
        const int j = c0 + tid;
        float s = -INFINITY;
        if (j < visible) {
            const int blk = table[(size_t)b * max_blocks + j / page];
            const int off = (blk * Hkv + g) * page + j % page;
            koff[tid] = off;
            const T* kr = kc + (size_t)off * hd;
            float dot = 0.f;
            for (int dd = 0; dd < hd; ++dd) dot += qs[dd] * ld_f32(kr + dd);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, block_max(s, red));
        const float pj = (j < visible) ? expf(s - m_new) : 0.f;
        ps[tid] = pj;
        const float csum = block_sum(pj, red);      // its barriers also publish ps and koff
        const float alpha = expf(m - m_new);        // first chunk: exp(-inf) = 0
        l = l * alpha + csum;
        m = m_new;
        if (active) {
            acc *= alpha;
            const int n = min(256, visible - c0);
            for (int jj = part; jj < n; jj += nparts)
                acc += ps[jj] * ld_f32(vc + (size_t)(koff[jj] / page) * page * hd + (size_t)d * page + koff[jj] % page);
        }
        __syncthreads();                            // ps/koff are rewritten by the next chunk
    }
    accs[tid] = active ? acc : 0.f;
    __syncthreads();
    if (tid < hd) {
        float sum = 0.f;
        for (int pp = 0; pp < nparts; ++pp) sum += accs[pp * hd + tid];
        st_f32(o + tid, l > 0.f ? sum / l : 0.f);
    }
}

extern "C" int ri_attention_generic(
        const void* q, int q_stride, void* out, int out_stride, int dtype,
        const void* kc, const void* vc, int num_pages, int page, int H, int Hkv, int hd,
        const int* table, int max_blocks, const int* row_of_token, const int* positions,
        const int* kv_lens, int T, float scale, int window, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && H > 0 && Hkv > 0 && H % Hkv == 0, "ri_attention_generic: bad head counts H=%d Hkv=%d", H, Hkv);
    RI_REQUIRE(hd > 0 && hd <= 256, "ri_attention_generic: head size %d not in [1, 256]", hd);
    RI_REQUIRE(page > 0 && max_blocks > 0 && num_pages > 0, "ri_attention_generic: bad cache sizes");
    RI_REQUIRE(q_stride >= H * hd && out_stride >= H * hd, "ri_attention_generic: row strides too small");
    RI_REQUIRE(window >= 0, "ri_attention_generic: window must be >= 0");
    if (T == 0) return 0;
    RI_REQUIRE(H <= 65535, "ri_attention_generic: too many heads for the grid");
    RI_REQUIRE(q && out && kc && vc && table && row_of_token && positions && kv_lens, "ri_attention_generic: null pointer");
    dim3 grid(T, H);
    if (dtype == RI_F32)
        attn_generic_kernel<float><<<grid, 256, 0, stream>>>((const float*)q, q_stride, (float*)out, out_stride, (const float*)kc, (const float*)vc, table, max_blocks, row_of_token, positions, kv_lens, H, Hkv, hd, page, scale, window);
    else if (dtype == RI_BF16)
        attn_generic_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kc, (const bf16_t*)vc, table, max_blocks, row_of_token, positions, kv_lens, H, Hkv, hd, page, scale, window);
    else
        return ri_fail("ri_attention_generic: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_attention_generic");
    return 0;
}
