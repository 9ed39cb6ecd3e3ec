// Embedding gather, residual add + RMSNorm, rotation + cache write, SwiGLU.
// The residual stream is 32-bit in both precisions; `act` tensors are float or bfloat16.
#include "common.h"

// ---------------------------------------------------------------------------
// x[t, :] = table[ids[t], :]        (reference: emb.cu:9-38; an id out of range gives zeros)
// ---------------------------------------------------------------------------
// A negative id -(k+1) stands for device_tokens[k]: the token a previous step sampled and left
// on the device, so that the next step can start before the host has seen it.
template <typename TW>
__global__ void embed_kernel(const int* __restrict__ ids, const int* __restrict__ device_tokens,
                             const TW* __restrict__ table, float* __restrict__ x, int d, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 && device_tokens != nullptr) id = device_tokens[-1 - id];
    float* xr = x + (size_t)t * d;
    if (id < 0 || id >= V) {
        for (int i = threadIdx.x; i < d; i += blockDim.x) xr[i] = 0.f;
        return;
    }
    const TW* row = table + (size_t)id * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) xr[i] = ld_f32(row + i);
}

extern "C" int ri_embed(const int* ids, const int* device_tokens, const void* table, int table_dtype,
                        float* x, int T, int d, int V, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && d > 0 && V > 0, "ri_embed: bad sizes T=%d d=%d V=%d", T, d, V);
    if (T == 0) return 0;
    RI_REQUIRE(ids && table && x, "ri_embed: null pointer");
    const int block = d >= 1024 ? 256 : (d >= 256 ? 128 : 64);
    if (table_dtype == RI_F32)
        embed_kernel<float><<<T, block, 0, stream>>>(ids, device_tokens, (const float*)table, x, d, V);
    else if (table_dtype == RI_BF16)
        embed_kernel<bf16_t><<<T, block, 0, stream>>>(ids, device_tokens, (const bf16_t*)table, x, d, V);
    else
        return ri_fail("ri_embed: unknown dtype %d", table_dtype);
    RI_LAUNCHED("ri_embed");
    return 0;
}

// ---------------------------------------------------------------------------
// r = rows ? rows[i] : i;  v = x[r] + sum_p delta[p][r];  (x[r] = v when not gathering)
// out[i] = v * rsqrt(mean(v^2) + eps) * w        all arithmetic in 32-bit, one rounding.
// (reference: fused_add_rmsnorm.cu:17-181 adds and scales in bf16.)
// delta may be a stack of `parts` 32-bit partial sums (what a product split over K leaves).
// VEC elements per thread and load: 4 when d % 4 == 0, else 1.
// ---------------------------------------------------------------------------
template <int VEC> struct VecLoad;
template <> struct VecLoad<1> {
    static __device__ __forceinline__ void ld(const float* p, float* v) { v[0] = *p; }
    static __device__ __forceinline__ void ld(const bf16_t* p, float* v) { v[0] = bf16_to_f32(*p); }
    static __device__ __forceinline__ void st(float* p, const float* v) { *p = v[0]; }
    static __device__ __forceinline__ void st(bf16_t* p, const float* v) { *p = f32_to_bf16(v[0]); }
};
template <> struct VecLoad<4> {
    static __device__ __forceinline__ void ld(const float* p, float* v) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    static __device__ __forceinline__ void ld(const bf16_t* p, float* v) {
        const uint2 t = *reinterpret_cast<const uint2*>(p);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
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

// PARTS > 0: that many partial sums, all requested before any is added; 0: a runtime count.
template <typename TD, typename TW, typename TO, int BLOCK, int VEC, int PARTS>
__global__ __launch_bounds__(BLOCK) void add_rmsnorm_kernel(
        float* __restrict__ x, const TD* __restrict__ delta, int parts_rt, size_t part_stride,
        const TW* __restrict__ w, TO* __restrict__ out, int d, float eps, const int* __restrict__ rows,
        float* __restrict__ x_rows) {
    __shared__ float red[16];
    using L = VecLoad<VEC>;
    const int i_out = blockIdx.x;
    const int r = rows ? rows[i_out] : i_out;
    float* xr = x + (size_t)r * d;
    const TD* dr = delta ? delta + (size_t)r * d : nullptr;
    TO* o = out + (size_t)i_out * d;
    const bool write_x = (dr != nullptr) && (rows == nullptr);
    float* xg = x_rows ? x_rows + (size_t)i_out * d : nullptr;      // gathered rows: the sums go here
    constexpr int CACHE = 4;                  // vectors a thread keeps in registers
    constexpr int NP = PARTS > 0 ? PARTS : 1;
    const int parts = PARTS > 0 ? PARTS : parts_rt;
    float v[CACHE][VEC], wv[CACHE][VEC];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = (threadIdx.x + k * BLOCK) * VEC;
#pragma unroll
        for (int e = 0; e < VEC; ++e) { v[k][e] = 0.f; wv[k][e] = 0.f; }
        if (i < d) {
            float t[NP][VEC];
            L::ld(xr + i, v[k]);
            L::ld(w + i, wv[k]);              // asked for early: it does not wait for the sum
            if (dr) {
                if (PARTS > 0) {
#pragma unroll
                    for (int p = 0; p < NP; ++p) L::ld(dr + p * part_stride + i, t[p]);
#pragma unroll
                    for (int p = 0; p < NP; ++p)
#pragma unroll
                        for (int e = 0; e < VEC; ++e) v[k][e] += t[p][e];
                } else {
                    for (int p = 0; p < parts; ++p) {
                        L::ld(dr + p * part_stride + i, t[0]);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) v[k][e] += t[0][e];
                    }
                }
            }
            if (write_x) L::st(xr + i, v[k]);
            if (xg) L::st(xg + i, v[k]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) ss += v[k][e] * v[k][e];
        }
    }
    for (int i = (threadIdx.x + CACHE * BLOCK) * VEC; i < d; i += BLOCK * VEC) {
        float a[VEC];
        L::ld(xr + i, a);
        if (dr) {
            for (int p = 0; p < parts; ++p) {
                float t[VEC];
                L::ld(dr + p * part_stride + i, t);
#pragma unroll
                for (int e = 0; e < VEC; ++e) a[e] += t[e];
            }
        }
        if (write_x) L::st(xr + i, a);
        if (xg) L::st(xg + i, a);
#pragma unroll
        for (int e = 0; e < VEC; ++e) ss += a[e] * a[e];
    }
    ss = block_sum(ss, red);
    const float rs = rsqrtf(ss / (float)d + eps);
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = (threadIdx.x + k * BLOCK) * VEC;
        if (i < d) {
            float y[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) y[e] = v[k][e] * rs * wv[k][e];
            L::st(o + i, y);
        }
    }
    for (int i = (threadIdx.x + CACHE * BLOCK) * VEC; i < d; i += BLOCK * VEC) {
        float a[VEC], ww[VEC], y[VEC];
        L::ld(xr + i, a);
        if (dr && !write_x) {                 // when x was written back it already holds the sum
            for (int p = 0; p < parts; ++p) {
                float t[VEC];
                L::ld(dr + p * part_stride + i, t);
#pragma unroll
                for (int e = 0; e < VEC; ++e) a[e] += t[e];
            }
        }
        L::ld(w + i, ww);
#pragma unroll
        for (int e = 0; e < VEC; ++e) y[e] = a[e] * rs * ww[e];
        L::st(o + i, y);
    }
}

template <typename TD, typename TW, typename TO>
static int launch_add_rmsnorm(float* x, const void* delta, int parts, size_t part_stride, const void* w,
                              void* out, int n_out, int d, float eps, const int* rows, float* x_rows, hipStream_t stream) {
#define RI_NORM_ARGS x, (const TD*)delta, parts, part_stride, (const TW*)w, (TO*)out, d, eps, rows, x_rows
#define RI_NORM_LAUNCH(BLOCK, VEC) do { \
        if (parts == 1) add_rmsnorm_kernel<TD, TW, TO, BLOCK, VEC, 1><<<n_out, BLOCK, 0, stream>>>(RI_NORM_ARGS); \
        else if (parts == 2) add_rmsnorm_kernel<TD, TW, TO, BLOCK, VEC, 2><<<n_out, BLOCK, 0, stream>>>(RI_NORM_ARGS); \
        else if (parts == 4) add_rmsnorm_kernel<TD, TW, TO, BLOCK, VEC, 4><<<n_out, BLOCK, 0, stream>>>(RI_NORM_ARGS); \
        else if (parts == 8) add_rmsnorm_kernel<TD, TW, TO, BLOCK, VEC, 8><<<n_out, BLOCK, 0, stream>>>(RI_NORM_ARGS); \
        else add_rmsnorm_kernel<TD, TW, TO, BLOCK, VEC, 0><<<n_out, BLOCK, 0, stream>>>(RI_NORM_ARGS); } while (0)
    if (d % 4 == 0) {
        // few rows that add up several partial sums each (a step of 17..64 tokens): a row's loads are
        // all in flight at once when every thread holds one vector of it
        if (parts >= 4 && n_out <= 256 && d >= 2048 && d <= 4096) RI_NORM_LAUNCH(1024, 4);
        else if (d <= 2048) RI_NORM_LAUNCH(128, 4);
        else if (d <= 4096) RI_NORM_LAUNCH(256, 4);
        else RI_NORM_LAUNCH(512, 4);
    } else {
        RI_NORM_LAUNCH(256, 1);
    }
#undef RI_NORM_LAUNCH
#undef RI_NORM_ARGS
    RI_LAUNCHED("ri_add_rmsnorm");
    return 0;
}

// delta: null, or [parts][rows of x][d] of delta_dtype with part_stride elements between parts
// rows: null, or the n_out rows of x to normalise (x itself is then left as it is); x_rows: null,
// or where the sums x + delta of those rows go ([n_out][d], 32-bit)
extern "C" int ri_add_rmsnorm(float* x, const void* delta, int delta_dtype, int parts, long long part_stride,
                              const void* w, int w_dtype, void* out, int out_dtype, int n_out, int d,
                              float eps, const int* rows, float* x_rows, hipStream_t stream) {
    RI_REQUIRE(!x_rows || rows, "ri_add_rmsnorm: x_rows goes with rows");
    RI_REQUIRE((uintptr_t)x_rows % 16 == 0, "ri_add_rmsnorm: operands must be 16-byte aligned");
    RI_REQUIRE(n_out >= 0 && d > 0, "ri_add_rmsnorm: bad sizes n_out=%d d=%d", n_out, d);
    RI_REQUIRE(eps > 0.f, "ri_add_rmsnorm: eps must be > 0");
    RI_REQUIRE(!delta || (parts >= 1 && part_stride >= 0), "ri_add_rmsnorm: bad parts");
    if (n_out == 0) return 0;
    RI_REQUIRE(x && w && out, "ri_add_rmsnorm: null pointer");
    RI_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)delta % 16 == 0,
               "ri_add_rmsnorm: operands must be 16-byte aligned");
    RI_REQUIRE(d % 4 != 0 || part_stride % 4 == 0, "ri_add_rmsnorm: part stride must be a multiple of 4");
    if (!delta) delta_dtype = out_dtype;
    const size_t ps = (size_t)part_stride;
    if (delta_dtype == RI_F32 && w_dtype == RI_F32 && out_dtype == RI_F32) return launch_add_rmsnorm<float, float, float>(x, delta, parts, ps, w, out, n_out, d, eps, rows, x_rows, stream);
    if (delta_dtype == RI_BF16 && w_dtype == RI_F32 && out_dtype == RI_BF16) return launch_add_rmsnorm<bf16_t, float, bf16_t>(x, delta, parts, ps, w, out, n_out, d, eps, rows, x_rows, stream);
    if (delta_dtype == RI_BF16 && w_dtype == RI_BF16 && out_dtype == RI_BF16) return launch_add_rmsnorm<bf16_t, bf16_t, bf16_t>(x, delta, parts, ps, w, out, n_out, d, eps, rows, x_rows, stream);
    if (delta_dtype == RI_F32 && w_dtype == RI_F32 && out_dtype == RI_BF16) return launch_add_rmsnorm<float, float, bf16_t>(x, delta, parts, ps, w, out, n_out, d, eps, rows, x_rows, stream);
    if (delta_dtype == RI_F32 && w_dtype == RI_BF16 && out_dtype == RI_BF16) return launch_add_rmsnorm<float, bf16_t, bf16_t>(x, delta, parts, ps, w, out, n_out, d, eps, rows, x_rows, stream);
    return ri_fail("ri_add_rmsnorm: unsupported dtypes delta=%d weight=%d out=%d", delta_dtype, w_dtype, out_dtype);
}

// ---------------------------------------------------------------------------
// Rotation of q (in place) and k by absolute position, pairing element i with i + rot/2
// (reference: rope.cu:84-133), and the write of rotated k and of v into the request's
// pages (reference: scatter_kv_batch.cu:236-304).  One block per token.
//   qkv row: [ q: H*hd | k: Hkv*hd | v: Hkv*hd ]     (k, v only if has_kv)
//   k cache: [num_pages][Hkv][page][hd]
//   v cache: [num_pages][Hkv][hd][page]   (position-contiguous, the layout the matrix cores
//            want for P.V; a choice of this engine, the reference keeps both row-major)
// ---------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
        TA* __restrict__ qkv, int row_stride, int H, int Hkv, int hd, int rot,
        const float* __restrict__ cos_t, const float* __restrict__ sin_t,
        const int* __restrict__ positions, const int* __restrict__ row_of_token,
        TA* __restrict__ kc, TA* __restrict__ vc, const int* __restrict__ table, int max_blocks,
        int page, int write_kv) {
    const int t = blockIdx.x;
    const int b = row_of_token[t];
    const int pos = positions[t];
    if (b < 0) return;                       // padding token
    TA* row = qkv + (size_t)t * row_stride;
    const int half = rot >> 1;
    const bool rotate = cos_t != nullptr;
    const float* cs = rotate ? cos_t + (size_t)pos * half : nullptr;
    const float* sn = rotate ? sin_t + (size_t)pos * half : nullptr;
    // one work item = one rotary pair of q or k, or one element that is only copied
    const int q_pairs = rotate ? H * half : 0;
    for (int idx = threadIdx.x; idx < q_pairs; idx += blockDim.x) {
        const int h = idx / half, i = idx - h * half;
        TA* qh = row + h * hd;
        const float a = ld_f32(qh + i), bb = ld_f32(qh + i + half);
        const float c = cs[i], s = sn[i];
        st_f32(qh + i, a * c - bb * s);
        st_f32(qh + i + half, a * s + bb * c);
    }
    if (!write_kv) return;
    const int blk = table[(size_t)b * max_blocks + pos / page];
    if (blk < 0) return;
    const int slot = pos % page;
    const TA* k = row + H * hd;
    const TA* v = k + Hkv * hd;
    for (int idx = threadIdx.x; idx < Hkv * hd; idx += blockDim.x) {
        const int g = idx / hd, dd = idx - g * hd;
        const TA* kh = k + g * hd;
        float val;
        if (rotate && dd < half) {
            val = ld_f32(kh + dd) * cs[dd] - ld_f32(kh + dd + half) * sn[dd];
        } else if (rotate && dd < rot) {
            const int i = dd - half;
            val = ld_f32(kh + i) * sn[i] + ld_f32(kh + dd) * cs[i];
        } else {
            val = ld_f32(kh + dd);
        }
        const size_t head = ((size_t)blk * Hkv + g) * page * hd;
        st_f32(kc + head + (size_t)slot * hd + dd, val);
        vc[head + (size_t)dd * page + slot] = v[idx];
    }
}

// Are the 16 tokens from t0 one request's consecutive positions that start a 16-slot stretch of a page?
__device__ __forceinline__ bool rope_value_run(int t0, int T, const int* __restrict__ row_of_token,
                                               const int* __restrict__ positions, int page) {
    if (t0 + 16 > T) return false;
    const int b0 = row_of_token[t0], p0 = positions[t0];
    bool run = b0 >= 0 && (p0 % page) % 16 == 0;
    for (int i = 1; run && i < 16; ++i) run = row_of_token[t0 + i] == b0 && positions[t0 + i] == p0 + i;
    return run;
}

// bfloat16 rows whose every head is rotated whole (rot == hd, hd % 16 == 0) and 16-byte aligned:
// eight elements a thread.  Blocks [0, T) rotate q and k of one token each and write k; blocks
// [T, T + ceil(T / 16)) look at 16 consecutive tokens each: where those are 16 consecutive
// positions of one request starting a 16-slot stretch of a page (the usual case in a prompt), a
// thread writes the 16 values of one feature as 32 contiguous bytes of the position-contiguous
// value cache; otherwise every token's own block writes its values, two bytes at a time.
__global__ __launch_bounds__(256) void rope_kv_write_bf16x8_kernel(
        bf16_t* __restrict__ qkv, int row_stride, int T, int H, int Hkv, int hd,
        const float* __restrict__ cos_t, const float* __restrict__ sin_t,
        const int* __restrict__ positions, const int* __restrict__ row_of_token,
        bf16_t* __restrict__ kc, bf16_t* __restrict__ vc, const int* __restrict__ table, int max_blocks,
        int page, int write_kv) {
    const int half = hd >> 1;
    if ((int)blockIdx.x < T) {
        const int t = blockIdx.x;
        const int b = row_of_token[t];
        if (b < 0) return;                       // padding token
        const int pos = positions[t];
        bf16_t* row = qkv + (size_t)t * row_stride;
        const float* cs = cos_t + (size_t)pos * half;
        const float* sn = sin_t + (size_t)pos * half;
        int blk = -1;
        if (write_kv) blk = table[(size_t)b * max_blocks + pos / page];
        const int slot = pos % page;
        const int vph = half >> 3;               // 8-element pieces in half a head
        const int heads = write_kv ? H + Hkv : H;
        for (int idx = threadIdx.x; idx < heads * vph; idx += 256) {
            const int h = idx / vph, i0 = (idx - h * vph) * 8;
            bf16_t* src = row + (size_t)h * hd;              // the k heads follow the q heads
            float a[8], bb[8], c[8], s[8], lo[8], hi[8];
            VecLoad<4>::ld(src + i0, a); VecLoad<4>::ld(src + i0 + 4, a + 4);
            VecLoad<4>::ld(src + half + i0, bb); VecLoad<4>::ld(src + half + i0 + 4, bb + 4);
            VecLoad<4>::ld(cs + i0, c); VecLoad<4>::ld(cs + i0 + 4, c + 4);
            VecLoad<4>::ld(sn + i0, s); VecLoad<4>::ld(sn + i0 + 4, s + 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) { lo[e] = a[e] * c[e] - bb[e] * s[e]; hi[e] = a[e] * s[e] + bb[e] * c[e]; }
            bf16_t* dst = src;
            if (h >= H) {
                if (blk < 0) continue;
                dst = kc + ((size_t)blk * Hkv + (h - H)) * page * hd + (size_t)slot * hd;
            }
            VecLoad<4>::st(dst + i0, lo); VecLoad<4>::st(dst + i0 + 4, lo + 4);
            VecLoad<4>::st(dst + half + i0, hi); VecLoad<4>::st(dst + half + i0 + 4, hi + 4);
        }
        // this token's values, unless the block of its group of 16 writes them all at once
        if (!write_kv || blk < 0 || rope_value_run(t & ~15, T, row_of_token, positions, page)) return;
        const bf16_t* v = row + (size_t)(H + Hkv) * hd;
        for (int idx = threadIdx.x; idx < Hkv * hd; idx += 256) {
            const int g = idx / hd, dd = idx - g * hd;
            vc[((size_t)blk * Hkv + g) * page * hd + (size_t)dd * page + slot] = v[idx];
        }
        return;
    }
    if (!write_kv) return;
    const int t0 = ((int)blockIdx.x - T) * 16;
    if (!rope_value_run(t0, T, row_of_token, positions, page)) return;
    const bf16_t* v0 = qkv + (size_t)t0 * row_stride + (size_t)(H + Hkv) * hd;
    {
        const int b0 = row_of_token[t0], p0 = positions[t0];
        const int blk = table[(size_t)b0 * max_blocks + p0 / page];
        if (blk < 0) return;
        const int slot0 = p0 % page;
        for (int idx = threadIdx.x; idx < Hkv * hd; idx += 256) {
            const int g = idx / hd, dd = idx - g * hd;
            uint32_t w[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                w[i] = (uint32_t)v0[(size_t)(2 * i) * row_stride + idx] | ((uint32_t)v0[(size_t)(2 * i + 1) * row_stride + idx] << 16);
            uint4* dst = reinterpret_cast<uint4*>(vc + ((size_t)blk * Hkv + g) * page * hd + (size_t)dd * page + slot0);
            dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
            dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
        }
    }
}

extern "C" int ri_rope_kv_write(void* qkv, int act_dtype, int T, int row_stride, int H, int Hkv, int hd,
                                int rot, const float* cos_t, const float* sin_t, int table_rows,
                                const int* positions, const int* row_of_token,
                                void* kc, void* vc, int num_pages, const int* table, int max_blocks,
                                int page, int has_kv, int write_kv, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && H > 0 && Hkv > 0 && hd > 0 && page > 0, "ri_rope_kv_write: bad sizes");
    RI_REQUIRE(row_stride >= H * hd + (has_kv ? 2 * Hkv * hd : 0), "ri_rope_kv_write: row stride %d too small", row_stride);
    RI_REQUIRE(!write_kv || has_kv, "ri_rope_kv_write: cannot write k/v that the row does not hold");
    if (cos_t) RI_REQUIRE(rot > 0 && rot % 2 == 0 && rot <= hd && sin_t && table_rows > 0, "ri_rope_kv_write: rot %d must be even and within head size %d", rot, hd);
    if (write_kv) RI_REQUIRE(kc && vc && table && max_blocks > 0 && num_pages > 0, "ri_rope_kv_write: no cache given");
    if (T == 0) return 0;
    RI_REQUIRE(qkv && positions && row_of_token, "ri_rope_kv_write: null pointer");
    const bool rows16 = row_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0 && hd % 16 == 0
        && (!write_kv || ((uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0 && page % 16 == 0));
    if (act_dtype == RI_BF16 && cos_t && rot == hd && rows16 && (!write_kv || has_kv)
            && (uintptr_t)cos_t % 16 == 0 && (uintptr_t)sin_t % 16 == 0) {
        const int blocks = T + (write_kv ? (T + 15) / 16 : 0);
        rope_kv_write_bf16x8_kernel<<<blocks, 256, 0, stream>>>((bf16_t*)qkv, row_stride, T, H, Hkv, hd, cos_t, sin_t, positions, row_of_token, (bf16_t*)kc, (bf16_t*)vc, table, max_blocks, page, write_kv);
        RI_LAUNCHED("ri_rope_kv_write");
        return 0;
    }
    if (act_dtype == RI_F32)
        rope_kv_write_kernel<float><<<T, 256, 0, stream>>>((float*)qkv, row_stride, H, Hkv, hd, rot, cos_t, sin_t, positions, row_of_token, (float*)kc, (float*)vc, table, max_blocks, page, write_kv);
    else if (act_dtype == RI_BF16)
        rope_kv_write_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)qkv, row_stride, H, Hkv, hd, rot, cos_t, sin_t, positions, row_of_token, (bf16_t*)kc, (bf16_t*)vc, table, max_blocks, page, write_kv);
    else
        return ri_fail("ri_rope_kv_write: unknown dtype %d", act_dtype);
    RI_LAUNCHED("ri_rope_kv_write");
    return 0;
}

// ---------------------------------------------------------------------------
// out[t, j] = silu(gu[t, j]) * gu[t, I + j],  silu(z) = z / (1 + exp(-z))  in 32-bit
// (reference: swiglu.cu:294-343)
// ---------------------------------------------------------------------------
template <typename TA>
__global__ void swiglu_kernel(const TA* __restrict__ gu, TA* __restrict__ out, int I) {
    const int t = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= I) return;
    const TA* row = gu + (size_t)t * 2 * I;
    const float g = ld_f32(row + j), u = ld_f32(row + I + j);
    st_f32(out + (size_t)t * I + j, g / (1.f + expf(-g)) * u);
}

// bfloat16 rows with I % 8 == 0: 16 bytes per thread and load
__global__ __launch_bounds__(256) void swiglu_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int I) {
    const int t = blockIdx.y;
    const int j = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (j >= I) return;
    const bf16_t* row = gu + (size_t)t * 2 * I;
    const uint4 g4 = *reinterpret_cast<const uint4*>(row + j);
    const uint4 u4 = *reinterpret_cast<const uint4*>(row + I + j);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
        const float y0 = g0 / (1.f + __expf(-g0)) * u0, y1 = g1 / (1.f + __expf(-g1)) * u1;
        ow[i] = (uint32_t)f32_to_bf16(y0) | ((uint32_t)f32_to_bf16(y1) << 16);
    }
    *reinterpret_cast<uint4*>(out + (size_t)t * I + j) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int ri_swiglu(const void* gate_up, void* out, int act_dtype, int T, int I, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && I > 0, "ri_swiglu: bad sizes T=%d I=%d", T, I);
    if (T == 0) return 0;
    RI_REQUIRE(T <= 65535, "ri_swiglu: T=%d exceeds the grid limit", T);
    RI_REQUIRE(gate_up && out, "ri_swiglu: null pointer");
    dim3 grid((I + 255) / 256, T);
    if (act_dtype == RI_F32)
        swiglu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gate_up, (float*)out, I);
    else if (act_dtype == RI_BF16 && I % 8 == 0 && (uintptr_t)gate_up % 16 == 0 && (uintptr_t)out % 16 == 0)
        swiglu_bf16x8_kernel<<<dim3((I / 8 + 255) / 256, T), 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, I);
    else if (act_dtype == RI_BF16)
        swiglu_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, I);
    else
        return ri_fail("ri_swiglu: unknown dtype %d", act_dtype);
    RI_LAUNCHED("ri_swiglu");
    return 0;
}
