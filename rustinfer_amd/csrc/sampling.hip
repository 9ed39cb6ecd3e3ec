// Choice of the next token from 32-bit logits: argmax, and temperature sampling with
// top-k / min-p / top-p filters.
#include "common.h"
#include "no_alloc.h"
#include <math.h>
#include <mutex>

// ---------------------------------------------------------------------------
// argmax over each row; ties go to the lowest index (reference: sampler.cu:65-78,81-164).
// NaN never wins.  Two phases as in the reference: slices of a row in parallel, then the
// best of the slices.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void better(float& best, int& besti, float v, int i) {
    if (v > best || (v == best && i < besti)) { best = v; besti = i; }
}

__device__ __forceinline__ void block_argmax(float& best, int& besti, float* sv, int* si) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(besti, o, 64);
        better(best, besti, ov, oi);
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    if (lane == 0) { sv[wave] = best; si[wave] = besti; }
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < nw; ++w) better(best, besti, sv[w], si[w]);
}

// zero_c / zero_m (may be null): [rows][zero_n] counters that the blocks of a row clear between them
// (the sampling kernels add to them afterwards).
__global__ __launch_bounds__(256) void argmax_slices_kernel(const float* __restrict__ logits, int V, int ld,
                                                            int slice, float* __restrict__ pv, int* __restrict__ pi,
                                                            unsigned int* __restrict__ zero_c = nullptr,
                                                            unsigned long long* __restrict__ zero_m = nullptr, int zero_n = 0) {
    __shared__ float sv[4];
    __shared__ int si[4];
    if (zero_c) {
        const int share = (zero_n + (int)gridDim.x - 1) / (int)gridDim.x;
        const int z0 = blockIdx.x * share, z1 = min(zero_n, z0 + share);
        for (int i = z0 + threadIdx.x; i < z1; i += 256) {
            zero_c[(size_t)blockIdx.y * zero_n + i] = 0;
            zero_m[(size_t)blockIdx.y * zero_n + i] = 0;
        }
    }
    const float* row = logits + (size_t)blockIdx.y * ld;
    const int lo = blockIdx.x * slice, hi = min(V, lo + slice);
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += 256) better(best, besti, row[i], i);
    block_argmax(best, besti, sv, si);
    if (threadIdx.x == 0) {
        pv[blockIdx.y * gridDim.x + blockIdx.x] = best;
        pi[blockIdx.y * gridDim.x + blockIdx.x] = besti;
    }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                          int n, int* __restrict__ out) {
    __shared__ float sv[1];
    __shared__ int si[1];
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = threadIdx.x; i < n; i += 64) better(best, besti, pv[blockIdx.x * n + i], pi[blockIdx.x * n + i]);
    block_argmax(best, besti, sv, si);
    if (threadIdx.x == 0) out[blockIdx.x] = besti == 0x7fffffff ? 0 : besti;
}

extern "C" int ri_argmax_slices(int V) { return V >= 8192 ? 64 : 1; }

// scratch: 2 * rows * ri_argmax_slices(V) 4-byte words
extern "C" int ri_argmax(const float* logits, int rows, int V, int ld, int* out, void* scratch,
                         hipStream_t stream) {
    RI_REQUIRE(rows >= 0 && V > 0 && ld >= V, "ri_argmax: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
    if (rows == 0) return 0;
    RI_REQUIRE(rows <= 65535, "ri_argmax: too many rows");
    RI_REQUIRE(logits && out && scratch, "ri_argmax: null pointer");
    const int n = ri_argmax_slices(V);
    const int slice = (V + n - 1) / n;
    float* pv = (float*)scratch;
    int* pi = (int*)scratch + (size_t)rows * n;
    argmax_slices_kernel<<<dim3(n, rows), 256, 0, stream>>>(logits, V, ld, slice, pv, pi);
    RI_LAUNCHED("ri_argmax");
    argmax_final_kernel<<<rows, 64, 0, stream>>>(pv, pi, n, out);
    RI_LAUNCHED("ri_argmax(final)");
    return 0;
}

// ---------------------------------------------------------------------------
// The same argmax for callers that cannot allocate (no_alloc.h): the slice maxima lie in a
// device array of the library instead of a buffer the caller brings.
// ---------------------------------------------------------------------------
#define RI_NO_ALLOC_MAX_DEVICES 64
// [rows][64] maxima (float) then [rows][64] places (int), at most; 512 KiB
static __device__ __align__(256) unsigned char scratch[(size_t)RI_ARGMAX_NO_ALLOC_MAX_ROWS * 64 * 8];
// In host code `scratch` is only a handle for the symbol: the array's address on a device comes
// from hipGetSymbolAddress with that device current, and each device has its own.
static void* g_scratch_ptr[RI_NO_ALLOC_MAX_DEVICES] = {};
static std::mutex g_scratch_mutex;

static int no_alloc_scratch(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    RI_REQUIRE(e == hipSuccess, "no_alloc: hipGetDevice failed: %s", hipGetErrorString(e));
    RI_REQUIRE(dev >= 0 && dev < RI_NO_ALLOC_MAX_DEVICES, "no_alloc: device %d beyond the %d this library keeps track of",
               dev, RI_NO_ALLOC_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        RI_REQUIRE(e == hipSuccess && p, "no_alloc: hipGetSymbolAddress failed on device %d: %s", dev,
                   hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

extern "C" int ri_no_alloc_init() {
    void* p = nullptr;
    return no_alloc_scratch(&p);
}

extern "C" int ri_argmax_no_alloc_max_rows() { return RI_ARGMAX_NO_ALLOC_MAX_ROWS; }

extern "C" int ri_argmax_no_alloc(const float* logits, int rows, int V, int ld, int* out, hipStream_t stream) {
    RI_REQUIRE(rows >= 0 && V > 0 && ld >= V, "ri_argmax_no_alloc: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
    if (rows == 0) return 0;
    RI_REQUIRE(rows <= RI_ARGMAX_NO_ALLOC_MAX_ROWS, "ri_argmax_no_alloc: %d rows exceed the %d this entry point "
               "has scratch for; use ri_argmax with a buffer of the caller's", rows, RI_ARGMAX_NO_ALLOC_MAX_ROWS);
    RI_REQUIRE(logits && out, "ri_argmax_no_alloc: null pointer");
    void* ptr = nullptr;
    if (no_alloc_scratch(&ptr)) return 1;
    const int n = ri_argmax_slices(V);          // at most 64: rows * n * 8 bytes fit the array
    const int slice = (V + n - 1) / n;
    float* pv = (float*)ptr;
    int* pi = (int*)ptr + (size_t)rows * n;
    argmax_slices_kernel<<<dim3(n, rows), 256, 0, stream>>>(logits, V, ld, slice, pv, pi);
    RI_LAUNCHED("ri_argmax_no_alloc");
    argmax_final_kernel<<<rows, 64, 0, stream>>>(pv, pi, n, out);
    RI_LAUNCHED("ri_argmax_no_alloc(final)");
    return 0;
}

// ---------------------------------------------------------------------------
// Temperature sampling with top-k / min-p / top-p, one block of 1024 threads per row.
//
// The reference samples on the host (sampler_stack.rs:242-351): logits / T, sort descending,
// keep the first top_k, w = exp(l - max), drop w < w0 * min_p, keep the shortest prefix whose
// share reaches top_p, then walk the kept tokens until the draw u * sum(w) is used up.
// Every filter keeps a prefix of the descending order, and the walk asks for the token at
// which the running sum passes a target, so no sort of the row is needed:
//   1. one pass puts every token into one of 2048 bins by its distance from the largest logit
//      (the bin number never decreases along the descending order) and adds up the count and
//      the weight of each bin.  The largest logit and these sums are found by kernels of many
//      blocks a row (slices of the vocabulary): one block a row would leave most of the chip
//      idle while it reads the row twice.  The blocks of the second kernel also leave their
//      slice's token ids ordered by bin (a counting sort in LDS);
//   2. a question "which token is the first whose running count / weight passes the target"
//      is answered on the bins by a prefix sum, and inside the one bin it falls into by
//      taking that bin's tokens from the slices' lists (a few loads; without lists, a pass over
//      the row: 11 us each time for the one block of a row), sorting them in LDS and a second
//      prefix sum.
// Measured at 128,256 tokens, 8 rows, temperature with top-k 50 and top-p 0.95 (three questions):
// 5 us for the maxima, 18 for the bins and lists, 26 for the questions; 124 us before the lists,
// with same-address LDS atomics where block-wide minima are taken now, and with each bin's totals
// read from 16 slices by the row's one block.
// Equal logits are ordered by token id.  Weights are summed as 64-bit fixed point (w * 2^32), so
// sums do not depend on the order of addition.  A bin with more tokens than LDS holds (many
// equal logits) is searched by the slower descent over the bits of an order-preserving key,
// eight at a time, with a histogram of counts and of weights per digit.
// ---------------------------------------------------------------------------
namespace {

constexpr int SAMPLE_BLOCK = 1024;
constexpr int SAMPLE_BINS = 2048;          // two per thread of the row's block
constexpr int SAMPLE_CAND = 4096;          // tokens of one bin that are sorted in LDS
constexpr float SAMPLE_ZERO_DIST = 23.f;   // exp(-23) * 2^32 < 1: the fixed-point weight is 0 beyond
constexpr float SAMPLE_BIN_SCALE = SAMPLE_BINS / 24.f;   // bins per unit of (max - logit); the last takes the rest
constexpr int SAMPLE_SLICE_THREADS = 512;
constexpr int SAMPLE_LIST_MAX = 8192;      // tokens of a slice that the second kernel can order in LDS

struct SampleShared {
    unsigned long long bmass[SAMPLE_BINS];         // per bin: weight and count of the whole row
    unsigned int bcnt[SAMPLE_BINS];
    union {
        unsigned long long cand[SAMPLE_CAND];          // (key << 32) | ~token of a bin's tokens
        struct {                                       // the digit descent
            unsigned long long mass[256];
            unsigned int cnt[256];
            unsigned int tcount[SAMPLE_BLOCK];
        } radix;
    };
    unsigned long long wave_sums[SAMPLE_BLOCK / 64], wave_sums2[SAMPLE_BLOCK / 64];
    unsigned int wave_min[SAMPLE_BLOCK / 64], wave_max[SAMPLE_BLOCK / 64];
    unsigned int slice_cnt[16], slice_off[16];         // a bin's tokens in each slice's list
    unsigned long long scan_mass;     // results handed from one thread to all
    unsigned long long res_mass, res_w;
    unsigned int scan_cnt, digit;
    unsigned int sel, last, ncand;
    unsigned int res_key, res_token, res_n;
    float red[16];
};

__device__ __forceinline__ uint32_t order_key(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);      // larger value -> larger key
}
__device__ __forceinline__ float key_value(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

struct RowView {
    const float* row;
    int V;
    float inv_t, lmax;
    // the row's token ids ordered by bin within each slice of the vocabulary (all but the last bin's), or null;
    // slice s lies at by_bin + s * per, its bin b begins loff[s * SAMPLE_BINS + b] in and has hcnt[...] tokens
    const unsigned int* by_bin = nullptr;
    const unsigned int* loff = nullptr;
    const unsigned int* hcnt = nullptr;
    int slices = 0, per = 0;
    __device__ __forceinline__ float fix(float raw) const {       // a raw logit -> logit / T, NaN -> -inf
        const float l = raw * inv_t;
        return l != l ? -INFINITY : l;
    }
    __device__ __forceinline__ float scaled(int i) const { return fix(row[i]); }
    __device__ __forceinline__ float weight(float l) const {
        if (lmax == INFINITY) return l == INFINITY ? 1.f : 0.f;
        if (lmax == -INFINITY) return 1.f;
        return expf(l - lmax);
    }
    // floor(w * 2^32) for a weight in [0, 1]; the 32-bit conversion is one instruction
    static __device__ __forceinline__ unsigned long long fixed(float wt) {
        return wt >= 1.f ? 4294967296ull : (unsigned long long)(uint32_t)(wt * 4294967296.0f);
    }
    __device__ __forceinline__ unsigned long long wfix(float l) const { return fixed(weight(l)); }
    // bin of a token: 0 holds the largest logits
    __device__ __forceinline__ int bin(float l) const {
        if (!(fabsf(lmax) < INFINITY)) return weight(l) > 0.f ? 0 : SAMPLE_BINS - 1;
        const float d = (lmax - l) * SAMPLE_BIN_SCALE;      // >= 0, +inf for l = -inf
        return (int)fminf(d, (float)(SAMPLE_BINS - 1));
    }
};

// Calls f(token, scaled logit) for every token of the row, each exactly once, in no particular
// order.  A thread asks for four 16-byte pieces before it looks at any: with one 4-byte load at a
// time the single CU that works on a row would have a few KB in flight and wait for memory.
template <typename F>
__device__ __forceinline__ void for_each_token(const RowView& rv, F&& f) {
    constexpr int UN = 4;
    const bool vec = ((uintptr_t)rv.row & 15) == 0;
    const int V4 = vec ? rv.V / 4 : 0;
    const float4* r4 = reinterpret_cast<const float4*>(rv.row);
    for (int i0 = threadIdx.x; i0 < V4; i0 += SAMPLE_BLOCK * UN) {
        float4 v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int idx = i0 + u * SAMPLE_BLOCK;
            v[u] = idx < V4 ? r4[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int idx = i0 + u * SAMPLE_BLOCK;
            if (idx < V4) {
                f(4 * idx + 0, rv.fix(v[u].x));
                f(4 * idx + 1, rv.fix(v[u].y));
                f(4 * idx + 2, rv.fix(v[u].z));
                f(4 * idx + 3, rv.fix(v[u].w));
            }
        }
    }
    for (int i = V4 * 4 + threadIdx.x; i < rv.V; i += SAMPLE_BLOCK) f(i, rv.scaled(i));
}

struct Boundary {            // an element of the descending order
    uint32_t key;            // its key; elements with this key are ordered by token id
    unsigned int j;          // its rank among the elements with this key (if token < 0)
    int token;               // its token id, or -1 if only (key, j) are known
    unsigned int n_before;   // elements before it
    unsigned long long mass_before, w;   // weight before it, and its own
};

enum { BY_COUNT = 0, BY_MASS_GT = 1, BY_MASS_GE = 2 };

__device__ __forceinline__ unsigned long long shfl_up_u64(unsigned long long v, int off) {
    const unsigned int lo = __shfl_up((unsigned int)v, off, 64), hi = __shfl_up((unsigned int)(v >> 32), off, 64);
    return ((unsigned long long)hi << 32) | lo;
}

__device__ __forceinline__ unsigned long long shfl_xor_u64(unsigned long long v, int off) {
    const unsigned int lo = __shfl_xor((unsigned int)v, off, 64), hi = __shfl_xor((unsigned int)(v >> 32), off, 64);
    return ((unsigned long long)hi << 32) | lo;
}

// Exclusive prefix sum over the threads of the block, and the total.  Contains two barriers.
__device__ unsigned long long block_scan_excl(unsigned long long v, unsigned long long& total, SampleShared& sh) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned long long inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long n = shfl_up_u64(inc, off);
        if (lane >= off) inc += n;
    }
    __syncthreads();
    if (lane == 63) sh.wave_sums[wave] = inc;
    __syncthreads();
    unsigned long long base = 0;
    total = 0;
    for (int w = 0; w < SAMPLE_BLOCK / 64; ++w) {
        const unsigned long long s = sh.wave_sums[w];
        if (w < wave) base += s;
        total += s;
    }
    return base + inc - v;
}

// The same for two values at once (the same two barriers).
__device__ void block_scan_excl2(unsigned long long v1, unsigned long long v2, unsigned long long& ex1,
                                 unsigned long long& ex2, SampleShared& sh) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned long long i1 = v1, i2 = v2;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long n1 = shfl_up_u64(i1, off), n2 = shfl_up_u64(i2, off);
        if (lane >= off) { i1 += n1; i2 += n2; }
    }
    __syncthreads();
    if (lane == 63) { sh.wave_sums[wave] = i1; sh.wave_sums2[wave] = i2; }
    __syncthreads();
    unsigned long long b1 = 0, b2 = 0;
    for (int w = 0; w < wave; ++w) { b1 += sh.wave_sums[w]; b2 += sh.wave_sums2[w]; }
    ex1 = b1 + i1 - v1;
    ex2 = b2 + i2 - v2;
}

// The smallest mn and the largest mx over the threads of the block.  Contains two barriers.
__device__ void block_min_max(unsigned int& mn, unsigned int& mx, SampleShared& sh) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        mn = min(mn, (unsigned int)__shfl_xor((int)mn, o, 64));
        mx = max(mx, (unsigned int)__shfl_xor((int)mx, o, 64));
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) { sh.wave_min[threadIdx.x >> 6] = mn; sh.wave_max[threadIdx.x >> 6] = mx; }
    __syncthreads();
    mn = sh.wave_min[0];
    mx = sh.wave_max[0];
    for (int w = 1; w < SAMPLE_BLOCK / 64; ++w) { mn = min(mn, sh.wave_min[w]); mx = max(mx, sh.wave_max[w]); }
}

// Find the first element e of the descending order with
//   BY_COUNT:   n_before(e) + 1 >  target            (the element of rank `target`)
//   BY_MASS_GT: mass_before(e) + w(e) >  target
//   BY_MASS_GE: mass_before(e) + w(e) >= target
// or the last element if none does, by descending the digits of the key.  All threads of the
// block call it and get the result.
__device__ Boundary descend(const RowView& rv, int mode, unsigned long long target, SampleShared& sh) {
    uint32_t prefix = 0, mask = 0;
    unsigned int n_before = 0;
    unsigned long long m_before = 0;
    unsigned int bucket_cnt = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += SAMPLE_BLOCK) { sh.radix.mass[i] = 0; sh.radix.cnt[i] = 0; }
        __syncthreads();
        for (int i = threadIdx.x; i < rv.V; i += SAMPLE_BLOCK) {
            const float l = rv.scaled(i);
            const uint32_t k = order_key(l);
            if ((k & mask) == prefix) {
                const unsigned int dg = (k >> shift) & 255u;
                atomicAdd(&sh.radix.cnt[dg], 1u);
                const unsigned long long w = rv.wfix(l);
                if (w) atomicAdd(&sh.radix.mass[dg], w);
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned int c = n_before, last = 256;
            unsigned long long m = m_before;
            int found = -1;
            for (int dg = 255; dg >= 0; --dg) {
                if (sh.radix.cnt[dg] == 0) continue;
                bool cross;
                if (mode == BY_COUNT) cross = (unsigned long long)c + sh.radix.cnt[dg] > target;
                else if (mode == BY_MASS_GT) cross = m + sh.radix.mass[dg] > target;
                else cross = m + sh.radix.mass[dg] >= target;
                if (cross) { found = dg; break; }
                last = dg;
                c += sh.radix.cnt[dg];
                m += sh.radix.mass[dg];
            }
            if (found < 0) {            // nothing crosses: stay on the last non-empty digit
                found = (int)last;
                c -= sh.radix.cnt[found];
                m -= sh.radix.mass[found];
            }
            sh.digit = (unsigned int)found;
            sh.scan_cnt = c;
            sh.scan_mass = m;
        }
        __syncthreads();
        prefix |= sh.digit << shift;
        mask |= 255u << shift;
        n_before = sh.scan_cnt;
        m_before = sh.scan_mass;
        bucket_cnt = sh.radix.cnt[sh.digit];
        __syncthreads();
    }
    // all elements with this key have the same weight
    Boundary b;
    b.key = prefix;
    b.token = -1;
    b.w = rv.wfix(key_value(prefix));
    unsigned long long j;
    if (mode == BY_COUNT) j = target - n_before;
    else if (b.w == 0) j = 0;
    else if (mode == BY_MASS_GT) j = target >= m_before ? (target - m_before) / b.w : 0;
    else j = target > m_before ? (target - m_before + b.w - 1) / b.w - 1 : 0;
    if (j >= bucket_cnt) j = bucket_cnt - 1;
    b.j = (unsigned int)j;
    b.n_before = n_before + b.j;
    b.mass_before = m_before + j * b.w;
    return b;
}

// Token id of the j-th (by id) element with the given key.
__device__ int locate(const RowView& rv, uint32_t key, unsigned int j, SampleShared& sh) {
    const int chunk = (rv.V + SAMPLE_BLOCK - 1) / SAMPLE_BLOCK;
    const int lo = threadIdx.x * chunk, hi = min(rv.V, lo + chunk);
    unsigned int c = 0;
    for (int i = lo; i < hi; ++i) c += order_key(rv.scaled(i)) == key;
    sh.radix.tcount[threadIdx.x] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned int acc = 0;
        sh.digit = 0;
        for (int t = 0; t < SAMPLE_BLOCK; ++t) {
            if (acc + sh.radix.tcount[t] > j) { sh.digit = t; sh.scan_cnt = j - acc; break; }
            acc += sh.radix.tcount[t];
        }
    }
    __syncthreads();
    const int owner = sh.digit;
    const unsigned int rank = sh.scan_cnt;
    __syncthreads();
    if ((int)threadIdx.x == owner) {
        unsigned int seen = 0;
        int tok = lo;
        for (int i = lo; i < hi; ++i)
            if (order_key(rv.scaled(i)) == key) { if (seen == rank) { tok = i; break; } ++seen; }
        sh.scan_cnt = (unsigned int)tok;
    }
    __syncthreads();
    const int tok = (int)sh.scan_cnt;
    __syncthreads();
    return tok;
}

// The same question as descend(), answered from the histogram over the bins (sh.bcnt, sh.bmass,
// filled by the caller) and a sort of the one bin the answer lies in.
__device__ Boundary select(const RowView& rv, int mode, unsigned long long target, SampleShared& sh) {
    // 1. the bin: thread t stands for bins 2t and 2t + 1
    const unsigned int bin0 = 2 * threadIdx.x;
    const unsigned int my_cnt[2] = {sh.bcnt[bin0], sh.bcnt[bin0 + 1]};
    const unsigned long long my_mass[2] = {sh.bmass[bin0], sh.bmass[bin0 + 1]};
    unsigned long long c_excl, m_excl;
    block_scan_excl2((unsigned long long)my_cnt[0] + my_cnt[1], my_mass[0] + my_mass[1], c_excl, m_excl, sh);
    if (threadIdx.x == 0) sh.ncand = 0;
    unsigned long long c_at[2] = {c_excl, c_excl + my_cnt[0]}, m_at[2] = {m_excl, m_excl + my_mass[0]};
    // the first bin that answers and the last one that holds anything: a thread's own, then the block's
    unsigned int first = SAMPLE_BINS, last = 0;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        if (!my_cnt[q]) continue;
        bool cross;
        if (mode == BY_COUNT) cross = c_at[q] + my_cnt[q] > target;
        else if (mode == BY_MASS_GT) cross = m_at[q] + my_mass[q] > target;
        else cross = m_at[q] + my_mass[q] >= target;
        if (cross) first = min(first, bin0 + q);
        last = bin0 + q;
    }
    block_min_max(first, last, sh);
    const unsigned int bin = first < SAMPLE_BINS ? first : last;        // nothing crosses: the last token of all
    if (threadIdx.x == bin / 2) {
        const int q = bin & 1;
        sh.scan_cnt = (unsigned int)c_at[q]; sh.scan_mass = m_at[q]; sh.digit = my_cnt[q];
    }
    __syncthreads();
    const unsigned int n_bin_before = sh.scan_cnt, n = sh.digit;
    const unsigned long long m_bin_before = sh.scan_mass;
    __syncthreads();
    if (n > SAMPLE_CAND) return descend(rv, mode, target, sh);          // many equal logits: the slow way

    // 2. the tokens of the bin, sorted by (logit descending, token ascending)
    unsigned int npad = 2;
    while (npad < n) npad <<= 1;
    for (unsigned int e = threadIdx.x; e < npad; e += SAMPLE_BLOCK) sh.cand[e] = 0;   // padding sorts last
    __syncthreads();
    if (rv.by_bin && bin != SAMPLE_BINS - 1) {
        // the bin's tokens from the slices' lists: wave w copies those of slices w, w + 16, ...
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        if ((int)threadIdx.x < rv.slices) {
            sh.slice_cnt[threadIdx.x] = rv.hcnt[(size_t)threadIdx.x * SAMPLE_BINS + bin];
            sh.slice_off[threadIdx.x] = rv.loff[(size_t)threadIdx.x * SAMPLE_BINS + bin];
        }
        __syncthreads();
        if (wave < rv.slices) {                                // at most 16 slices, 16 waves
            unsigned int at = 0;                               // where the slice's tokens go among the candidates
            for (int s0 = 0; s0 < wave; ++s0) at += sh.slice_cnt[s0];
            const unsigned int c = sh.slice_cnt[wave];
            const unsigned int* src = rv.by_bin + (size_t)wave * rv.per + sh.slice_off[wave];
            for (unsigned int e = lane; e < c; e += 64) {
                const unsigned int tok = src[e];
                sh.cand[at + e] = ((unsigned long long)order_key(rv.scaled((int)tok)) << 32) | (0xffffffffu - tok);
            }
        }
    } else {
        for_each_token(rv, [&](int i, float l) {
            if ((unsigned int)rv.bin(l) == bin) {
                const unsigned int pos = atomicAdd(&sh.ncand, 1u);
                if (pos < (unsigned int)SAMPLE_CAND)
                    sh.cand[pos] = ((unsigned long long)order_key(l) << 32) | (0xffffffffu - (unsigned int)i);
            }
        });
    }
    __syncthreads();
    for (unsigned int k = 2; k <= npad; k <<= 1) {
        for (unsigned int j = k >> 1; j > 0; j >>= 1) {
            for (unsigned int e = threadIdx.x; e < npad; e += SAMPLE_BLOCK) {
                const unsigned int partner = e ^ j;
                if (partner > e) {
                    const unsigned long long x = sh.cand[e], y = sh.cand[partner];
                    const bool descending = (e & k) == 0;
                    if ((x < y) == descending) { sh.cand[e] = y; sh.cand[partner] = x; }
                }
            }
            __syncthreads();
        }
    }
    // 3. running weight inside the bin: thread t owns the elements [t * per, (t + 1) * per)
    const unsigned int per = (npad + SAMPLE_BLOCK - 1) / SAMPLE_BLOCK;       // 1, 2 or 4
    const unsigned int e0 = threadIdx.x * per;
    unsigned long long wloc[4] = {0, 0, 0, 0}, sum = 0;
    for (unsigned int q = 0; q < per; ++q) {
        const unsigned int e = e0 + q;
        if (e < n) wloc[q] = rv.wfix(key_value((uint32_t)(sh.cand[e] >> 32)));
        sum += wloc[q];
    }
    unsigned long long tot_w;
    const unsigned long long base = m_bin_before + block_scan_excl(sum, tot_w, sh);   // weight before this thread's first element
    if (threadIdx.x == 0) sh.sel = n;                                          // first element that answers
    __syncthreads();
    {
        unsigned long long run = base;
        for (unsigned int q = 0; q < per; ++q) {
            const unsigned int e = e0 + q;
            if (e >= n) break;
            bool cross;
            if (mode == BY_COUNT) cross = (unsigned long long)n_bin_before + e + 1 > target;
            else if (mode == BY_MASS_GT) cross = run + wloc[q] > target;
            else cross = run + wloc[q] >= target;
            if (cross) { atomicMin(&sh.sel, e); break; }
            run += wloc[q];
        }
    }
    __syncthreads();
    const unsigned int pick = sh.sel < n ? sh.sel : n - 1;                     // nothing answers: the last one
    __syncthreads();
    if (pick >= e0 && pick < e0 + per) {
        unsigned long long before = base;
        for (unsigned int q = 0; q < pick - e0; ++q) before += wloc[q];
        const unsigned long long c = sh.cand[pick];
        sh.res_key = (unsigned int)(c >> 32);
        sh.res_token = 0xffffffffu - (unsigned int)c;
        sh.res_mass = before;
        sh.res_w = wloc[pick - e0];
        sh.res_n = n_bin_before + pick;
    }
    __syncthreads();
    Boundary b;
    b.key = sh.res_key;
    b.j = 0;
    b.token = (int)sh.res_token;
    b.n_before = sh.res_n;
    b.mass_before = sh.res_mass;
    b.w = sh.res_w;
    __syncthreads();
    return b;
}

}  // namespace

// Scratch of a row, written by the slice kernels and read by the row's block:
//   slice maxima of the raw logits with their places (as the argmax kernels leave them), and per
//   slice of the second kernel the bins' weights and counts and the sums over the slice.
struct SampleScratch {
    const float* smax; const int* sarg; int nmax;          // [rows][nmax]
    unsigned int* hcnt;                                     // [rows][slices][SAMPLE_BINS]
    unsigned long long* stot; unsigned long long* smp_mass; unsigned int* smp_cnt;   // [rows][slices]
    unsigned int* loff;                                     // [rows][slices][SAMPLE_BINS]: where a bin begins in the slice's list
    unsigned int* by_bin;                                   // [rows][V]: token ids, slice after slice, bin after bin; or null
    unsigned long long* tmass; unsigned int* tcnt;          // [rows][SAMPLE_BINS]: the slices added up (cleared by the first kernel)
    int slices, per;                                        // per: tokens a slice
};

// Calls f(token, scaled logit) for the tokens [lo, hi) of the row, eight loads a thread under way.
template <typename F>
__device__ __forceinline__ void for_each_of_slice(const RowView& rv, int lo, int hi, F&& f) {
    constexpr int UN = 8;
    for (int i0 = lo + threadIdx.x; i0 < hi; i0 += SAMPLE_SLICE_THREADS * UN) {
        float v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int i = i0 + u * SAMPLE_SLICE_THREADS;
            v[u] = i < hi ? rv.row[i] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int i = i0 + u * SAMPLE_SLICE_THREADS;
            if (i < hi) f(i, rv.fix(v[u]));
        }
    }
}

__device__ __forceinline__ bool sample_row_is_greedy(float temp, int k, float p) {
    return !(temp > 0.f) || k == 1 || !(p > 0.f);                                   // sampler.rs:44-46
}

// Second kernel: one block per (slice, row) bins its part of the vocabulary, and (LIST) leaves
// its tokens ordered by bin: a counting sort in LDS with the histogram it has just made, written
// out in one piece to the slice's stretch of the row's list ([lo, hi) of by_bin; where in it each
// bin begins goes to loff).  Within a bin the order is whatever the atomics gave: whoever reads a
// bin sorts it.  The last bin (everything 24 and more below the largest logit, often nearly the
// whole row) is left out of the list; a question that ends there reads the row instead.
// Dynamic LDS: hc [BINS], hm [BINS] 64-bit; (LIST) the slice's SAMPLE_LIST_MAX token ids take hm's
// place, and as much again behind it, once the weights have been added to the row's totals.
template <bool LIST>
__global__ __launch_bounds__(SAMPLE_SLICE_THREADS) void sample_bins_kernel(
        const float* __restrict__ logits, int V, int ld, const float* __restrict__ temperature,
        const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ min_p,
        SampleScratch sc) {
    extern __shared__ __align__(16) unsigned long long bins_lds[];
    unsigned int* hc = reinterpret_cast<unsigned int*>(bins_lds);             // [SAMPLE_BINS]
    unsigned long long* hm = bins_lds + SAMPLE_BINS / 2;                      // [SAMPLE_BINS]
    unsigned int* buf = reinterpret_cast<unsigned int*>(hm);                  // [SAMPLE_LIST_MAX], after hm's last use
    __shared__ unsigned long long sums[2];
    __shared__ unsigned int sum_cnt;
    __shared__ unsigned int wave_tot[SAMPLE_SLICE_THREADS / 64];
    const int r = blockIdx.y, sl = blockIdx.x;
    const int per = (V + sc.slices - 1) / sc.slices;
    const int lo = sl * per, hi = min(V, lo + per);
    const float* row = logits + (size_t)r * ld;
    // LIST: the slice's values stay in registers for the second pass; all of them are asked for
    // here, before anything else, so that the row's parameters and maxima arrive meanwhile
    constexpr int NV = LIST ? SAMPLE_LIST_MAX / SAMPLE_SLICE_THREADS : 1;
    float lv[NV];
    if constexpr (LIST) {
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int i = lo + (int)threadIdx.x + u * SAMPLE_SLICE_THREADS;
            lv[u] = i < hi ? row[i] : 0.f;
        }
    }
    const float temp = temperature[r];
    if (sample_row_is_greedy(temp, top_k[r], top_p[r])) return;
    RowView rv;
    rv.row = row;
    rv.V = V;
    rv.inv_t = 1.f / temp;
    float raw = -INFINITY;
    for (int i = 0; i < sc.nmax; ++i) raw = fmaxf(raw, sc.smax[(size_t)r * sc.nmax + i]);
    rv.lmax = rv.fix(raw);
    for (int i = threadIdx.x; i < SAMPLE_BINS; i += SAMPLE_SLICE_THREADS) { hm[i] = 0; hc[i] = 0; }
    if (threadIdx.x == 0) { sums[0] = 0; sums[1] = 0; sum_cnt = 0; }
    __syncthreads();
    const float mp = min_p[r];
    const bool far_weights = mp > 0.f && mp < 2e-10f;          // min_p so small that far tokens may pass it
    const bool finite_max = fabsf(rv.lmax) < INFINITY;
    unsigned long long tot = 0, mp_mass = 0;
    unsigned int mp_cnt = 0, last_cnt = 0;
    if constexpr (LIST) {
#pragma unroll
        for (int u = 0; u < NV; ++u) lv[u] = rv.fix(lv[u]);
    }
    auto visit = [&](auto&& f) {
        if constexpr (LIST) {
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                const int i = lo + (int)threadIdx.x + u * SAMPLE_SLICE_THREADS;
                if (i < hi) f(i, lv[u]);
            }
        } else {
            for_each_of_slice(rv, lo, hi, f);
        }
    };
    visit([&](int, float l) {
        const int bn = rv.bin(l);
        const bool near = !finite_max || rv.lmax - l < SAMPLE_ZERO_DIST;
        unsigned long long w = 0;
        if (near || far_weights) {
            const float wt = rv.weight(l);
            w = RowView::fixed(wt);
            if (mp > 0.f && wt >= mp) { mp_mass += w; ++mp_cnt; }
        }
        tot += w;
        if (bn == SAMPLE_BINS - 1 && w == 0) { ++last_cnt; return; }     // where most of a peaked row ends up
        atomicAdd(&hc[bn], 1u);
        if (w) atomicAdd(&hm[bn], w);
    });
    if (last_cnt) atomicAdd(&hc[SAMPLE_BINS - 1], last_cnt);
    if (tot) atomicAdd(&sums[0], tot);
    if (mp_mass) atomicAdd(&sums[1], mp_mass);
    if (mp_cnt) atomicAdd(&sum_cnt, mp_cnt);
    __syncthreads();
    const size_t base = ((size_t)r * sc.slices + sl) * SAMPLE_BINS;
    // the slice's counts for whoever reads its list, and counts and weights added to the row's totals
    for (int i = threadIdx.x; i < SAMPLE_BINS; i += SAMPLE_SLICE_THREADS) {
        const unsigned int c = hc[i];
        const unsigned long long m = hm[i];
        sc.hcnt[base + i] = c;
        if (c) atomicAdd(&sc.tcnt[(size_t)r * SAMPLE_BINS + i], c);
        if (m) atomicAdd(&sc.tmass[(size_t)r * SAMPLE_BINS + i], m);
    }
    if (threadIdx.x == 0) {
        sc.stot[(size_t)r * sc.slices + sl] = sums[0];
        sc.smp_mass[(size_t)r * sc.slices + sl] = sums[1];
        sc.smp_cnt[(size_t)r * sc.slices + sl] = sum_cnt;
    }
    if constexpr (LIST) {
        // where each bin begins in this slice's list: the exclusive prefix of the counts (a thread's
        // PER consecutive bins, the threads of a wave, the waves); hc then serves as the cursors
        constexpr int PER = SAMPLE_BINS / SAMPLE_SLICE_THREADS;
        __syncthreads();
        unsigned int cnt[PER], sum = 0;
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int b = threadIdx.x * PER + q;
            cnt[q] = b == SAMPLE_BINS - 1 ? 0u : hc[b];
            sum += cnt[q];
        }
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        unsigned int inc = sum;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const unsigned int n = __shfl_up(inc, o, 64);
            if (lane >= o) inc += n;
        }
        if (lane == 63) wave_tot[wave] = inc;
        __syncthreads();
        unsigned int at = inc - sum, listed = 0;
        for (int w = 0; w < SAMPLE_SLICE_THREADS / 64; ++w) {
            if (w < wave) at += wave_tot[w];
            listed += wave_tot[w];
        }
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int b = threadIdx.x * PER + q;
            hc[b] = at;
            sc.loff[base + b] = at;
            at += cnt[q];
        }
        __syncthreads();
        visit([&](int i, float l) {
            const int bn = rv.bin(l);
            if (bn == SAMPLE_BINS - 1) return;
            const unsigned int pos = atomicAdd(&hc[bn], 1u);
            buf[pos] = (unsigned int)i;
        });
        __syncthreads();
        unsigned int* dst = sc.by_bin + (size_t)r * V + lo;
        for (unsigned int e = threadIdx.x; e < listed; e += SAMPLE_SLICE_THREADS) dst[e] = buf[e];
    }
}

// Third kernel: one block per row answers the questions.
// LP: log-probabilities are asked for (a kernel of its own, so that the usual one is not burdened).
template <bool LP>
__global__ __launch_bounds__(SAMPLE_BLOCK) void sample_kernel(
        const float* __restrict__ logits, int V, int ld,
        const float* __restrict__ temperature, const int* __restrict__ top_k,
        const float* __restrict__ top_p, const float* __restrict__ min_p,
        const double* __restrict__ draws, SampleScratch sc, int* __restrict__ out,
        float* __restrict__ out_lp, int* __restrict__ top_ids, float* __restrict__ top_lp,
        const int* __restrict__ want_top) {
    __shared__ SampleShared sh;
    const int r = blockIdx.x;
    RowView rv;
    rv.row = logits + (size_t)r * ld;
    rv.V = V;
    const float temp = temperature[r];
    const bool is_greedy = sample_row_is_greedy(temp, top_k[r], top_p[r]);
    rv.inv_t = is_greedy ? 1.f : 1.f / temp;
    // the largest logit and where it is (lowest id on ties), from the slices
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = threadIdx.x; i < sc.nmax; i += SAMPLE_BLOCK) {
        const float v = sc.smax[(size_t)r * sc.nmax + i];
        const int at = sc.sarg[(size_t)r * sc.nmax + i];
        if (v > best || (v == best && at < besti)) { best = v; besti = at; }
    }
    const float raw_max = block_max(best, sh.red);
    rv.lmax = rv.fix(raw_max);
    if (is_greedy) {
        int cand = (best == raw_max) ? besti : 0x7fffffff;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
        if ((threadIdx.x & 63) == 0) sh.radix.tcount[threadIdx.x >> 6] = (unsigned int)cand;
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned int m = sh.radix.tcount[0];
            for (int w = 1; w < SAMPLE_BLOCK / 64; ++w) m = min(m, sh.radix.tcount[w]);
            out[r] = m == 0x7fffffffu ? 0 : (int)m;
        }
        if (LP && out_lp) {
            // log-softmax of the raw logits at their maximum: -ln sum exp(l - max)
            // (sampler_stack.rs:248-256, log_softmax_at :353-365); no list of the best for greedy rows
            unsigned long long part = 0, total;
            for_each_token(rv, [&](int, float l) { part += rv.wfix(l); });
            __syncthreads();
            (void)block_scan_excl(part, total, sh);
            if (threadIdx.x == 0) out_lp[r] = (float)(-(log((double)total) - 32.0 * 0.6931471805599453));
        }
        if (LP && top_ids && threadIdx.x < 5) { top_ids[r * 5 + threadIdx.x] = -1; top_lp[r * 5 + threadIdx.x] = -INFINITY; }
        return;
    }
    // count and weight of every bin, of the whole row, and of the part min_p keeps
    // (w >= w0 * min_p, w0 = 1): the slices' sums added up
    const float mp = min_p[r];
    unsigned long long tot = 0, mp_mass = 0, mp_cnt = 0;
    rv.slices = sc.slices;
    rv.per = sc.per;
    rv.hcnt = sc.hcnt + (size_t)r * sc.slices * SAMPLE_BINS;
    if (sc.by_bin) {
        rv.by_bin = sc.by_bin + (size_t)r * V;
        rv.loff = sc.loff + (size_t)r * sc.slices * SAMPLE_BINS;
    }
    {
        for (int b = threadIdx.x; b < SAMPLE_BINS; b += SAMPLE_BLOCK) {
            sh.bmass[b] = sc.tmass[(size_t)r * SAMPLE_BINS + b];
            sh.bcnt[b] = sc.tcnt[(size_t)r * SAMPLE_BINS + b];
        }
        if ((int)threadIdx.x < sc.slices) {
            tot = sc.stot[(size_t)r * sc.slices + threadIdx.x];
            mp_mass = sc.smp_mass[(size_t)r * sc.slices + threadIdx.x];
            mp_cnt = sc.smp_cnt[(size_t)r * sc.slices + threadIdx.x];
        }
    }
    // the slices' sums (at most 16 of each, in the first threads): the first wave adds them up
    if (threadIdx.x < 64) {
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) {
            tot += shfl_xor_u64(tot, o);
            mp_mass += shfl_xor_u64(mp_mass, o);
            mp_cnt += shfl_xor_u64(mp_cnt, o);
        }
        if (threadIdx.x == 0) { sh.res_mass = tot; sh.res_w = mp_mass; sh.scan_mass = mp_cnt; }
    }
    __syncthreads();
    unsigned long long keep_mass = sh.res_mass;
    const unsigned long long mpm = sh.res_w;
    const unsigned int mpc = (unsigned int)sh.scan_mass;
    unsigned int keep_n = (unsigned int)V;
    __syncthreads();
    const int k = top_k[r];
    if (k > 0 && k < V) {
        const Boundary b = select(rv, BY_COUNT, (unsigned long long)(k - 1), sh);
        keep_n = b.n_before + 1;
        keep_mass = b.mass_before + b.w;
    }
    if (mp > 0.f && mpc >= 1 && mpc < keep_n) { keep_n = mpc; keep_mass = mpm; }
    const float p = top_p[r];
    if (p < 1.f) {
        const double want = (double)p * (double)keep_mass;
        unsigned long long tgt = (unsigned long long)want;
        if ((double)tgt < want) ++tgt;                       // ceil: cum >= p * total
        if (tgt < 1) tgt = 1;
        const Boundary b = select(rv, BY_MASS_GE, tgt, sh);
        if (b.n_before + 1 < keep_n) { keep_n = b.n_before + 1; keep_mass = b.mass_before + b.w; }
    }
    double u = draws[r];
    u = u < 0.0 ? 0.0 : (u > 1.0 - 2.220446049250313e-16 ? 1.0 - 2.220446049250313e-16 : u);
    unsigned long long target = (unsigned long long)(u * (double)keep_mass);
    if (keep_mass > 0 && target >= keep_mass) target = keep_mass - 1;
    Boundary b = select(rv, BY_MASS_GT, target, sh);
    if (b.n_before >= keep_n)                                // rounding put it past the kept prefix
        b = select(rv, BY_COUNT, (unsigned long long)(keep_n - 1), sh);
    const int tok = b.token >= 0 ? b.token : locate(rv, b.key, b.j, sh);
    if (threadIdx.x == 0) out[r] = tok;
    // ln(w / sum of the kept weights) of the chosen token and, where asked for, of the five
    // best kept tokens in their order (sampler_stack.rs:335-350); ln w is taken from the logit
    // itself, not from the fixed-point weight, so that small probabilities keep their digits
    if (LP && (out_lp || top_ids)) {
        const double log_total = log((double)keep_mass) - 32.0 * 0.6931471805599453;
        auto log_prob = [&](uint32_t key) -> float {
            const float l = key_value(key);
            const float lw = fabsf(rv.lmax) < INFINITY ? l - rv.lmax : logf(rv.weight(l));
            return (float)((double)lw - log_total);
        };
        if (out_lp && threadIdx.x == 0) out_lp[r] = log_prob(b.key);
        if (top_ids) {
            const bool want = !want_top || want_top[r] != 0;
            for (int j = 0; j < 5; ++j) {
                int id = -1;
                float lp = -INFINITY;
                if (want && (unsigned int)j < keep_n) {
                    const Boundary bj = select(rv, BY_COUNT, (unsigned long long)j, sh);
                    id = bj.token >= 0 ? bj.token : locate(rv, bj.key, bj.j, sh);
                    lp = log_prob(bj.key);
                }
                if (threadIdx.x == 0) { top_ids[r * 5 + j] = id; top_lp[r * 5 + j] = lp; }
            }
        }
    }
}

extern "C" int ri_sample_slices(int V) {
    const int n = (V + 8191) / 8192;
    return n < 1 ? 1 : (n > 16 ? 16 : n);
}

// bytes of scratch for `rows` rows of V logits
extern "C" size_t ri_sample_scratch_bytes(int rows, int V) {
    const size_t nmax = ri_argmax_slices(V), sl = ri_sample_slices(V);
    return (size_t)rows * (nmax * 8 + sl * ((size_t)SAMPLE_BINS * 8 + 24) + (size_t)SAMPLE_BINS * 12 + (size_t)V * 4) + 64;
}

// out_logprob [rows], top_ids / top_logprobs [rows][5], want_top [rows] may be null: the natural
// logarithm of the chosen token's probability among the kept ones (greedy rows: log-softmax of the
// raw logits at the maximum), and the five most probable kept tokens with theirs (-1 / -inf where
// fewer are kept, for greedy rows, and for rows whose want_top is 0).
extern "C" int ri_sample(const float* logits, int rows, int V, int ld, const float* temperature,
                         const int* top_k, const float* top_p, const float* min_p,
                         const double* draws, int* out, void* scratch, size_t scratch_bytes,
                         float* out_logprob, int* top_ids, float* top_logprobs, const int* want_top,
                         hipStream_t stream) {
    RI_REQUIRE(rows >= 0 && V > 0 && ld >= V, "ri_sample: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
    if (rows == 0) return 0;
    RI_REQUIRE(rows <= 65535, "ri_sample: too many rows");
    RI_REQUIRE(logits && temperature && top_k && top_p && min_p && draws && out && scratch, "ri_sample: null pointer");
    RI_REQUIRE((top_ids == nullptr) == (top_logprobs == nullptr), "ri_sample: top_ids and top_logprobs come together");
    RI_REQUIRE(scratch_bytes >= ri_sample_scratch_bytes(rows, V) && (uintptr_t)scratch % 8 == 0, "ri_sample: scratch too small or misaligned");
    const int nmax = ri_argmax_slices(V), sl = ri_sample_slices(V);
    // carve the scratch: 8-byte things first
    char* p = (char*)scratch;
    SampleScratch sc;
    sc.nmax = nmax;
    sc.slices = sl;
    sc.stot = (unsigned long long*)p;    p += (size_t)rows * sl * 8;
    sc.smp_mass = (unsigned long long*)p; p += (size_t)rows * sl * 8;
    sc.tmass = (unsigned long long*)p;   p += (size_t)rows * SAMPLE_BINS * 8;
    sc.hcnt = (unsigned int*)p;          p += (size_t)rows * sl * SAMPLE_BINS * 4;
    sc.smp_cnt = (unsigned int*)p;       p += (size_t)rows * sl * 4;
    sc.loff = (unsigned int*)p;          p += (size_t)rows * sl * SAMPLE_BINS * 4;
    sc.tcnt = (unsigned int*)p;          p += (size_t)rows * SAMPLE_BINS * 4;
    sc.by_bin = (unsigned int*)p;        p += (size_t)rows * V * 4;
    float* smax = (float*)p;             p += (size_t)rows * nmax * 4;
    int* sarg = (int*)p;
    sc.smax = smax;
    sc.sarg = sarg;
    const int slice = (V + nmax - 1) / nmax;
    argmax_slices_kernel<<<dim3(nmax, rows), 256, 0, stream>>>(logits, V, ld, slice, smax, sarg, sc.tcnt, sc.tmass, SAMPLE_BINS);
    RI_LAUNCHED("ri_sample(maxima)");
    sc.per = (V + sl - 1) / sl;
    constexpr size_t hist_lds = (size_t)SAMPLE_BINS * 12, list_lds = (size_t)SAMPLE_BINS * 4 + (size_t)SAMPLE_LIST_MAX * 4;
    static_assert(list_lds >= hist_lds && list_lds <= 64 * 1024, "the list covers the weights' place; within what a kernel may take unasked");
    if (sc.per <= SAMPLE_LIST_MAX) {
        sample_bins_kernel<true><<<dim3(sl, rows), SAMPLE_SLICE_THREADS, list_lds, stream>>>(logits, V, ld, temperature, top_k, top_p, min_p, sc);
    } else {
        // a vocabulary whose slices LDS does not hold: no lists, the last kernel reads the row instead
        sc.by_bin = nullptr;
        sample_bins_kernel<false><<<dim3(sl, rows), SAMPLE_SLICE_THREADS, hist_lds, stream>>>(logits, V, ld, temperature, top_k, top_p, min_p, sc);
    }
    RI_LAUNCHED("ri_sample(bins)");
    if (out_logprob || top_ids)
        sample_kernel<true><<<rows, SAMPLE_BLOCK, 0, stream>>>(logits, V, ld, temperature, top_k, top_p, min_p, draws, sc, out,
                                                               out_logprob, top_ids, top_logprobs, want_top);
    else
        sample_kernel<false><<<rows, SAMPLE_BLOCK, 0, stream>>>(logits, V, ld, temperature, top_k, top_p, min_p, draws, sc, out,
                                                                nullptr, nullptr, nullptr, nullptr);
    RI_LAUNCHED("ri_sample");
    return 0;
}
