// Choice of the next token from 32-bit logits: argmax, and temperature sampling with
// top-k / min-p / top-p filters.
#include "common.h"
#include <math.h>

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

__global__ __launch_bounds__(256) void argmax_slices_kernel(const float* __restrict__ logits, int V, int ld,
                                                            int slice, float* __restrict__ pv, int* __restrict__ pi) {
    __shared__ float sv[4];
    __shared__ int si[4];
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
// Temperature sampling with top-k / min-p / top-p, one block of 1024 threads per row.
//
// The reference samples on the host (sampler_stack.rs:242-351): logits / T, sort descending,
// keep the first top_k, w = exp(l - max), drop w < w0 * min_p, keep the shortest prefix whose
// share reaches top_p, then walk the kept tokens until the draw u * sum(w) is used up.
// Every filter keeps a prefix of the descending order, and the walk asks for the token at
// which the running sum passes a target, so no sort is needed: the kernel descends the bits
// of an order-preserving key, eight at a time, with a histogram of counts and of weights
// per digit.  Equal logits are ordered by token id.  Weights are summed as 64-bit fixed
// point (w * 2^32), so sums do not depend on the order of addition and the sum of a digit
// equals the sum of its sub-digits exactly.
// ---------------------------------------------------------------------------
namespace {

constexpr int SAMPLE_BLOCK = 1024;

struct SampleShared {
    unsigned long long mass[256];
    unsigned int cnt[256];
    unsigned long long scan_mass;     // results of the digit walk
    unsigned int scan_cnt;
    unsigned int digit;
    unsigned int tcount[SAMPLE_BLOCK];
    float red[16];
};

__device__ __forceinline__ uint32_t order_key(float v) {
    const uint32_t u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);      // larger value -> larger key
}

struct RowView {
    const float* row;
    int V;
    float inv_t, lmax;
    __device__ __forceinline__ float scaled(int i) const {
        const float l = row[i] * inv_t;
        return l != l ? -INFINITY : l;
    }
    __device__ __forceinline__ float weight(float l) const {
        if (lmax == INFINITY) return l == INFINITY ? 1.f : 0.f;
        if (lmax == -INFINITY) return 1.f;
        return expf(l - lmax);
    }
    __device__ __forceinline__ unsigned long long wfix(float l) const {
        return (unsigned long long)(weight(l) * 4294967296.0f);
    }
};

struct Boundary {            // an element of the descending order
    uint32_t key;            // its key; elements with this key are ordered by token id
    unsigned int j;          // its rank among the elements with this key
    unsigned int n_before;   // elements before it
    unsigned long long mass_before, w;   // weight before it, and its own
};

enum { BY_COUNT = 0, BY_MASS_GT = 1, BY_MASS_GE = 2 };

// Find the first element e of the descending order with
//   BY_COUNT:   n_before(e) + 1 >  target            (the element of rank `target`)
//   BY_MASS_GT: mass_before(e) + w(e) >  target
//   BY_MASS_GE: mass_before(e) + w(e) >= target
// or the last element if none does.  All threads of the block call it and get the result.
__device__ Boundary descend(const RowView& rv, int mode, unsigned long long target, SampleShared& sh) {
    uint32_t prefix = 0, mask = 0;
    unsigned int n_before = 0;
    unsigned long long m_before = 0;
    unsigned int bucket_cnt = 0;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int i = threadIdx.x; i < 256; i += SAMPLE_BLOCK) { sh.mass[i] = 0; sh.cnt[i] = 0; }
        __syncthreads();
        for (int i = threadIdx.x; i < rv.V; i += SAMPLE_BLOCK) {
            const float l = rv.scaled(i);
            const uint32_t k = order_key(l);
            if ((k & mask) == prefix) {
                const unsigned int dg = (k >> shift) & 255u;
                atomicAdd(&sh.cnt[dg], 1u);
                const unsigned long long w = rv.wfix(l);
                if (w) atomicAdd(&sh.mass[dg], w);
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned int c = n_before, last = 256;
            unsigned long long m = m_before;
            int found = -1;
            for (int dg = 255; dg >= 0; --dg) {
                if (sh.cnt[dg] == 0) continue;
                bool cross;
                if (mode == BY_COUNT) cross = (unsigned long long)c + sh.cnt[dg] > target;
                else if (mode == BY_MASS_GT) cross = m + sh.mass[dg] > target;
                else cross = m + sh.mass[dg] >= target;
                if (cross) { found = dg; break; }
                last = dg;
                c += sh.cnt[dg];
                m += sh.mass[dg];
            }
            if (found < 0) {            // nothing crosses: stay on the last non-empty digit
                found = (int)last;
                c -= sh.cnt[found];
                m -= sh.mass[found];
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
        bucket_cnt = sh.cnt[sh.digit];
        __syncthreads();
    }
    // all elements with this key have the same weight
    Boundary b;
    b.key = prefix;
    const uint32_t bits = (prefix & 0x80000000u) ? (prefix & 0x7fffffffu) : ~prefix;
    b.w = rv.wfix(__uint_as_float(bits));
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
    sh.tcount[threadIdx.x] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned int acc = 0;
        sh.digit = 0;
        for (int t = 0; t < SAMPLE_BLOCK; ++t) {
            if (acc + sh.tcount[t] > j) { sh.digit = t; sh.scan_cnt = j - acc; break; }
            acc += sh.tcount[t];
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

}  // namespace

__global__ __launch_bounds__(SAMPLE_BLOCK) void sample_kernel(
        const float* __restrict__ logits, int V, int ld,
        const float* __restrict__ temperature, const int* __restrict__ top_k,
        const float* __restrict__ top_p, const float* __restrict__ min_p,
        const double* __restrict__ draws, int* __restrict__ out) {
    __shared__ SampleShared sh;
    const int r = blockIdx.x;
    RowView rv;
    rv.row = logits + (size_t)r * ld;
    rv.V = V;
    const float temp = temperature[r];
    const bool is_greedy = !(temp > 0.f) || top_k[r] == 1 || !(top_p[r] > 0.f);   // sampler.rs:44-46
    rv.inv_t = is_greedy ? 1.f : 1.f / temp;
    // maximum (and, for greedy rows, where it is: lowest id on ties)
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += SAMPLE_BLOCK) {
        const float l = rv.scaled(i);
        if (l > best || (l == best && i < besti)) { best = l; besti = i; }
    }
    rv.lmax = block_max(best, sh.red);
    if (is_greedy) {
        int cand = (best == rv.lmax) ? besti : 0x7fffffff;
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) cand = min(cand, __shfl_xor(cand, o, 64));
        if ((threadIdx.x & 63) == 0) sh.tcount[threadIdx.x >> 6] = (unsigned int)cand;
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned int m = sh.tcount[0];
            for (int w = 1; w < SAMPLE_BLOCK / 64; ++w) m = min(m, sh.tcount[w]);
            out[r] = m == 0x7fffffffu ? 0 : (int)m;
        }
        return;
    }
    // the whole row: count and weight; and the part min_p keeps (w >= w0 * min_p, w0 = 1)
    const float mp = min_p[r];
    unsigned long long tot = 0, mp_mass = 0;
    unsigned int mp_cnt = 0;
    for (int i = threadIdx.x; i < V; i += SAMPLE_BLOCK) {
        const float l = rv.scaled(i);
        const unsigned long long w = rv.wfix(l);
        tot += w;
        if (mp > 0.f && rv.weight(l) >= mp) { mp_mass += w; ++mp_cnt; }
    }
    for (int i = threadIdx.x; i < 256; i += SAMPLE_BLOCK) { sh.mass[i] = 0; sh.cnt[i] = 0; }
    __syncthreads();
    atomicAdd(&sh.mass[0], tot);
    atomicAdd(&sh.mass[1], mp_mass);
    atomicAdd(&sh.cnt[0], mp_cnt);
    __syncthreads();
    unsigned long long keep_mass = sh.mass[0];
    unsigned int keep_n = (unsigned int)V;
    const unsigned long long mpm = sh.mass[1];
    const unsigned int mpc = sh.cnt[0];
    __syncthreads();
    const int k = top_k[r];
    if (k > 0 && k < V) {
        const Boundary b = descend(rv, BY_COUNT, (unsigned long long)(k - 1), sh);
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
        const Boundary b = descend(rv, BY_MASS_GE, tgt, sh);
        if (b.n_before + 1 < keep_n) { keep_n = b.n_before + 1; keep_mass = b.mass_before + b.w; }
    }
    double u = draws[r];
    u = u < 0.0 ? 0.0 : (u > 1.0 - 2.220446049250313e-16 ? 1.0 - 2.220446049250313e-16 : u);
    unsigned long long target = (unsigned long long)(u * (double)keep_mass);
    if (keep_mass > 0 && target >= keep_mass) target = keep_mass - 1;
    const Boundary b = descend(rv, BY_MASS_GT, target, sh);
    unsigned int j = b.j;
    uint32_t key = b.key;
    if (b.n_before >= keep_n) {                              // rounding put it past the kept prefix
        const Boundary last = descend(rv, BY_COUNT, (unsigned long long)(keep_n - 1), sh);
        key = last.key;
        j = last.j;
    }
    const int tok = locate(rv, key, j, sh);
    if (threadIdx.x == 0) out[r] = tok;
}

extern "C" int ri_sample(const float* logits, int rows, int V, int ld, const float* temperature,
                         const int* top_k, const float* top_p, const float* min_p,
                         const double* draws, int* out, hipStream_t stream) {
    RI_REQUIRE(rows >= 0 && V > 0 && ld >= V, "ri_sample: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
    if (rows == 0) return 0;
    RI_REQUIRE(logits && temperature && top_k && top_p && min_p && draws && out, "ri_sample: null pointer");
    sample_kernel<<<rows, SAMPLE_BLOCK, 0, stream>>>(logits, V, ld, temperature, top_k, top_p, min_p, draws, out);
    RI_LAUNCHED("ri_sample");
    return 0;
}
