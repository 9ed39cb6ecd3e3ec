// Choice of the next token from 32-bit logits: argmax, and temperature sampling with
// top-k / min-p / top-p filters.
#include "common.h"
#include <math.h>

// ---------------------------------------------------------------------------
// argmax over each row; ties go to the lowest index (reference: sampler.cu:65-78,81-164).
// NaN never wins.  One block of 1024 threads per row.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, int V,
                                                      int ld, int* __restrict__ out) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const float* row = logits + (size_t)blockIdx.x * ld;
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += 1024) {
        const float v = row[i];
        if (v > best || (v == best && i < besti)) { best = v; besti = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64);
        const int oi = __shfl_xor(besti, o, 64);
        if (ov > best || (ov == best && oi < besti)) { best = ov; besti = oi; }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { sv[wave] = best; si[wave] = besti; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < besti)) { best = sv[w]; besti = si[w]; }
        out[blockIdx.x] = besti == 0x7fffffff ? 0 : besti;
    }
}

extern "C" int ri_argmax(const float* logits, int rows, int V, int ld, int* out, hipStream_t stream) {
    RI_REQUIRE(rows >= 0 && V > 0 && ld >= V, "ri_argmax: bad sizes rows=%d V=%d ld=%d", rows, V, ld);
    if (rows == 0) return 0;
    RI_REQUIRE(logits && out, "ri_argmax: null pointer");
    argmax_kernel<<<rows, 1024, 0, stream>>>(logits, V, ld, out);
    RI_LAUNCHED("ri_argmax");
    return 0;
}
