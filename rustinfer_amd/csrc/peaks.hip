// What this GPU reaches with nothing in the way: a kernel that only reads memory, one that copies
// it, a loop of matrix instructions on registers and a loop of 32-bit FMAs.  The benchmark prices
// the engine's steps against these figures beside the published peaks: a decode step that reads
// its weights at the rate a bare read reaches cannot be made faster by a better kernel.
// (The reference prices nothing; this is the engine's own measuring tool.)
#include "common.h"

namespace {

typedef __bf16 kbf16x8_t __attribute__((ext_vector_type(8)));
typedef float kf32x4_t __attribute__((ext_vector_type(4)));
typedef float kf32x16_t __attribute__((ext_vector_type(16)));

// Every block walks the buffer with a stride of the whole grid, 16 bytes a lane and load, eight
// non-temporal loads in flight; what is read is folded into one word a block so that no load can
// be dropped.  (Of the forms tried over 4 GiB this one reads fastest: 6.9 TB/s against 6.1 with
// plain loads and 6.2 with a contiguous stretch a block.)
__global__ __launch_bounds__(256) void peak_read_kernel(const ri_u32x4_t* __restrict__ src, size_t n16, uint32_t* __restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    uint32_t acc = 0;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        ri_u32x4_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const ri_u32x4_t a = __builtin_nontemporal_load(src + i);
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x9e3779b9u) sink[blockIdx.x & 1023] = acc;     // practically never: the sink stays as it is
}

__global__ __launch_bounds__(256) void peak_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        dst[i] = a; dst[i + stride] = b; dst[i + 2 * stride] = c; dst[i + 3 * stride] = d;
    }
    for (; i < n16; i += stride) dst[i] = src[i];
}

// Four independent chains of 32x32x16 bfloat16 matrix instructions a wave, operands in registers.
__global__ __launch_bounds__(256) void peak_mfma_bf16_kernel(int iters, float* __restrict__ sink) {
    kbf16x8_t a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(0.001f * (threadIdx.x + i)); b[i] = (__bf16)(0.002f * (i + 1)); }
    kf32x16_t c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    for (int it = 0; it < iters; ++it) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
    if (s == 12345.678f) sink[blockIdx.x] = s;
}

// Eight independent chains of 32-bit FMAs a lane.
__global__ __launch_bounds__(256) void peak_fma_f32_kernel(int iters, float x, float* __restrict__ sink) {
    float r[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = 0.001f * (threadIdx.x + i);
    const float m = 1.0f - x, add = x;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) r[i] = fmaf(r[i], m, add);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += r[i];
    if (s == 12345.678f) sink[blockIdx.x] = s;
}

}  // namespace

// what: 0 read, 1 copy (bytes counted once read and once written), 2 bfloat16 matrix
// instructions, 3 32-bit FMA.  buf: device memory of `bytes` bytes (read: the source; copy: first
// half source, second half destination); sink: 16 KB of device memory nobody reads.
// Launches `reps` kernels on the stream; work_out receives the bytes moved or the
// floating-point operations done by one of them.  The caller times the stream.
extern "C" int ri_measure_peak(int what, void* buf, size_t bytes, void* sink, int reps, double* work_out, hipStream_t stream) {
    RI_REQUIRE(what >= 0 && what <= 3 && reps > 0 && sink && work_out, "ri_measure_peak: bad arguments");
    hipDeviceProp_t prop;
    int dev = 0;
    RI_REQUIRE(hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess, "ri_measure_peak: no device properties");
    const int cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    if (what <= 1) {
        RI_REQUIRE(buf && bytes >= (1u << 20) && (uintptr_t)buf % 16 == 0, "ri_measure_peak: needs a 16-byte aligned buffer of at least 1 MiB");
        const size_t n16 = what == 0 ? bytes / 16 : bytes / 32;
        const int grid = cus * 8;
        for (int r = 0; r < reps; ++r) {
            if (what == 0) peak_read_kernel<<<cus * 64, 256, 0, stream>>>((const ri_u32x4_t*)buf, n16, (uint32_t*)sink);
            else peak_copy_kernel<<<grid, 256, 0, stream>>>((const uint4*)buf, (uint4*)buf + n16, n16);
        }
        *work_out = what == 0 ? (double)n16 * 16 : (double)n16 * 32;
    } else {
        const int grid = cus * 8, iters = 4096;
        RI_REQUIRE(grid <= 4096, "ri_measure_peak: more compute units than the sink is sized for");
        for (int r = 0; r < reps; ++r) {
            if (what == 2) peak_mfma_bf16_kernel<<<grid, 256, 0, stream>>>(iters, (float*)sink);
            else peak_fma_f32_kernel<<<grid, 256, 0, stream>>>(iters, 1e-7f, (float*)sink);
        }
        // a matrix instruction: 2 * 32 * 32 * 16 operations a wave; an FMA: 2 a lane
        *work_out = what == 2 ? (double)grid * 4 * iters * 4 * (2.0 * 32 * 32 * 16) : (double)grid * 256 * iters * 8 * 2.0;
    }
    RI_LAUNCHED("ri_measure_peak");
    return 0;
}
