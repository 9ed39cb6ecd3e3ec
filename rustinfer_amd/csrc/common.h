// Shared helpers of the gfx950 kernels: dtypes, error reporting, reductions.
// Every entry point is extern "C", takes raw device pointers and a HIP stream, checks its
// operands on the host and returns 0, or non-zero with a message in ri_last_error().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

enum { RI_F32 = 0, RI_BF16 = 1 };

typedef uint16_t bf16_t;   // raw bfloat16 bits

extern "C" const char* ri_last_error();
int ri_fail(const char* fmt, ...);

#define RI_REQUIRE(cond, ...) do { if (!(cond)) return ri_fail(__VA_ARGS__); } while (0)
#define RI_LAUNCHED(name) do { hipError_t e_ = hipGetLastError(); \
    if (e_ != hipSuccess) return ri_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); } while (0)

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest, ties to even; NaN stays NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

// A 16-byte load of data that is read once (weights, the keys and values of a decoding step): the
// non-temporal form.  A kernel that only reads memory reaches a tenth more bandwidth with it than
// with plain loads on this GPU (6.9 against 6.1 TB/s over 4 GiB).
typedef unsigned int ri_u32x4_t __attribute__((ext_vector_type(4)));
template <typename T>
__device__ __forceinline__ T ld_stream16(const void* p) {
    static_assert(sizeof(T) == 16, "ld_stream16 loads 16 bytes");
    const ri_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const ri_u32x4_t*>(p));
    return __builtin_bit_cast(T, v);
}

__device__ __forceinline__ float ld_f32(const float* p) { return *p; }
__device__ __forceinline__ float ld_f32(const bf16_t* p) { return bf16_to_f32(*p); }
__device__ __forceinline__ void st_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void st_f32(bf16_t* p, float v) { *p = f32_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Block-wide reductions for blocks of up to 1024 threads (16 waves); `red` holds 16 floats.
// Every thread gets the result.  Contains two barriers.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nw; ++i) r += red[i];
    return r;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
    for (int i = 1; i < nw; ++i) r = fmaxf(r, red[i]);
    return r;
}
