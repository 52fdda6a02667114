// Shared device/host helpers for the gfx950 kernels of the llama decoder-layer step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

typedef __bf16 bf16_t;
typedef bf16_t bf16x2 __attribute__((ext_vector_type(2)));
typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define EZL_OK 0
#define EZL_EINVAL (-1)
#define EZL_EUNSUPPORTED (-2)
#define EZL_EHIP (-3)

#define EZL_WAVE 64

// thread-local last-error text, read back through ezl_last_error()
void ezl_set_error(const char* fmt, ...);

#define EZL_REQUIRE(cond, code, ...)      \
    do {                                  \
        if (!(cond)) {                    \
            ezl_set_error(__VA_ARGS__);   \
            return (code);                \
        }                                 \
    } while (0)

// surfaces launch-configuration errors without synchronising the device
#define EZL_LAUNCH_CHECK(name)                                                     \
    do {                                                                           \
        hipError_t e__ = hipGetLastError();                                        \
        if (e__ != hipSuccess) {                                                   \
            ezl_set_error("%s: launch failed: %s", (name), hipGetErrorString(e__)); \
            return EZL_EHIP;                                                       \
        }                                                                          \
    } while (0)

static inline bool ezl_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

#ifdef __HIPCC__
// 8 bf16 <-> 8 fp32 (one 128-bit HBM transaction per lane)
struct alignas(16) bf16x8_raw {
    bf16x8 v;
};

__device__ __forceinline__ bf16x8 ld_bf16x8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ void st_bf16x8(bf16_t* p, bf16x8 v) { *reinterpret_cast<bf16x8*>(p) = v; }
// Streaming forms for large tensors that are read or written once per kernel.  Measured inside the training step: they help
// the kernels that move hundreds of MB (SwiGLU backward 92 -> 78 us, RMSNorm backward 42 -> 34 us) and hurt where a 33 MB
// tensor goes from one kernel straight into the next (the consumer then misses the last-level cache), so only the former
// use them.
__device__ __forceinline__ bf16x8 ld_bf16x8_nt(const bf16_t* p) { return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p)); }
__device__ __forceinline__ void st_bf16x8_nt(bf16_t* p, bf16x8 v) { __builtin_nontemporal_store(v, reinterpret_cast<bf16x8*>(p)); }

__device__ __forceinline__ void unpack8(bf16x8 v, float* f) {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)v[i];
}
__device__ __forceinline__ bf16x8 pack8(const float* f) {
    bf16x8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (bf16_t)f[i];
    return v;
}

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

// out[col] (+)= sum_r partial[r][col];  64 columns per block, 16 row groups (loads of a group issued eight at a time)
// folded through LDS in a fixed order.
constexpr int kColsumThreads = 1024;
template <int UNUSED>
__global__ __launch_bounds__(kColsumThreads) void ezl_colsum_kernel(const float* __restrict__ partial, int nrows, int ncols,
                                                                    bf16_t* __restrict__ out_bf16, float* __restrict__ out_f32,
                                                                    int accumulate) {
    constexpr int G = kColsumThreads / 64;
    __shared__ float s[G][64];
    const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int col = blockIdx.x * 64 + c;
    float acc = 0.f;
    if (col < ncols) {
        int r = g;
        for (; r + 7 * G < nrows; r += 8 * G) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[(size_t)(r + u * G) * ncols + col];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; r < nrows; r += G) acc += partial[(size_t)r * ncols + col];
    }
    s[g][c] = acc;
    __syncthreads();
    if (g == 0 && col < ncols) {
        float v = 0.f;
#pragma unroll
        for (int i = 0; i < G; ++i) v += s[i][c];
        if (out_f32) out_f32[col] = accumulate ? out_f32[col] + v : v;
        else out_bf16[col] = (bf16_t)v;
    }
}
#endif
