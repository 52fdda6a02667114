// Optimizer step for the parameters of the decoder stack on gfx950 (HBM-bound): fp32 master weights, fp32 gradient
// buffers, bf16 model weights.
//
// Restates what the reference's Megatron path runs after backward: apex `FusedAdam` in its default AdamW mode
// (built at llm/utils/model/optimizer_helper.py:93-95 from configs/megatron/llama_7b_sft.yaml:106-112) under
// DeepSpeed's bf16 optimizer with `gradient_clipping: 1.0` (llama_7b_sft.yaml:13): global L2 norm of all gradients,
// clip coefficient max_norm / (norm + 1e-6) applied when below one, then per element
//     m = b1 m + (1 - b1) g;  v = b2 v + (1 - b2) g^2;  p -= lr (m / bc1 / (sqrt(v / bc2) + eps) + wd p)
// with bc = 1 - beta^step, and the bf16 weight refreshed from the fp32 master value.
// The norm is reduced in a fixed order (per-block partials, then one block), so a step is bit-reproducible; the clip
// coefficient stays on the device: nothing here synchronises with the host.
#include "common.h"

namespace {

constexpr int kOptBlock = 256;
constexpr int kSumsqPartials = 256;  // partial sums written per ezl_sumsq_f32 call

// partials[b] = sum of x[i]^2 over block b's share (grid-stride over 4-float vectors, four loads in flight per thread,
// tail by block 0)
constexpr int kSumsqBlock = 1024;
__global__ __launch_bounds__(kSumsqBlock) void sumsq_partial_kernel(const float* __restrict__ x, int64_t n, float* __restrict__ partials) {
    __shared__ float red[kSumsqBlock / 64];
    const int64_t n4 = n >> 2;
    const int64_t stride = (int64_t)gridDim.x * kSumsqBlock;
    float acc = 0.f;
    int64_t i = (int64_t)blockIdx.x * kSumsqBlock + threadIdx.x;
    for (; i + 3 * stride < n4; i += 4 * stride) {
        f32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = reinterpret_cast<const f32x4*>(x)[i + u * stride];
#pragma unroll
        for (int u = 0; u < 4; ++u) acc += v[u][0] * v[u][0] + v[u][1] * v[u][1] + v[u][2] * v[u][2] + v[u][3] * v[u][3];
    }
    for (; i < n4; i += stride) {
        const f32x4 v = reinterpret_cast<const f32x4*>(x)[i];
        acc += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const float v = x[(n4 << 2) + threadIdx.x];
        acc += v * v;
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < kSumsqBlock / 64; ++k) t += red[k];
        partials[blockIdx.x] = t;
    }
}

// out[0] = sqrt(sum partials), out[1] = clip coefficient: max_norm / (norm + 1e-6) if that is below one, else 1
__global__ __launch_bounds__(1024) void clip_coef_kernel(const float* __restrict__ partials, int64_t count, float max_norm,
                                                         float* __restrict__ out) {
    __shared__ double red[16];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < count; i += 1024) acc += (double)partials[i];
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < 16; ++i) t += red[i];
        const float norm = (float)sqrt(t);
        float coef = 1.0f;
        if (max_norm > 0.f) {
            const float c = max_norm / (norm + 1e-6f);
            if (c < 1.0f) coef = c;
        }
        out[0] = norm;
        out[1] = coef;
    }
}

struct AdamArgs {
    float lr, beta1, beta2, eps, weight_decay, inv_bc1, inv_bc2;
};

__device__ __forceinline__ void adam_one(float& p, float& m, float& v, float g, const AdamArgs& a) {
    m = a.beta1 * m + (1.0f - a.beta1) * g;
    v = a.beta2 * v + (1.0f - a.beta2) * g * g;
    const float denom = sqrtf(v * a.inv_bc2) + a.eps;
    const float update = (m * a.inv_bc1) / denom + a.weight_decay * p;
    p = p - a.lr * update;
}

__global__ __launch_bounds__(kOptBlock) void adamw_kernel(float* __restrict__ master, float* __restrict__ exp_avg,
                                                         float* __restrict__ exp_avg_sq, const float* __restrict__ grad,
                                                         bf16_t* __restrict__ param, int64_t n, AdamArgs a,
                                                         const float* __restrict__ norm_coef) {
    const float coef = norm_coef ? norm_coef[1] : 1.0f;
    const int64_t n4 = n >> 2;
    const int64_t stride = (int64_t)gridDim.x * kOptBlock;
    auto update = [&](int64_t i, f32x4 p, f32x4 m, f32x4 v, const f32x4 g) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float pk = p[k], mk = m[k], vk = v[k];
            adam_one(pk, mk, vk, g[k] * coef, a);
            p[k] = pk; m[k] = mk; v[k] = vk;
        }
        reinterpret_cast<f32x4*>(master)[i] = p;
        reinterpret_cast<f32x4*>(exp_avg)[i] = m;
        reinterpret_cast<f32x4*>(exp_avg_sq)[i] = v;
        if (param) {
            bf16x4 o;
#pragma unroll
            for (int k = 0; k < 4; ++k) o[k] = (bf16_t)p[k];
            reinterpret_cast<bf16x4*>(param)[i] = o;
        }
    };
    int64_t i = (int64_t)blockIdx.x * kOptBlock + threadIdx.x;
    for (; i + stride < n4; i += 2 * stride) {  // two vectors of every stream in flight per thread
        const int64_t j = i + stride;
        const f32x4 p0 = reinterpret_cast<f32x4*>(master)[i], p1 = reinterpret_cast<f32x4*>(master)[j];
        const f32x4 m0 = reinterpret_cast<f32x4*>(exp_avg)[i], m1 = reinterpret_cast<f32x4*>(exp_avg)[j];
        const f32x4 v0 = reinterpret_cast<f32x4*>(exp_avg_sq)[i], v1 = reinterpret_cast<f32x4*>(exp_avg_sq)[j];
        const f32x4 g0 = reinterpret_cast<const f32x4*>(grad)[i], g1 = reinterpret_cast<const f32x4*>(grad)[j];
        update(i, p0, m0, v0, g0);
        update(j, p1, m1, v1, g1);
    }
    if (i < n4)
        update(i, reinterpret_cast<f32x4*>(master)[i], reinterpret_cast<f32x4*>(exp_avg)[i], reinterpret_cast<f32x4*>(exp_avg_sq)[i],
               reinterpret_cast<const f32x4*>(grad)[i]);
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = (n4 << 2) + threadIdx.x;
        float p = master[i], m = exp_avg[i], v = exp_avg_sq[i];
        adam_one(p, m, v, grad[i] * coef, a);
        master[i] = p;
        exp_avg[i] = m;
        exp_avg_sq[i] = v;
        if (param) param[i] = (bf16_t)p;
    }
}

inline unsigned opt_grid(int64_t n4, int64_t cap) {
    int64_t g = (n4 + kOptBlock - 1) / kOptBlock;
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return (unsigned)g;
}

}  // namespace

extern "C" int64_t ezl_sumsq_partials(void) { return kSumsqPartials; }

extern "C" int ezl_sumsq_f32(const void* x, int64_t n, void* partials, void* stream) {
    EZL_REQUIRE(n >= 0 && partials && (n == 0 || x), EZL_EINVAL, "ezl_sumsq_f32: null pointer");
    EZL_REQUIRE(ezl_aligned16(x), EZL_EINVAL, "ezl_sumsq_f32: x must be 16-byte aligned");
    // always kSumsqPartials blocks, so every slot of `partials` is written (zeros for blocks without work)
    hipLaunchKernelGGL(sumsq_partial_kernel, dim3(kSumsqPartials), dim3(kSumsqBlock), 0, (hipStream_t)stream, (const float*)x, n,
                       (float*)partials);
    EZL_LAUNCH_CHECK("ezl_sumsq_f32");
    return EZL_OK;
}

extern "C" int ezl_clip_coef(const void* partials, int64_t count, float max_norm, void* norm_coef_out, void* stream) {
    EZL_REQUIRE(count >= 0 && norm_coef_out && (count == 0 || partials), EZL_EINVAL, "ezl_clip_coef: null pointer");
    hipLaunchKernelGGL(clip_coef_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const float*)partials, count, max_norm,
                       (float*)norm_coef_out);
    EZL_LAUNCH_CHECK("ezl_clip_coef");
    return EZL_OK;
}

extern "C" int ezl_adamw_step(void* master, void* exp_avg, void* exp_avg_sq, const void* grad, void* param_bf16, int64_t n,
                              float lr, float beta1, float beta2, float eps, float weight_decay, int64_t step,
                              int bias_correction, const void* norm_coef, void* stream) {
    EZL_REQUIRE(n >= 0 && (n == 0 || (master && exp_avg && exp_avg_sq && grad)), EZL_EINVAL, "ezl_adamw_step: null pointer");
    EZL_REQUIRE(step >= 1, EZL_EINVAL, "ezl_adamw_step: step counts from 1");
    EZL_REQUIRE(ezl_aligned16(master) && ezl_aligned16(exp_avg) && ezl_aligned16(exp_avg_sq) && ezl_aligned16(grad) &&
                    (((uintptr_t)param_bf16 & 7) == 0),
                EZL_EINVAL, "ezl_adamw_step: fp32 buffers must be 16-byte aligned, the bf16 weight 8-byte aligned");
    if (n == 0) return EZL_OK;
    AdamArgs a;
    a.lr = lr; a.beta1 = beta1; a.beta2 = beta2; a.eps = eps; a.weight_decay = weight_decay;
    a.inv_bc1 = bias_correction ? (float)(1.0 / (1.0 - pow((double)beta1, (double)step))) : 1.0f;
    a.inv_bc2 = bias_correction ? (float)(1.0 / (1.0 - pow((double)beta2, (double)step))) : 1.0f;
    hipLaunchKernelGGL(adamw_kernel, dim3(opt_grid(n >> 2, 256 * 16)), dim3(kOptBlock), 0, (hipStream_t)stream, (float*)master,
                       (float*)exp_avg, (float*)exp_avg_sq, (const float*)grad, (bf16_t*)param_bf16, n, a, (const float*)norm_coef);
    EZL_LAUNCH_CHECK("ezl_adamw_step");
    return EZL_OK;
}
