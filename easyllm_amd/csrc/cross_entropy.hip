// Vocab-parallel cross entropy at TP=1 for gfx950 (HBM-bound).
//
// Restates base_modules/functions/cross_entropy.py:24-112 and llama/losses.py:20-56 of the
// reference without its fp32 [T, V] copy and ~10 passes:
//   * ezl_ce_prepare      weights w = loss_mask * (label != -100) and N = sum(w)      (losses.py:21-23,45)
//   * ezl_ce_fwd          per-token loss + logsumexp                                  (cross_entropy.py:24-89)
//   * ezl_ce_bwd          (softmax - onehot[valid]) * grad_out                        (cross_entropy.py:91-112)
//   * ezl_ce_fused        loss rows AND d loss / d logits in one visit of the logits, for the
//                         mean-reduced loss: grad = (softmax - onehot) * w / N
//   * ezl_ce_reduce       loss = sum(loss_row * w) / N                                (losses.py:55)
// A row of logits (bf16 or fp32) is owned by one 512-thread block.  When the row fits 64 KiB of
// LDS it is staged there during the max pass, so HBM sees one read and (for bwd/fused) one write.
// Integer semantics are exact: a label outside [0, V - cut) is "masked": pred = 0, no one-hot.
#include "common.h"

namespace {

constexpr int kCeBlock = 512;
constexpr int kCeWaves = kCeBlock / 64;
constexpr float kLog2e = 1.4426950408889634f;

template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float* f) { unpack8(ld_bf16x8(p), f); }
    static __device__ __forceinline__ void store(bf16_t* p, const float* f) { st_bf16x8(p, pack8(f)); }
};
template <> struct Vec8<float> {
    static __device__ __forceinline__ void load(const float* p, float* f) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
        f[0] = a[0]; f[1] = a[1]; f[2] = a[2]; f[3] = a[3]; f[4] = b[0]; f[5] = b[1]; f[6] = b[2]; f[7] = b[3];
    }
    static __device__ __forceinline__ void store(float* p, const float* f) {
        f32x4 a = {f[0], f[1], f[2], f[3]}, b = {f[4], f[5], f[6], f[7]};
        *reinterpret_cast<f32x4*>(p) = a;
        *reinterpret_cast<f32x4*>(p + 4) = b;
    }
};

__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    __syncthreads();  // red may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int i = 1; i < kCeWaves; ++i) r = fmaxf(r, red[i]);
    return r;
}
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < kCeWaves; ++i) r += red[i];
    return r;
}

// Max and sum(exp(x - max)) over columns [0, vend) of one row; optionally stages the row in LDS.
template <typename T, bool IN_LDS>
__device__ __forceinline__ void row_max_sumexp(const T* __restrict__ xrow, T* __restrict__ srow, int V, int vend, float* red,
                                               float& m_out, float& s_out) {
    const int v8 = V >> 3;
    float m = -INFINITY;
    for (int i = threadIdx.x; i < v8; i += kCeBlock) {
        float f[8];
        Vec8<T>::load(xrow + i * 8, f);
        if (IN_LDS) Vec8<T>::store(srow + i * 8, f);
        if (i * 8 + 8 <= vend) {  // whole vector inside [0, vend): no per-element compare
#pragma unroll
            for (int k = 0; k < 8; ++k) m = fmaxf(m, f[k]);
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (i * 8 + k < vend) m = fmaxf(m, f[k]);
        }
    }
    m = block_max(m, red);  // barriers inside also publish the staged row
    float s = 0.f;
    const float mb = m * kLog2e;
    for (int i = threadIdx.x; i < v8; i += kCeBlock) {
        float f[8];
        Vec8<T>::load((IN_LDS ? (const T*)srow : xrow) + i * 8, f);
        // the argument is never positive, so the bare instruction (no range fix-up) is exact enough: results below
        // 2^-126 may flush to zero
        if (i * 8 + 8 <= vend) {
#pragma unroll
            for (int k = 0; k < 8; ++k) s += __builtin_amdgcn_exp2f(f[k] * kLog2e - mb);
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (i * 8 + k < vend) s += __builtin_amdgcn_exp2f(f[k] * kLog2e - mb);
        }
    }
    s = block_sum(s, red);
    m_out = m;
    s_out = s;
}

// grad[c] = (exp(x[c] - lse) - [c == target]) * scale   for every column (cut columns included)
template <typename T, bool IN_LDS>
__device__ __forceinline__ void row_write_grad(const T* __restrict__ xrow, const T* __restrict__ srow, T* __restrict__ grow,
                                               int V, float lse, int target, float scale) {
    const int v8 = V >> 3;
    const float lb = lse * kLog2e;
    for (int i = threadIdx.x; i < v8; i += kCeBlock) {
        float f[8];
        Vec8<T>::load((IN_LDS ? srow : xrow) + i * 8, f);
        // columns past vend (cut_size) may exceed the row maximum, so this exp can overflow to +inf exactly as the
        // reference's does; the bare instruction handles that range too
#pragma unroll
        for (int k = 0; k < 8; ++k) f[k] = __builtin_amdgcn_exp2f(f[k] * kLog2e - lb);
        if ((target >> 3) == i) {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if ((target & 7) == k) f[k] -= 1.0f;
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) f[k] *= scale;
        Vec8<T>::store(grow + i * 8, f);
    }
}

template <typename T>
__device__ __forceinline__ void row_write_zero(T* __restrict__ grow, int V) {
    float z[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = threadIdx.x; i < (V >> 3); i += kCeBlock) Vec8<T>::store(grow + i * 8, z);
}

template <typename T, bool IN_LDS>
__global__ __launch_bounds__(kCeBlock) void ce_fwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                          float* __restrict__ loss, float* __restrict__ lse_out, int64_t rows,
                                                          int V, int vend) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    __shared__ float red[kCeWaves];
    T* srow = reinterpret_cast<T*>(smem_raw);
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const T* xrow = logits + r * V;
        float m, s;
        row_max_sumexp<T, IN_LDS>(xrow, srow, V, vend, red, m, s);
        if (threadIdx.x == 0) {
            const int64_t t = labels[r];
            const bool masked = t < 0 || t >= vend;
            const float pred = masked ? 0.f : ((float)xrow[t] - m);  // cross_entropy.py:58-65 (shifted logit)
            loss[r] = logf(s) - pred;                                // :83
            lse_out[r] = m + logf(s);
        }
        __syncthreads();  // the staged row is overwritten by the next iteration
    }
}

template <typename T>
__global__ __launch_bounds__(kCeBlock) void ce_bwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                          const float* __restrict__ lse, const float* __restrict__ grad_out,
                                                          T* __restrict__ grad, int64_t rows, int V, int vend) {
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const int64_t t = labels[r];
        const int target = (t < 0 || t >= vend) ? -1 : (int)t;
        row_write_grad<T, false>(logits + r * V, nullptr, grad + r * V, V, lse[r], target, grad_out[r]);
    }
}

template <typename T, bool IN_LDS>
__global__ __launch_bounds__(kCeBlock) void ce_fused_kernel(const T* __restrict__ logits, const int64_t* __restrict__ labels,
                                                            const float* __restrict__ weights, const float* __restrict__ count,
                                                            float* __restrict__ loss, T* __restrict__ grad, int64_t rows, int V,
                                                            int vend) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    __shared__ float red[kCeWaves];
    T* srow = reinterpret_cast<T*>(smem_raw);
    const float inv_n = 1.0f / count[0];
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const float w = weights[r];
        T* grow = grad + r * V;
        if (w == 0.f) {  // ignored position: exact zero gradient, contributes nothing to the loss
            row_write_zero<T>(grow, V);
            if (threadIdx.x == 0) loss[r] = 0.f;
            continue;
        }
        const T* xrow = logits + r * V;
        const int64_t t = labels[r];
        const bool masked = t < 0 || t >= vend;
        // read the target logit before the row is overwritten in place
        const float xt = masked ? 0.f : (float)xrow[t];
        float m, s;
        row_max_sumexp<T, IN_LDS>(xrow, srow, V, vend, red, m, s);
        const float lse = m + logf(s);
        if (threadIdx.x == 0) loss[r] = masked ? logf(s) : (lse - xt);
        row_write_grad<T, IN_LDS>(xrow, srow, grow, V, lse, masked ? -1 : (int)t, w * inv_n);
        __syncthreads();
    }
}

// Fused loss + gradient for bf16 rows of up to 512 * 8 * NCH columns, held in registers: the kernel is bound by vector
// ALU work as much as by HBM (a transcendental costs four issue slots), so exp(x - max) is computed once per element with
// the bare v_exp_f32 (its argument is never positive; anything below 2^-126 may flush to zero) and kept in fp32 registers
// for the gradient, vectors past the row end are filled with -inf instead of being branched around, and the raw
// vectors of the block's next row are fetched while the current row is worked on.  HAS_CUT: columns [vend, V) are
// excluded from max and sum but still receive their softmax gradient (reference semantics of cut_size).
template <int NCH, bool HAS_CUT>
__global__ __launch_bounds__(kCeBlock) void ce_fused_reg_kernel(const bf16_t* __restrict__ logits, const int64_t* __restrict__ labels,
                                                                const float* __restrict__ weights, const float* __restrict__ count,
                                                                float* __restrict__ loss, bf16_t* __restrict__ grad, int64_t rows,
                                                                int V, int vend) {
    __shared__ float red[kCeWaves];
    const int v8 = V >> 3;
    const float inv_n = 1.0f / count[0];
    bf16x8 nxt[NCH];
    auto fetch = [&](int64_t r) {
        const bf16_t* src = logits + r * V;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int i = threadIdx.x + j * kCeBlock;
            if (i < v8) {
                nxt[j] = ld_bf16x8(src + i * 8);
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) nxt[j][k] = (bf16_t)(-INFINITY);
            }
        }
    };
    int64_t r = blockIdx.x;
    if (r < rows) fetch(r);
    for (; r < rows; r += gridDim.x) {
        const float w = weights[r];
        bf16_t* grow = grad + r * V;
        const int64_t t = labels[r];
        const bool masked = t < 0 || t >= vend;
        const int tvec = masked ? -1 : (int)(t >> 3), tsub = (int)(t & 7);
        float e[NCH][8];
        float m = -INFINITY, xt = 0.f;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int i = threadIdx.x + j * kCeBlock;
            unpack8(nxt[j], e[j]);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if (!HAS_CUT || i * 8 + k < vend) m = fmaxf(m, e[j][k]);
            }
            if (i == tvec) {  // exactly one thread holds the target logit
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (tsub == k) xt = e[j][k];
            }
        }
        if (r + gridDim.x < rows) fetch(r + gridDim.x);
        if (w == 0.f) {  // ignored position: exact zero gradient, contributes nothing to the loss
            row_write_zero<bf16_t>(grow, V);
            if (threadIdx.x == 0) loss[r] = 0.f;
            continue;
        }
        m = block_max(m, red);
        const float mb = m * kLog2e;
        float ssum = 0.f;
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int i = threadIdx.x + j * kCeBlock;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                e[j][k] = __builtin_amdgcn_exp2f(e[j][k] * kLog2e - mb);
                if (!HAS_CUT || i * 8 + k < vend) ssum += e[j][k];
            }
        }
        ssum = block_sum(ssum, red);
        xt = block_sum(xt, red);  // every other thread contributes 0
        const float lse = m + logf(ssum);
        if (threadIdx.x == 0) loss[r] = masked ? logf(ssum) : (lse - xt);
        const float scale = w * inv_n;
        const float ps = scale / ssum;  // exp(x - lse) * scale = e * scale / sum
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
            const int i = threadIdx.x + j * kCeBlock;
            float g[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) g[k] = e[j][k] * ps;
            if (i == tvec) {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (tsub == k) g[k] -= scale;
            }
            if (i < v8) st_bf16x8(grow + i * 8, pack8(g));
        }
    }
}

// Fused loss + gradient for bf16 rows too long for the kernel above (a 152064-entry vocabulary): one 1024-thread block per
// CU owns a row and keeps it RAW (bf16) on chip, so the logits are read from HBM exactly once and the gradient is written
// once.  The first 9 x 1024 vectors of 8 logits live in LDS (144 KiB, thread t owns vector t of every 1024: private
// slots, no barriers), the remaining NR x 1024 in registers.  exp is evaluated twice per element (sum pass, gradient
// pass): fp32 copies would not fit.  While the gradient pass runs, each finished vector's slot is refilled with the
// block's next row -- registers by a plain load, LDS slots by a buffer load straight to LDS, which needs no registers at
// all -- so the HBM pipe is busy under the vector ALU work.  Vectors past the row end hold -inf (exp = 0) and are never
// stored.  For the refills to stay in flight while later slots are read, the LDS reads must not wait for them: the kernel
// has a single LDS array (the reduction cells sit behind the row) and reads it through a __restrict__ pointer, which keeps
// the reads' no-alias tag (with a second LDS variable the compiler re-tags every access and each read then waits for all
// loads in flight, vmcnt(0)); and the loads are buffer loads, because a global load to LDS in flight turns every counted
// wait on LDS reads into a full drain.
constexpr int kWideBlock = 1024;
constexpr int kWideWaves = kWideBlock / 64;
constexpr int kWideLds = 9;  // vectors per thread kept in LDS

typedef __attribute__((address_space(3))) void ce_lds_void;

__device__ __forceinline__ bf16x8 ce_lds_vec(const bf16_t* __restrict__ row, int i) { return *reinterpret_cast<const bf16x8*>(row + i * 8); }

template <int NR, bool HAS_CUT>
__global__ __launch_bounds__(kWideBlock) void ce_fused_wide_kernel(const bf16_t* __restrict__ logits, const int64_t* __restrict__ labels,
                                                                   const float* __restrict__ weights, const float* __restrict__ count,
                                                                   float* __restrict__ loss, bf16_t* __restrict__ grad, int64_t rows,
                                                                   int V, int vend) {
    __shared__ __attribute__((aligned(16))) bf16_t srow[kWideLds * kWideBlock * 8 + 4 * kWideWaves];  // the row, then red[2][waves]
    float* red = reinterpret_cast<float*>(srow + kWideLds * kWideBlock * 8);
    const int v8 = V >> 3;  // >= kWideLds * kWideBlock (checked by the host): every LDS vector lies inside the row
    const float inv_n = 1.0f / count[0];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    bf16x8 raw[NR > 0 ? NR : 1];
    auto fetch_reg = [&](const bf16_t* src, int j) {  // register vector j = row vector (kWideLds + j) * 1024 + tid
        const int i = tid + (kWideLds + j) * kWideBlock;
        if (i < v8) {
            raw[j] = ld_bf16x8_nt(src + (int64_t)i * 8);
        } else {
#pragma unroll
            for (int k = 0; k < 8; ++k) raw[j][k] = (bf16_t)(-INFINITY);
        }
    };
    auto fetch_lds = [&](const bf16_t* src, int j) {  // one wave instruction fills the 64 slots of this wave in chunk j
        const __amdgpu_buffer_rsrc_t g = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(src), 0, 0xffffffffu, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(g, (ce_lds_void*)(srow + (j * kWideBlock + wv * 64) * 8), 16, tid * 16,
                                                 j * kWideBlock * 16, 0, 0);
    };
    auto lds_vec = [&](int j) { return ce_lds_vec(srow, tid + j * kWideBlock); };

    int64_t r = blockIdx.x;
    if (r < rows) {
        const bf16_t* src = logits + r * V;
#pragma unroll
        for (int j = 0; j < kWideLds; ++j) fetch_lds(src, j);
#pragma unroll
        for (int j = 0; j < NR; ++j) fetch_reg(src, j);
    }
    for (; r < rows; r += gridDim.x) {
        const float w = weights[r];
        bf16_t* grow = grad + r * V;
        const int64_t rn = r + gridDim.x;
        const bf16_t* next = logits + (rn < rows ? rn : r) * V;  // a block's last row re-reads itself (never used)
        if (w == 0.f) {  // ignored position: exact zero gradient, contributes nothing to the loss
            bf16x8 z;
#pragma unroll
            for (int k = 0; k < 8; ++k) z[k] = (bf16_t)0.0f;
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this row's own loads into LDS have landed before they are replaced
#pragma unroll
            for (int j = 0; j < kWideLds; ++j) {
                st_bf16x8(grow + (int64_t)(tid + j * kWideBlock) * 8, z);
                fetch_lds(next, j);
            }
#pragma unroll
            for (int j = 0; j < NR; ++j) {
                const int i = tid + (kWideLds + j) * kWideBlock;
                if (i < v8) st_bf16x8(grow + (int64_t)i * 8, z);
                fetch_reg(next, j);
            }
            if (tid == 0) loss[r] = 0.f;
            continue;
        }
        const int64_t t = labels[r];
        const bool masked = t < 0 || t >= vend;
        // the target logit straight from memory (the row is being read anyway): the first two passes stay free of target tests
        const float xt = masked ? 0.f : (float)logits[r * V + t];
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the row is on chip (LDS part included)
        asm volatile("" ::: "memory");           // ... and the compiler may not reuse LDS values read before this point
        // ---- pass 1: row maximum over the columns below vend
        float m = -INFINITY;
        auto max_of = [&](const bf16x8 v, int i) {
            float f[8];
            unpack8(v, f);
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (!HAS_CUT || i * 8 + k < vend) m = fmaxf(m, f[k]);
        };
#pragma unroll
        for (int j = 0; j < kWideLds; ++j) max_of(lds_vec(j), tid + j * kWideBlock);
#pragma unroll
        for (int j = 0; j < NR; ++j) max_of(raw[j], tid + (kWideLds + j) * kWideBlock);
        m = wave_max(m);
        __syncthreads();  // red is free again (read by every thread at the end of the previous row)
        if (lane == 0) red[wv] = m;
        __syncthreads();
        m = red[0];
#pragma unroll
        for (int i = 1; i < kWideWaves; ++i) m = fmaxf(m, red[i]);
        const float mb = m * kLog2e;
        // ---- pass 2: sum of exp(x - max) over the columns below vend
        float ssum = 0.f;
        auto sum_of = [&](const bf16x8 v, int i) {
            float f[8];
            unpack8(v, f);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float e = __builtin_amdgcn_exp2f(f[k] * kLog2e - mb);
                if (!HAS_CUT || i * 8 + k < vend) ssum += e;
            }
        };
#pragma unroll
        for (int j = 0; j < kWideLds; ++j) sum_of(lds_vec(j), tid + j * kWideBlock);
#pragma unroll
        for (int j = 0; j < NR; ++j) {
            asm volatile("" : "+v"(raw[j]));  // opaque: the fp32 copies of pass 1 must not be kept alive
            sum_of(raw[j], tid + (kWideLds + j) * kWideBlock);
        }
        ssum = wave_sum(ssum);
        if (lane == 0) red[kWideWaves + wv] = ssum;
        __syncthreads();
        ssum = 0.f;
#pragma unroll
        for (int i = 0; i < kWideWaves; ++i) ssum += red[kWideWaves + i];
        const float lse = m + logf(ssum);
        if (tid == 0) loss[r] = masked ? logf(ssum) : (lse - xt);
        const float scale = w * inv_n;
        const float ps = scale / ssum;  // exp(x - lse) * scale = exp(x - max) * scale / sum
        // ---- pass 3: gradient; the exponentials are evaluated again on purpose.  The copy of `mb` is opaque to the
        // compiler, which would otherwise recognise the expression of pass 2, keep all of that pass's results alive across
        // the block reduction and spill them.
        float mb2 = mb;
        asm volatile("" : "+v"(mb2));
        // one-hot term: the vector that holds the target column belongs to chunk tj (uniform over the block: a scalar test
        // per chunk), and inside it to thread towner, element tsub
        const int tj = masked ? -1 : (int)(t >> 3) / kWideBlock, towner = (int)(t >> 3) % kWideBlock, tsub = (int)(t & 7);
        auto grad_of = [&](const bf16x8 v, bool holds_target) {
            float g[8];
            unpack8(v, g);
#pragma unroll
            for (int k = 0; k < 8; ++k) g[k] = __builtin_amdgcn_exp2f(g[k] * kLog2e - mb2) * ps;
            if (holds_target) {
#pragma unroll
                for (int k = 0; k < 8; ++k) g[k] -= (k == tsub && tid == towner) ? scale : 0.f;
            }
            return pack8(g);
        };
#pragma unroll
        for (int j = 0; j < kWideLds; ++j) {
            const int i = tid + j * kWideBlock;
            st_bf16x8_nt(grow + (int64_t)i * 8, grad_of(lds_vec(j), j == tj));
            // the LDS read above has returned (its value was used): the slot may be refilled with the next row
            fetch_lds(next, j);
        }
#pragma unroll
        for (int j = 0; j < NR; ++j) {
            const int i = tid + (kWideLds + j) * kWideBlock;
            asm volatile("" : "+v"(raw[j]));
            const bf16x8 gv = grad_of(raw[j], kWideLds + j == tj);
            if (i < v8) st_bf16x8_nt(grow + (int64_t)i * 8, gv);
            fetch_reg(next, j);  // this vector's registers are free: start the next row's fetch behind the store
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // no LDS write of this block may still be in flight when it ends
}

// weights[i] = mask[i] * (labels[i] != ignore_index); count[0] = sum(weights) -- one block, fixed order
__global__ __launch_bounds__(1024) void ce_prepare_kernel(const int64_t* __restrict__ labels, const void* __restrict__ mask,
                                                          int mask_dtype, int64_t ignore_index, float* __restrict__ weights,
                                                          float* __restrict__ count, int64_t n) {
    __shared__ float red[16];
    float acc = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        float mv = 1.0f;
        if (mask_dtype == 1) mv = reinterpret_cast<const float*>(mask)[i];
        else if (mask_dtype == 2) mv = reinterpret_cast<const unsigned char*>(mask)[i] ? 1.0f : 0.0f;
        else if (mask_dtype == 3) mv = (float)reinterpret_cast<const int64_t*>(mask)[i];
        else if (mask_dtype == 4) mv = (float)reinterpret_cast<const bf16_t*>(mask)[i];
        const float w = labels[i] != ignore_index ? mv : 0.0f;
        weights[i] = w;
        acc += w;
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int i = 0; i < 16; ++i) t += red[i];
        count[0] = t;
    }
}

// out[0] = sum(loss[i] * weights[i]) / count[0]
__global__ __launch_bounds__(1024) void ce_reduce_kernel(const float* __restrict__ loss, const float* __restrict__ weights,
                                                         const float* __restrict__ count, float* __restrict__ out, int64_t n) {
    __shared__ float red[16];
    float acc = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 1024) acc += loss[i] * weights[i];
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = 0.f;
        for (int i = 0; i < 16; ++i) t += red[i];
        out[0] = t / count[0];
    }
}

// x[i] *= s[0] unless s[0] == 1 (the usual case for loss.backward(): nothing is touched)
template <typename T>
__global__ __launch_bounds__(256) void scale_by_scalar_kernel(T* __restrict__ x, const float* __restrict__ s, int64_t n8) {
    const float sc = s[0];
    if (sc == 1.0f) return;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
        float f[8];
        Vec8<T>::load(x + i * 8, f);
#pragma unroll
        for (int k = 0; k < 8; ++k) f[k] *= sc;
        Vec8<T>::store(x + i * 8, f);
    }
}

int ce_check(const char* name, const void* logits, int64_t rows, int64_t V, int64_t cut, int dtype) {
    EZL_REQUIRE(dtype == 0 || dtype == 1, EZL_EUNSUPPORTED, "%s: dtype must be 0 (bf16) or 1 (fp32)", name);
    EZL_REQUIRE(rows >= 0 && V > 0 && V % 8 == 0 && V < (1LL << 31), EZL_EUNSUPPORTED, "%s: vocab must be a multiple of 8", name);
    EZL_REQUIRE(cut >= 0 && cut < V, EZL_EINVAL, "%s: bad cut_size", name);
    EZL_REQUIRE(rows == 0 || logits, EZL_EINVAL, "%s: null logits", name);
    EZL_REQUIRE(ezl_aligned16(logits), EZL_EINVAL, "%s: logits must be 16-byte aligned", name);
    return EZL_OK;
}

inline unsigned ce_grid(int64_t rows) { return (unsigned)(rows < 256 * 8 ? (rows < 1 ? 1 : rows) : 256 * 8); }

}  // namespace

extern "C" int ezl_ce_prepare(const void* labels, const void* loss_mask, int mask_dtype, int64_t ignore_index, void* weights,
                              void* count, int64_t n, void* stream) {
    EZL_REQUIRE(n >= 0 && count && (n == 0 || (labels && weights)), EZL_EINVAL, "ezl_ce_prepare: null pointer");
    EZL_REQUIRE(mask_dtype >= 0 && mask_dtype <= 4 && (mask_dtype == 0 || loss_mask), EZL_EINVAL, "ezl_ce_prepare: bad loss_mask");
    hipLaunchKernelGGL(ce_prepare_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const int64_t*)labels, loss_mask,
                       mask_dtype, ignore_index, (float*)weights, (float*)count, n);
    EZL_LAUNCH_CHECK("ezl_ce_prepare");
    return EZL_OK;
}

extern "C" int ezl_ce_fwd(const void* logits, const void* labels, void* loss, void* lse, int64_t rows, int64_t vocab,
                          int64_t cut_size, int dtype, void* stream) {
    int rc = ce_check("ezl_ce_fwd", logits, rows, vocab, cut_size, dtype);
    if (rc) return rc;
    EZL_REQUIRE(rows == 0 || (labels && loss && lse), EZL_EINVAL, "ezl_ce_fwd: null pointer");
    if (rows == 0) return EZL_OK;
    const int V = (int)vocab, vend = (int)(vocab - cut_size);
    const size_t row_bytes = (size_t)V * (dtype == 0 ? 2 : 4);
    const bool in_lds = row_bytes <= 65536;
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(TT, L)                                                                                                  \
    hipLaunchKernelGGL((ce_fwd_kernel<TT, L>), dim3(ce_grid(rows)), dim3(kCeBlock), (L) ? row_bytes : 0, st, (const TT*)logits, \
                       (const int64_t*)labels, (float*)loss, (float*)lse, rows, V, vend)
    if (dtype == 0) { if (in_lds) LAUNCH(bf16_t, true); else LAUNCH(bf16_t, false); }
    else { if (in_lds) LAUNCH(float, true); else LAUNCH(float, false); }
#undef LAUNCH
    EZL_LAUNCH_CHECK("ezl_ce_fwd");
    return EZL_OK;
}

extern "C" int ezl_ce_bwd(const void* logits, const void* labels, const void* lse, const void* grad_out, void* grad,
                          int64_t rows, int64_t vocab, int64_t cut_size, int dtype, void* stream) {
    int rc = ce_check("ezl_ce_bwd", logits, rows, vocab, cut_size, dtype);
    if (rc) return rc;
    EZL_REQUIRE(rows == 0 || (labels && lse && grad_out && grad), EZL_EINVAL, "ezl_ce_bwd: null pointer");
    EZL_REQUIRE(ezl_aligned16(grad), EZL_EINVAL, "ezl_ce_bwd: grad must be 16-byte aligned");
    if (rows == 0) return EZL_OK;
    const int V = (int)vocab, vend = (int)(vocab - cut_size);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == 0)
        hipLaunchKernelGGL((ce_bwd_kernel<bf16_t>), dim3(ce_grid(rows)), dim3(kCeBlock), 0, st, (const bf16_t*)logits,
                           (const int64_t*)labels, (const float*)lse, (const float*)grad_out, (bf16_t*)grad, rows, V, vend);
    else
        hipLaunchKernelGGL((ce_bwd_kernel<float>), dim3(ce_grid(rows)), dim3(kCeBlock), 0, st, (const float*)logits,
                           (const int64_t*)labels, (const float*)lse, (const float*)grad_out, (float*)grad, rows, V, vend);
    EZL_LAUNCH_CHECK("ezl_ce_bwd");
    return EZL_OK;
}

extern "C" int ezl_ce_fused(const void* logits, const void* labels, const void* weights, const void* count, void* loss_rows,
                            void* grad, int64_t rows, int64_t vocab, int64_t cut_size, int dtype, void* stream) {
    int rc = ce_check("ezl_ce_fused", logits, rows, vocab, cut_size, dtype);
    if (rc) return rc;
    EZL_REQUIRE(rows == 0 || (labels && weights && count && loss_rows && grad), EZL_EINVAL, "ezl_ce_fused: null pointer");
    EZL_REQUIRE(ezl_aligned16(grad), EZL_EINVAL, "ezl_ce_fused: grad must be 16-byte aligned");
    if (rows == 0) return EZL_OK;
    const int V = (int)vocab, vend = (int)(vocab - cut_size);
    const size_t row_bytes = (size_t)V * (dtype == 0 ? 2 : 4);
    const bool in_lds = row_bytes <= 65536;
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(KERNEL, TT, SMEM)                                                                                         \
    hipLaunchKernelGGL((KERNEL), dim3(ce_grid(rows)), dim3(kCeBlock), SMEM, st, (const TT*)logits, (const int64_t*)labels, \
                       (const float*)weights, (const float*)count, (float*)loss_rows, (TT*)grad, rows, V, vend)
    if (dtype == 0) {
        const bool cut = vend != V;
        if (V <= kCeBlock * 8 * 2) { if (cut) LAUNCH((ce_fused_reg_kernel<2, true>), bf16_t, 0); else LAUNCH((ce_fused_reg_kernel<2, false>), bf16_t, 0); }
        else if (V <= kCeBlock * 8 * 4) { if (cut) LAUNCH((ce_fused_reg_kernel<4, true>), bf16_t, 0); else LAUNCH((ce_fused_reg_kernel<4, false>), bf16_t, 0); }
        else if (V <= kCeBlock * 8 * 8) { if (cut) LAUNCH((ce_fused_reg_kernel<8, true>), bf16_t, 0); else LAUNCH((ce_fused_reg_kernel<8, false>), bf16_t, 0); }
        else if (V >= kWideBlock * 8 * kWideLds && V <= kWideBlock * 8 * (kWideLds + 13)) {
            // one block per CU (1024 threads, 144 KiB of LDS); every block walks rows blockIdx.x, + gridDim.x, ...
            const unsigned g = (unsigned)(rows < 256 ? rows : 256);
#define LAUNCH_WIDE(NR)                                                                                                       \
    do {                                                                                                                      \
        if (cut) hipLaunchKernelGGL((ce_fused_wide_kernel<NR, true>), dim3(g), dim3(kWideBlock), 0, st, (const bf16_t*)logits, \
                                    (const int64_t*)labels, (const float*)weights, (const float*)count, (float*)loss_rows,    \
                                    (bf16_t*)grad, rows, V, vend);                                                            \
        else hipLaunchKernelGGL((ce_fused_wide_kernel<NR, false>), dim3(g), dim3(kWideBlock), 0, st, (const bf16_t*)logits,    \
                                (const int64_t*)labels, (const float*)weights, (const float*)count, (float*)loss_rows,        \
                                (bf16_t*)grad, rows, V, vend);                                                                \
    } while (0)
            if (V <= kWideBlock * 8 * (kWideLds + 4)) LAUNCH_WIDE(4);
            else if (V <= kWideBlock * 8 * (kWideLds + 7)) LAUNCH_WIDE(7);
            else if (V <= kWideBlock * 8 * (kWideLds + 10)) LAUNCH_WIDE(10);
            else LAUNCH_WIDE(13);
#undef LAUNCH_WIDE
        } else LAUNCH((ce_fused_kernel<bf16_t, false>), bf16_t, 0);
    } else {
        if (in_lds) LAUNCH((ce_fused_kernel<float, true>), float, row_bytes); else LAUNCH((ce_fused_kernel<float, false>), float, 0);
    }
#undef LAUNCH
    EZL_LAUNCH_CHECK("ezl_ce_fused");
    return EZL_OK;
}

extern "C" int ezl_ce_reduce(const void* loss_rows, const void* weights, const void* count, void* loss_out, int64_t n,
                             void* stream) {
    EZL_REQUIRE(n >= 0 && count && loss_out && (n == 0 || (loss_rows && weights)), EZL_EINVAL, "ezl_ce_reduce: null pointer");
    hipLaunchKernelGGL(ce_reduce_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const float*)loss_rows,
                       (const float*)weights, (const float*)count, (float*)loss_out, n);
    EZL_LAUNCH_CHECK("ezl_ce_reduce");
    return EZL_OK;
}

extern "C" int ezl_scale_by_scalar(void* x, const void* scalar_f32, int64_t n, int dtype, void* stream) {
    EZL_REQUIRE(dtype == 0 || dtype == 1, EZL_EUNSUPPORTED, "ezl_scale_by_scalar: dtype must be 0 (bf16) or 1 (fp32)");
    EZL_REQUIRE(n >= 0 && n % 8 == 0 && (n == 0 || (x && scalar_f32)) && ezl_aligned16(x), EZL_EINVAL,
                "ezl_scale_by_scalar: bad argument");
    if (n == 0) return EZL_OK;
    int64_t g = (n / 8 + 255) / 256;
    if (g > 256 * 16) g = 256 * 16;
    if (dtype == 0)
        hipLaunchKernelGGL((scale_by_scalar_kernel<bf16_t>), dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, (bf16_t*)x,
                           (const float*)scalar_f32, n / 8);
    else
        hipLaunchKernelGGL((scale_by_scalar_kernel<float>), dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, (float*)x,
                           (const float*)scalar_f32, n / 8);
    EZL_LAUNCH_CHECK("ezl_scale_by_scalar");
    return EZL_OK;
}
