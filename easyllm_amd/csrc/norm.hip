// RMSNorm forward / backward for gfx950 (HBM-bound).
//
// Restates base_modules/layers/fused_layer_norm.py:49-71 of the reference (the fp32-accumulate
// form its fused path uses): y = x * rsqrt(mean(x^2) + eps) * w, with the optional residual add
// of llama/transformer.py:786 fused in front (sum rounded to bf16 first, as the reference's bf16
// tensor add does).
//
// Layout: rows of h bf16, h % 8 == 0.  Up to h = 8192 a row is held in registers (read from HBM exactly once): forward by
// TPR = min(256, h/8 rounded up to a wave) threads whose row sums meet through a double-buffered LDS cell; backward by one
// wave (h <= 2048), two waves (h <= 4096) or four (wider rows).  Rows up to 32768 wide go through two-pass kernels.
#include "common.h"

#include <mutex>

namespace {

template <int NCHUNK, bool HAS_RES>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ res,
                                                          const bf16_t* __restrict__ w, bf16_t* __restrict__ y,
                                                          bf16_t* __restrict__ sum_out, float* __restrict__ rstd_out,
                                                          int T, int h, float eps, int tpr) {
    __shared__ float red[2][4][4];  // [parity][row slot][wave in slot]
    const int rpb = 256 / tpr;             // row slots per block
    const int slot = threadIdx.x / tpr;    // which row slot
    const int tin = threadIdx.x % tpr;     // thread within the row
    const int wis = tin >> 6;              // wave within the slot
    const int nws = tpr >> 6;              // waves per slot
    const int lane = threadIdx.x & 63;
    float wv[NCHUNK][8];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
        const int col = (c * tpr + tin) * 8;
        if (col < h) unpack8(ld_bf16x8(w + col), wv[c]);
    }
    int parity = 0;
    // every thread of the block runs the same number of iterations (barrier inside)
    for (int row0 = blockIdx.x * rpb; row0 < T; row0 += gridDim.x * rpb) {
        const int row = row0 + slot;
        const bool live = row < T;
        const size_t base = (size_t)row * h;
        float xv[NCHUNK][8];
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int col = (c * tpr + tin) * 8;
            if (live && col < h) {
                unpack8(ld_bf16x8(x + base + col), xv[c]);
                if (HAS_RES) {
                    float r[8];
                    unpack8(ld_bf16x8(res + base + col), r);
#pragma unroll
                    for (int i = 0; i < 8; ++i) xv[c][i] = (float)(bf16_t)(xv[c][i] + r[i]);
                    st_bf16x8(sum_out + base + col, pack8(xv[c]));
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) ss += xv[c][i] * xv[c][i];
            }
        }
        ss = wave_sum(ss);
        if (nws > 1) {
            if (lane == 0) red[parity][slot][wis] = ss;
            __syncthreads();
            ss = 0.f;
            for (int i = 0; i < nws; ++i) ss += red[parity][slot][i];
            parity ^= 1;
        }
        const float rs = rsqrtf(ss / (float)h + eps);
        if (live && tin == 0) rstd_out[row] = rs;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int col = (c * tpr + tin) * 8;
            if (live && col < h) {
                float o[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = xv[c][i] * rs * wv[c][i];
                st_bf16x8(y + base + col, pack8(o));
            }
        }
    }
}

// Backward: dx = rstd * (g - xhat * mean(g * xhat)),  g = dy * w, xhat = x * rstd;  dw = sum_rows dy * xhat.
// ---- backward with one wave per row (h <= 2048) ----------------------------------------------------------------
// A row is owned by ONE wave: lane l holds the 8 columns (c * 64 + l) * 8 .. + 7 of chunk c, so every chunk is one
// coalesced 1 KiB access, the row sums need wave shuffles only and there is no barrier inside the row loop: the waves
// of a CU run out of step and keep HBM busy while others compute.  Loads and stores carry the streaming hint (in the
// step: 42 -> 34 us); the forward kernel keeps the block-per-row form and plain accesses, which measured faster there
// (its input was written by the kernel before it and its output is read by the one after, 33 MB each).
// Backward, 8 waves per block: each wave keeps the dw partial of its lanes' columns over all rows it visits; at the end the
// 8 waves of a block are folded through LDS in a fixed order and one partial row per block goes to HBM.
template <int NCHUNK, bool HAS_DRES>
__global__ __launch_bounds__(512) void rmsnorm_bwd_wave_kernel(const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x,
                                                               const bf16_t* __restrict__ w, const float* __restrict__ rstd,
                                                               const bf16_t* __restrict__ dres, bf16_t* __restrict__ dx,
                                                               float* __restrict__ dw_partial, int T, int h) {
    extern __shared__ float fold[];  // h floats
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    bf16x8 wr[NCHUNK];
    float dwacc[NCHUNK][8];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
        const int col = (c * 64 + lane) * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) { dwacc[c][i] = 0.f; wr[c][i] = (bf16_t)0.0f; }
        if (col < h) wr[c] = ld_bf16x8(w + col);
    }
    const float inv_h = 1.0f / (float)h;
    for (int row = blockIdx.x * 8 + wave; row < T; row += gridDim.x * 8) {
        const size_t base = (size_t)row * h;
        const float rs = rstd[row];
        bf16x8 xr[NCHUNK], dyr[NCHUNK], drr[NCHUNK];
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int col = (c * 64 + lane) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) { xr[c][i] = (bf16_t)0.0f; dyr[c][i] = (bf16_t)0.0f; }
            if (col < h) {
                xr[c] = ld_bf16x8_nt(x + base + col);
                dyr[c] = ld_bf16x8_nt(dy + base + col);
                if (HAS_DRES) drr[c] = ld_bf16x8_nt(dres + base + col);
            }
        }
        float dot = 0.f;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) dot += (float)dyr[c][i] * (float)wr[c][i] * ((float)xr[c][i] * rs);
        dot = wave_sum(dot);
        const float cmean = dot * inv_h;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const int col = (c * 64 + lane) * 8;
            // opaque to the compiler: the fp32 copies made for the dot product must not be kept alive (they would not fit)
            asm volatile("" : "+v"(xr[c]), "+v"(dyr[c]));
            if (col < h) {
                float o[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float xhat = (float)xr[c][i] * rs;
                    const float dyv = (float)dyr[c][i];
                    o[i] = rs * (dyv * (float)wr[c][i] - xhat * cmean);
                    if (HAS_DRES) o[i] += (float)drr[c][i];
                    dwacc[c][i] += dyv * xhat;
                }
                st_bf16x8_nt(dx + base + col, pack8(o));
            }
        }
    }
    for (int s = 0; s < 8; ++s) {  // wave 0 stores, the others add in turn: a fixed order
        if (wave == s) {
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c) {
                const int col = (c * 64 + lane) * 8;
                if (col < h) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        if (s == 0) fold[col + i] = dwacc[c][i];
                        else fold[col + i] += dwacc[c][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    for (int j = threadIdx.x; j < h; j += 512) dw_partial[(size_t)blockIdx.x * h + j] = fold[j];
}

// ---- backward with two or four waves per row (2048 < h <= 8192) ---------------------------------------------------
// The same scheme with a row shared by NSPLIT (2 or 4) waves: wave part p owns NCHUNK * 512 columns from p * NCHUNK * 512
// on, so the per-lane state (operands, weight, dw partials) is that of a row of 1/NSPLIT of the width, stays in registers
// and leaves room for a second set of operand registers: the loads of a wave's next row are issued before the current row
// is worked on, so HBM requests are in flight all the time.  (With one row per wave and nothing prefetched a wave loads,
// waits, computes and stores in turn, and at T = h = 4096 each wave sees only two rows: 45 us for backward + column sum
// against 29 us with the prefetch.)  The partial sums of a row meet in an LDS cell (double buffered by iteration parity:
// one barrier per row).  A block is 4 waves = 4 / NSPLIT rows per pass, two blocks per CU.
template <int NCHUNK, int NSPLIT, bool HAS_DRES>
__global__ __launch_bounds__(256, 2) void rmsnorm_bwd_split_kernel(const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x,
                                                                   const bf16_t* __restrict__ w, const float* __restrict__ rstd,
                                                                   const bf16_t* __restrict__ dres, bf16_t* __restrict__ dx,
                                                                   float* __restrict__ dw_partial, int T, int h) {
    constexpr int RPB = 4 / NSPLIT;  // rows per block pass
    extern __shared__ float fold[];  // h floats
    __shared__ float cell[2][RPB][NSPLIT];  // [parity][row slot][part]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform values stay in scalar registers
    const int slot = wave / NSPLIT, part = wave % NSPLIT;
    const int col0 = (part * NCHUNK * 64 + lane) * 8;  // this lane's first column; chunk c is 512 c further
    bf16x8 wr[NCHUNK];
    float dwacc[NCHUNK][8];
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) {
        const int col = col0 + c * 512;
#pragma unroll
        for (int i = 0; i < 8; ++i) { dwacc[c][i] = 0.f; wr[c][i] = (bf16_t)0.0f; }
        if (col < h) wr[c] = ld_bf16x8(w + col);
    }
    const float inv_h = 1.0f / (float)h;
    int parity = 0;
    bf16x8 nxr[NCHUNK], ndyr[NCHUNK], ndrr[NCHUNK];
    float nrs = 0.f;
    auto fetch = [&](int row) {  // the operands of this wave's share of `row` into the next-row registers
        const bool live = row < T;
        nrs = live ? rstd[row] : 0.f;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
#pragma unroll
            for (int i = 0; i < 8; ++i) { nxr[c][i] = (bf16_t)0.0f; ndyr[c][i] = (bf16_t)0.0f; }
            if (live && col0 + c * 512 < h) {
                nxr[c] = ld_bf16x8_nt(x + (size_t)row * h + col0 + c * 512);
                ndyr[c] = ld_bf16x8_nt(dy + (size_t)row * h + col0 + c * 512);
                if (HAS_DRES) ndrr[c] = ld_bf16x8_nt(dres + (size_t)row * h + col0 + c * 512);
            }
        }
    };
    fetch(blockIdx.x * RPB + slot);
    // every wave of the block runs the same number of iterations (barrier inside)
    for (int row0 = blockIdx.x * RPB; row0 < T; row0 += gridDim.x * RPB) {
        const int row = row0 + slot;
        const bool live = row < T;
        bf16x8 xr[NCHUNK], dyr[NCHUNK], drr[NCHUNK];
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            xr[c] = nxr[c];
            dyr[c] = ndyr[c];
            if (HAS_DRES) drr[c] = ndrr[c];
        }
        const float rs = nrs;
        if (row0 + (int)gridDim.x * RPB < T) fetch(row + gridDim.x * RPB);
        float dot = 0.f;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
#pragma unroll
            for (int i = 0; i < 8; ++i) dot += (float)dyr[c][i] * (float)wr[c][i] * ((float)xr[c][i] * rs);
        dot = wave_sum(dot);
        if (lane == 0) cell[parity][slot][part] = dot;
        __syncthreads();
        float rowdot = cell[parity][slot][0];  // same order in every wave of the row
#pragma unroll
        for (int q = 1; q < NSPLIT; ++q) rowdot += cell[parity][slot][q];
        const float cmean = rowdot * inv_h;
        parity ^= 1;
        bf16_t* dxrow = dx + (size_t)row * h + col0;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            asm volatile("" : "+v"(xr[c]), "+v"(dyr[c]));  // do not keep the fp32 copies of the dot product alive
            if (live && col0 + c * 512 < h) {
                float o[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float xhat = (float)xr[c][i] * rs;
                    const float dyv = (float)dyr[c][i];
                    o[i] = rs * (dyv * (float)wr[c][i] - xhat * cmean);
                    if (HAS_DRES) o[i] += (float)drr[c][i];
                    dwacc[c][i] += dyv * xhat;
                }
                st_bf16x8_nt(dxrow + c * 512, pack8(o));
            }
        }
    }
    for (int s2 = 0; s2 < RPB; ++s2) {  // row slot 0 stores, the next adds: a fixed order
        if (slot == s2) {
#pragma unroll
            for (int c = 0; c < NCHUNK; ++c) {
                const int col = col0 + c * 512;
                if (col < h) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        if (s2 == 0) fold[col + i] = dwacc[c][i];
                        else fold[col + i] += dwacc[c][i];
                    }
                }
            }
        }
        __syncthreads();
    }
    for (int j = threadIdx.x; j < h; j += 256) dw_partial[(size_t)blockIdx.x * h + j] = fold[j];
}

// ---- rows wider than 8192 (up to kWideMaxH) --------------------------------------------------------------------------
// The reference leaves such rows to its unfused path (fused_layer_norm.py:56, :68-71).  Here a block of 1024 threads walks a
// row twice -- once for the row statistic, once to produce the output (the second read comes from cache) -- so nothing
// depends on the row fitting into registers.  Backward keeps the dw column sums of the block's rows in LDS, every thread
// adding only to its own columns (no atomics, fixed order), and writes one partial row per block.
constexpr int kWideMaxH = 32768;
constexpr int kWideThreads = 1024;

__device__ __forceinline__ float block_sum_1024(float v, float (*red)[kWideThreads / 64], int& parity) {
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[parity][threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kWideThreads / 64; ++i) t += red[parity][i];
    parity ^= 1;  // the next sum uses the other set of cells: one barrier per sum
    return t;
}

template <bool HAS_RES>
__global__ __launch_bounds__(kWideThreads) void rmsnorm_fwd_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ res,
                                                                        const bf16_t* __restrict__ w, bf16_t* __restrict__ y,
                                                                        bf16_t* __restrict__ sum_out, float* __restrict__ rstd_out,
                                                                        int T, int h, float eps) {
    __shared__ float red[2][kWideThreads / 64];
    const int h8 = h >> 3;
    int parity = 0;
    for (int row = blockIdx.x; row < T; row += gridDim.x) {
        const size_t base = (size_t)row * h;
        float ss = 0.f;
        for (int c = threadIdx.x; c < h8; c += kWideThreads) {
            float v[8];
            unpack8(ld_bf16x8(x + base + c * 8), v);
            if (HAS_RES) {
                float r[8];
                unpack8(ld_bf16x8(res + base + c * 8), r);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (float)(bf16_t)(v[i] + r[i]);
                st_bf16x8(sum_out + base + c * 8, pack8(v));
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
        }
        ss = block_sum_1024(ss, red, parity);
        const float rs = rsqrtf(ss / (float)h + eps);
        if (threadIdx.x == 0) rstd_out[row] = rs;
        for (int c = threadIdx.x; c < h8; c += kWideThreads) {
            float v[8], wv[8], o[8];
            unpack8(ld_bf16x8(x + base + c * 8), v);
            if (HAS_RES) {  // recomputed rather than read back from sum_out
                float r[8];
                unpack8(ld_bf16x8(res + base + c * 8), r);
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = (float)(bf16_t)(v[i] + r[i]);
            }
            unpack8(ld_bf16x8(w + c * 8), wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = v[i] * rs * wv[i];
            st_bf16x8(y + base + c * 8, pack8(o));
        }
    }
}

template <bool HAS_DRES>
__global__ __launch_bounds__(kWideThreads) void rmsnorm_bwd_wide_kernel(const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x,
                                                                        const bf16_t* __restrict__ w, const float* __restrict__ rstd,
                                                                        const bf16_t* __restrict__ dres, bf16_t* __restrict__ dx,
                                                                        float* __restrict__ dw_partial, int T, int h) {
    __shared__ float fold[kWideMaxH];  // dw sums over this block's rows; thread t owns columns 8 (c * 1024 + t) .. + 7
    __shared__ float red[2][kWideThreads / 64];
    const int h8 = h >> 3;
    for (int c = threadIdx.x; c < h8; c += kWideThreads)
#pragma unroll
        for (int i = 0; i < 8; ++i) fold[c * 8 + i] = 0.f;
    int parity = 0;
    const float inv_h = 1.0f / (float)h;
    for (int row = blockIdx.x; row < T; row += gridDim.x) {
        const size_t base = (size_t)row * h;
        const float rs = rstd[row];
        float dot = 0.f;
        for (int c = threadIdx.x; c < h8; c += kWideThreads) {
            float xv[8], dyv[8], wv[8];
            unpack8(ld_bf16x8(x + base + c * 8), xv);
            unpack8(ld_bf16x8(dy + base + c * 8), dyv);
            unpack8(ld_bf16x8(w + c * 8), wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) dot += dyv[i] * wv[i] * (xv[i] * rs);
        }
        const float cmean = block_sum_1024(dot, red, parity) * inv_h;
        for (int c = threadIdx.x; c < h8; c += kWideThreads) {
            float xv[8], dyv[8], wv[8], o[8];
            unpack8(ld_bf16x8(x + base + c * 8), xv);
            unpack8(ld_bf16x8(dy + base + c * 8), dyv);
            unpack8(ld_bf16x8(w + c * 8), wv);
            if (HAS_DRES) unpack8(ld_bf16x8(dres + base + c * 8), o);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float xhat = xv[i] * rs;
                const float g = rs * (dyv[i] * wv[i] - xhat * cmean);
                o[i] = HAS_DRES ? o[i] + g : g;
                fold[c * 8 + i] += dyv[i] * xhat;
            }
            st_bf16x8(dx + base + c * 8, pack8(o));
        }
    }
    for (int c = threadIdx.x; c < h8; c += kWideThreads)
#pragma unroll
        for (int i = 0; i < 8; ++i) dw_partial[(size_t)blockIdx.x * h + c * 8 + i] = fold[c * 8 + i];
}

int tpr_for(int h) {
    int t = (h / 8 + 63) / 64 * 64;
    return t < 64 ? 64 : (t > 256 ? 256 : t);
}

}  // namespace

extern "C" int ezl_rmsnorm_fwd(const void* x, const void* residual, const void* weight, void* y, void* sum_out,
                               void* rstd, int64_t rows, int64_t h, float eps, void* stream) {
    EZL_REQUIRE(rows >= 0 && h > 0 && h % 8 == 0 && h <= kWideMaxH, EZL_EUNSUPPORTED,
                "ezl_rmsnorm_fwd: need h %% 8 == 0 and h <= %d (got h=%lld)", kWideMaxH, (long long)h);
    EZL_REQUIRE(rows == 0 || (x && weight && y && rstd), EZL_EINVAL, "ezl_rmsnorm_fwd: null pointer");
    EZL_REQUIRE((residual == nullptr) == (sum_out == nullptr), EZL_EINVAL,
                "ezl_rmsnorm_fwd: residual and sum_out go together");
    EZL_REQUIRE(ezl_aligned16(x) && ezl_aligned16(weight) && ezl_aligned16(y) && ezl_aligned16(residual) &&
                    ezl_aligned16(sum_out),
                EZL_EINVAL, "ezl_rmsnorm_fwd: pointers must be 16-byte aligned");
    if (rows == 0) return EZL_OK;
    hipStream_t st = (hipStream_t)stream;
    EZL_REQUIRE(rows < (1LL << 31), EZL_EUNSUPPORTED, "ezl_rmsnorm_fwd: too many rows");
    if (h > 8192) {
        const unsigned g = (unsigned)(rows < 512 ? rows : 512);
        if (residual)
            hipLaunchKernelGGL(rmsnorm_fwd_wide_kernel<true>, dim3(g), dim3(kWideThreads), 0, st, (const bf16_t*)x, (const bf16_t*)residual,
                               (const bf16_t*)weight, (bf16_t*)y, (bf16_t*)sum_out, (float*)rstd, (int)rows, (int)h, eps);
        else
            hipLaunchKernelGGL(rmsnorm_fwd_wide_kernel<false>, dim3(g), dim3(kWideThreads), 0, st, (const bf16_t*)x, (const bf16_t*)residual,
                               (const bf16_t*)weight, (bf16_t*)y, (bf16_t*)sum_out, (float*)rstd, (int)rows, (int)h, eps);
        EZL_LAUNCH_CHECK("ezl_rmsnorm_fwd");
        return EZL_OK;
    }
    const int tpr = tpr_for((int)h);
    const int nchunk = ((int)h + tpr * 8 - 1) / (tpr * 8);
    const int rpb = 256 / tpr;
    int64_t grid = (rows + rpb - 1) / rpb;
    if (grid > 256 * 16) grid = 256 * 16;
#define LAUNCH(NC, RES)                                                                                             \
    hipLaunchKernelGGL((rmsnorm_fwd_kernel<NC, RES>), dim3((unsigned)grid), dim3(256), 0, st, (const bf16_t*)x,      \
                       (const bf16_t*)residual, (const bf16_t*)weight, (bf16_t*)y, (bf16_t*)sum_out, (float*)rstd, \
                       (int)rows, (int)h, eps, tpr)
    if (residual) {
        if (nchunk == 1) LAUNCH(1, true); else if (nchunk == 2) LAUNCH(2, true); else LAUNCH(4, true);
    } else {
        if (nchunk == 1) LAUNCH(1, false); else if (nchunk == 2) LAUNCH(2, false); else LAUNCH(4, false);
    }
#undef LAUNCH
    EZL_LAUNCH_CHECK("ezl_rmsnorm_fwd");
    return EZL_OK;
}

namespace {
// blocks (= fp32 partial rows of h) the backward kernels want: 8 waves per CU in both forms
int64_t rmsnorm_bwd_blocks(int64_t h) { return h <= 4096 ? 256 : (h <= 8192 ? 512 : 256); }
}  // namespace

extern "C" int64_t ezl_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t h) {
    (void)rows;
    return rmsnorm_bwd_blocks(h) * h * (int64_t)sizeof(float);
}

namespace {

int rmsnorm_bwd_check(const char* name, const void* dy, const void* x, const void* weight, const void* rstd, const void* dresidual,
                      const void* dx, const void* dw_bf16, const void* dw_f32, int64_t rows, int64_t h) {
    EZL_REQUIRE(rows >= 0 && h > 0 && h % 8 == 0 && h <= kWideMaxH, EZL_EUNSUPPORTED, "%s: need h %% 8 == 0 and h <= %d (got h=%lld)",
                name, kWideMaxH, (long long)h);
    EZL_REQUIRE(weight && (rows == 0 || (dy && x && rstd && dx)), EZL_EINVAL, "%s: null pointer", name);
    EZL_REQUIRE((dw_bf16 != nullptr) != (dw_f32 != nullptr), EZL_EINVAL, "%s: exactly one of dw_bf16 / dw_f32", name);
    EZL_REQUIRE(ezl_aligned16(dy) && ezl_aligned16(x) && ezl_aligned16(weight) && ezl_aligned16(dx) && ezl_aligned16(dresidual),
                EZL_EINVAL, "%s: pointers must be 16-byte aligned", name);
    EZL_REQUIRE(rows < (1LL << 31), EZL_EUNSUPPORTED, "%s: too many rows", name);
    return EZL_OK;
}

// both entry points: `partials` holds one fp32 row of h per block (at most max_blocks blocks; the narrow-row kernel uses up
// to 256, the wide-row one up to 512), every used row fully written
int rmsnorm_bwd_launch(const void* dy, const void* x, const void* weight, const void* rstd, const void* dresidual, void* dx,
                       void* dw_bf16, void* dw_f32, int accumulate, float* partials, int64_t max_blocks, int64_t rows, int64_t h,
                       hipStream_t st) {
    const size_t smem = (size_t)h * sizeof(float);
    int64_t grid;
#define LAUNCH_SPLIT(NC, NS, DR)                                                                                           \
    hipLaunchKernelGGL((rmsnorm_bwd_split_kernel<NC, NS, DR>), dim3((unsigned)grid), dim3(256), smem, st, (const bf16_t*)dy, \
                       (const bf16_t*)x, (const bf16_t*)weight, (const float*)rstd, (const bf16_t*)dresidual, (bf16_t*)dx,  \
                       partials, (int)rows, (int)h)
    if (h <= 2048) {  // one wave per row, 8 rows per block
        const int nchunk = ((int)h + 511) / 512;
        grid = (rows + 7) / 8;
        if (grid > max_blocks) grid = max_blocks;
        if (grid < 1) grid = 1;  // rows == 0 still produces a zero dw
#define LAUNCH(NC, DR)                                                                                                    \
    hipLaunchKernelGGL((rmsnorm_bwd_wave_kernel<NC, DR>), dim3((unsigned)grid), dim3(512), smem, st, (const bf16_t*)dy,    \
                       (const bf16_t*)x, (const bf16_t*)weight, (const float*)rstd, (const bf16_t*)dresidual, (bf16_t*)dx, \
                       partials, (int)rows, (int)h)
#define LAUNCH_NC(DR)                                  \
    do {                                               \
        if (nchunk <= 1) LAUNCH(1, DR);                \
        else if (nchunk <= 2) LAUNCH(2, DR);           \
        else LAUNCH(4, DR);                            \
    } while (0)
        if (dresidual) LAUNCH_NC(true); else LAUNCH_NC(false);
#undef LAUNCH_NC
#undef LAUNCH
    } else if (h <= 4096) {  // two waves per row (3 or 4 chunks of 512 columns each), 2 rows per block pass
        grid = (rows + 1) / 2;
        if (grid > max_blocks) grid = max_blocks;
        if (grid < 1) grid = 1;
        if (h <= 3072) { if (dresidual) LAUNCH_SPLIT(3, 2, true); else LAUNCH_SPLIT(3, 2, false); }
        else { if (dresidual) LAUNCH_SPLIT(4, 2, true); else LAUNCH_SPLIT(4, 2, false); }
    } else if (h <= 8192) {  // four waves per row, one row per block pass
        grid = rows < max_blocks ? rows : max_blocks;
        if (grid < 1) grid = 1;
        if (h <= 6144) { if (dresidual) LAUNCH_SPLIT(3, 4, true); else LAUNCH_SPLIT(3, 4, false); }
        else { if (dresidual) LAUNCH_SPLIT(4, 4, true); else LAUNCH_SPLIT(4, 4, false); }
    } else {  // rows that do not fit into registers: two passes per row, dw sums in LDS
        grid = rows < max_blocks ? rows : max_blocks;
        if (grid < 1) grid = 1;
        if (dresidual)
            hipLaunchKernelGGL(rmsnorm_bwd_wide_kernel<true>, dim3((unsigned)grid), dim3(kWideThreads), 0, st, (const bf16_t*)dy, (const bf16_t*)x,
                               (const bf16_t*)weight, (const float*)rstd, (const bf16_t*)dresidual, (bf16_t*)dx, partials, (int)rows, (int)h);
        else
            hipLaunchKernelGGL(rmsnorm_bwd_wide_kernel<false>, dim3((unsigned)grid), dim3(kWideThreads), 0, st, (const bf16_t*)dy, (const bf16_t*)x,
                               (const bf16_t*)weight, (const float*)rstd, (const bf16_t*)dresidual, (bf16_t*)dx, partials, (int)rows, (int)h);
    }
#undef LAUNCH_SPLIT
    EZL_LAUNCH_CHECK("ezl_rmsnorm_bwd");
    hipLaunchKernelGGL(ezl_colsum_kernel<0>, dim3((unsigned)((h + 63) / 64)), dim3(kColsumThreads), 0, st, (const float*)partials,
                       (int)grid, (int)h, (bf16_t*)dw_bf16, (float*)dw_f32, accumulate);
    EZL_LAUNCH_CHECK("ezl_rmsnorm_bwd(colsum)");
    return EZL_OK;
}

}  // namespace

extern "C" int ezl_rmsnorm_bwd(const void* dy, const void* x, const void* weight, const void* rstd,
                               const void* dresidual, void* dx, void* dw_bf16, void* dw_f32, int accumulate,
                               void* workspace, int64_t workspace_bytes, int64_t rows, int64_t h, void* stream) {
    if (const int rc = rmsnorm_bwd_check("ezl_rmsnorm_bwd", dy, x, weight, rstd, dresidual, dx, dw_bf16, dw_f32, rows, h)) return rc;
    EZL_REQUIRE(workspace && workspace_bytes >= ezl_rmsnorm_bwd_workspace_bytes(rows, h), EZL_EINVAL,
                "ezl_rmsnorm_bwd: workspace missing or too small");
    return rmsnorm_bwd_launch(dy, x, weight, rstd, dresidual, dx, dw_bf16, dw_f32, accumulate, (float*)workspace,
                              rmsnorm_bwd_blocks(h), rows, h, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------------------------------
// ezl_rmsnorm_bwd without a workspace argument, for callers that cannot obtain device memory (code under HIP graph
// capture, serving loops, harnesses that forbid allocation): the per-block dw partials live in a file-scope device array
// of the largest size the kernels can need (512 blocks x h <= 8192 floats = 16 MiB), held by every GPU the library runs on
// until the process ends.  All calls on one GPU share that array: calls that overlap on one GPU (different streams or
// host threads) race on it.  Nothing in it needs clearing: every row of partials that is read has been written by the
// same call.
namespace {

constexpr int kScratchBlocks = 512, kScratchMaxH = 8192;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) float scratch[kScratchBlocks * kScratchMaxH];

// The array's name is only a host-side handle; its device address differs per GPU and is looked up once per device,
// with that device current.
float* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int scratch_for_current_device(float** out, hipStream_t stream) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    EZL_REQUIRE(e == hipSuccess && dev >= 0 && dev < kMaxDevices, EZL_EHIP, "ezl_rmsnorm_bwd_noalloc: cannot identify the current device (%s)",
                hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        // The lookup is a runtime call that may load the code object: not something to do while the stream records a graph.
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &cap);
        EZL_REQUIRE(e == hipSuccess && cap == hipStreamCaptureStatusNone, EZL_EINVAL,
                    "ezl_rmsnorm_bwd_noalloc: the first call on a device must not be made under stream capture (call it once before)");
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        EZL_REQUIRE(e == hipSuccess && p, EZL_EHIP, "ezl_rmsnorm_bwd_noalloc: hipGetSymbolAddress failed (%s)", hipGetErrorString(e));
        g_scratch_ptr[dev] = static_cast<float*>(p);
    }
    *out = g_scratch_ptr[dev];
    return EZL_OK;
}

}  // namespace

extern "C" int64_t ezl_rmsnorm_bwd_noalloc_max_h(void) { return kScratchMaxH; }

extern "C" int ezl_rmsnorm_bwd_noalloc(const void* dy, const void* x, const void* weight, const void* rstd, const void* dresidual,
                                       void* dx, void* dw_bf16, void* dw_f32, int accumulate, int64_t rows, int64_t h, void* stream) {
    EZL_REQUIRE(h <= kScratchMaxH, EZL_EUNSUPPORTED, "ezl_rmsnorm_bwd_noalloc: h = %lld exceeds the built-in scratch (h <= %d)",
                (long long)h, kScratchMaxH);
    if (const int rc = rmsnorm_bwd_check("ezl_rmsnorm_bwd_noalloc", dy, x, weight, rstd, dresidual, dx, dw_bf16, dw_f32, rows, h)) return rc;
    const int64_t blocks = rmsnorm_bwd_blocks(h);  // as in ezl_rmsnorm_bwd, so that both give the same bits
    static_assert(kScratchBlocks >= 512, "the scratch holds the partial rows of the widest launch");
    float* partials = nullptr;
    if (const int rc = scratch_for_current_device(&partials, (hipStream_t)stream)) return rc;
    return rmsnorm_bwd_launch(dy, x, weight, rstd, dresidual, dx, dw_bf16, dw_f32, accumulate, partials, blocks, rows, h, (hipStream_t)stream);
}
