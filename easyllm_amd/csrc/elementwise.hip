// HBM-bound elementwise / gather kernels of the llama decoder-layer step (gfx950):
// SwiGLU, rotary embedding, token-embedding gather / scatter-add, [b,s,h] <-> [s,b,h] row moves,
// bf16 add and bf16 <-> fp32 casts.  All use 128-bit accesses (8 bf16 per lane).
#include "common.h"

namespace {

constexpr int kBlock = 256;

inline unsigned grid_for(int64_t items, int per_block, int64_t cap = 256 * 32) {
    int64_t g = (items + per_block - 1) / per_block;
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return (unsigned)g;
}

// 1 / (1 + 2^(-x log2 e)) with the bare exp2 / rcp instructions (1 ulp each); saturates correctly at both ends
__device__ __forceinline__ float sigmoidf_fast(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// ---------------------------------------------------------------------------------------------
// SwiGLU: out = silu(gate) * up     (llama/transformer.py:220-222, glu_activations.py:56-61)
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void swiglu_fwd_kernel(const bf16_t* __restrict__ gate, const bf16_t* __restrict__ up,
                                                            bf16_t* __restrict__ out, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += (int64_t)gridDim.x * kBlock) {
        float g[8], u[8], o[8];
        unpack8(ld_bf16x8_nt(gate + i * 8), g);
        unpack8(ld_bf16x8_nt(up + i * 8), u);
#pragma unroll
        for (int k = 0; k < 8; ++k) o[k] = g[k] * sigmoidf_fast(g[k]) * u[k];
        st_bf16x8_nt(out + i * 8, pack8(o));
    }
}

// dgate = dout * up * s * (1 + g * (1 - s)),  dup = dout * g * s,  s = sigmoid(g)
__global__ __launch_bounds__(kBlock) void swiglu_bwd_kernel(const bf16_t* __restrict__ dout, const bf16_t* __restrict__ gate,
                                                            const bf16_t* __restrict__ up, bf16_t* __restrict__ dgate,
                                                            bf16_t* __restrict__ dup, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += (int64_t)gridDim.x * kBlock) {
        float g[8], u[8], d[8], dg[8], du[8];
        unpack8(ld_bf16x8_nt(gate + i * 8), g);
        unpack8(ld_bf16x8_nt(up + i * 8), u);
        unpack8(ld_bf16x8_nt(dout + i * 8), d);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float s = sigmoidf_fast(g[k]);
            dg[k] = d[k] * u[k] * s * (1.0f + g[k] * (1.0f - s));
            du[k] = d[k] * g[k] * s;
        }
        st_bf16x8_nt(dgate + i * 8, pack8(dg));
        st_bf16x8_nt(dup + i * 8, pack8(du));
    }
}

// ---------------------------------------------------------------------------------------------
// Rotary embedding (llama/positional_embeddings.py:17-36, 94-96, 105-122)
// ---------------------------------------------------------------------------------------------
// cos/sin table [npos, d/2] in fp32: theta = (p / scale_factor) * inv_freq[j]  (:21-23)
__global__ __launch_bounds__(kBlock) void rope_table_kernel(const float* __restrict__ inv_freq, float* __restrict__ cosb,
                                                            float* __restrict__ sinb, int64_t npos, int half,
                                                            float scale_factor) {
    const int64_t n = npos * half;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
        const int64_t p = i / half;
        const int j = (int)(i % half);
        const float t = (float)p / scale_factor;
        const float th = t * inv_freq[j];
        cosb[i] = cosf(th);
        sinb[i] = sinf(th);
    }
}

// x [rows = s*b (s-major), nheads, d] with a row stride; one work item = 8 low-half + 8 high-half
// elements of one head.  out1 = x1*c - sign*x2*s ; out2 = x2*c + sign*x1*s  (sign = -1: backward).
// Two tensors that share their rows (q and k of one layer: nheads0 + nheads1 heads per row) go through one launch; the
// second is absent when nheads1 == 0.
struct RopeSide {
    const bf16_t* x;
    bf16_t* out;
    int64_t in_stride, out_stride;
};

__global__ __launch_bounds__(kBlock) void rope_kernel(RopeSide a, RopeSide b2, const float* __restrict__ cosb,
                                                      const float* __restrict__ sinb, const int64_t* __restrict__ position_ids,
                                                      int64_t rows, int s, int b, int nheads0, int nheads1, int d, int64_t npos,
                                                      float sign) {
    const int half = d >> 1;
    const int per_head = half >> 3;
    const int nheads = nheads0 + nheads1;
    const int64_t items = rows * nheads * per_head;
    for (int64_t it = (int64_t)blockIdx.x * kBlock + threadIdx.x; it < items; it += (int64_t)gridDim.x * kBlock) {
        const int j8 = (int)(it % per_head);
        const int64_t rh = it / per_head;
        int head = (int)(rh % nheads);
        const int64_t row = rh / nheads;
        const int si = (int)(row / b), bi = (int)(row % b);
        int64_t pos = position_ids ? position_ids[(int64_t)bi * s + si] : si;
        pos = pos < 0 ? 0 : (pos >= npos ? npos - 1 : pos);
        const float* cp = cosb + pos * half + j8 * 8;
        const float* sp = sinb + pos * half + j8 * 8;
        const bool second = head >= nheads0;
        head -= second ? nheads0 : 0;
        const bf16_t* xi = (second ? b2.x : a.x) + row * (second ? b2.in_stride : a.in_stride) + (int64_t)head * d + j8 * 8;
        bf16_t* xo = (second ? b2.out : a.out) + row * (second ? b2.out_stride : a.out_stride) + (int64_t)head * d + j8 * 8;
        float av[8], c[8], o1[8], o2[8];
        unpack8(ld_bf16x8(xi), av);
        unpack8(ld_bf16x8(xi + half), c);
        const f32x4 c0 = *reinterpret_cast<const f32x4*>(cp), c1 = *reinterpret_cast<const f32x4*>(cp + 4);
        const f32x4 s0 = *reinterpret_cast<const f32x4*>(sp), s1 = *reinterpret_cast<const f32x4*>(sp + 4);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float cs = k < 4 ? c0[k] : c1[k - 4];
            const float sn = sign * (k < 4 ? s0[k] : s1[k - 4]);
            o1[k] = av[k] * cs - c[k] * sn;
            o2[k] = c[k] * cs + av[k] * sn;
        }
        st_bf16x8(xo, pack8(o1));
        st_bf16x8(xo + half, pack8(o2));
    }
}

// ---------------------------------------------------------------------------------------------
// Token embedding (base_modules/layers/vocab_parallel_emb.py:106-137, TP=1)
// ---------------------------------------------------------------------------------------------
// ORs 1 into *bad_flag if some id >= limit, 2 if some id < 0 (the range test of an index tensor, without a host sync)
__global__ __launch_bounds__(kBlock) void ids_in_range_kernel(const int64_t* __restrict__ ids, int64_t n, int64_t limit,
                                                              int* __restrict__ bad_flag) {
    int bad = 0;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
        const int64_t id = ids[i];
        bad |= id >= limit ? 1 : (id < 0 ? 2 : 0);
    }
    if (bad) atomicOr(bad_flag, bad);
}

// out[r, :] = W[ids[r], :]; an id outside [0, V) raises the flag and yields a zero row.
// One wave per row; a lane's loads (up to 8 vectors of 8 at a time: a row of 4096 in one go) are all in flight before its
// first store.
__global__ __launch_bounds__(kBlock) void embed_gather_kernel(const int64_t* __restrict__ ids, const bf16_t* __restrict__ W,
                                                              bf16_t* __restrict__ out, int64_t rows, int h, int64_t V,
                                                              int* __restrict__ bad_flag) {
    const int h8 = h >> 3;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int64_t r = (int64_t)blockIdx.x * 4 + wave; r < rows; r += (int64_t)gridDim.x * 4) {
        const int64_t id = ids[r];
        const bool ok = id >= 0 && id < V;
        if (!ok && lane == 0) atomicOr(bad_flag, id >= V ? 1 : 2);
        const bf16_t* src = W + (ok ? id : 0) * h;
        bf16_t* dst = out + r * h;
        for (int c0 = lane; c0 < h8; c0 += 512) {
            bf16x8 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
#pragma unroll
                for (int k = 0; k < 8; ++k) v[u][k] = (bf16_t)0.0f;
                if (ok && c0 + u * 64 < h8) v[u] = ld_bf16x8(src + (c0 + u * 64) * 8);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c0 + u * 64 < h8) st_bf16x8(dst + (c0 + u * 64) * 8, v[u]);
        }
    }
}

// dW[id, :] += sum of dY[r, :] over all rows r with ids[r] == id, in increasing row order (bit-reproducible), in time
// linear in the number of rows.  The rows are bucketed by id through four int32 tables in the workspace:
//   cnt[V]   rows per id                      first[V]  smallest row holding the id (its block does the sum)
//   off[V]   start of the id's bucket         bucket[T] rows grouped by id (order inside a group: as the atomics fell)
// The owner block of an id sorts that id's bucket by row number before summing, so the order the atomics produced never
// reaches the result.
constexpr int kBucketLds = 1024;  // buckets up to this size are sorted in LDS by rank; longer ones through a row bitmap

__global__ __launch_bounds__(kBlock) void embed_tables_init_kernel(int* __restrict__ cnt, int* __restrict__ first,
                                                                   int* __restrict__ fill, int* __restrict__ cursor, int64_t V) {
    if (blockIdx.x == 0 && threadIdx.x == 0) *cursor = 0;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < V; i += (int64_t)gridDim.x * kBlock) {
        cnt[i] = 0;
        fill[i] = 0;
        first[i] = 0x7fffffff;
    }
}

__global__ __launch_bounds__(kBlock) void embed_count_kernel(const int64_t* __restrict__ ids, int* __restrict__ cnt,
                                                             int* __restrict__ first, int64_t rows, int64_t V) {
    for (int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x; r < rows; r += (int64_t)gridDim.x * kBlock) {
        const int64_t id = ids[r];
        if (id < 0 || id >= V) continue;
        atomicAdd(cnt + id, 1);
        atomicMin(first + id, (int)r);
    }
}

// off[id] = start of id's range in the bucket array.  The ranges only have to be disjoint -- every bucket is put into row
// order before it is summed, and where it lies does not reach the result -- so the owner row of each id (its smallest row)
// takes the next cnt[id] entries from a running cursor; no prefix sum over the vocabulary is needed.
__global__ __launch_bounds__(kBlock) void embed_assign_kernel(const int64_t* __restrict__ ids, const int* __restrict__ cnt,
                                                              const int* __restrict__ first, int* __restrict__ off,
                                                              int* __restrict__ cursor, int64_t rows, int64_t V) {
    for (int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x; r < rows; r += (int64_t)gridDim.x * kBlock) {
        const int64_t id = ids[r];
        if (id < 0 || id >= V || first[id] != (int)r) continue;
        off[id] = atomicAdd(cursor, cnt[id]);
    }
}

__global__ __launch_bounds__(kBlock) void embed_bucket_kernel(const int64_t* __restrict__ ids, const int* __restrict__ off,
                                                              int* __restrict__ fill, int* __restrict__ bucket, int64_t rows,
                                                              int64_t V) {
    for (int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x; r < rows; r += (int64_t)gridDim.x * kBlock) {
        const int64_t id = ids[r];
        if (id < 0 || id >= V) continue;
        bucket[off[id] + atomicAdd(fill + id, 1)] = (int)r;
    }
}

// p[0 .. n4) = 0 in 16-byte pieces: a block clears one contiguous 16 KiB chunk (4 stores per thread), chunks dealt to blocks in
// order, so the blocks running at any moment sweep one window of the buffer.
__global__ __launch_bounds__(kBlock) void zero_f32x4_kernel(f32x4* __restrict__ p, int64_t n4) {
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    for (int64_t c = blockIdx.x; c * (4 * kBlock) < n4; c += gridDim.x) {
        const int64_t i0 = c * (4 * kBlock) + threadIdx.x;
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i0 + u * kBlock < n4) p[i0 + u * kBlock] = z;
    }
}

// overwrite: dW[id] = sum instead of dW[id] += sum, and the rows of ids that do not occur are zero-filled (the whole
// [V, h] gradient is then defined by this launch: no separate fill pass).
constexpr int kWindowRows = 2048;  // an id with more than kBucketLds rows is ordered through a bitmap over this many row numbers

template <int MAXC>
__global__ __launch_bounds__(kBlock) void embed_scatter_bucket_kernel(const int64_t* __restrict__ ids, const bf16_t* __restrict__ dY,
                                                                      float* __restrict__ dW, const int* __restrict__ cnt,
                                                                      const int* __restrict__ first, const int* __restrict__ off,
                                                                      const int* __restrict__ bucket, int64_t rows, int h,
                                                                      int64_t V, int overwrite) {
    static_assert(kWindowRows == 32 * 64 && kWindowRows >= kBucketLds, "one bitmap word per lane of the first wave");
    __shared__ int list[kWindowRows];  // rows of the current id in increasing order (first kBucketLds entries double as `sorted`)
    __shared__ int raw[kBucketLds];
    __shared__ unsigned bits[64];
    __shared__ int wtot;
    int* sorted = list;
    const int h8 = h >> 3;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int64_t t = blockIdx.x; t < rows; t += gridDim.x) {
        const int64_t id = ids[t];
        if (id < 0 || id >= V) continue;
        if (first[id] != (int)t) continue;  // the block of the smallest row of an id owns it (uniform over the block)
        const int n = cnt[id];
        const int* mine = bucket + off[id];
        float acc[MAXC][8];
#pragma unroll
        for (int c = 0; c < MAXC; ++c)
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[c][k] = 0.f;
        auto add_row = [&](int64_t jj) {
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int col = (c * kBlock + threadIdx.x);
                if (col < h8) {
                    float g[8];
                    unpack8(ld_bf16x8(dY + jj * h + col * 8), g);
#pragma unroll
                    for (int k = 0; k < 8; ++k) acc[c][k] += g[k];
                }
            }
        };
        // rows lst[0 .. m-1] in that order, the loads of four rows in flight at a time
        auto add_rows = [&](const int* lst, int m) {
            int i = 0;
            for (; i + 4 <= m; i += 4) {
                bf16x8 v[4][MAXC];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int64_t jj = lst[i + u];
#pragma unroll
                    for (int c = 0; c < MAXC; ++c) {
                        const int col = (c * kBlock + threadIdx.x);
                        if (col < h8) v[u][c] = ld_bf16x8(dY + jj * h + col * 8);
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int c = 0; c < MAXC; ++c) {
                        const int col = (c * kBlock + threadIdx.x);
                        if (col < h8) {
#pragma unroll
                            for (int k = 0; k < 8; ++k) acc[c][k] += (float)v[u][c][k];
                        }
                    }
            }
            for (; i < m; ++i) add_row(lst[i]);
        };
        if (n == 1) {
            add_row(t);
        } else if (n <= kBucketLds) {
            __syncthreads();  // the previous id's LDS use is over
            for (int i = threadIdx.x; i < n; i += kBlock) raw[i] = mine[i];
            __syncthreads();
            for (int i = threadIdx.x; i < n; i += kBlock) {  // rows are distinct: rank = number of smaller rows
                const int v = raw[i];
                int rank = 0;
                for (int j = 0; j < n; ++j) rank += raw[j] < v;
                sorted[rank] = v;
            }
            __syncthreads();
            add_rows(sorted, n);
        } else {
            // A frequent id (padding, say): its rows are put in order through a bitmap over row numbers, a window of
            // kWindowRows rows at a time -- every lane of the first wave owns one 32-row word, counts its bits, and after a
            // scan over the wave writes its rows into the ordered list.  n / kBlock bucket reads per thread and window.
            for (int64_t w0 = 0; w0 < rows; w0 += kWindowRows) {
                __syncthreads();  // the previous window's (or id's) LDS use is over
                if (threadIdx.x < 64) bits[threadIdx.x] = 0u;
                __syncthreads();
                for (int i = threadIdx.x; i < n; i += kBlock) {
                    const int64_t r = (int64_t)mine[i] - w0;
                    if (r >= 0 && r < kWindowRows) atomicOr(&bits[r >> 5], 1u << (r & 31));
                }
                __syncthreads();
                if (wv == 0) {
                    unsigned m = bits[lane];
                    const int mine_n = __builtin_popcount(m);
                    int incl = mine_n;
#pragma unroll
                    for (int o = 1; o < 64; o <<= 1) {
                        const int v = __shfl_up(incl, o, 64);
                        if (lane >= o) incl += v;
                    }
                    if (lane == 63) wtot = incl;
                    int pos = incl - mine_n;
                    while (m) {
                        list[pos++] = (int)w0 + 32 * lane + __builtin_ctz(m);
                        m &= m - 1;
                    }
                }
                __syncthreads();
                add_rows(list, wtot);
            }
        }
#pragma unroll
        for (int c = 0; c < MAXC; ++c) {
            const int col = (c * kBlock + threadIdx.x);
            if (col < h8) {
                float* dst = dW + id * h + col * 8;
                f32x4 lo, hi;
                if (overwrite) {
#pragma unroll
                    for (int k = 0; k < 4; ++k) { lo[k] = acc[c][k]; hi[k] = acc[c][4 + k]; }
                } else {
                    lo = *reinterpret_cast<f32x4*>(dst);
                    hi = *reinterpret_cast<f32x4*>(dst + 4);
#pragma unroll
                    for (int k = 0; k < 4; ++k) { lo[k] += acc[c][k]; hi[k] += acc[c][4 + k]; }
                }
                *reinterpret_cast<f32x4*>(dst) = lo;
                *reinterpret_cast<f32x4*>(dst + 4) = hi;
            }
        }
    }
    if (overwrite) {
        // ids that do not occur: zero rows.  Rows are dealt round-robin to the blocks, so that the blocks running at any
        // moment write one contiguous window of the buffer; a block reads the counts of up to kBlock of its rows at once, so
        // that the fill streams instead of waiting for one count per row.
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
        for (int64_t v0 = blockIdx.x; v0 < V; v0 += (int64_t)gridDim.x * kBlock) {
            const int64_t left = (V - v0 + gridDim.x - 1) / gridDim.x;  // rows v0, v0 + grid, ... below V
            const int m = left < kBlock ? (int)left : kBlock;
            __syncthreads();
            if ((int)threadIdx.x < m) raw[threadIdx.x] = cnt[v0 + (int64_t)threadIdx.x * gridDim.x];
            __syncthreads();
            for (int r = 0; r < m; ++r) {
                if (raw[r] != 0) continue;
                f32x4* dst = reinterpret_cast<f32x4*>(dW + (v0 + (int64_t)r * gridDim.x) * h);
                for (int i = threadIdx.x; i < (h >> 2); i += kBlock) __builtin_nontemporal_store(z, dst + i);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Unpadding by a key-padding mask (FlashAttention.forward, llama/transformer.py:117-141: unpad_input / pad_input)
// ---------------------------------------------------------------------------------------------
// mask [rows, s_len] (non-zero = keep), flattened to n = rows * s_len tokens.  One block walks the tokens 1024 at a time
// with a running count:  idx[p] = flat index of the p-th kept token (entries past the last kept token: -1),
// inv[i] = position of token i among the kept ones, or -1;  cu[r + 1] = kept tokens in rows 0..r (cu[0] = 0).
__global__ __launch_bounds__(1024) void mask_compact_kernel(const unsigned char* __restrict__ mask, int64_t n, int s_len,
                                                            int* __restrict__ idx, int* __restrict__ inv, int* __restrict__ cu) {
    __shared__ int wsum[16];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    int base = 0;
    if (tid == 0) cu[0] = 0;
    for (int64_t i0 = 0; i0 < n; i0 += 1024) {
        const int64_t i = i0 + tid;
        const int m = (i < n && mask[i]) ? 1 : 0;
        int incl = m;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o, 64);
            if (lane >= o) incl += v;
        }
        __syncthreads();  // wsum of the previous round has been read
        if (lane == 63) wsum[wv] = incl;
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            before += k < wv ? wsum[k] : 0;
            total += wsum[k];
        }
        const int upto = base + before + incl;  // kept tokens among 0..i
        if (i < n) {
            inv[i] = m ? upto - 1 : -1;
            if (m) idx[upto - 1] = (int)i;
            if ((i + 1) % s_len == 0) cu[(i + 1) / s_len] = upto;
        }
        base += total;
    }
    for (int64_t i = base + tid; i < n; i += 1024) idx[i] = -1;
}

// out row r = src row idx[r] (zeros where idx[r] is negative or past the source); a row number maps to memory as
// (r / s_len) * batch_stride + (r % s_len) * seq_stride on either side, so [s, b, ...] activations are read and
// written where they lie.
__global__ __launch_bounds__(kBlock) void rows_gather_kernel(const bf16_t* __restrict__ src, const int* __restrict__ idx,
                                                             bf16_t* __restrict__ out, int64_t n_out, int width, int64_t n_src,
                                                             int src_s_len, int64_t src_ss, int64_t src_sb, int out_s_len,
                                                             int64_t out_ss, int64_t out_sb) {
    const int w8 = width >> 3;
    for (int64_t r = blockIdx.x; r < n_out; r += gridDim.x) {
        const int64_t j = idx[r];
        const bool ok = j >= 0 && j < n_src;
        const bf16_t* s = src + (ok ? (j / src_s_len) * src_sb + (j % src_s_len) * src_ss : 0);
        bf16_t* o = out + (r / out_s_len) * out_sb + (r % out_s_len) * out_ss;
        for (int c = threadIdx.x; c < w8; c += kBlock) {
            bf16x8 v;
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = (bf16_t)0.0f;
            if (ok) v = ld_bf16x8(s + c * 8);
            st_bf16x8(o + c * 8, v);
        }
    }
}

// y[j, i, :] = x[i, j, :]  for x [d0, d1, inner]   (llama/llama.py:157-168,175-179)
__global__ __launch_bounds__(kBlock) void transpose01_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ y, int64_t d0,
                                                             int64_t d1, int inner) {
    const int i8 = inner >> 3;
    const int64_t rows = d0 * d1;
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const int64_t i = r / d1, j = r % d1;
        const bf16_t* src = x + r * inner;
        bf16_t* dst = y + (j * d0 + i) * inner;
        for (int c = threadIdx.x; c < i8; c += kBlock) st_bf16x8(dst + c * 8, ld_bf16x8(src + c * 8));
    }
}

__global__ __launch_bounds__(kBlock) void add_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ b,
                                                     bf16_t* __restrict__ out, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += (int64_t)gridDim.x * kBlock) {
        float x[8], y[8];
        unpack8(ld_bf16x8(a + i * 8), x);
        unpack8(ld_bf16x8(b + i * 8), y);
#pragma unroll
        for (int k = 0; k < 8; ++k) x[k] += y[k];
        st_bf16x8(out + i * 8, pack8(x));
    }
}

__global__ __launch_bounds__(kBlock) void bf16_to_f32_kernel(const bf16_t* __restrict__ in, float* __restrict__ out, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += (int64_t)gridDim.x * kBlock) {
        float x[8];
        unpack8(ld_bf16x8(in + i * 8), x);
        f32x4 lo = {x[0], x[1], x[2], x[3]}, hi = {x[4], x[5], x[6], x[7]};
        *reinterpret_cast<f32x4*>(out + i * 8) = lo;
        *reinterpret_cast<f32x4*>(out + i * 8 + 4) = hi;
    }
}

__global__ __launch_bounds__(kBlock) void f32_to_bf16_kernel(const float* __restrict__ in, bf16_t* __restrict__ out, int64_t n8) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += (int64_t)gridDim.x * kBlock) {
        const f32x4 lo = *reinterpret_cast<const f32x4*>(in + i * 8), hi = *reinterpret_cast<const f32x4*>(in + i * 8 + 4);
        float x[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        st_bf16x8(out + i * 8, pack8(x));
    }
}

// out[r, :] = x[r, :] + bias   (column_parallel_linear.py:43-44)
__global__ __launch_bounds__(kBlock) void bias_add_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ bias,
                                                          bf16_t* __restrict__ out, int64_t rows, int n) {
    const int n8 = n >> 3;
    const int64_t items = rows * n8;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < items; i += (int64_t)gridDim.x * kBlock) {
        const int c = (int)(i % n8);
        float a[8], b[8];
        unpack8(ld_bf16x8(x + i * 8), a);
        unpack8(ld_bf16x8(bias + c * 8), b);
#pragma unroll
        for (int k = 0; k < 8; ++k) a[k] += b[k];
        st_bf16x8(out + i * 8, pack8(a));
    }
}

// partial[blockIdx.y][col] = sum over rows r = blockIdx.y, blockIdx.y + gridDim.y, ... of dy[r][col]   (:100)
__global__ __launch_bounds__(kBlock) void bias_grad_partial_kernel(const bf16_t* __restrict__ dy, float* __restrict__ partial,
                                                                   int64_t rows, int n) {
    const int col = (blockIdx.x * kBlock + threadIdx.x) * 8;
    if (col >= n) return;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        float v[8];
        unpack8(ld_bf16x8(dy + r * n + col), v);
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[k] += v[k];
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) partial[(int64_t)blockIdx.y * n + col + k] = acc[k];
}

}  // namespace

extern "C" int ezl_swiglu_fwd(const void* gate, const void* up, void* out, int64_t n, void* stream) {
    EZL_REQUIRE(n >= 0 && n % 8 == 0, EZL_EUNSUPPORTED, "ezl_swiglu_fwd: n must be a multiple of 8");
    EZL_REQUIRE(ezl_aligned16(gate) && ezl_aligned16(up) && ezl_aligned16(out) && (n == 0 || (gate && up && out)), EZL_EINVAL,
                "ezl_swiglu_fwd: null or misaligned pointer");
    if (n == 0) return EZL_OK;
    hipLaunchKernelGGL(swiglu_fwd_kernel, dim3(grid_for(n / 8, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                       (const bf16_t*)gate, (const bf16_t*)up, (bf16_t*)out, n / 8);
    EZL_LAUNCH_CHECK("ezl_swiglu_fwd");
    return EZL_OK;
}

extern "C" int ezl_swiglu_bwd(const void* dout, const void* gate, const void* up, void* dgate, void* dup, int64_t n,
                              void* stream) {
    EZL_REQUIRE(n >= 0 && n % 8 == 0, EZL_EUNSUPPORTED, "ezl_swiglu_bwd: n must be a multiple of 8");
    EZL_REQUIRE(ezl_aligned16(dout) && ezl_aligned16(gate) && ezl_aligned16(up) && ezl_aligned16(dgate) && ezl_aligned16(dup) &&
                    (n == 0 || (dout && gate && up && dgate && dup)),
                EZL_EINVAL, "ezl_swiglu_bwd: null or misaligned pointer");
    if (n == 0) return EZL_OK;
    hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(grid_for(n / 8, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                       (const bf16_t*)dout, (const bf16_t*)gate, (const bf16_t*)up, (bf16_t*)dgate, (bf16_t*)dup, n / 8);
    EZL_LAUNCH_CHECK("ezl_swiglu_bwd");
    return EZL_OK;
}

extern "C" int ezl_rope_table(const void* inv_freq, void* cos_out, void* sin_out, int64_t npos, int64_t half_dim,
                              float scale_factor, void* stream) {
    EZL_REQUIRE(npos > 0 && half_dim > 0 && scale_factor > 0.f && inv_freq && cos_out && sin_out, EZL_EINVAL,
                "ezl_rope_table: bad argument");
    hipLaunchKernelGGL(rope_table_kernel, dim3(grid_for(npos * half_dim, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                       (const float*)inv_freq, (float*)cos_out, (float*)sin_out, npos, (int)half_dim, scale_factor);
    EZL_LAUNCH_CHECK("ezl_rope_table");
    return EZL_OK;
}

namespace {
int rope_launch(const char* name, const void* x0, void* out0, int64_t nh0, int64_t is0, int64_t os0, const void* x1, void* out1,
                int64_t nh1, int64_t is1, int64_t os1, const void* cos_table, const void* sin_table, const void* position_ids,
                int64_t s, int64_t b, int64_t d, int64_t npos, int backward, void* stream) {
    EZL_REQUIRE(s >= 0 && b > 0 && nh0 > 0 && nh1 >= 0 && d > 0 && d % 16 == 0, EZL_EUNSUPPORTED,
                "%s: head dim must be a multiple of 16 (got %lld)", name, (long long)d);
    EZL_REQUIRE(is0 % 8 == 0 && os0 % 8 == 0 && is0 >= nh0 * d && os0 >= nh0 * d, EZL_EINVAL, "%s: bad row stride", name);
    EZL_REQUIRE(nh1 == 0 || (is1 % 8 == 0 && os1 % 8 == 0 && is1 >= nh1 * d && os1 >= nh1 * d), EZL_EINVAL, "%s: bad row stride", name);
    EZL_REQUIRE(npos >= 1 && (position_ids || npos >= s), EZL_EINVAL, "%s: cos/sin table shorter than the sequence", name);
    EZL_REQUIRE((s == 0 || (x0 && out0 && (nh1 == 0 || (x1 && out1)))) && cos_table && sin_table && ezl_aligned16(x0) &&
                    ezl_aligned16(out0) && ezl_aligned16(x1) && ezl_aligned16(out1) && ezl_aligned16(cos_table) &&
                    ezl_aligned16(sin_table),
                EZL_EINVAL, "%s: null or misaligned pointer", name);
    EZL_REQUIRE(s < (1LL << 31) && b < (1LL << 31) && nh0 + nh1 < (1LL << 24), EZL_EUNSUPPORTED, "%s: shape too large", name);
    if (s == 0) return EZL_OK;
    const int64_t items = s * b * (nh0 + nh1) * (d / 16);
    const RopeSide a = {(const bf16_t*)x0, (bf16_t*)out0, is0, os0};
    const RopeSide c = {(const bf16_t*)x1, (bf16_t*)out1, is1, os1};
    hipLaunchKernelGGL(rope_kernel, dim3(grid_for(items, kBlock)), dim3(kBlock), 0, (hipStream_t)stream, a, c,
                       (const float*)cos_table, (const float*)sin_table, (const int64_t*)position_ids, s * b, (int)s, (int)b,
                       (int)nh0, (int)nh1, (int)d, npos, backward ? -1.0f : 1.0f);
    EZL_LAUNCH_CHECK(name);
    return EZL_OK;
}
}  // namespace

extern "C" int ezl_rope_apply(const void* x, void* out, const void* cos_table, const void* sin_table,
                              const void* position_ids, int64_t s, int64_t b, int64_t nheads, int64_t d,
                              int64_t in_row_stride, int64_t out_row_stride, int64_t npos, int backward, void* stream) {
    return rope_launch("ezl_rope_apply", x, out, nheads, in_row_stride, out_row_stride, nullptr, nullptr, 0, 0, 0, cos_table,
                       sin_table, position_ids, s, b, d, npos, backward, stream);
}

extern "C" int ezl_rope_apply_pair(const void* q, void* q_out, int64_t nq, int64_t q_in_stride, int64_t q_out_stride,
                                   const void* k, void* k_out, int64_t nk, int64_t k_in_stride, int64_t k_out_stride,
                                   const void* cos_table, const void* sin_table, const void* position_ids, int64_t s, int64_t b,
                                   int64_t d, int64_t npos, int backward, void* stream) {
    EZL_REQUIRE(nk > 0, EZL_EINVAL, "ezl_rope_apply_pair: the second tensor needs at least one head");
    return rope_launch("ezl_rope_apply_pair", q, q_out, nq, q_in_stride, q_out_stride, k, k_out, nk, k_in_stride, k_out_stride,
                       cos_table, sin_table, position_ids, s, b, d, npos, backward, stream);
}

extern "C" int ezl_ids_in_range(const void* ids, int64_t n, int64_t limit, void* bad_flag, void* stream) {
    EZL_REQUIRE(n >= 0 && bad_flag && (n == 0 || ids), EZL_EINVAL, "ezl_ids_in_range: null pointer");
    if (n == 0) return EZL_OK;
    hipLaunchKernelGGL(ids_in_range_kernel, dim3(grid_for(n, kBlock, 256)), dim3(kBlock), 0, (hipStream_t)stream, (const int64_t*)ids,
                       n, limit, (int*)bad_flag);
    EZL_LAUNCH_CHECK("ezl_ids_in_range");
    return EZL_OK;
}

extern "C" int ezl_embed_gather(const void* ids, const void* weight, void* out, void* bad_flag, int64_t rows, int64_t h,
                                int64_t vocab, void* stream) {
    EZL_REQUIRE(rows >= 0 && h > 0 && h % 8 == 0 && h < (1LL << 31) && vocab > 0, EZL_EUNSUPPORTED,
                "ezl_embed_gather: h must be a multiple of 8");
    EZL_REQUIRE(bad_flag && (rows == 0 || (ids && weight && out)) && ezl_aligned16(weight) && ezl_aligned16(out), EZL_EINVAL,
                "ezl_embed_gather: null or misaligned pointer");
    if (rows == 0) return EZL_OK;
    hipLaunchKernelGGL(embed_gather_kernel, dim3(grid_for((rows + 3) / 4, 1)), dim3(kBlock), 0, (hipStream_t)stream, (const int64_t*)ids,
                       (const bf16_t*)weight, (bf16_t*)out, rows, (int)h, vocab, (int*)bad_flag);
    EZL_LAUNCH_CHECK("ezl_embed_gather");
    return EZL_OK;
}

extern "C" int64_t ezl_embed_scatter_add_workspace_bytes(int64_t rows, int64_t vocab) {
    if (rows < 0 || vocab <= 0) return -1;
    return (4 * vocab + rows + 4) * (int64_t)sizeof(int);
}

extern "C" int ezl_embed_scatter_add(const void* ids, const void* dy, void* dweight_f32, void* workspace, int64_t workspace_bytes,
                                     int64_t rows, int64_t h, int64_t vocab, int accumulate, void* stream) {
    EZL_REQUIRE(rows >= 0 && h > 0 && h % 8 == 0 && h < (1LL << 31) && vocab > 0, EZL_EUNSUPPORTED,
                "ezl_embed_scatter_add: h must be a multiple of 8");
    EZL_REQUIRE((rows == 0 || (ids && dy && dweight_f32)) && ezl_aligned16(dy), EZL_EINVAL,
                "ezl_embed_scatter_add: null or misaligned pointer");
    if (rows == 0 && accumulate) return EZL_OK;
    EZL_REQUIRE(dweight_f32, EZL_EINVAL, "ezl_embed_scatter_add: null or misaligned pointer");
    EZL_REQUIRE(h <= 8192 * 2, EZL_EUNSUPPORTED, "ezl_embed_scatter_add: h must be <= 16384");
    EZL_REQUIRE(rows < (1LL << 31) && vocab < (1LL << 31), EZL_EUNSUPPORTED, "ezl_embed_scatter_add: more than 2^31 rows or ids");
    EZL_REQUIRE(((uintptr_t)dweight_f32 & 15) == 0, EZL_EINVAL, "ezl_embed_scatter_add: dweight must be 16-byte aligned");
    EZL_REQUIRE(workspace && ((uintptr_t)workspace & 3) == 0 && workspace_bytes >= ezl_embed_scatter_add_workspace_bytes(rows, vocab),
                EZL_EINVAL, "ezl_embed_scatter_add: workspace missing or smaller than ezl_embed_scatter_add_workspace_bytes()");
    int* cnt = (int*)workspace;
    int* first = cnt + vocab;
    int* off = first + vocab;
    int* fill = off + vocab;
    int* bucket = fill + vocab;
    int* cursor = bucket + rows;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(embed_tables_init_kernel, dim3(grid_for(vocab, kBlock, 1024)), dim3(kBlock), 0, st, cnt, first, fill, cursor, vocab);
    hipLaunchKernelGGL(embed_count_kernel, dim3(grid_for(rows, kBlock, 1024)), dim3(kBlock), 0, st, (const int64_t*)ids, cnt, first,
                       rows, vocab);
    hipLaunchKernelGGL(embed_assign_kernel, dim3(grid_for(rows, kBlock, 1024)), dim3(kBlock), 0, st, (const int64_t*)ids, cnt, first, off,
                       cursor, rows, vocab);
    hipLaunchKernelGGL(embed_bucket_kernel, dim3(grid_for(rows, kBlock, 1024)), dim3(kBlock), 0, st, (const int64_t*)ids, off, fill,
                       bucket, rows, vocab);
    EZL_LAUNCH_CHECK("ezl_embed_scatter_add(tables)");
    // one workgroup per token row (accumulate) or per vocabulary row, whichever is more: the zero fill of the rows that
    // received nothing is most of the traffic when the result overwrites the buffer
    // Overwriting a large table ([152064, 5120] fp32 = 3.1 GB, say) is mostly a zero fill, and a flat fill kernel in front
    // of the adding form writes it faster than the per-row fill inside the scatter kernel does (measured 502 against 580 us
    // at that size); for a table of 0.5 GB the fused form wins (99 against 116 us) because the two parts overlap.
    const bool flat_fill = !accumulate && vocab * h >= (int64_t)1 << 28;
    if (flat_fill) {
        const int64_t n4 = vocab * h / 4;
        hipLaunchKernelGGL(zero_f32x4_kernel, dim3(grid_for(n4, 4 * kBlock, (int64_t)1 << 20)), dim3(kBlock), 0, st, (f32x4*)dweight_f32, n4);
    }
    const int overwrite = accumulate || flat_fill ? 0 : 1;
    const dim3 grid(grid_for(overwrite ? (rows > vocab ? rows : vocab) : rows, 1));
    if (h <= 8 * kBlock * 2)
        hipLaunchKernelGGL((embed_scatter_bucket_kernel<2>), grid, dim3(kBlock), 0, st, (const int64_t*)ids, (const bf16_t*)dy,
                           (float*)dweight_f32, cnt, first, off, bucket, rows, (int)h, vocab, overwrite);
    else if (h <= 8 * kBlock * 4)
        hipLaunchKernelGGL((embed_scatter_bucket_kernel<4>), grid, dim3(kBlock), 0, st, (const int64_t*)ids, (const bf16_t*)dy,
                           (float*)dweight_f32, cnt, first, off, bucket, rows, (int)h, vocab, overwrite);
    else
        hipLaunchKernelGGL((embed_scatter_bucket_kernel<8>), grid, dim3(kBlock), 0, st, (const int64_t*)ids, (const bf16_t*)dy,
                           (float*)dweight_f32, cnt, first, off, bucket, rows, (int)h, vocab, overwrite);
    EZL_LAUNCH_CHECK("ezl_embed_scatter_add");
    return EZL_OK;
}

extern "C" int ezl_transpose01(const void* x, void* y, int64_t d0, int64_t d1, int64_t inner, void* stream) {
    EZL_REQUIRE(d0 >= 0 && d1 >= 0 && inner > 0 && inner % 8 == 0 && inner < (1LL << 31), EZL_EUNSUPPORTED,
                "ezl_transpose01: inner must be a multiple of 8");
    EZL_REQUIRE((d0 * d1 == 0 || (x && y)) && ezl_aligned16(x) && ezl_aligned16(y), EZL_EINVAL,
                "ezl_transpose01: null or misaligned pointer");
    if (d0 * d1 == 0) return EZL_OK;
    hipLaunchKernelGGL(transpose01_kernel, dim3(grid_for(d0 * d1, 1)), dim3(kBlock), 0, (hipStream_t)stream, (const bf16_t*)x,
                       (bf16_t*)y, d0, d1, (int)inner);
    EZL_LAUNCH_CHECK("ezl_transpose01");
    return EZL_OK;
}

extern "C" int ezl_add(const void* a, const void* b, void* out, int64_t n, void* stream) {
    EZL_REQUIRE(n >= 0 && n % 8 == 0, EZL_EUNSUPPORTED, "ezl_add: n must be a multiple of 8");
    EZL_REQUIRE((n == 0 || (a && b && out)) && ezl_aligned16(a) && ezl_aligned16(b) && ezl_aligned16(out), EZL_EINVAL,
                "ezl_add: null or misaligned pointer");
    if (n == 0) return EZL_OK;
    hipLaunchKernelGGL(add_kernel, dim3(grid_for(n / 8, kBlock)), dim3(kBlock), 0, (hipStream_t)stream, (const bf16_t*)a,
                       (const bf16_t*)b, (bf16_t*)out, n / 8);
    EZL_LAUNCH_CHECK("ezl_add");
    return EZL_OK;
}

extern "C" int ezl_cast_bf16_to_f32(const void* in, void* out, int64_t n, void* stream) {
    EZL_REQUIRE(n >= 0 && n % 8 == 0, EZL_EUNSUPPORTED, "ezl_cast_bf16_to_f32: n must be a multiple of 8");
    EZL_REQUIRE((n == 0 || (in && out)) && ezl_aligned16(in) && ezl_aligned16(out), EZL_EINVAL,
                "ezl_cast_bf16_to_f32: null or misaligned pointer");
    if (n == 0) return EZL_OK;
    hipLaunchKernelGGL(bf16_to_f32_kernel, dim3(grid_for(n / 8, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                       (const bf16_t*)in, (float*)out, n / 8);
    EZL_LAUNCH_CHECK("ezl_cast_bf16_to_f32");
    return EZL_OK;
}

extern "C" int ezl_cast_f32_to_bf16(const void* in, void* out, int64_t n, void* stream) {
    EZL_REQUIRE(n >= 0 && n % 8 == 0, EZL_EUNSUPPORTED, "ezl_cast_f32_to_bf16: n must be a multiple of 8");
    EZL_REQUIRE((n == 0 || (in && out)) && ezl_aligned16(in) && ezl_aligned16(out), EZL_EINVAL,
                "ezl_cast_f32_to_bf16: null or misaligned pointer");
    if (n == 0) return EZL_OK;
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(grid_for(n / 8, kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                       (const float*)in, (bf16_t*)out, n / 8);
    EZL_LAUNCH_CHECK("ezl_cast_f32_to_bf16");
    return EZL_OK;
}

extern "C" int ezl_bias_add(const void* x, const void* bias, void* out, int64_t rows, int64_t n, void* stream) {
    EZL_REQUIRE(rows >= 0 && n > 0 && n % 8 == 0 && n < (1LL << 31), EZL_EUNSUPPORTED, "ezl_bias_add: n must be a multiple of 8");
    EZL_REQUIRE((rows == 0 || (x && bias && out)) && ezl_aligned16(x) && ezl_aligned16(bias) && ezl_aligned16(out), EZL_EINVAL,
                "ezl_bias_add: null or misaligned pointer");
    if (rows == 0) return EZL_OK;
    hipLaunchKernelGGL(bias_add_kernel, dim3(grid_for(rows * (n / 8), kBlock)), dim3(kBlock), 0, (hipStream_t)stream,
                       (const bf16_t*)x, (const bf16_t*)bias, (bf16_t*)out, rows, (int)n);
    EZL_LAUNCH_CHECK("ezl_bias_add");
    return EZL_OK;
}

extern "C" int64_t ezl_bias_grad_workspace_bytes(int64_t rows, int64_t n) {
    (void)rows;
    return (int64_t)64 * n * (int64_t)sizeof(float);
}

extern "C" int ezl_bias_grad(const void* dy, void* db_bf16, void* db_f32, int accumulate, void* workspace,
                             int64_t workspace_bytes, int64_t rows, int64_t n, void* stream) {
    EZL_REQUIRE(rows >= 0 && n > 0 && n % 8 == 0 && n < (1LL << 31), EZL_EUNSUPPORTED, "ezl_bias_grad: n must be a multiple of 8");
    EZL_REQUIRE(dy && workspace && ezl_aligned16(dy) && ((db_bf16 != nullptr) != (db_f32 != nullptr)), EZL_EINVAL,
                "ezl_bias_grad: bad pointer arguments");
    EZL_REQUIRE(workspace_bytes >= ezl_bias_grad_workspace_bytes(rows, n), EZL_EINVAL, "ezl_bias_grad: workspace too small");
    const dim3 grid((unsigned)((n / 8 + kBlock - 1) / kBlock), 64);
    hipLaunchKernelGGL(bias_grad_partial_kernel, grid, dim3(kBlock), 0, (hipStream_t)stream, (const bf16_t*)dy, (float*)workspace,
                       rows, (int)n);
    EZL_LAUNCH_CHECK("ezl_bias_grad");
    hipLaunchKernelGGL(ezl_colsum_kernel<0>, dim3((unsigned)((n + 63) / 64)), dim3(kColsumThreads), 0, (hipStream_t)stream,
                       (const float*)workspace, 64, (int)n, (bf16_t*)db_bf16, (float*)db_f32, accumulate);
    EZL_LAUNCH_CHECK("ezl_bias_grad(colsum)");
    return EZL_OK;
}

extern "C" int ezl_mask_compact(const void* mask_u8, int64_t rows, int64_t s_len, void* idx, void* inv, void* cu_seqlens, void* stream) {
    EZL_REQUIRE(rows >= 0 && s_len > 0 && rows * s_len < (1LL << 31), EZL_EINVAL, "ezl_mask_compact: bad shape");
    EZL_REQUIRE(cu_seqlens && (rows == 0 || (mask_u8 && idx && inv)), EZL_EINVAL, "ezl_mask_compact: null pointer");
    hipLaunchKernelGGL(mask_compact_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, (const unsigned char*)mask_u8, rows * s_len,
                       (int)s_len, (int*)idx, (int*)inv, (int*)cu_seqlens);
    EZL_LAUNCH_CHECK("ezl_mask_compact");
    return EZL_OK;
}

extern "C" int ezl_rows_gather(const void* src, const void* idx, void* out, int64_t n_out, int64_t width, int64_t n_src,
                               int64_t src_s_len, int64_t src_seq_stride, int64_t src_batch_stride, int64_t out_s_len,
                               int64_t out_seq_stride, int64_t out_batch_stride, void* stream) {
    EZL_REQUIRE(n_out >= 0 && n_src >= 0 && width > 0 && width % 8 == 0 && width < (1LL << 31), EZL_EUNSUPPORTED,
                "ezl_rows_gather: width must be a multiple of 8");
    EZL_REQUIRE(src_s_len > 0 && out_s_len > 0 && src_s_len < (1LL << 31) && out_s_len < (1LL << 31) && src_seq_stride % 8 == 0 &&
                    src_batch_stride % 8 == 0 && out_seq_stride % 8 == 0 && out_batch_stride % 8 == 0,
                EZL_EINVAL, "ezl_rows_gather: strides must be multiples of 8 elements");
    EZL_REQUIRE((n_out == 0 || (idx && out && (src || n_src == 0))) && ezl_aligned16(src) && ezl_aligned16(out), EZL_EINVAL,
                "ezl_rows_gather: null or misaligned pointer");
    if (n_out == 0) return EZL_OK;
    hipLaunchKernelGGL(rows_gather_kernel, dim3(grid_for(n_out, 1)), dim3(kBlock), 0, (hipStream_t)stream, (const bf16_t*)src,
                       (const int*)idx, (bf16_t*)out, n_out, (int)width, n_src, (int)src_s_len, src_seq_stride, src_batch_stride,
                       (int)out_s_len, out_seq_stride, out_batch_stride);
    EZL_LAUNCH_CHECK("ezl_rows_gather");
    return EZL_OK;
}
