// Causal, variable-length flash attention forward + backward for gfx950 (bf16 MFMA, fp32 softmax).
//
// Replaces the flash_attn_varlen_{qkv,kv}packed_func calls of the reference's FlashAttention
// (llama/transformer.py:83-143): tokens are flattened to (b s); documents are the batch rows or the
// cu_seqlens segments; attention is causal inside each document; softmax scale defaults to
// 1/sqrt(d); query head i reads kv head i / (nq / nk) (MHA and GQA).
//
// Tensors are addressed as  token n -> (n / s_len) * batch_stride + (n % s_len) * seq_stride, heads
// contiguous inside a token, so the [s, b, heads*d] activations of the layer are consumed and
// produced in place (no [s,b]<->[b,s] copies, cf. transformer.py:478,491).
//
// The forward and the dK/dV kernel use the 32x32x16 bf16 MFMA, the dQ kernel the 16x16x32 one (measured faster there, slower
// in dK/dV); all with "transposed" score tiles so that the softmax statistics of a query are per-lane scalars:
//   forward       S^T = K Q^T (keys x queries), online softmax per lane, O^T += V^T P^T
//   dK/dV kernel  S = Q K^T (queries x keys), dV^T += dO^T P, dK^T += Q^T dS   (block owns 128 keys)
//   dQ kernel     S^T = K Q^T, dP^T = V dO^T, dQ^T += K^T dS^T                 (block owns 128 queries)
// Operands whose reduction index is the strided one (V^T, K^T, Q^T, dO^T) are read from their
// natural [row][d] LDS tiles with ds_read_b64_tr_b16; the accumulator registers of the score tile
// are reused directly as the B operand of the second MFMA (the k index is permuted consistently).
// LDS rows are padded to (d*2 + 48) bytes, which keeps both the 128-bit row reads and the transpose
// reads free of bank conflicts.  K/V (or Q/dO) tiles are double buffered and filled through
// registers one tile ahead.  dQ uses its own pass instead of atomics, so results are deterministic.
#include "common.h"

#include <type_traits>

namespace {

constexpr int kThreads = 256;
#ifndef EZL_DKDV_MIN_BLOCKS
#define EZL_DKDV_MIN_BLOCKS 512  // dK/dV workgroups wanted before (kv head, key block) pairs stop being split
#endif
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
typedef __attribute__((address_space(3))) void lds_void;

struct AttnParams {
    const bf16_t* q; const bf16_t* k; const bf16_t* v; const bf16_t* o; const bf16_t* dout;
    bf16_t* out; bf16_t* dq; bf16_t* dk; bf16_t* dv;
    float* lse; float* delta;
    float* part;  // dK/dV kernel with nsplit > 1: fp32 partial sums [nsplit][2 (dK, dV)][T][nk][d]
    int nsplit;   // workgroups that share a (kv head, key block): each takes nq / nk / nsplit of the group's query heads
    const int* cu;
    int ndocs, s_len, T, nq, nk;
    float scale;
    int64_t q_ss, q_sb, k_ss, k_sb, v_ss, v_sb, o_ss, o_sb;          // forward tensors
    int64_t do_ss, do_sb, dq_ss, dq_sb, dk_ss, dk_sb, dv_ss, dv_sb;  // backward tensors
};

__device__ __forceinline__ int64_t tok_off(int n, int s_len, int64_t ss, int64_t sb) {
    const int b = n / s_len;
    return (int64_t)b * sb + (int64_t)(n - b * s_len) * ss;
}

// Work list of the three kernels.  A document is cut at batch-row boundaries (the reference's collator never emits one
// that crosses a row: it appends every row's length to that row's boundaries), so inside a piece token i lives at
// tok_off(piece_start) + i * seq_stride and no per-token division is needed.  A piece of n tokens has ceil(n / 128) blocks;
// block j of a piece (queries, or keys counted from the piece's END for the dK/dV kernel) walks j + 1 blocks of the other
// operand, so its running time grows with j.
//
// Blocks are handed out longest first over ALL pieces and heads (rank 0 = the largest j anywhere): the hardware starts
// workgroups in the order of their ids, and with the long blocks of some head started late -- as happens when ids run head
// by head -- the last of them finish long after everything else (98 instead of 66 block-times for 4 heads x 32 blocks on
// the 64 slots of an XCD).  rank -> (piece, j): level j holds the pieces with more than j blocks, levels are laid out from
// the highest down; the level is found by bisection on count(j) = number of blocks with index >= j, the piece inside the
// level by a prefix sum, both computed by the whole workgroup (every thread must call this, before any other use of LDS).
// Dense batches (no cu_seqlens) have a closed form.
__device__ __forceinline__ int doc_bounds(const int* __restrict__ cu, int d, int s_len, int T, int& e) {
    int a = cu ? cu[d] : d * s_len;
    e = cu ? cu[d + 1] : (d + 1) * s_len;
    a = a < 0 ? 0 : a;
    e = e > T ? T : e;
    return a;
}

struct BlockSearch {
    int* s_wave;  // [16]
    int tid, nthr, lane, wv, nwaves;
    // sum over the workgroup; uniform result
    __device__ __forceinline__ int reduce(int v) const {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        __syncthreads();  // s_wave of the previous reduction has been read
        if (lane == 0) s_wave[wv] = v;
        __syncthreads();
        int t = 0;
        for (int i = 0; i < nwaves; ++i) t += s_wave[i];
        return t;
    }
};

// lds: kFindBlockInts ints of LDS for the search.  It is handed in by the kernel, carved from its one LDS array, instead of
// being declared here: with several LDS variables in a kernel the compiler tags every LDS access with the variable it
// belongs to and thereby drops the no-alias tags of the fragment reads, after which each read waits for all tile loads in
// flight (vmcnt(0)) because it might alias their destination.
constexpr int kFindBlockInts = 20;
__device__ __forceinline__ bool find_block(const int* __restrict__ cu, int ndocs, int s_len, int T, int rank, int blk_rows,
                                           int& doc_start, int& doc_len, int& blk, int* lds) {
    const int nb_row = (s_len + blk_rows - 1) / blk_rows;
    if (!cu) {  // every piece is a whole batch row: level j holds all ndocs rows
        if (rank >= ndocs * nb_row) return false;
        blk = nb_row - 1 - rank / ndocs;
        doc_start = (rank % ndocs) * s_len;
        doc_len = s_len;
        return true;
    }
    int* s_wave = lds;        // [16]
    int* s_found = lds + 16;  // [4]
    BlockSearch bs;
    bs.s_wave = s_wave;
    bs.tid = threadIdx.x; bs.nthr = blockDim.x; bs.lane = bs.tid & 63; bs.wv = bs.tid >> 6; bs.nwaves = bs.nthr >> 6;
    // blocks with index >= j over this thread's documents (pieces enumerated on the fly; one piece unless a document
    // crosses a batch row)
    auto count_ge = [&](int j) {
        int c = 0;
        for (int d = bs.tid; d < ndocs; d += bs.nthr) {
            int e;
            const int a = doc_bounds(cu, d, s_len, T, e);
            for (int x = a; x < e;) {
                const int row_end = (x / s_len + 1) * s_len;
                const int e1 = e < row_end ? e : row_end;
                const int nb = (e1 - x + blk_rows - 1) / blk_rows;
                c += nb > j ? nb - j : 0;
                x = e1;
            }
        }
        return bs.reduce(c);
    };
    if (rank >= count_ge(0)) return false;
    int lo = 0, hi = nb_row, c_hi = 0;  // count(lo) > rank >= count(hi)
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        const int c = count_ge(mid);
        if (c > rank) lo = mid;
        else { hi = mid; c_hi = c; }
    }
    const int j = lo;
    const int want = rank - c_hi;  // the want-th piece (in document order) that has more than j blocks
    if (bs.tid == 0) s_found[0] = 0;
    int base = 0;
    for (int d0 = 0; d0 < ndocs; d0 += bs.nthr) {
        const int d = d0 + bs.tid;
        int mine = 0, a = 0, e = 0;
        if (d < ndocs) {
            a = doc_bounds(cu, d, s_len, T, e);
            for (int x = a; x < e;) {
                const int row_end = (x / s_len + 1) * s_len;
                const int e1 = e < row_end ? e : row_end;
                mine += (e1 - x + blk_rows - 1) / blk_rows > j;
                x = e1;
            }
        }
        int incl = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(incl, o, 64);
            if (bs.lane >= o) incl += v;
        }
        __syncthreads();
        if (bs.lane == 63) s_wave[bs.wv] = incl;
        __syncthreads();
        int before = 0, total = 0;
        for (int i = 0; i < bs.nwaves; ++i) {
            const int v = s_wave[i];
            before += i < bs.wv ? v : 0;
            total += v;
        }
        const int first = base + before + incl - mine;  // rank inside the level of this thread's first qualifying piece
        if (mine > 0 && want >= first && want < first + mine) {
            int rel = want - first;
            for (int x = a; x < e;) {
                const int row_end = (x / s_len + 1) * s_len;
                const int e1 = e < row_end ? e : row_end;
                if ((e1 - x + blk_rows - 1) / blk_rows > j) {
                    if (rel == 0) {
                        s_found[1] = x;
                        s_found[2] = e1 - x;
                        s_found[0] = 1;
                        break;
                    }
                    --rel;
                }
                x = e1;
            }
        }
        base += total;
        if (want < base) break;  // uniform
    }
    __syncthreads();
    if (!s_found[0]) return false;
    doc_start = __builtin_amdgcn_readfirstlane(s_found[1]);
    doc_len = __builtin_amdgcn_readfirstlane(s_found[2]);
    blk = j;
    return true;
}

// The hardware deals consecutive workgroups (x fastest, then y) round-robin to the 8 XCDs, each with an L2 of its own.
// With the plain (block, head) numbering every XCD would touch the K / V rows of every head and its L2 would keep missing;
// renumbered, an XCD owns nheads / 8 heads, and inside an XCD the ids run over ranks (longest blocks first, see above) with
// the XCD's heads innermost: blocks of equal length of all its heads start together and walk the keys in step.
// by: head, rank: position in the longest-first work list of one head.
__device__ __forceinline__ void xcd_head_blocks(int nheads, int& rank, int& by) {
    const int lin = blockIdx.y * gridDim.x + blockIdx.x;
    if ((nheads & 7) == 0) {
        const int hpx = nheads >> 3, idx = lin >> 3;
        by = (lin & 7) * hpx + idx % hpx;
        rank = idx / hpx;
    } else {
        by = lin % nheads;
        rank = lin / nheads;
    }
}

template <int D>
struct Tile {
    static constexpr int LD = D + 24;             // padded row stride in elements
    static constexpr int CH = D / 8;              // 128-bit chunks per row
    static constexpr int ROWS = 64;
    static constexpr int ELEMS = ROWS * LD;

    // ---- tile rows straight from global memory into LDS (buffer_load ... lds, 16 bytes per lane) ----
    // One wave instruction fills 1 KiB of consecutive LDS, i.e. 1024 / (2 LD) padded rows: instruction q of a tile covers
    // bytes 1024 q .. 1024 q + 1023 of its LDS image, and the lane that falls on row padding re-reads the row's first chunk.
    // Rows at or past the document's end re-read its last row: finite values that only ever meet masked probabilities.
    // NWAVES waves share the NQ instructions of a tile: wave w issues q = w, w + NWAVES, ...
    static constexpr int NQ = (ROWS * LD * 2 + 1023) / 1024;
    static_assert(ROWS * LD * 2 % 1024 == 0, "a tile is a whole number of 1 KiB pieces");
    template <int NWAVES>
    struct Direct {
        static constexpr int NJ = (NQ + NWAVES - 1) / NWAVES;
        uint32_t off[NJ];  // global byte offset of this lane's chunk from the tile's first row, per instruction
        // last: last valid row of the tile (63, or fewer in a document's ragged last tile: later rows re-read it)
        __device__ __forceinline__ void init(int64_t ss, int lane, int wave, int last) {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int q = wave + NWAVES * j;
                const int byte = q * 1024 + lane * 16;
                int row = byte / (LD * 2);
                int colb = byte - row * (LD * 2);
                colb = colb < D * 2 ? colb : 0;
                row = row < last ? row : last;
                off[j] = (uint32_t)row * (uint32_t)(ss * 2) + (uint32_t)colb;
            }
        }
        // tile_rows: global address of the tile's first row (head column included); stage: its LDS image
        __device__ __forceinline__ void issue(const bf16_t* tile_rows, bf16_t* stage, int wave) const {
            // (the buffer form of the load: while a global load to LDS is in flight the compiler, which books it as a flat
            // access, turns every counted wait on LDS reads into a full drain)
            const __amdgpu_buffer_rsrc_t g = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<char*>(reinterpret_cast<const char*>(tile_rows)), 0, 0xffffffffu, 0x00020000);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int q = wave + NWAVES * j;
                if (q < NQ) __builtin_amdgcn_raw_ptr_buffer_load_lds(g, (lds_void*)(stage + q * 512), 16, off[j], 0, 0, 0);
            }
        }
    };
    // operand whose k index is d:   lane -> row (row0 + lane&31), d = kd*16 + 8*(lane>>5) ..+7
    static __device__ __forceinline__ bf16x8 frag_kc(const bf16_t* __restrict__ s, int row0, int kd, int lane) {
        return *reinterpret_cast<const bf16x8*>(s + (row0 + (lane & 31)) * LD + kd * 16 + (lane >> 5) * 8);
    }
    // operand whose k index is the tile row: lane -> d column (col0 + lane&31); k values are tile rows
    // krow0 + 4g + {0..3} and krow0 + 8 + 4g + {0..3}, g = lane>>5 -- the order in which a 32x32
    // accumulator block holds 16 consecutive rows, so accumulators convert straight to the B operand.
    static __device__ __forceinline__ bf16x8 frag_tr(const bf16_t* __restrict__ s, int krow0, int col0, int lane) {
        const int q = lane >> 4;
        const bf16_t* p = s + (krow0 + 4 * (lane >> 5) + ((lane & 15) >> 2)) * LD + col0 + (q & 1) * 16 + ((lane & 3) << 2);
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p));
        const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p + 8 * LD));
        bf16x8 v;
        v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
        v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
        return v;
    }
    // ---- fragments of the 16x16x32 MFMA (l16 = lane & 15, j4 = lane >> 4) ----
    // (the tile pointers are __restrict__ so that the reads carry a no-alias tag: an untagged LDS read waits for every tile
    // load in flight)
    // A operand whose k index is d: 16 tile rows row0 .., d = 32 ds + 8 j4 .. + 7
    static __device__ __forceinline__ bf16x8 frag_kc16(const bf16_t* __restrict__ s, int row0, int ds, int lane) {
        return *reinterpret_cast<const bf16x8*>(s + (row0 + (lane & 15)) * LD + ds * 32 + (lane >> 4) * 8);
    }
    // A operand whose k index is the tile row: lane -> d column col0 + l16; k slots 8 j4 + e are tile rows krow0 + 4 j4 + e
    // (e < 4) and krow0 + 16 + 4 j4 + e - 4 (e >= 4): the order in which two stacked 16-row accumulator tiles hold them
    static __device__ __forceinline__ bf16x8 frag_tr16(const bf16_t* __restrict__ s, int krow0, int col0, int lane) {
        const bf16_t* a = s + (krow0 + 4 * (lane >> 4) + ((lane & 15) >> 2)) * LD + col0 + ((lane & 3) << 2);
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(a));
        const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(a + 16 * LD));
        bf16x8 v;
        v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
        v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
        return v;
    }
};

// registers 8t .. 8t+7 of an accumulator block as a bf16 B operand
__device__ __forceinline__ bf16x8 acc_to_b(const f32x16& a, int t) {
    bf16x8 v;
    if (t == 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (bf16_t)a[e];
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (bf16_t)a[8 + e];
    }
    return v;
}

// row of register r inside a 32-row accumulator block
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// one operand row per lane, straight from global memory, as D/16 B-operand fragments
template <int D>
__device__ __forceinline__ void load_row_frags(const bf16_t* __restrict__ rowp, int lane, bf16x8* f) {
#pragma unroll
    for (int kd = 0; kd < D / 16; ++kd) f[kd] = *reinterpret_cast<const bf16x8*>(rowp + kd * 16 + (lane >> 5) * 8);
}

// =================================================================================================
// forward
// =================================================================================================
// f(integral_constant<int, I>) for I = I0 .. N-1, so that the body sees its index as a constant expression
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// The loop over the key tiles below the diagonal is software-pipelined inside each wave: iteration t issues the MFMAs of
// S(t+1) = K(t+1) Q^T and then of O += V(t) P(t), one per step, and between them the vector ALU work that turns S(t) into
// P(t) and, once S(t+1) is complete, takes its row maxima.  A sched_barrier after every step keeps that interleaving.  The
// K tiles therefore run one tile ahead of the V tiles in LDS.  The two tiles on the diagonal are done afterwards, one at a
// time with the mask.
template <int D>
__global__ __launch_bounds__(kThreads, 2) void attn_fwd_kernel(AttnParams p) {
    using TL = Tile<D>;
    // K0 V0 K1 V1: tile t of K or V in stage t & 1; then the block search's scratch
    __shared__ __attribute__((aligned(16))) bf16_t smem[4 * TL::ELEMS + 2 * kFindBlockInts];
    int doc_start, doc_len, qb;
    int bx, by;
    xcd_head_blocks(p.nq, bx, by);
    if (!find_block(p.cu, p.ndocs, p.s_len, p.T, bx, 128, doc_start, doc_len, qb, reinterpret_cast<int*>(smem + 4 * TL::ELEMS)))
        return;  // bx = rank: longest rows first
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hq = by, hk = hq / (p.nq / p.nk);
    const int q0 = qb * 128, qw0 = q0 + wave * 32;
    const int qi = qw0 + (lane & 31);                        // this lane's query (document relative)
    const int qtok = doc_start + (qi < doc_len ? qi : doc_len - 1);
    bf16x8 qf[D / 16];
    load_row_frags<D>(p.q + tok_off(qtok, p.s_len, p.q_ss, p.q_sb) + (int64_t)hq * D, lane, qf);

    const int kend = (q0 + 128 < doc_len ? q0 + 128 : doc_len);
    const int ntiles = (kend + 63) / 64;
    const int nmain = 2 * qb;  // tiles wholly below the diagonal for every query of the workgroup
    const int64_t kh = (int64_t)hk * D;
    const bf16_t* kbase = p.k + tok_off(doc_start, p.s_len, p.k_ss, p.k_sb) + kh;
    const bf16_t* vbase = p.v + tok_off(doc_start, p.s_len, p.v_ss, p.v_sb) + kh;
    typename TL::template Direct<kThreads / 64> kld, vld;
    kld.init(p.k_ss, lane, wave, 63);
    vld.init(p.v_ss, lane, wave, 63);
    // which: 0 = K tile t, 1 = V tile t
    auto issue_one = [&](int t, int which) {
        const int row0 = t * 64;
        bf16_t* dst = smem + (t & 1) * 2 * TL::ELEMS + which * TL::ELEMS;
        const bf16_t* src = (which ? vbase + (int64_t)row0 * p.v_ss : kbase + (int64_t)row0 * p.k_ss);
        if (row0 + 64 <= doc_len) {
            if (which) vld.issue(src, dst, wave);
            else kld.issue(src, dst, wave);
        } else {  // the document's ragged last tile: rows past its end re-read its last row
            typename TL::template Direct<kThreads / 64> e;
            e.init(which ? p.v_ss : p.k_ss, lane, wave, doc_len - 1 - row0);
            e.issue(src, dst, wave);
        }
    };
    issue_one(0, 0);
    issue_one(0, 1);
    if (ntiles > 1) issue_one(1, 0);
    // every load issued so far (the per-lane operand rows included) has landed before the loop starts
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    f32x16 oacc[D / 32];
#pragma unroll
    for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;
    const float sl2 = p.scale * kLog2e;
    const float tau = 8.0f / sl2;  // 2^8 in units of the raw scores

    constexpr int KD = D / 16;   // K fragments per 32 keys
    constexpr int NKF = 2 * KD;  // K fragments of a tile
    constexpr int NVF = 4 * (D / 32);  // V fragments of a tile
    constexpr int NSTEP = NKF + NVF;
    auto scores1 = [&](int t, f32x16 (&s)[2]) {
        const bf16_t* sK = smem + (t & 1) * 2 * TL::ELEMS;
        bf16x8 fk[2][4];
        constexpr int KG = D / 64, NG = 2 * KG;
        auto ldk = [&](int g, int buf) {
#pragma unroll
            for (int i = 0; i < 4; ++i) fk[buf][i] = TL::frag_kc(sK, (g / KG) * 32, (g % KG) * 4 + i, lane);
        };
        ldk(0, 0);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[kb][r] = 0.f;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            if (g + 1 < NG) ldk(g + 1, (g + 1) & 1);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                s[g / KG] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fk[g & 1][i], qf[(g % KG) * 4 + i], s[g / KG], 0, 0, 0);
        }
    };
    auto rowmax = [&](const f32x16 (&s)[2]) {
        float v = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) v = fmaxf(v, s[kb][r]);
        return fmaxf(v, __shfl_xor(v, 32, 64));
    };
    // The reference point m of the exponentials only has to bound them, not equal the running maximum: it is moved (and
    // O, l rescaled) only when some row of the wave has outgrown it by more than a factor 2^8, which after the first tiles
    // is rare.  Probabilities then reach at most 2^8 before the final division by l.
    auto rescale = [&](float mloc) {
        const float mnew = fmaxf(m, mloc);
        const float alpha = __builtin_amdgcn_exp2f((m - (mnew == -INFINITY ? 0.f : mnew)) * sl2);  // m = -inf: 0
        lsum *= alpha;
#pragma unroll
        for (int i = 0; i < D / 32; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[i][r] *= alpha;
        m = mnew;
    };

    f32x16 cur[2], nxt[2];
    scores1(0, cur);  // tile 0 concerns every wave
    float mloc = rowmax(cur);
    bool need = true;
    // every wave has finished reading K(0) before the first iteration refills its stage with K(2)
    __syncthreads();
    for (int t = 0; t < nmain; ++t) {
        if (need) rescale(mloc);
        // K stage t & 1: K(t) was last read by the scores of the previous iteration (t = 0: by scores1 above), i.e. before
        // the barrier every wave has passed since
        if (t + 2 < ntiles) issue_one(t + 2, 0);
        issue_one(t + 1, 1);                      // V stage (t+1) & 1: V(t-1) likewise; t + 1 <= nmain < ntiles
        {
            const bf16_t* sK = smem + ((t + 1) & 1) * 2 * TL::ELEMS;
            const bf16_t* sV = smem + (t & 1) * 2 * TL::ELEMS + TL::ELEMS;
            const float moff = m * sl2;
            float ps = 0.f, mx = -INFINITY;
            bf16x8 pf[4];
            bf16x8 fr[4];
            auto frag = [&](int i) {
                if (i < NKF) return TL::frag_kc(sK, (i / KD) * 32, i % KD, lane);
                const int j = i - NKF;
                return TL::frag_tr(sV, (j / (D / 32)) * 16, (j % (D / 32)) * 32, lane);
            };
            fr[0] = frag(0);
            fr[1] = frag(1);
            fr[2] = frag(2);
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) nxt[kb][r] = 0.f;
            static_for<0, NSTEP>([&](auto ST) {
                constexpr int i = decltype(ST)::value;
                if constexpr (i + 3 < NSTEP) fr[(i + 3) % 4] = frag(i + 3);
                if constexpr (i < NKF) {
                    nxt[i / KD] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[i % 4], qf[i % KD], nxt[i / KD], 0, 0, 0);
                } else {
                    constexpr int j = i - NKF;
                    oacc[j % (D / 32)] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[i % 4], pf[j / (D / 32)], oacc[j % (D / 32)], 0, 0, 0);
                }
                // P(t): the 32 probabilities of this lane, 32 / NKF per step during the first NKF steps (16 keys' worth,
                // one B operand of the O MFMAs, every NKF / 4 steps)
                if constexpr (i < NKF) {
                    constexpr int per = 32 / NKF;  // probabilities per step
#pragma unroll
                    for (int n = i * per; n < (i + 1) * per; ++n)
                        cur[n / 16][n % 16] = __builtin_amdgcn_exp2f(__builtin_fmaf(cur[n / 16][n % 16], sl2, -moff));
                }
                // the sums and the conversion to bf16 trail the exponentials by one step, so that no instruction waits for
                // the result of the one before it
                if constexpr (i >= 1 && i <= NKF) {
                    constexpr int per = 32 / NKF;
#pragma unroll
                    for (int n = (i - 1) * per; n < i * per; ++n) {
                        const int g = n / 8, e = n % 8;
                        ps += cur[n / 16][n % 16];
                        pf[g][e] = (bf16_t)cur[n / 16][n % 16];
                    }
                }
                if constexpr (i >= NKF) {  // S(t+1) is complete: out of the accumulators, and its maximum
                    constexpr int per = 32 / NVF;
#pragma unroll
                    for (int n = (i - NKF) * per; n < (i - NKF + 1) * per; ++n) {
                        cur[n / 16][n % 16] = nxt[n / 16][n % 16];
                        mx = fmaxf(mx, cur[n / 16][n % 16]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            lsum += ps;
            mloc = fmaxf(mx, __shfl_xor(mx, 32, 64));
            need = __builtin_amdgcn_ballot_w64(mloc > m + tau) != 0;
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's pieces of the tiles in flight are in LDS
        __syncthreads();
    }
    // ---- the tiles on the diagonal; cur holds S(nmain) ----
    for (int t = nmain; t < ntiles; ++t) {
        if (t + 2 < ntiles) issue_one(t + 2, 0);
        if (t + 1 < ntiles) issue_one(t + 1, 1);
        const bf16_t* sV = smem + (t & 1) * 2 * TL::ELEMS + TL::ELEMS;
        const int key0 = t * 64;
        if (key0 <= qw0 + 31) {  // otherwise every key of the tile is after every query of this wave
            bf16x8 fv[2][D / 32];
            auto ldv = [&](int g, int buf) {
#pragma unroll
                for (int db = 0; db < D / 32; ++db) fv[buf][db] = TL::frag_tr(sV, (g >> 1) * 32 + 16 * (g & 1), db * 32, lane);
            };
            ldv(0, 0);
            if (key0 + 63 > qw0) {  // the tile touches the diagonal: mask keys after the query
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        if (key0 + kb * 32 + acc_row(r, lane) > qi) cur[kb][r] = -INFINITY;
            }
            const float ml = rowmax(cur);
            if (__builtin_amdgcn_ballot_w64(ml > m + tau) != 0) rescale(ml);
            const float moff = (m == -INFINITY ? 0.f : m) * sl2;
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(cur[kb][r], sl2, -moff));
                    cur[kb][r] = pe;
                    psum += pe;
                }
            lsum += psum;
            // O^T += V^T P^T, 4 groups of (16 keys x all d blocks)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (g + 1 < 4) ldv(g + 1, (g + 1) & 1);
                const bf16x8 pfr = acc_to_b(cur[g >> 1], g & 1);
#pragma unroll
                for (int db = 0; db < D / 32; ++db)
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fv[g & 1][db], pfr, oacc[db], 0, 0, 0);
            }
        }
        if (t + 1 < ntiles && (t + 1) * 64 <= qw0 + 31) scores1(t + 1, cur);  // K(t+1) arrived before the previous barrier
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    }
    const float ltot = lsum + __shfl_xor(lsum, 32, 64);
    if (qi < doc_len) {
        const float inv = 1.0f / ltot;
        bf16_t* orow = p.out + tok_off(doc_start + qi, p.s_len, p.o_ss, p.o_sb) + (int64_t)hq * D;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                bf16x4 w;
#pragma unroll
                for (int e = 0; e < 4; ++e) w[e] = (bf16_t)(oacc[db][r4 * 4 + e] * inv);
                *reinterpret_cast<bf16x4*>(orow + db * 32 + 8 * r4 + 4 * (lane >> 5)) = w;
            }
        if (lane < 32) p.lse[(int64_t)hq * p.T + doc_start + qi] = m * p.scale + __builtin_amdgcn_logf(ltot) * kLn2;
    }
}

// =================================================================================================
// backward, dK and dV: a block owns 128 keys of one kv head and walks the queries at or after them
// =================================================================================================
// 8 waves: wave w works on keys 32 (w & 3) .. +31 and, of every 64-query tile, on the 32-query half (w >> 2); the two
// waves that share a key group sit on the same SIMD, so the elementwise phase of one overlaps the MFMAs of the other.
// To leave room for two waves per SIMD the K / V operand rows live in LDS (read as fragments per use) instead of in
// registers; the two partial dK / dV of a key group are added through LDS at the end, always in the same order.
constexpr int kDkdvThreads = 512;

template <int D>
__global__ __launch_bounds__(kDkdvThreads) void attn_bwd_dkdv_kernel(AttnParams p) {
    using TL = Tile<D>;
    constexpr int LD = TL::LD, CH = TL::CH;
    constexpr int KV_ELEMS = 128 * LD;     // K (or V) rows of the block's 128 keys
    constexpr int STAGE = 2 * TL::ELEMS;   // Q tile + dO tile, 64 rows each
    constexpr int NCH_KV = 128 * CH / kDkdvThreads, NCH_Q = 64 * CH / kDkdvThreads;
    __shared__ __attribute__((aligned(16))) bf16_t smem[2 * KV_ELEMS + 2 * STAGE];  // K V | (Q dO) x 2 stages
    __shared__ __attribute__((aligned(16))) float sstat[2][2][64];                   // [stage][lse*log2e | delta][query]
    static_assert(sizeof(bf16_t) * (2 * KV_ELEMS + 2 * STAGE) >= sizeof(float) * 4 * 2 * (D / 32) * 16 * 64,
                  "the final reduction parks four waves' accumulators in the tile memory");
    int doc_start, doc_len, kbk;
    int bx, by;
    xcd_head_blocks(p.nk * p.nsplit, bx, by);
    __shared__ int s_find[kFindBlockInts];  // (no tile loads straight into LDS in this kernel: several LDS variables do no harm)
    if (!find_block(p.cu, p.ndocs, p.s_len, p.T, bx, 128, doc_start, doc_len, kbk, s_find)) return;
    kbk = (doc_len + 127) / 128 - 1 - kbk;  // rank 0 = most blocks of queries to walk = the piece's first keys
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = wave & 3, half = wave >> 2;
    // With a large GQA group a (kv head, key block) is long and there are few of them: the group's query heads are dealt
    // to nsplit workgroups, each leaving fp32 partial sums that attn_dkdv_combine_kernel adds in a fixed order.
    const int hk = by / p.nsplit, part = by - hk * p.nsplit;
    const int group = p.nq / p.nk / p.nsplit, hq0 = hk * (p.nq / p.nk) + part * group;
    const int k0 = kbk * 128, kw0 = k0 + kg * 32;
    const int tok_end = doc_start + doc_len;
    const int kj = kw0 + (lane & 31);  // this lane's key (document relative)
    bf16_t* sK = smem;
    bf16_t* sV = smem + KV_ELEMS;
    bf16_t* sQ0 = smem + 2 * KV_ELEMS;

    {   // K / V rows of the block: rows past the document's end re-read its last row (always masked)
        const bf16_t* kdoc = p.k + tok_off(doc_start, p.s_len, p.k_ss, p.k_sb) + (int64_t)hk * D;
        const bf16_t* vdoc = p.v + tok_off(doc_start, p.s_len, p.v_ss, p.v_sb) + (int64_t)hk * D;
        bf16x8 rk[NCH_KV], rv[NCH_KV];
#pragma unroll
        for (int i = 0; i < NCH_KV; ++i) {
            const int c = tid + kDkdvThreads * i;
            int n = k0 + c / CH;
            n = n < doc_len ? n : doc_len - 1;
            rk[i] = *reinterpret_cast<const bf16x8*>(kdoc + (int64_t)n * p.k_ss + (c % CH) * 8);
            rv[i] = *reinterpret_cast<const bf16x8*>(vdoc + (int64_t)n * p.v_ss + (c % CH) * 8);
        }
#pragma unroll
        for (int i = 0; i < NCH_KV; ++i) {
            const int c = tid + kDkdvThreads * i;
            *reinterpret_cast<bf16x8*>(sK + (c / CH) * LD + (c % CH) * 8) = rk[i];
            *reinterpret_cast<bf16x8*>(sV + (c / CH) * LD + (c % CH) * 8) = rv[i];
        }
    }

    f32x16 dkacc[D / 32], dvacc[D / 32];
#pragma unroll
    for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dkacc[i][r] = 0.f; dvacc[i][r] = 0.f; }

    const int qt0 = k0 / 64;                      // first query tile that can see these keys
    const int nqt = (doc_len + 63) / 64 - qt0;    // query tiles per head
    const int total = nqt * group;                // flattened (head in group, query tile) iterations
    const float sl2 = p.scale * kLog2e;

    const bf16_t* qdoc = p.q + tok_off(doc_start, p.s_len, p.q_ss, p.q_sb);
    const bf16_t* dodoc = p.dout + tok_off(doc_start, p.s_len, p.do_ss, p.do_sb);
    bf16x8 rq[NCH_Q], rdo[NCH_Q];
    float rstat = 0.f;  // threads 0..63: lse*log2e of query tid; 64..127: delta of query tid-64
    auto load_iter = [&](int it) {
        const int hq = hq0 + it / nqt;
        const int row0 = (qt0 + it % nqt) * 64;
#pragma unroll
        for (int i = 0; i < NCH_Q; ++i) {
            const int c = tid + kDkdvThreads * i;
            int n = row0 + c / CH;
            n = n < doc_len ? n : doc_len - 1;
            rq[i] = *reinterpret_cast<const bf16x8*>(qdoc + (int64_t)hq * D + (int64_t)n * p.q_ss + (c % CH) * 8);
            rdo[i] = *reinterpret_cast<const bf16x8*>(dodoc + (int64_t)hq * D + (int64_t)n * p.do_ss + (c % CH) * 8);
        }
        if (tid < 128) {
            const int n = doc_start + row0 + (tid & 63);
            rstat = 0.f;
            if (n < tok_end) rstat = tid < 64 ? p.lse[(int64_t)hq * p.T + n] * kLog2e : p.delta[(int64_t)hq * p.T + n];
        }
    };
    auto store_iter = [&](int stage) {
        bf16_t* sq = sQ0 + stage * STAGE;
#pragma unroll
        for (int i = 0; i < NCH_Q; ++i) {
            const int c = tid + kDkdvThreads * i;
            *reinterpret_cast<bf16x8*>(sq + (c / CH) * LD + (c % CH) * 8) = rq[i];
            *reinterpret_cast<bf16x8*>(sq + TL::ELEMS + (c / CH) * LD + (c % CH) * 8) = rdo[i];
        }
        if (tid < 128) sstat[stage][tid >> 6][tid & 63] = rstat;
    };
    load_iter(0);
    store_iter(0);
    if (total > 1) load_iter(1);
    __syncthreads();

    for (int it = 0; it < total; ++it) {
        const int cur = it & 1;
        const bf16_t* sQ = sQ0 + cur * STAGE;
        const bf16_t* sdO = sQ + TL::ELEMS;
        if (it + 1 < total) store_iter(cur ^ 1);
        if (it + 2 < total) load_iter(it + 2);
        const int qbase = (qt0 + it % nqt) * 64;
        const int qs0 = qbase + half * 32;
        if (!(qs0 + 31 < kw0 || qs0 >= doc_len)) {  // else: all queries before this wave's keys / past the end
            // S = Q K^T and dP = dO V^T, one d-step (4 fragments, 2 MFMAs) at a time with the next step's fragments in flight
            constexpr int NS = D / 16;
            f32x16 sacc, dpacc;
            bf16x8 fq[2], fo[2], fk[2], fv[2];
            auto lda = [&](int g, int buf) {
                fq[buf] = TL::frag_kc(sQ, half * 32, g, lane);
                fk[buf] = TL::frag_kc(sK, kg * 32, g, lane);
                fo[buf] = TL::frag_kc(sdO, half * 32, g, lane);
                fv[buf] = TL::frag_kc(sV, kg * 32, g, lane);
            };
            lda(0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; dpacc[r] = 0.f; }
#pragma unroll
            for (int g = 0; g < NS; ++g) {
                if (g + 1 < NS) lda(g + 1, (g + 1) & 1);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fq[g & 1], fk[g & 1], sacc, 0, 0, 0);
                dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fo[g & 1], fv[g & 1], dpacc, 0, 0, 0);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
            for (int g = 0; g < NS; ++g) {
                if (g + 1 < NS) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
            // dO^T / Q^T fragments, two d blocks at a time; the first pair's latency hides under the elementwise math
            constexpr int NT = 2 * (D / 64);  // (16-query step, d-block pair) groups
            bf16x8 fto[2][2], ftq[2][2];
            auto ldt = [&](int gt, int buf) {
                const int tt = gt / (D / 64), dbp = gt % (D / 64);
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    fto[buf][i] = TL::frag_tr(sdO, half * 32 + 16 * tt, (2 * dbp + i) * 32, lane);
                    ftq[buf][i] = TL::frag_tr(sQ, half * 32 + 16 * tt, (2 * dbp + i) * 32, lane);
                }
            };
            ldt(0, 0);
            // accumulator register r <-> query qs0 + acc_row(r); lane <-> key kj.  Only a tile that meets the diagonal of this
            // wave's keys or the document's end needs the mask (a wave-uniform property).
            auto probabilities = [&](auto MASKED) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int ql = half * 32 + 8 * r4 + 4 * (lane >> 5);
                    const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sstat[cur][0][ql]);
                    const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sstat[cur][1][ql]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = r4 * 4 + e;
                        float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[r], sl2, -l4[e]));
                        if constexpr (decltype(MASKED)::value) {
                            const int qidx = qbase + ql + e;
                            if (kj > qidx || qidx >= doc_len) pe = 0.f;
                        }
                        sacc[r] = pe;
                        dpacc[r] = pe * (dpacc[r] - d4[e]);
                    }
                }
            };
            if (qs0 < kw0 + 31 || qs0 + 32 > doc_len) probabilities(std::true_type{});
            else probabilities(std::false_type{});
#pragma unroll
            for (int gt = 0; gt < NT; ++gt) {
                if (gt + 1 < NT) ldt(gt + 1, (gt + 1) & 1);
                const int tt = gt / (D / 64), dbp = gt % (D / 64);
                const bf16x8 pf = acc_to_b(sacc, tt);
                const bf16x8 dsf = acc_to_b(dpacc, tt);
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    dvacc[2 * dbp + i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fto[gt & 1][i], pf, dvacc[2 * dbp + i], 0, 0, 0);
                    dkacc[2 * dbp + i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ftq[gt & 1][i], dsf, dkacc[2 * dbp + i], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }

    // fold the two halves of every key group: waves 4..7 park their accumulators in LDS (32 KiB each, lane-contiguous),
    // waves 0..3 add them to their own and write the rows out
    float* red = reinterpret_cast<float*>(smem) + (size_t)kg * (2 * (D / 32) * 16 * 64);
    if (half == 1) {
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                red[(db * 16 + r) * 64 + lane] = dkacc[db][r];
                red[((D / 32 + db) * 16 + r) * 64 + lane] = dvacc[db][r];
            }
    }
    __syncthreads();
    if (half == 0 && kj < doc_len) {
        if (p.nsplit > 1) {  // fp32 partial sums of this workgroup's query heads, unscaled
            const int64_t slab = (int64_t)p.T * p.nk * D;
            float* pk = p.part + (int64_t)part * 2 * slab + ((int64_t)(doc_start + kj) * p.nk + hk) * D;
            float* pv = pk + slab;
#pragma unroll
            for (int db = 0; db < D / 32; ++db)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    f32x4 a, b;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = r4 * 4 + e;
                        a[e] = dkacc[db][r] + red[(db * 16 + r) * 64 + lane];
                        b[e] = dvacc[db][r] + red[((D / 32 + db) * 16 + r) * 64 + lane];
                    }
                    const int dcol = db * 32 + 8 * r4 + 4 * (lane >> 5);
                    *reinterpret_cast<f32x4*>(pk + dcol) = a;
                    *reinterpret_cast<f32x4*>(pv + dcol) = b;
                }
            return;
        }
        bf16_t* dkrow = p.dk + tok_off(doc_start + kj, p.s_len, p.dk_ss, p.dk_sb) + (int64_t)hk * D;
        bf16_t* dvrow = p.dv + tok_off(doc_start + kj, p.s_len, p.dv_ss, p.dv_sb) + (int64_t)hk * D;
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                bf16x4 a, b;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = r4 * 4 + e;
                    a[e] = (bf16_t)((dkacc[db][r] + red[(db * 16 + r) * 64 + lane]) * p.scale);
                    b[e] = (bf16_t)(dvacc[db][r] + red[((D / 32 + db) * 16 + r) * 64 + lane]);
                }
                const int dcol = db * 32 + 8 * r4 + 4 * (lane >> 5);
                *reinterpret_cast<bf16x4*>(dkrow + dcol) = a;
                *reinterpret_cast<bf16x4*>(dvrow + dcol) = b;
            }
    }
}

// dK = scale * sum_parts partial dK, dV = sum_parts partial dV, parts added in index order; one thread per 8 columns
template <int D>
__global__ __launch_bounds__(kThreads) void attn_dkdv_combine_kernel(AttnParams p) {
    const int64_t slab = (int64_t)p.T * p.nk * D;
    const int64_t chunks = slab / 8;
    for (int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x; c < chunks; c += (int64_t)gridDim.x * kThreads) {
        const int64_t e0 = c * 8;
        const int n = (int)(e0 / ((int64_t)p.nk * D));
        const int rem = (int)(e0 - (int64_t)n * p.nk * D);  // head * D + column
        float k8[8], v8[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { k8[i] = 0.f; v8[i] = 0.f; }
        for (int s = 0; s < p.nsplit; ++s) {
            const float* pk = p.part + (int64_t)s * 2 * slab + e0;
            const f32x4 a0 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pk));
            const f32x4 a1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pk + 4));
            const f32x4 b0 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pk + slab));
            const f32x4 b1 = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pk + slab + 4));
#pragma unroll
            for (int i = 0; i < 4; ++i) { k8[i] += a0[i]; k8[4 + i] += a1[i]; v8[i] += b0[i]; v8[4 + i] += b1[i]; }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) k8[i] *= p.scale;
        st_bf16x8(p.dk + tok_off(n, p.s_len, p.dk_ss, p.dk_sb) + rem, pack8(k8));
        st_bf16x8(p.dv + tok_off(n, p.s_len, p.dv_ss, p.dv_sb) + rem, pack8(v8));
    }
}

// =================================================================================================
// backward, dQ: a block owns 128 queries of one head (32 per wave) and walks the keys at or before them
// =================================================================================================
// MFMA 16x16x32: A operand lane l = row (l & 15), k = 8 (l >> 4) .. + 7; B operand lane l = column (l & 15), same k; result
// lane l = column (l & 15), rows 4 (l >> 4) .. + 3 in four registers.  A wave owns 32 queries = two 16-query groups qg.
//   S^T[16 keys x 16 q] = K frag (16 keys x 32 d, LDS) x Q frag (16 q x 32 d, registers), 4 d steps; likewise dP^T from V, dO
//   dQ^T[16 d x 16 q] += K^T frag (16 d x 32 keys, transposed LDS read) x dS^T (32 keys x 16 q, from the accumulators)
// A fragment read from LDS feeds two MFMAs (the two query groups), as one 32x32x16 fragment feeds one MFMA of twice the work.
typedef float f32x4v __attribute__((ext_vector_type(4)));

template <int D>
__global__ __launch_bounds__(kThreads, 2) void attn_bwd_dq_kernel(AttnParams p) {
    using TL = Tile<D>;
    constexpr int LD = TL::LD;
    __shared__ __attribute__((aligned(16))) bf16_t smem[4 * TL::ELEMS + 2 * kFindBlockInts];  // K0 V0 K1 V1, block search scratch
    int doc_start, doc_len, qb;
    int bx, by;
    xcd_head_blocks(p.nq, bx, by);
    if (!find_block(p.cu, p.ndocs, p.s_len, p.T, bx, 128, doc_start, doc_len, qb, reinterpret_cast<int*>(smem + 4 * TL::ELEMS))) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hq = by, hk = hq / (p.nq / p.nk);
    const int q0 = qb * 128, qw0 = q0 + wave * 32;
    const int j4 = lane >> 4, l16 = lane & 15;
    constexpr int NDS = D / 32;  // d steps of 32
    int qi[2];
    bf16x8 qf[2][NDS], dof[2][NDS];
    float lse2[2], dlt[2];
#pragma unroll
    for (int qg = 0; qg < 2; ++qg) {
        qi[qg] = qw0 + 16 * qg + l16;
        const int qtok = doc_start + (qi[qg] < doc_len ? qi[qg] : doc_len - 1);
        const bf16_t* qrow = p.q + tok_off(qtok, p.s_len, p.q_ss, p.q_sb) + (int64_t)hq * D;
        const bf16_t* dorow = p.dout + tok_off(qtok, p.s_len, p.do_ss, p.do_sb) + (int64_t)hq * D;
        const bf16_t* orow = p.o + tok_off(qtok, p.s_len, p.o_ss, p.o_sb) + (int64_t)hq * D;
        float acc = 0.f;
#pragma unroll
        for (int ds = 0; ds < NDS; ++ds) {
            qf[qg][ds] = *reinterpret_cast<const bf16x8*>(qrow + ds * 32 + j4 * 8);
            dof[qg][ds] = *reinterpret_cast<const bf16x8*>(dorow + ds * 32 + j4 * 8);
            const bf16x8 ov = *reinterpret_cast<const bf16x8*>(orow + ds * 32 + j4 * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc += (float)ov[e] * (float)dof[qg][ds][e];
        }
        // delta = sum_d dO * O of this lane's query: the four lanes l16 + 16 j hold a quarter of the row each
        acc += __shfl_xor(acc, 16, 64);
        acc += __shfl_xor(acc, 32, 64);
        dlt[qg] = acc;
        lse2[qg] = p.lse[(int64_t)hq * p.T + qtok] * kLog2e;
        if (j4 == 0 && qi[qg] < doc_len) p.delta[(int64_t)hq * p.T + doc_start + qi[qg]] = acc;
    }

    const int kend = (q0 + 128 < doc_len ? q0 + 128 : doc_len);
    const int ntiles = (kend + 63) / 64;
    const int64_t kh = (int64_t)hk * D;
    const bf16_t* kbase = p.k + tok_off(doc_start, p.s_len, p.k_ss, p.k_sb) + kh;
    const bf16_t* vbase = p.v + tok_off(doc_start, p.s_len, p.v_ss, p.v_sb) + kh;
    typename TL::template Direct<kThreads / 64> kld, vld;
    kld.init(p.k_ss, lane, wave, 63);
    vld.init(p.v_ss, lane, wave, 63);
    auto issue_tile = [&](int t, int stage) {
        const int row0 = t * 64;
        bf16_t* sk = smem + stage * 2 * TL::ELEMS;
        if (row0 + 64 <= doc_len) {
            kld.issue(kbase + (int64_t)row0 * p.k_ss, sk, wave);
            vld.issue(vbase + (int64_t)row0 * p.v_ss, sk + TL::ELEMS, wave);
        } else {  // the document's ragged last tile: rows past its end re-read its last row
            typename TL::template Direct<kThreads / 64> ke, ve;
            ke.init(p.k_ss, lane, wave, doc_len - 1 - row0);
            ve.init(p.v_ss, lane, wave, doc_len - 1 - row0);
            ke.issue(kbase + (int64_t)row0 * p.k_ss, sk, wave);
            ve.issue(vbase + (int64_t)row0 * p.v_ss, sk + TL::ELEMS, wave);
        }
    };
    issue_tile(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    f32x4v dqacc[D / 16][2];
#pragma unroll
    for (int i = 0; i < D / 16; ++i)
#pragma unroll
        for (int qg = 0; qg < 2; ++qg)
#pragma unroll
            for (int r = 0; r < 4; ++r) dqacc[i][qg][r] = 0.f;
    const float sl2 = p.scale * kLog2e;

    for (int t = 0; t < ntiles; ++t) {
        const int cur = t & 1;
        const bf16_t* sK = smem + cur * 2 * TL::ELEMS;
        const bf16_t* sV = sK + TL::ELEMS;
        if (t + 1 < ntiles) issue_tile(t + 1, cur ^ 1);  // that stage was last read before the barrier that ended tile t-1
        const int key0 = t * 64;
        if (key0 <= qw0 + 31) {
            const bool on_diag = key0 + 63 > qw0;
#pragma unroll
            for (int pb = 0; pb < 2; ++pb) {  // 32 keys at a time
                f32x4v sacc[2][2], dpacc[2][2];  // [16-key group][query group]
#pragma unroll
                for (int kg = 0; kg < 2; ++kg)
#pragma unroll
                    for (int qg = 0; qg < 2; ++qg)
#pragma unroll
                        for (int r = 0; r < 4; ++r) { sacc[kg][qg][r] = 0.f; dpacc[kg][qg][r] = 0.f; }
                // S^T and dP^T: per (key group, d step) one K and one V fragment, four MFMAs; next fragments in flight
                constexpr int NST = 2 * NDS;
                bf16x8 fk[2], fv[2];
                auto ld = [&](int st, int buf) {
                    fk[buf] = TL::frag_kc16(sK, pb * 32 + (st / NDS) * 16, st % NDS, lane);
                    fv[buf] = TL::frag_kc16(sV, pb * 32 + (st / NDS) * 16, st % NDS, lane);
                };
                ld(0, 0);
#pragma unroll
                for (int st = 0; st < NST; ++st) {
                    if (st + 1 < NST) ld(st + 1, (st + 1) & 1);
                    const int kg = st / NDS, ds = st % NDS;
#pragma unroll
                    for (int qg = 0; qg < 2; ++qg) {
                        sacc[kg][qg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fk[st & 1], qf[qg][ds], sacc[kg][qg], 0, 0, 0);
                        dpacc[kg][qg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fv[st & 1], dof[qg][ds], dpacc[kg][qg], 0, 0, 0);
                    }
                }
                // K^T fragments of the first d tiles: issued before the elementwise math
                constexpr int NDT = D / 16;
                bf16x8 ftk[2];
                ftk[0] = TL::frag_tr16(sK, pb * 32, 0, lane);
                bf16x8 dsf[2];
                // register r of tile (kg, qg) <-> key key0 + 32 pb + 16 kg + 4 j4 + r, query qi[qg]; the mask is needed only on
                // the tile that meets the diagonal (a wave-uniform property: two instantiations of the loop)
                auto dscores = [&](auto MASKED) {
#pragma unroll
                    for (int qg = 0; qg < 2; ++qg) {
#pragma unroll
                        for (int kg = 0; kg < 2; ++kg)
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kg][qg][r], sl2, -lse2[qg]));
                                if constexpr (decltype(MASKED)::value) {
                                    if (key0 + pb * 32 + kg * 16 + 4 * j4 + r > qi[qg]) pe = 0.f;
                                }
                                dsf[qg][kg * 4 + r] = (bf16_t)(pe * (dpacc[kg][qg][r] - dlt[qg]));
                            }
                    }
                };
                if (on_diag) dscores(std::true_type{});
                else dscores(std::false_type{});
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    if (dt + 1 < NDT) ftk[(dt + 1) & 1] = TL::frag_tr16(sK, pb * 32, (dt + 1) * 16, lane);
#pragma unroll
                    for (int qg = 0; qg < 2; ++qg)
                        dqacc[dt][qg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ftk[dt & 1], dsf[qg], dqacc[dt][qg], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's pieces of the next tile are in LDS
        __syncthreads();
    }
#pragma unroll
    for (int qg = 0; qg < 2; ++qg) {
        if (qi[qg] >= doc_len) continue;
        bf16_t* dqrow = p.dq + tok_off(doc_start + qi[qg], p.s_len, p.dq_ss, p.dq_sb) + (int64_t)hq * D;
#pragma unroll
        for (int dt = 0; dt < D / 16; ++dt) {
            bf16x4 w;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[e] = (bf16_t)(dqacc[dt][qg][e] * p.scale);
            *reinterpret_cast<bf16x4*>(dqrow + dt * 16 + 4 * j4) = w;
        }
    }
}
// (explicit: the launches below alone have left the host-side launch stubs of some of these kernels undefined)
template __global__ void attn_fwd_kernel<128>(AttnParams);
template __global__ void attn_fwd_kernel<64>(AttnParams);
template __global__ void attn_bwd_dkdv_kernel<128>(AttnParams);
template __global__ void attn_bwd_dkdv_kernel<64>(AttnParams);
template __global__ void attn_dkdv_combine_kernel<128>(AttnParams);
template __global__ void attn_dkdv_combine_kernel<64>(AttnParams);
template __global__ void attn_bwd_dq_kernel<128>(AttnParams);
template __global__ void attn_bwd_dq_kernel<64>(AttnParams);

int check_common(const char* name, int64_t T, int64_t s_len, int64_t nq, int64_t nk, int64_t d, int64_t ndocs, const int64_t* strides,
                 int nstrides) {
    EZL_REQUIRE(d == 64 || d == 128, EZL_EUNSUPPORTED, "%s: head dim must be 64 or 128 (got %lld)", name, (long long)d);
    EZL_REQUIRE(nq > 0 && nk > 0 && nq % nk == 0, EZL_EINVAL, "%s: nq must be a positive multiple of nk", name);
    EZL_REQUIRE(T >= 0 && T < (1LL << 30) && (T == 0 || (s_len > 0 && T % s_len == 0)) && ndocs > 0 && ndocs < (1LL << 24), EZL_EINVAL,
                "%s: bad token / document counts", name);
    EZL_REQUIRE(nq < 65536, EZL_EUNSUPPORTED, "%s: too many heads", name);
    for (int i = 0; i < nstrides; ++i) EZL_REQUIRE(strides[i] % 8 == 0, EZL_EINVAL, "%s: strides must be multiples of 8 elements", name);
    return EZL_OK;
}

}  // namespace

// strides[8]: q_seq, q_batch, k_seq, k_batch, v_seq, v_batch, out_seq, out_batch (elements)
extern "C" int ezl_attn_fwd(const void* q, const void* k, const void* v, void* out, void* lse, const void* cu_seqlens, int64_t ndocs,
                            int64_t total_tokens, int64_t s_len, int64_t nq, int64_t nk, int64_t d, float scale,
                            const int64_t* strides, void* stream) {
    int rc = check_common("ezl_attn_fwd", total_tokens, s_len, nq, nk, d, ndocs, strides, 8);
    if (rc) return rc;
    if (total_tokens == 0) return EZL_OK;
    EZL_REQUIRE(q && k && v && out && lse && ezl_aligned16(q) && ezl_aligned16(k) && ezl_aligned16(v) && ezl_aligned16(out), EZL_EINVAL,
                "ezl_attn_fwd: null or misaligned pointer");
    AttnParams p = {};
    p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.out = (bf16_t*)out; p.lse = (float*)lse;
    p.cu = (const int*)cu_seqlens; p.ndocs = (int)ndocs; p.s_len = (int)s_len; p.T = (int)total_tokens; p.nq = (int)nq; p.nk = (int)nk;
    p.scale = scale;
    p.q_ss = strides[0]; p.q_sb = strides[1]; p.k_ss = strides[2]; p.k_sb = strides[3];
    p.v_ss = strides[4]; p.v_sb = strides[5]; p.o_ss = strides[6]; p.o_sb = strides[7];
    const dim3 grid((unsigned)((total_tokens + 127) / 128 + ndocs + total_tokens / s_len), (unsigned)nq);
    if (d == 128) hipLaunchKernelGGL(attn_fwd_kernel<128>, grid, dim3(kThreads), 0, (hipStream_t)stream, p);
    else hipLaunchKernelGGL(attn_fwd_kernel<64>, grid, dim3(kThreads), 0, (hipStream_t)stream, p);
    EZL_LAUNCH_CHECK("ezl_attn_fwd");
    return EZL_OK;
}

namespace {
// workgroups per (kv head, key block) of the dK/dV kernel: enough of them for two rounds of the 256 CUs, so that a long
// block from the start of a document and a short one from its end share a CU (measured at 64 q / 8 kv heads, s = 4096:
// 1080 us unsplit, 582 us with 2 parts, 578 us with 4 parts, whose partial sums cost twice as much to add)
int attn_bwd_split(int64_t total_tokens, int64_t ndocs, int64_t nq, int64_t nk) {
    const int64_t group = nq / nk;
    const int64_t blocks = nk * ((total_tokens + 127) / 128 + ndocs - 1);
    int split = 1;
    while (blocks * split < EZL_DKDV_MIN_BLOCKS && group % (split * 2) == 0) split *= 2;
    return split;
}
}  // namespace

extern "C" int64_t ezl_attn_bwd_workspace_bytes(int64_t total_tokens, int64_t ndocs, int64_t nq, int64_t nk, int64_t d) {
    if (total_tokens < 0 || ndocs <= 0 || nq <= 0 || nk <= 0 || nq % nk != 0 || d <= 0) return -1;
    const int split = attn_bwd_split(total_tokens, ndocs, nq, nk);
    return split > 1 ? (int64_t)split * 2 * total_tokens * nk * d * (int64_t)sizeof(float) : 0;
}

// strides[16]: q, k, v, out (as above), then dout, dq, dk, dv (seq, batch each)
extern "C" int ezl_attn_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout, const void* lse,
                            void* delta, void* dq, void* dk, void* dv, const void* cu_seqlens, int64_t ndocs, int64_t total_tokens,
                            int64_t s_len, int64_t nq, int64_t nk, int64_t d, float scale, const int64_t* strides, void* workspace,
                            int64_t workspace_bytes, void* stream) {
    int rc = check_common("ezl_attn_bwd", total_tokens, s_len, nq, nk, d, ndocs, strides, 16);
    if (rc) return rc;
    if (total_tokens == 0) return EZL_OK;
    EZL_REQUIRE(q && k && v && out && dout && lse && delta && dq && dk && dv, EZL_EINVAL, "ezl_attn_bwd: null pointer");
    EZL_REQUIRE(ezl_aligned16(q) && ezl_aligned16(k) && ezl_aligned16(v) && ezl_aligned16(out) && ezl_aligned16(dout) &&
                    ezl_aligned16(dq) && ezl_aligned16(dk) && ezl_aligned16(dv),
                EZL_EINVAL, "ezl_attn_bwd: misaligned pointer");
    const int64_t need = ezl_attn_bwd_workspace_bytes(total_tokens, ndocs, nq, nk, d);
    EZL_REQUIRE(need == 0 || (workspace && ezl_aligned16(workspace) && workspace_bytes >= need), EZL_EINVAL,
                "ezl_attn_bwd: workspace missing, misaligned or smaller than ezl_attn_bwd_workspace_bytes()");
    AttnParams p = {};
    p.q = (const bf16_t*)q; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v; p.o = (const bf16_t*)out; p.dout = (const bf16_t*)dout;
    p.lse = (float*)const_cast<void*>(lse); p.delta = (float*)delta; p.dq = (bf16_t*)dq; p.dk = (bf16_t*)dk; p.dv = (bf16_t*)dv;
    p.cu = (const int*)cu_seqlens; p.ndocs = (int)ndocs; p.s_len = (int)s_len; p.T = (int)total_tokens; p.nq = (int)nq; p.nk = (int)nk;
    p.scale = scale;
    p.nsplit = attn_bwd_split(total_tokens, ndocs, nq, nk);
    p.part = p.nsplit > 1 ? (float*)workspace : nullptr;
    p.q_ss = strides[0]; p.q_sb = strides[1]; p.k_ss = strides[2]; p.k_sb = strides[3];
    p.v_ss = strides[4]; p.v_sb = strides[5]; p.o_ss = strides[6]; p.o_sb = strides[7];
    p.do_ss = strides[8]; p.do_sb = strides[9]; p.dq_ss = strides[10]; p.dq_sb = strides[11];
    p.dk_ss = strides[12]; p.dk_sb = strides[13]; p.dv_ss = strides[14]; p.dv_sb = strides[15];
    hipStream_t st = (hipStream_t)stream;
    const unsigned nblk = (unsigned)((total_tokens + 127) / 128 + ndocs + total_tokens / s_len);
    const dim3 gridq(nblk, (unsigned)nq);
    const dim3 gridk(nblk, (unsigned)(nk * p.nsplit));
    int64_t gc = (total_tokens * nk * d / 8 + kThreads - 1) / kThreads;
    if (gc > 256 * 16) gc = 256 * 16;
    // the dQ kernel goes first: it also produces delta = rowsum(dO * O), which the dK/dV kernel reads
    if (d == 128) {
        hipLaunchKernelGGL(attn_bwd_dq_kernel<128>, gridq, dim3(kThreads), 0, st, p);
        hipLaunchKernelGGL(attn_bwd_dkdv_kernel<128>, gridk, dim3(kDkdvThreads), 0, st, p);
        if (p.nsplit > 1) hipLaunchKernelGGL(attn_dkdv_combine_kernel<128>, dim3((unsigned)gc), dim3(kThreads), 0, st, p);
    } else {
        hipLaunchKernelGGL(attn_bwd_dq_kernel<64>, gridq, dim3(kThreads), 0, st, p);
        hipLaunchKernelGGL(attn_bwd_dkdv_kernel<64>, gridk, dim3(kDkdvThreads), 0, st, p);
        if (p.nsplit > 1) hipLaunchKernelGGL(attn_dkdv_combine_kernel<64>, dim3((unsigned)gc), dim3(kThreads), 0, st, p);
    }
    EZL_LAUNCH_CHECK("ezl_attn_bwd");
    return EZL_OK;
}
