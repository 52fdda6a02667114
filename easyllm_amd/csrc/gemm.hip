// bf16 MFMA GEMM for gfx950: C[M,N] = A * B with fp32 accumulation.
//
// Replaces the three matmuls of the reference's linear layers
// (base_modules/layers/column_parallel_linear.py:42 forward, :68 input gradient, :99 weight
// gradient; row_parallel_linear.py:113; llama/lm_head.py:62):
//   forward   Y[T,out]  = X[T,in]   * W[out,in]^T    A k-contiguous, B k-contiguous
//   dgrad     dX[T,in]  = dY[T,out] * W[out,in]      A k-contiguous, B n-contiguous
//   wgrad     dW[out,in]= dY[T,out]^T * X[T,in]      A m-contiguous, B n-contiguous   (fp32 or bf16 out)
//
// Tiling: 256x256 block tile, K step 64, 8 waves (2x4), each wave owns 128x64.  Operand tiles are double buffered in LDS
// (2 stages x 2 operands x 32 KiB).  An operand whose reduction dimension is the strided one is kept as it lies in
// memory ([k][256]) and read with ds_read_b64_tr_b16 (the LDS transpose read), so nothing is ever transposed in HBM.
//
// Main kernel (K % 64 == 0): MFMA 16x16x32 (8x4 tiles per wave); tiles go HBM -> LDS directly
// (buffer_load_dwordx4 ... lds, no staging registers, no ds_write); bank conflicts are avoided by an XOR swizzle applied on
// the global-address side.  A K tile is consumed in four phases (k half x M half) of 16 MFMAs; the fragments of the
// next phase are read during the current one, the barrier that publishes the next stage sits in front of the last
// phase, and the loads of tile kt+2 are issued under that phase's MFMAs.  A second kernel with register staging,
// padded tiles and MFMA 32x32x16 covers K tails (K % 64 != 0).
// The forward form and the fp32 weight-gradient form on long reductions run a 4-wave variant of the main kernel (128x128
// wave tiles, one wave per SIMD).
// Blocks are renumbered so that each XCD (own L2) works on a contiguous band of tiles, 8 tiles tall.
//
// Tile counts that leave the last round of workgroups mostly empty (320 tiles on 256 CUs, or 64 tiles in all) are evened out
// by splitting the reduction of the tiles of that last round over several workgroups (given a workspace): each writes an
// fp32 partial tile and a small kernel adds the partials in a fixed order, so results stay bit-reproducible.
#include "common.h"

#include <type_traits>

namespace {

// =================================================================================================
// K-tail kernel: register-staged loads, padded tiles
// =================================================================================================
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int LDK = BK + 8;     // row stride (elements) of a k-contiguous tile  [256][72]
constexpr int LDN = 256 + 32;   // row stride (elements) of a k-major tile       [64][288]
constexpr int TILE = 256 * LDK; // == 64 * LDN elements per operand per stage
static_assert(TILE == 64 * LDN, "both tile layouts must have the same footprint");

typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;

// ---- global -> register staging of one operand tile (2048 x 128-bit chunks over NT threads) ----
template <bool KC, int NT, bool KTAIL>
struct Stager {
    static constexpr int NCH = 2048 / NT;   // chunks per thread
    static constexpr int RSTEP = NT / 8;    // KC: tile rows between two chunks of a thread
    static constexpr int KSTEP = NT / 32;   // non-KC: k rows between two chunks of a thread
    uint32_t off[NCH];  // element offsets of this thread's chunks at k = 0
    int kpos;           // (KC) k column of all chunks / (non-KC) k row of chunk 0
    // dim = extent of the non-reduction dimension, first = first row/col of the block tile
    __device__ __forceinline__ void init(int tid, int first, int dim, int64_t ld) {
        if (KC) {
            kpos = (tid & 7) * 8;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                int r = first + (tid >> 3) + RSTEP * i;
                r = r < dim ? r : dim - 1;  // rows past the edge re-read the last row; their results are never stored
                off[i] = (uint32_t)((int64_t)r * ld + kpos);
            }
        } else {
            kpos = tid >> 5;
            int c = first + (tid & 31) * 8;
            c = c + 8 <= dim ? c : dim - 8;
#pragma unroll
            for (int i = 0; i < NCH; ++i) off[i] = (uint32_t)((int64_t)(kpos + KSTEP * i) * ld + c);
        }
    }
    // k0 = first k of the tile; kadv = element offset of that k (k0 for KC, k0 * ld otherwise)
    __device__ __forceinline__ void load(const bf16_t* __restrict__ base, int k0, int64_t kadv, int K, bf16x8* r) const {
        const bf16_t* p = base + kadv;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (KTAIL) {
                const bool ok = KC ? (k0 + kpos < K) : (k0 + kpos + KSTEP * i < K);
                bf16x8 z;
#pragma unroll
                for (int j = 0; j < 8; ++j) z[j] = (bf16_t)0.0f;
                r[i] = ok ? *reinterpret_cast<const bf16x8*>(p + off[i]) : z;
            } else {
                r[i] = *reinterpret_cast<const bf16x8*>(p + off[i]);
            }
        }
    }
    __device__ __forceinline__ void store(bf16_t* __restrict__ s, int tid, const bf16x8* r) const {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (KC) *reinterpret_cast<bf16x8*>(s + ((tid >> 3) + RSTEP * i) * LDK + (tid & 7) * 8) = r[i];
            else *reinterpret_cast<bf16x8*>(s + ((tid >> 5) + KSTEP * i) * LDN + (tid & 31) * 8) = r[i];
        }
    }
};

// ---- LDS -> MFMA operand fragment: 32 rows(or cols) x 16 k, lane holds 8 k of one row ----------
// lane l: row = l & 31, k = 8 * (l >> 5) + 0..7
template <bool KC>
__device__ __forceinline__ bf16x8 frag(const bf16_t* __restrict__ s, int row0, int ks, int lane) {
    if (KC) {
        return *reinterpret_cast<const bf16x8*>(s + (row0 + (lane & 31)) * LDK + ks * 16 + (lane >> 5) * 8);
    } else {
        // a 16-lane group reads a 4(k) x 16(row) block; lane i of the group receives column i
        const int q = lane >> 4;
        const bf16_t* p = s + (ks * 16 + (q >> 1) * 8 + ((lane & 15) >> 2)) * LDN + row0 + (q & 1) * 16 + ((lane & 3) << 2);
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p));
        const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p + 4 * LDN));
        bf16x8 v;
        v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
        v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
        return v;
    }
}

template <typename OutT> __device__ __forceinline__ void store_out(OutT* p, float v, bool accumulate);
template <> __device__ __forceinline__ void store_out<bf16_t>(bf16_t* p, float v, bool accumulate) {
    *p = (bf16_t)(accumulate ? v + (float)*p : v);
}
template <> __device__ __forceinline__ void store_out<float>(float* p, float v, bool accumulate) {
    *p = accumulate ? v + *p : v;
}

// WAVES_M x WAVES_N waves tile the 256x256 block; a wave owns (256/WAVES_M) x (256/WAVES_N)
template <bool A_KC, bool B_KC, typename OutT, bool KTAIL, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void gemm_staged_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B,
                                                                      OutT* __restrict__ C, int M, int N, int K, int64_t lda,
                                                                      int64_t ldb, int64_t ldc, int accumulate, int tiles_m,
                                                                      int tiles_n) {
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int TM = BM / WAVES_M / 32, TN = BN / WAVES_N / 32;  // MFMA tiles per wave
    __shared__ __attribute__((aligned(16))) bf16_t smem[4 * TILE];  // A0 B0 A1 B1
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // XCD-aware renumbering: hardware deals consecutive block ids round-robin to the 8 XCDs
    const int nblocks = tiles_m * tiles_n;
    int pid = blockIdx.x;
    {
        const int per = nblocks >> 3, rem = nblocks & 7, xcd = pid & 7, idx = pid >> 3;
        pid = xcd * per + (xcd < rem ? xcd : rem) + idx;
    }
    constexpr int GROUP_M = 8;
    const int group_size = GROUP_M * tiles_n;
    const int group = pid / group_size;
    const int first_m = group * GROUP_M;
    const int gm = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    const int tm = first_m + (pid % group_size) % gm;
    const int tn = (pid % group_size) / gm;
    const int m0 = tm * BM, n0 = tn * BN;

    Stager<A_KC, NT, KTAIL> sa;
    Stager<B_KC, NT, KTAIL> sb;
    // per-thread offsets are 32-bit and relative to the block's first row / column: operands of any size are addressable
    A += A_KC ? (int64_t)m0 * lda : (int64_t)m0;
    B += B_KC ? (int64_t)n0 * ldb : (int64_t)n0;
    sa.init(tid, 0, M - m0, lda);
    sb.init(tid, 0, N - n0, ldb);
    constexpr int NCH = 2048 / NT;
    bf16x8 ra[NCH], rb[NCH];

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int nk = (K + BK - 1) / BK;
    const int64_t astep = A_KC ? BK : (int64_t)BK * lda;
    const int64_t bstep = B_KC ? BK : (int64_t)BK * ldb;

    sa.load(A, 0, 0, K, ra);
    sb.load(B, 0, 0, K, rb);
    sa.store(smem, tid, ra);
    sb.store(smem + TILE, tid, rb);
    if (nk > 1) {
        sa.load(A, BK, astep, K, ra);
        sb.load(B, BK, bstep, K, rb);
    }
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        const bf16_t* sA = smem + cur * 2 * TILE;
        const bf16_t* sB = sA + TILE;
        if (kt + 1 < nk) {  // tile kt+1 sits in registers: park it in the other stage
            sa.store(smem + (cur ^ 1) * 2 * TILE, tid, ra);
            sb.store(smem + (cur ^ 1) * 2 * TILE + TILE, tid, rb);
        }
        if (kt + 2 < nk) {  // and start fetching tile kt+2, to land during this step's MFMAs
            sa.load(A, (kt + 2) * BK, (int64_t)(kt + 2) * astep, K, ra);
            sb.load(B, (kt + 2) * BK, (int64_t)(kt + 2) * bstep, K, rb);
        }
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = frag<A_KC>(sA, wm * (TM * 32) + i * 32, ks, lane);
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = frag<B_KC>(sB, wn * (TN * 32) + j * 32, ks, lane);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // epilogue: lane holds column (lane & 31); register r is row 8*(r/4) + 4*(lane>>5) + r%4
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n0 + wn * (TN * 32) + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * (TM * 32) + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row < M && col < N) store_out<OutT>(C + (int64_t)row * ldc + col, acc[i][j][r], accumulate != 0);
            }
        }
    }
}


// =================================================================================================
// main kernel: direct-to-LDS loads, XOR-swizzled tiles
// =================================================================================================
constexpr int DTILE = 256 * 64;  // elements per operand per stage of the swizzled layout (32 KiB)

typedef __attribute__((address_space(3))) void lds_void;

// tile id (in the banded order described above) -> tile coordinates
__device__ __forceinline__ void tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
    constexpr int GROUP_M = 8;
    const int group_size = GROUP_M * tiles_n;
    const int group = pid / group_size;
    const int first_m = group * GROUP_M;
    const int gm = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    tm = first_m + (pid % group_size) % gm;
    tn = (pid % group_size) / gm;
}

// Work split of a launch whose main kernel runs (K % 64 == 0): tile ids below `full` are one workgroup each; every later
// tile is computed by `nsplit` workgroups that each take a contiguous share of the K tiles and leave an fp32 partial tile.
struct SplitPlan {
    int full, nsplit;
    float* partial;  // [tiles - full][nsplit][256 x 256]
};


#define SG_MFMA 0x008
#define SG_VMEM_R 0x020
#define SG_DS_R 0x100

// One operand tile = 32 wave-instructions of 1 KiB each (buffer_load_dwordx4 ... lds: lane l lands at base + 16 l).
//   k-contiguous tile [256 rows][64 k]:  instruction q covers rows 8q..8q+7; chunk c of row r sits in slot c ^ ((r>>1)&7)
//   k-major tile      [64 k][256 cols]:  instruction q covers k rows 2q, 2q+1; chunk c of k row sits in slot c ^ kmajor_swizzle(k)
// Wave w issues instructions q = w*NI .. w*NI+NI-1, i.e. one contiguous NI KiB piece of the tile: M0 (the LDS base) is
// written once per tile and the instruction offset i*1024 selects the KiB.  That offset is also added to the global
// address, so the per-lane byte offsets are stored with i*1024 already subtracted; they are kept 4 KiB high (and the
// buffer's base 4 KiB low) so that they stay non-negative.  The address is buffer base (scalar, advanced per K tile) +
// 32-bit lane offset + immediate: no vector address arithmetic inside the K loop.
// The buffer form of the load is used rather than the global one because the compiler books a global load to LDS as a
// flat access that may touch both memories, and while one is in flight it turns every counted wait on the LDS fragment
// reads into a full drain (lgkmcnt(0)); with buffer loads the waits inside the K loop are exact counts.
// chunk (16 B) permutation of a k-major tile row: keeps the transpose reads of one wave instruction on distinct banks
__device__ __forceinline__ int kmajor_swizzle(int krow) { return ((krow & 3) << 2) ^ (((krow >> 3) & 1) << 1); }

template <bool KC, int NW>
struct Loader {
    static constexpr int NI = 32 / NW;
    static_assert(NI * 1024 <= 4096, "instruction offsets are limited to 12 bits");
    uint32_t off[NI];  // byte offsets from (operand base + k advance - 4096)
    __device__ __forceinline__ void init(int lane, int wave, int first, int dim, int64_t ld) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int q = wave * NI + i;
            int64_t e;
            if (KC) {
                const int row = 8 * q + (lane >> 3);
                const int c = (lane & 7) ^ ((row >> 1) & 7);
                int gr = first + row;
                gr = gr < dim ? gr : dim - 1;
                e = (int64_t)gr * ld + c * 8;
            } else {
                const int krow = 2 * q + (lane >> 5);
                const int c = (lane & 31) ^ kmajor_swizzle(krow);
                int col = first + c * 8;
                col = col + 8 <= dim ? col : dim - 8;
                e = (int64_t)krow * ld + col;
            }
            off[i] = (uint32_t)(e * 2 + 4096 - i * 1024);
        }
    }
    // gbase: operand base advanced to the tile's first k, as a byte pointer
    template <int I>
    __device__ __forceinline__ void issue_one(__amdgpu_buffer_rsrc_t gbase, bf16_t* piece) const {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(gbase, (lds_void*)piece, 16, off[I], 0, I * 1024, 0);
    }
    __device__ __forceinline__ void issue(const bf16_t* __restrict__ gtile, bf16_t* stage, int wave) const {
        // an unbounded raw buffer that starts 4 KiB below the tile
        const __amdgpu_buffer_rsrc_t gbase = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<char*>(reinterpret_cast<const char*>(gtile)) - 4096, 0, 0xffffffffu, 0x00020000);
        bf16_t* piece = stage + wave * (NI * 512);
        issue_one<0>(gbase, piece);
        if constexpr (NI > 1) issue_one<1>(gbase, piece);
        if constexpr (NI > 2) issue_one<2>(gbase, piece);
        if constexpr (NI > 3) issue_one<3>(gbase, piece);
    }
};

// ---- LDS -> MFMA 16x16x32 operand fragment: 16 rows (or columns) x 32 k; lane l holds row l & 15, k = 8 (l >> 4) + 0..7 ----
template <bool KC>
__device__ __forceinline__ bf16x8 sfrag(const bf16_t* __restrict__ s, int row0, int ks, int lane) {
    if (KC) {
        const int row = row0 + (lane & 15);
        const int c = (ks * 4 + (lane >> 4)) ^ ((row >> 1) & 7);
        return *reinterpret_cast<const bf16x8*>(s + row * 64 + c * 8);
    } else {
        // a 16-lane group reads an 8(k) x 16(row) block as two 4 x 16 transpose reads; lane i of the group receives column i
        const int krow = ks * 32 + (lane >> 4) * 8 + ((lane & 15) >> 2);
        const int col = row0 + ((lane & 3) << 2);
        const int c = (col >> 3) ^ kmajor_swizzle(krow);
        const bf16_t* p = s + krow * 256 + c * 8 + (col & 7);
        const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p));
        const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p + 4 * 256));  // k + 4: same swizzle
        bf16x8 v;
        v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
        v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
        return v;
    }
}

// Instruction-scheduling recipe for one phase (compile-time unrolled): one MFMA, then up to PER LDS reads while reads are
// left, then up to PER_V global->LDS loads while loads are left.
template <int MASK, int N>
__device__ __forceinline__ void sched_group() {
    if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, 0);
}
template <int G, int NM, int RD, int PER, int NLD, int PER_V>
struct SchedPhase {
    static __device__ __forceinline__ void run() {
        if constexpr (G < NM) {
            sched_group<SG_MFMA, 1>();
            constexpr int left = RD - G * PER;
            constexpr int ds_slots = PER > 0 ? (RD + PER - 1) / PER : 0;
            constexpr int vleft = G >= ds_slots ? NLD - (G - ds_slots) * PER_V : 0;
            sched_group<SG_DS_R, (left > PER ? PER : (left > 0 ? left : 0))>();
            sched_group<SG_VMEM_R, (vleft > PER_V ? PER_V : (vleft > 0 ? vleft : 0))>();
            SchedPhase<G + 1, NM, RD, PER, NLD, PER_V>::run();
        }
    }
};

template <typename OutT> struct Out4;
template <> struct Out4<bf16_t> { typedef bf16x4 type; };
template <> struct Out4<float> { typedef f32x4 type; };

// 8 waves (2 x 4), each owning 128 x 64 of the 256 x 256 block tile as 8 x 4 MFMA 16x16x32 tiles.  The 16x16x32 shape is
// used because it sustains a higher clock than 32x32x16 under the board's power limit (fewer accumulator-register
// accesses per flop).  A 64-wide K tile is worked off in four phases (k half, M half): a phase issues 16 MFMAs on 4 A and
// 4 B fragments while the fragments of the next phase are read from LDS into the other register set.
//
// MULTI: the reduction runs over up to three (A, B) pairs in turn, C (=|+=) A0 B0 + A1 B1 + A2 B2, all pairs with the same
// leading dimensions: the input gradient of several linears that share their input (q / k / v, gate / up) in one launch,
// summed in fp32, instead of one launch per pair that reads and rewrites the bf16 result.  K is the total reduction
// length; pair 1 starts at K tile t1, pair 2 at t2 (INT_MAX when absent).
struct KSegments {
    const bf16_t* A1;
    const bf16_t* B1;
    const bf16_t* A2;
    const bf16_t* B2;
    int t1, t2;
};

template <bool A_KC, bool B_KC, typename OutT, bool MULTI = false>
__global__ __launch_bounds__(512) void gemm_d2l_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B, OutT* __restrict__ C,
                                                       int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int accumulate,
                                                       int tiles_m, int tiles_n, const SplitPlan plan, const KSegments seg = KSegments()) {
    constexpr int NW = 8, WAVES_N = 4;
    __shared__ __attribute__((aligned(1024))) bf16_t smem[4 * DTILE];  // A0 B0 A1 B1
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    int pid = blockIdx.x, part = 0;
    const bool split = pid >= plan.full;
    if (!split) {  // XCD-aware renumbering over the whole-tile workgroups
        const int per = plan.full >> 3, rem = plan.full & 7, xcd = pid & 7, idx = pid >> 3;
        pid = xcd * per + (xcd < rem ? xcd : rem) + idx;
    } else {
        const int u = pid - plan.full;
        pid = plan.full + u / plan.nsplit;
        part = u - (pid - plan.full) * plan.nsplit;
    }
    int tm, tn;
    tile_of(pid, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    Loader<A_KC, NW> la;
    Loader<B_KC, NW> lb;
    // per-lane offsets are 32-bit and relative to the block's first row / column (a scalar 64-bit advance of the operand
    // base), so operands of more than 2^31 elements are addressable
    const int64_t a_blk = A_KC ? (int64_t)m0 * lda : (int64_t)m0;
    const int64_t b_blk = B_KC ? (int64_t)n0 * ldb : (int64_t)n0;
    la.init(lane, wave, 0, M - m0, lda);
    lb.init(lane, wave, 0, N - n0, ldb);

    f32x4 acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    int nk = K / BK, kt0 = 0;  // this workgroup's K tiles: kt0 .. kt0 + nk - 1
    if (split) {
        kt0 = (int)((int64_t)nk * part / plan.nsplit);
        nk = (int)((int64_t)nk * (part + 1) / plan.nsplit) - kt0;
    }
    const int64_t astep = A_KC ? BK : (int64_t)BK * lda;
    const int64_t bstep = B_KC ? BK : (int64_t)BK * ldb;
    const int arow = wm * 128, brow = wn * 64;

    bf16x8 fa[2][4], fb[2][4];
    auto read_a = [&](const bf16_t* sA, int ks, int half, int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[buf][i] = sfrag<A_KC>(sA, arow + half * 64 + i * 16, ks, lane);
    };
    auto read_b = [&](const bf16_t* sA, int ks, int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j) fb[buf][j] = sfrag<B_KC>(sA + DTILE, brow + j * 16, ks, lane);
    };
    // B is the first MFMA operand: the accumulator then holds C^T fragments, i.e. a lane owns 4 consecutive columns of one
    // row of C, which it can store as one vector.
    auto mfmas = [&](int half, int abuf, int bbuf) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[half * 4 + i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[bbuf][j], fa[abuf][i], acc[half * 4 + i][j], 0, 0, 0);
    };
    auto issue_tile = [&](int t, int stage) {
        const bf16_t* Ab = A;
        const bf16_t* Bb = B;
        t += kt0;
        if constexpr (MULTI) {  // scalar selects: which pair K tile t belongs to
            const bool s1 = t >= seg.t1, s2 = t >= seg.t2;
            Ab = s2 ? seg.A2 : (s1 ? seg.A1 : A);
            Bb = s2 ? seg.B2 : (s1 ? seg.B1 : B);
            t -= s2 ? seg.t2 : (s1 ? seg.t1 : 0);
        }
        la.issue(Ab + a_blk + (int64_t)t * astep, smem + stage * 2 * DTILE, wave);
        lb.issue(Bb + b_blk + (int64_t)t * bstep, smem + stage * 2 * DTILE + DTILE, wave);
    };

    issue_tile(0, 0);
    if (nk > 1) issue_tile(1, 1);
    // Pull the remaining kernel arguments into registers now: a scalar load still in flight inside the K loop shares the
    // counter of the LDS reads and would turn every counted wait on them into a full drain.
    asm volatile("" ::"s"(C), "s"(ldc), "s"(accumulate), "s"(plan.partial), "s"(plan.full), "s"(plan.nsplit));
    if constexpr (MULTI) asm volatile("" ::"s"(seg.A1), "s"(seg.B1), "s"(seg.A2), "s"(seg.B2), "s"(seg.t1), "s"(seg.t2));
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
    __syncthreads();
    read_b(smem, 0, 0);
    read_a(smem, 0, 0, 0);

    constexpr int RA = A_KC ? 4 : 8, RB = B_KC ? 4 : 8;  // LDS reads per fragment set
    constexpr int NM = 16;                                // MFMAs per phase
    constexpr int NLD = 2 * (32 / NW);                    // global->LDS loads per wave and tile pair
    // phases 0 and 2 fetch the A fragments of the other M half; phases 1 and 3 fetch B and A of the next k half
#define EZL_PHASE_SCHED(RD, LD) SchedPhase<0, NM, (RD), ((RD) + 11) / 12, (LD), 1>::run()
#define EZL_STEP(HAS_NEXT, DO_LOAD)                                                                       \
    {                                                                                                     \
        const int cur = kt & 1;                                                                           \
        const bf16_t* sA = smem + cur * 2 * DTILE;                                                         \
        read_a(sA, 0, 1, 1);                                                                              \
        mfmas(0, 0, 0);                                                                                   \
        EZL_PHASE_SCHED(RA, 0);                                                                           \
        read_b(sA, 1, 1);                                                                                 \
        read_a(sA, 1, 0, 0);                                                                              \
        mfmas(1, 1, 0);                                                                                   \
        EZL_PHASE_SCHED(RA + RB, 0);                                                                      \
        read_a(sA, 1, 1, 1);                                                                              \
        mfmas(0, 0, 1);                                                                                   \
        EZL_PHASE_SCHED(RA, 0);                                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                                \
        __builtin_amdgcn_s_waitcnt(0x0F70);                                                               \
        __syncthreads();                                                                                  \
        __builtin_amdgcn_sched_barrier(0);                                                                \
        if (HAS_NEXT) {                                                                                   \
            read_b(smem + (cur ^ 1) * 2 * DTILE, 0, 0);                                                    \
            read_a(smem + (cur ^ 1) * 2 * DTILE, 0, 0, 0);                                                 \
        }                                                                                                 \
        if (DO_LOAD) issue_tile(kt + 2, cur);                                                             \
        mfmas(1, 1, 1);                                                                                   \
        EZL_PHASE_SCHED((HAS_NEXT) ? RA + RB : 0, (DO_LOAD) ? NLD : 0);                                   \
        __builtin_amdgcn_sched_barrier(0);                                                                \
    }

    int kt = 0;
    for (; kt + 2 < nk; ++kt) EZL_STEP(true, true)
    if (kt + 1 < nk) {
        EZL_STEP(true, false)
        ++kt;
    }
    EZL_STEP(false, false)
#undef EZL_STEP
#undef EZL_PHASE_SCHED

    // epilogue: acc[i][j] register r is C[m0 + arow + 16 i + (lane & 15)][n0 + brow + 16 j + 4 (lane >> 4) + r]
    typedef typename Out4<OutT>::type out4_t;
    if (split) {  // this workgroup's share of the reduction, as a dense fp32 tile; gemm_split_reduce_kernel adds the shares
        float* tile = plan.partial + ((size_t)(pid - plan.full) * plan.nsplit + part) * (size_t)(BM * BN);
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<f32x4*>(tile + (arow + i * 16 + (lane & 15)) * BN + brow + j * 16 + 4 * (lane >> 4)) = acc[i][j];
        return;
    }
    if constexpr (sizeof(OutT) == 2) {
        // bf16: 8-byte stores of 4 columns reach only half the write bandwidth of 16-byte ones (3.8 vs 6.7 TB/s on a
        // 4096 x 32000 output).  Lanes l and l ^ 16 trade halves of two neighbouring column tiles, so that the lane of
        // the even 16-lane row ends up with 8 consecutive columns of tile 2 jp and its partner with those of tile 2 jp + 1.
        if ((N % 8 == 0) && (ldc % 8 == 0) && (((uintptr_t)C & 15) == 0)) {
            const int g = lane >> 4;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int row = m0 + arow + i * 16 + (lane & 15);
#pragma unroll
                for (int jp = 0; jp < 2; ++jp) {
                    float lo[4], hi[4];  // columns +0..3 and +4..7 of this lane's 8
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float ta = acc[i][2 * jp][r], tb = acc[i][2 * jp + 1][r];  // scalars: a bit_cast of a vector element reads element 0
                        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(ta), __float_as_uint(tb), false, false);
                        lo[r] = __uint_as_float(sw[0]);
                        hi[r] = __uint_as_float(sw[1]);
                    }
                    const int col = n0 + brow + (2 * jp + (g & 1)) * 16 + 8 * (g >> 1);
                    if (row >= M || col >= N) continue;
                    bf16_t* dst = C + (int64_t)row * ldc + col;
                    bf16x8 v;
                    if (accumulate) {
                        const bf16x8 old = *reinterpret_cast<const bf16x8*>(dst);
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            v[r] = (bf16_t)(lo[r] + (float)old[r]);
                            v[4 + r] = (bf16_t)(hi[r] + (float)old[4 + r]);
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            v[r] = (bf16_t)lo[r];
                            v[4 + r] = (bf16_t)hi[r];
                        }
                    }
                    *reinterpret_cast<bf16x8*>(dst) = v;
                }
            }
            return;
        }
    }
    const bool vec_ok = (N % 4 == 0) && (ldc % 4 == 0) && (((uintptr_t)C & 15) == 0);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = m0 + arow + i * 16 + (lane & 15);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + brow + j * 16 + 4 * (lane >> 4);
            if (row >= M || col >= N) continue;
            OutT* dst = C + (int64_t)row * ldc + col;
            if (vec_ok) {
                out4_t v;
                if (accumulate) {
                    const out4_t old = *reinterpret_cast<const out4_t*>(dst);
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = (OutT)(acc[i][j][r] + (float)old[r]);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] = (OutT)acc[i][j][r];
                }
                *reinterpret_cast<out4_t*>(dst) = v;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (col + r < N) store_out<OutT>(dst + r, acc[i][j][r], accumulate != 0);
            }
        }
    }
}


// =================================================================================================
// 4-wave form of the main kernel: 2 x 2 waves, each owning 128 x 128 of the block tile
// =================================================================================================
// One wave per SIMD with 8 x 8 MFMA 16x16x32 tiles: the 256 accumulator registers live in AGPRs, a K tile costs a third
// fewer LDS fragment reads than with 128 x 64 wave tiles, and nothing else runs on the SIMD to cover a stall, so the K loop
// is laid out step by step (one MFMA per step, a sched_barrier after each):
//   phase A of tile kt: 64 MFMAs on k half 0 (fragment set 0); the 16 fragments of k half 1 are read meanwhile
//   wait for the loads in flight + barrier: tile kt + 1 has landed, every wave is done reading the stage of tile kt
//   phase B of tile kt: 64 MFMAs on k half 1 (set 1); the fragments of tile kt + 1, k half 0 are read meanwhile and the
//                       16 wave loads of tile kt + 2 go out into the stage of tile kt
// The loop's back edge sits right behind the barrier, where no LDS read is in flight, so inside the body the compiler's
// waits on the fragment reads are exact counts.  Reads are issued in the first half of a phase (one every second MFMA) and
// have landed long before the next phase needs them; loads are issued one every fourth MFMA over the whole of phase B:
// the CU's address unit takes 16 cycles per 1 KiB wave load, i.e. the four waves' loads keep it busy for all of phase B,
// and issued any faster they fill its queue and the issuing wave stalls with its MFMAs behind it (measured on all-zero
// operands, 4096 x 4096 x K: 0.96 us per K tile with this spacing, 1.12 with one load every second MFMA, 1.23 back to
// back; the 8-wave kernel 1.05).  Used for the forward form (both operands k-contiguous, bf16 result) and for the
// weight-gradient form with an fp32 result on long reductions; for input gradients and short reductions the 8-wave
// kernel, which hides more of the prologue and the epilogue, is as fast or faster.
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// one operand tile for 4 waves: wave w issues instructions q = 8 w .. 8 w + 7 (8 KiB), in two groups of four that share an
// LDS base (the instruction offset reaches 4 KiB)
template <bool KC>
struct Loader4 {
    uint32_t off[8];
    __device__ __forceinline__ void init(int lane, int wave, int dim, int64_t ld) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int q = wave * 8 + i;
            int64_t e;
            if (KC) {
                const int row = 8 * q + (lane >> 3);
                const int c = (lane & 7) ^ ((row >> 1) & 7);
                const int gr = row < dim ? row : dim - 1;
                e = (int64_t)gr * ld + c * 8;
            } else {
                const int krow = 2 * q + (lane >> 5);
                const int c = (lane & 31) ^ kmajor_swizzle(krow);
                int col = c * 8;
                col = col + 8 <= dim ? col : dim - 8;
                e = (int64_t)krow * ld + col;
            }
            off[i] = (uint32_t)(e * 2 + 4096 - (i & 3) * 1024);
        }
    }
    // gbase: buffer that starts 4 KiB below the tile
    template <int I>
    __device__ __forceinline__ void issue_one(__amdgpu_buffer_rsrc_t gbase, bf16_t* stage, int wave) const {
        bf16_t* piece = stage + wave * 4096 + (I >> 2) * 2048;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(gbase, (lds_void*)piece, 16, off[I], 0, (I & 3) * 1024, 0);
    }
};

// C must allow 16-byte stores (N and ldc multiples of 8 for bf16, of 4 for fp32, aligned base) and, for bf16, its
// tile-relative byte offsets must fit 31 bits: the host side checks.
template <bool A_KC, bool B_KC, typename OutT>
__global__ __launch_bounds__(256, 1) void gemm_w4_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B, OutT* __restrict__ C,
                                                         int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int accumulate,
                                                         int tiles_m, int tiles_n, const SplitPlan plan) {
    __shared__ __attribute__((aligned(1024))) bf16_t smem[4 * DTILE];  // A0 B0 A1 B1
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    int pid = blockIdx.x, part = 0;
    const bool split = pid >= plan.full;
    if (!split) {  // XCD-aware renumbering over the whole-tile workgroups
        const int per = plan.full >> 3, rem = plan.full & 7, xcd = pid & 7, idx = pid >> 3;
        pid = xcd * per + (xcd < rem ? xcd : rem) + idx;
    } else {  // a tile of the split last round: this workgroup's share of its K tiles
        const int u = pid - plan.full;
        pid = plan.full + u / plan.nsplit;
        part = u - (pid - plan.full) * plan.nsplit;
    }
    int tm, tn;
    tile_of(pid, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    Loader4<A_KC> la;
    Loader4<B_KC> lb;
    const int64_t a_blk = A_KC ? (int64_t)m0 * lda : (int64_t)m0;
    const int64_t b_blk = B_KC ? (int64_t)n0 * ldb : (int64_t)n0;
    la.init(lane, wave, M - m0, lda);
    lb.init(lane, wave, N - n0, ldb);

    f32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    int nk = K / BK, kt0 = 0;  // this workgroup's K tiles: kt0 .. kt0 + nk - 1
    if (split) {
        kt0 = (int)((int64_t)nk * part / plan.nsplit);
        nk = (int)((int64_t)nk * (part + 1) / plan.nsplit) - kt0;
    }
    const int64_t astep = A_KC ? BK : (int64_t)BK * lda;
    const int64_t bstep = B_KC ? BK : (int64_t)BK * ldb;
    const int arow = wm * 128, brow = wn * 128;

    bf16x8 fa[2][8], fb[2][8];
    // fragment f of a k half: f < 8 the B fragment f, else the A fragment f - 8
    auto read_frag = [&](const bf16_t* sA, int ks, int buf, auto F) {
        constexpr int f = decltype(F)::value;
        if constexpr (f < 8) fb[buf][f] = sfrag<B_KC>(sA + DTILE, brow + f * 16, ks, lane);
        else fa[buf][f - 8] = sfrag<A_KC>(sA, arow + (f - 8) * 16, ks, lane);
    };
    __amdgpu_buffer_rsrc_t ga, gb;
    auto tile_bases = [&](int t) {
        t += kt0;
        ga = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(reinterpret_cast<const char*>(A + a_blk + (int64_t)t * astep)) - 4096, 0,
                                               0xffffffffu, 0x00020000);
        gb = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(reinterpret_cast<const char*>(B + b_blk + (int64_t)t * bstep)) - 4096, 0,
                                               0xffffffffu, 0x00020000);
    };
    // load l of a tile pair: l < 8 piece l of the A tile, else piece l - 8 of the B tile
    auto issue_load = [&](int stage, auto L) {
        constexpr int l = decltype(L)::value;
        if constexpr (l < 8) la.template issue_one<l>(ga, smem + stage * 2 * DTILE, wave);
        else lb.template issue_one<l - 8>(gb, smem + stage * 2 * DTILE + DTILE, wave);
    };
    auto issue_tile = [&](int t, int stage) {
        tile_bases(t);
        static_for<0, 16>([&](auto L) { issue_load(stage, L); });
    };

    issue_tile(0, 0);
    if (nk > 1) issue_tile(1, 1);
    // the remaining kernel arguments, pulled into registers now (a scalar load in flight inside the K loop would share the
    // counter of the LDS reads)
    asm volatile("" ::"s"(C), "s"(ldc), "s"(accumulate), "s"(plan.partial), "s"(plan.full), "s"(plan.nsplit));
    if (nk > 1) __builtin_amdgcn_s_waitcnt(0x4070);  // vmcnt(16) lgkmcnt(0): tile 0 has landed, tile 1 is still on its way
    else __builtin_amdgcn_s_waitcnt(0x0070);         // vmcnt(0) lgkmcnt(0)
    __syncthreads();
    static_for<0, 16>([&](auto F) { read_frag(smem, 0, 0, F); });

    constexpr int RSTEP = 2;  // a fragment read every RSTEP MFMAs (16 reads: the first half of a phase)
    constexpr int LSTEP = 4;  // a tile load every LSTEP MFMAs (16 loads: all of phase B)
    auto phase_a = [&](int kt) {
        const bf16_t* sA = smem + (kt & 1) * 2 * DTILE;
        static_for<0, 64>([&](auto S) {
            constexpr int m = decltype(S)::value, i = m >> 3, j = m & 7;
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[0][j], fa[0][i], acc[i][j], 0, 0, 0);
            if constexpr (m % RSTEP == 0 && m / RSTEP < 16) read_frag(sA, 1, 1, std::integral_constant<int, m / RSTEP>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto phase_b = [&](int kt, auto HAS_NEXT, auto DO_LOAD) {
        constexpr bool has_next = decltype(HAS_NEXT)::value, do_load = decltype(DO_LOAD)::value;
        const int cur = kt & 1;
        const bf16_t* sN = smem + (cur ^ 1) * 2 * DTILE;
        if constexpr (do_load) tile_bases(kt + 2);
        static_for<0, 64>([&](auto S) {
            constexpr int m = decltype(S)::value, i = m >> 3, j = m & 7;
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[1][j], fa[1][i], acc[i][j], 0, 0, 0);
            if constexpr (has_next && m % RSTEP == 0 && m / RSTEP < 16) read_frag(sN, 0, 0, std::integral_constant<int, m / RSTEP>{});
            if constexpr (do_load && m % LSTEP == LSTEP - 1) issue_load(cur, std::integral_constant<int, m / LSTEP>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto publish = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): the next tile has landed, this wave's reads are done
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    };
    phase_a(0);
    publish();
    int kt = 0;
    for (; kt + 2 < nk; ++kt) {
        phase_b(kt, std::true_type{}, std::true_type{});
        phase_a(kt + 1);
        publish();
    }
    if (kt + 1 < nk) {
        phase_b(kt, std::true_type{}, std::false_type{});
        phase_a(kt + 1);
        publish();
        ++kt;
    }
    phase_b(kt, std::false_type{}, std::false_type{});

    if (split) {  // this workgroup's share of the reduction, as a dense fp32 tile; gemm_split_reduce_kernel adds the shares
        float* tile = plan.partial + ((size_t)(pid - plan.full) * plan.nsplit + part) * (size_t)(BM * BN);
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                *reinterpret_cast<f32x4*>(tile + (arow + i * 16 + (lane & 15)) * BN + brow + j * 16 + 4 * (lane >> 4)) = acc[i][j];
        return;
    }
    // the accumulators stay in their AGPRs until here (otherwise the last phase copies each finished tile out to VGPRs
    // right behind its MFMA and runs out of registers)
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));
    if constexpr (sizeof(OutT) == 4) {  // fp32 results (weight gradients): the 4 columns a lane owns as one 16-byte store
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = m0 + arow + i * 16 + (lane & 15);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int col = n0 + brow + j * 16 + 4 * (lane >> 4);
                if (row >= M || col >= N) continue;
                float* dst = C + (int64_t)row * ldc + col;
                f32x4 v = acc[i][j];
                if (accumulate) {
                    const f32x4 old = *reinterpret_cast<const f32x4*>(dst);
#pragma unroll
                    for (int r = 0; r < 4; ++r) v[r] += old[r];
                }
                *reinterpret_cast<f32x4*>(dst) = v;
            }
        }
    } else {

    // epilogue: acc[i][j] register r is C[m0 + arow + 16 i + (lane & 15)][n0 + brow + 16 j + 4 (lane >> 4) + r]
    // C is addressed as a buffer that starts at the tile's corner and ends behind the tile's last valid row: a store to a row
    // past M drops out by the buffer's range check, one to a column past N by an offset that is out of range.  The epilogue is
    // thus straight-line code (no branch per store, and `accumulate` decided once), whose 32 independent chains of
    // register moves, conversions and stores the compiler interleaves; with a branch per store it took twice as long.
    constexpr int SZ = 2;
    const int mrem = M - m0 < BM ? M - m0 : BM;
    const __amdgpu_buffer_rsrc_t cbuf = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<char*>(C + (int64_t)m0 * ldc + n0), 0, (uint32_t)(((int64_t)mrem * ldc - n0) * SZ), 0x00020000);
    const uint32_t row_off = (uint32_t)(arow + (lane & 15)) * (uint32_t)(ldc * SZ);
    const uint32_t row_step = (uint32_t)(16 * ldc * SZ);  // scalar: rows 16 i
    constexpr uint32_t kOut = 0x80000000u;
    auto epilogue = [&](auto ACC) {
        constexpr bool accum = decltype(ACC)::value;
        {  // lanes l and l ^ 16 trade halves of two neighbouring column tiles: 16-byte stores
            const int g = lane >> 4;
            uint32_t voff[4];
#pragma unroll
            for (int jp = 0; jp < 4; ++jp) {
                const int col = brow + (2 * jp + (g & 1)) * 16 + 8 * (g >> 1);
                voff[jp] = n0 + col < N ? row_off + (uint32_t)col * SZ : kOut;
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
#pragma unroll
                for (int jp = 0; jp < 4; ++jp) {
                    float lo[4], hi[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float ta = acc[i][2 * jp][r], tb = acc[i][2 * jp + 1][r];
                        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(ta), __float_as_uint(tb), false, false);
                        lo[r] = __uint_as_float(sw[0]);
                        hi[r] = __uint_as_float(sw[1]);
                    }
                    bf16x8 v;
                    if constexpr (accum) {
                        const bf16x8 old = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(cbuf, voff[jp], i * row_step, 0));
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            v[r] = (bf16_t)(lo[r] + (float)old[r]);
                            v[4 + r] = (bf16_t)(hi[r] + (float)old[4 + r]);
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            v[r] = (bf16_t)lo[r];
                            v[4 + r] = (bf16_t)hi[r];
                        }
                    }
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), cbuf, voff[jp], i * row_step, 0);
                }
            }
        }
    };
    if (accumulate) epilogue(std::true_type{});
    else epilogue(std::false_type{});
    }
}

// C tile (=|+=) sum of the nsplit fp32 partial tiles, added in index order.  One block per 16 rows of a tile: a thread owns 16
// consecutive columns of one row.
template <typename OutT>
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(OutT* __restrict__ C, int M, int N, int64_t ldc, int accumulate,
                                                                int tiles_m, int tiles_n, const SplitPlan plan) {
    const int t = blockIdx.x >> 4;  // split tile
    int tm, tn;
    tile_of(plan.full + t, tiles_m, tiles_n, tm, tn);
    const int rl = (blockIdx.x & 15) * 16 + (threadIdx.x >> 4), cl = (threadIdx.x & 15) * 16;
    const int row = tm * BM + rl, col = tn * BN + cl;
    if (row >= M || col >= N) return;
    float v[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = 0.f;
    const float* src = plan.partial + (size_t)t * plan.nsplit * (size_t)(BM * BN) + (size_t)rl * BN + cl;
    for (int p = 0; p < plan.nsplit; ++p, src += BM * BN) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(src) + q);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[4 * q + e] += x[e];
        }
    }
    OutT* dst = C + (int64_t)row * ldc + col;
    if (col + 16 <= N && ldc % 8 == 0 && ((uintptr_t)C & 15) == 0) {  // whole 16-column piece, 16-byte aligned
        constexpr int VE = 16 / (int)sizeof(OutT);  // elements per 16-byte vector
        typedef OutT vec_t __attribute__((ext_vector_type(VE)));
#pragma unroll
        for (int q = 0; q < 16 / VE; ++q) {
            vec_t o;
            if (accumulate) {
                const vec_t old = *reinterpret_cast<const vec_t*>(dst + q * VE);
#pragma unroll
                for (int e = 0; e < VE; ++e) o[e] = (OutT)(v[q * VE + e] + (float)old[e]);
            } else {
#pragma unroll
                for (int e = 0; e < VE; ++e) o[e] = (OutT)v[q * VE + e];
            }
            *reinterpret_cast<vec_t*>(dst + q * VE) = o;
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e)
        if (col + e < N) store_out<OutT>(dst + e, v[e], accumulate != 0);
}

// Split the tiles of a mostly empty last round?  cus workgroups run at a time (one per CU: the kernel uses 128 KiB of LDS).
constexpr int kCus = 256;
SplitPlan make_plan(int64_t tiles, int64_t nk, void* workspace, int64_t workspace_bytes) {
    SplitPlan p;
    p.full = (int)tiles; p.nsplit = 1; p.partial = nullptr;
    const int64_t r = tiles % kCus;
    // A last round that is more than 3/8 full is left alone: split two ways it measured slower (128 tiles, K = 4096: 88 against
    // 81 us -- under the power limit a half-empty round runs at a higher clock, and the partial tiles cost a pass of their own).
    if (r == 0 || r > 96) return p;
    int s = (int)(kCus / r);
    while (s > 1 && nk / s < 8) --s;  // a share of fewer than 8 K tiles is mostly prologue
    if (s < 2) return p;
    if (!workspace || workspace_bytes < r * s * (int64_t)(BM * BN) * (int64_t)sizeof(float)) return p;
    p.full = (int)(tiles - r); p.nsplit = s; p.partial = (float*)workspace;
    return p;
}
int64_t plan_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % BK != 0) return 0;
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    SplitPlan p = make_plan(tiles, K / BK, (void*)16, INT64_MAX);
    return p.nsplit > 1 ? (tiles - p.full) * p.nsplit * (int64_t)(BM * BN) * (int64_t)sizeof(float) : 0;
}

// the 4-wave kernel pays off from this many K tiles on (4096 x 4096 x K, forward form: 57 against 54 us at 32 tiles, 98
// against 103 at 64, 179 against 194 at 128)
constexpr int kW4MinKTiles = 48;

template <bool A_KC, bool B_KC, typename OutT>
void launch(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int accumulate,
            void* workspace, int64_t workspace_bytes, hipStream_t st) {
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const dim3 grid((unsigned)(tiles_m * tiles_n)), block(512);
    if (K % BK == 0) {
        const SplitPlan plan = make_plan((int64_t)tiles_m * tiles_n, K / BK, workspace, workspace_bytes);
        const int split_tiles = tiles_m * tiles_n - plan.full;
        // The 4-wave kernel: forward form with a bf16 result, and weight-gradient form with an fp32 result (inside the steps
        // 0.4 - 0.8 % faster than the 8-wave kernel although a single launch at K = 4096 is not: it moves a third fewer LDS
        // bytes, and the steps are bound by power).  With a k-strided B only (input gradients) it gained nothing.
        if constexpr ((A_KC && B_KC && sizeof(OutT) == 2) || (!A_KC && !B_KC && sizeof(OutT) == 4)) {
            const int vec = 16 / (int)sizeof(OutT);
            // (a launch that is split tiles only is judged by the length of a share)
            const int w4_ktiles = plan.nsplit > 1 && plan.full == 0 ? K / BK / plan.nsplit : K / BK;
            if (w4_ktiles >= kW4MinKTiles && N % vec == 0 && ldc % vec == 0 && ezl_aligned16(C) &&
                (int64_t)ldc * (int64_t)sizeof(OutT) * BM < (1LL << 31)) {  // tile-relative byte offsets of C fit 31 bits
                hipLaunchKernelGGL((gemm_w4_kernel<A_KC, B_KC, OutT>), dim3((unsigned)(plan.full + split_tiles * plan.nsplit)), dim3(256), 0, st,
                                   (const bf16_t*)A, (const bf16_t*)B, (OutT*)C, M, N, K, lda, ldb, ldc, accumulate, tiles_m, tiles_n, plan);
                if (plan.nsplit > 1)
                    hipLaunchKernelGGL((gemm_split_reduce_kernel<OutT>), dim3((unsigned)(split_tiles * 16)), dim3(256), 0, st, (OutT*)C, M, N,
                                       ldc, accumulate, tiles_m, tiles_n, plan);
                return;
            }
        }
        hipLaunchKernelGGL((gemm_d2l_kernel<A_KC, B_KC, OutT>), dim3((unsigned)(plan.full + split_tiles * plan.nsplit)), block, 0, st,
                           (const bf16_t*)A, (const bf16_t*)B, (OutT*)C, M, N, K, lda, ldb, ldc, accumulate, tiles_m, tiles_n, plan);
        if (plan.nsplit > 1)
            hipLaunchKernelGGL((gemm_split_reduce_kernel<OutT>), dim3((unsigned)(split_tiles * 16)), dim3(256), 0, st, (OutT*)C, M, N, ldc,
                               accumulate, tiles_m, tiles_n, plan);
    } else
        hipLaunchKernelGGL((gemm_staged_kernel<A_KC, B_KC, OutT, true, 2, 4>), grid, block, 0, st, (const bf16_t*)A,
                           (const bf16_t*)B, (OutT*)C, M, N, K, lda, ldb, ldc, accumulate, tiles_m, tiles_n);
}

// C = 0 for an empty reduction (a fill kernel rather than a memset node, so the call can be captured into a graph)
template <typename OutT>
__global__ __launch_bounds__(256) void zero_c_kernel(OutT* __restrict__ C, int64_t M, int64_t N, int64_t ldc) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < M * N; i += (int64_t)gridDim.x * 256)
        C[(i / N) * ldc + (i % N)] = (OutT)0.0f;
}

}  // namespace


// a_kc / b_kc: 1 if the operand's reduction index is its contiguous one
//   A: a_kc ? A[m * lda + k] : A[k * lda + m]        B: b_kc ? B[n * ldb + k] : B[k * ldb + n]
// out_dtype: 0 bf16, 1 fp32.  accumulate: C += A*B instead of C = A*B.
// bytes of workspace with which a launch of this shape evens out a mostly empty last round of tiles (0: none needed)
extern "C" int64_t ezl_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) { return plan_bytes(M, N, K); }

extern "C" int ezl_gemm_bf16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                             int64_t ldc, int a_kc, int b_kc, int out_dtype, int accumulate, void* workspace,
                             int64_t workspace_bytes, void* stream) {
    EZL_REQUIRE(M >= 0 && N >= 0 && K >= 0, EZL_EINVAL, "ezl_gemm_bf16: negative size");
    EZL_REQUIRE(out_dtype == 0 || out_dtype == 1, EZL_EUNSUPPORTED, "ezl_gemm_bf16: out_dtype must be 0 (bf16) or 1 (fp32)");
    if (M == 0 || N == 0) return EZL_OK;
    EZL_REQUIRE(C, EZL_EINVAL, "ezl_gemm_bf16: null pointer");
    if (K == 0) {  // empty reduction (a weight gradient over zero tokens): C = 0, or C unchanged when accumulating
        EZL_REQUIRE(ldc >= N, EZL_EINVAL, "ezl_gemm_bf16: leading dimension too small");
        if (!accumulate) {
            if (out_dtype == 0) hipLaunchKernelGGL(zero_c_kernel<bf16_t>, dim3(256), dim3(256), 0, (hipStream_t)stream, (bf16_t*)C, M, N, ldc);
            else hipLaunchKernelGGL(zero_c_kernel<float>, dim3(256), dim3(256), 0, (hipStream_t)stream, (float*)C, M, N, ldc);
            EZL_LAUNCH_CHECK("ezl_gemm_bf16(zero)");
        }
        return EZL_OK;
    }
    EZL_REQUIRE(A && B, EZL_EINVAL, "ezl_gemm_bf16: null pointer");
    EZL_REQUIRE(ezl_aligned16(A) && ezl_aligned16(B) && lda % 8 == 0 && ldb % 8 == 0, EZL_EINVAL,
                "ezl_gemm_bf16: operands must be 16-byte aligned with leading dimensions that are multiples of 8");
    // every 128-bit chunk must lie wholly inside or wholly outside the matrix
    EZL_REQUIRE(a_kc ? (K % 8 == 0) : (M % 8 == 0), EZL_EUNSUPPORTED, "ezl_gemm_bf16: contiguous extent of A must be a multiple of 8");
    EZL_REQUIRE(b_kc ? (K % 8 == 0) : (N % 8 == 0), EZL_EUNSUPPORTED, "ezl_gemm_bf16: contiguous extent of B must be a multiple of 8");
    EZL_REQUIRE(lda >= (a_kc ? K : M) && ldb >= (b_kc ? K : N) && ldc >= N, EZL_EINVAL, "ezl_gemm_bf16: leading dimension too small");
    // 32-bit byte offsets inside one 256-row (or 64-k-row) tile; the tile bases advance in 64 bits
    EZL_REQUIRE(lda < (1LL << 22) && ldb < (1LL << 22) && M < (1LL << 31) && N < (1LL << 31) && K < (1LL << 31), EZL_EUNSUPPORTED,
                "ezl_gemm_bf16: a dimension of 2^31 or more, or a leading dimension of 2^22 or more");
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    EZL_REQUIRE(tiles < (1LL << 31), EZL_EUNSUPPORTED, "ezl_gemm_bf16: too many tiles");
    hipStream_t st = (hipStream_t)stream;
    EZL_REQUIRE(!workspace || ezl_aligned16(workspace), EZL_EINVAL, "ezl_gemm_bf16: workspace must be 16-byte aligned");
#define EZL_GEMM_CASE(AK, BKC, OT) \
    launch<AK, BKC, OT>(A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, accumulate, workspace, workspace_bytes, st)
    if (out_dtype == 0) {
        if (a_kc && b_kc) EZL_GEMM_CASE(true, true, bf16_t);
        else if (a_kc && !b_kc) EZL_GEMM_CASE(true, false, bf16_t);
        else if (!a_kc && !b_kc) EZL_GEMM_CASE(false, false, bf16_t);
        else EZL_GEMM_CASE(false, true, bf16_t);
    } else {
        if (a_kc && b_kc) EZL_GEMM_CASE(true, true, float);
        else if (a_kc && !b_kc) EZL_GEMM_CASE(true, false, float);
        else if (!a_kc && !b_kc) EZL_GEMM_CASE(false, false, float);
        else EZL_GEMM_CASE(false, true, float);
    }
#undef EZL_GEMM_CASE
    EZL_LAUNCH_CHECK("ezl_gemm_bf16");
    return EZL_OK;
}

// C (=|+=) sum_i A[i] * B[i] over `count` operand pairs that share M, N and the leading dimensions; K[i] is the reduction
// length of pair i.  The input gradient dx = sum_i dy_i W_i of linears that share their input is one such sum.  With up to
// three pairs in the (a_kc = 1, b_kc = 0, bf16 output) form and every K[i] a positive multiple of 64 it is a single launch
// that adds the products in fp32 and rounds once; otherwise the pairs go out as ezl_gemm_bf16 calls that accumulate into C.
extern "C" int ezl_gemm_bf16_ksplit(int count, const void* const* A, const void* const* B, void* C, int64_t M, int64_t N,
                                    const int64_t* K, int64_t lda, int64_t ldb, int64_t ldc, int a_kc, int b_kc, int out_dtype,
                                    int accumulate, void* workspace, int64_t workspace_bytes, void* stream) {
    EZL_REQUIRE(count >= 1 && A && B && K, EZL_EINVAL, "ezl_gemm_bf16_ksplit: bad count or null argument array");
    bool one_launch = count <= 3 && a_kc == 1 && b_kc == 0 && out_dtype == 0 && M > 0 && N > 0;
    int64_t ktot = 0;
    for (int i = 0; i < count; ++i) {
        EZL_REQUIRE(K[i] >= 0, EZL_EINVAL, "ezl_gemm_bf16_ksplit: negative size");
        one_launch = one_launch && K[i] > 0 && K[i] % BK == 0;
        ktot += K[i];
    }
    if (!one_launch || count == 1) {
        for (int i = 0; i < count; ++i)
            if (const int rc = ezl_gemm_bf16(A[i], B[i], C, M, N, K[i], lda, ldb, ldc, a_kc, b_kc, out_dtype, i == 0 ? accumulate : 1,
                                             workspace, workspace_bytes, stream))
                return rc;
        return EZL_OK;
    }
    EZL_REQUIRE(C, EZL_EINVAL, "ezl_gemm_bf16: null pointer");
    for (int i = 0; i < count; ++i) {
        EZL_REQUIRE(A[i] && B[i], EZL_EINVAL, "ezl_gemm_bf16: null pointer");
        EZL_REQUIRE(ezl_aligned16(A[i]) && ezl_aligned16(B[i]) && lda % 8 == 0 && ldb % 8 == 0, EZL_EINVAL,
                    "ezl_gemm_bf16: operands must be 16-byte aligned with leading dimensions that are multiples of 8");
        EZL_REQUIRE(lda >= K[i] && lda < (1LL << 22) && ldb < (1LL << 22), EZL_EUNSUPPORTED,
                    "ezl_gemm_bf16: leading dimension too small, or 2^22 or more");
    }
    EZL_REQUIRE(N % 8 == 0 && ldb >= N && ldc >= N && M < (1LL << 31) && N < (1LL << 31) && ktot < (1LL << 31), EZL_EUNSUPPORTED,
                "ezl_gemm_bf16: contiguous extent of B must be a multiple of 8");
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    EZL_REQUIRE(tiles < (1LL << 31), EZL_EUNSUPPORTED, "ezl_gemm_bf16: too many tiles");
    KSegments seg;
    seg.A1 = (const bf16_t*)A[1]; seg.B1 = (const bf16_t*)B[1];
    seg.t1 = (int)(K[0] / BK);
    seg.A2 = count > 2 ? (const bf16_t*)A[2] : seg.A1; seg.B2 = count > 2 ? (const bf16_t*)B[2] : seg.B1;
    seg.t2 = count > 2 ? (int)((K[0] + K[1]) / BK) : 0x7fffffff;
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    EZL_REQUIRE(!workspace || ezl_aligned16(workspace), EZL_EINVAL, "ezl_gemm_bf16: workspace must be 16-byte aligned");
    const SplitPlan plan = make_plan(tiles, ktot / BK, workspace, workspace_bytes);
    const int split_tiles = (int)tiles - plan.full;
    hipLaunchKernelGGL((gemm_d2l_kernel<true, false, bf16_t, true>), dim3((unsigned)(plan.full + split_tiles * plan.nsplit)), dim3(512), 0,
                       (hipStream_t)stream, (const bf16_t*)A[0], (const bf16_t*)B[0], (bf16_t*)C, (int)M, (int)N, (int)ktot, lda, ldb, ldc,
                       accumulate, tiles_m, tiles_n, plan, seg);
    if (plan.nsplit > 1)
        hipLaunchKernelGGL((gemm_split_reduce_kernel<bf16_t>), dim3((unsigned)(split_tiles * 16)), dim3(256), 0, (hipStream_t)stream,
                           (bf16_t*)C, (int)M, (int)N, ldc, accumulate, tiles_m, tiles_n, plan);
    EZL_LAUNCH_CHECK("ezl_gemm_bf16_ksplit");
    return EZL_OK;
}
