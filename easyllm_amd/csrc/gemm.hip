// bf16 MFMA GEMM for gfx950: C[M,N] = A * B with fp32 accumulation.
//
// Replaces the three matmuls of the reference's linear layers
// (base_modules/layers/column_parallel_linear.py:42 forward, :68 input gradient, :99 weight
// gradient; row_parallel_linear.py:113; llama/lm_head.py:62):
//   forward   Y[T,out]  = X[T,in]   * W[out,in]^T    A k-contiguous, B k-contiguous
//   dgrad     dX[T,in]  = dY[T,out] * W[out,in]      A k-contiguous, B n-contiguous
//   wgrad     dW[out,in]= dY[T,out]^T * X[T,in]      A m-contiguous, B n-contiguous   (fp32 or bf16 out)
//
// Tiling: 256x256 block tile, K step 64, 4 waves (2x2), each wave owns 128x128 = 4x4 MFMA
// 32x32x16 tiles (256 fp32 accumulators per lane).  Both operand tiles are staged in LDS, double
// buffered (2 x 2 x 36 KiB of the 160 KiB), filled through registers with 128-bit global loads that
// are issued one full K step ahead of their use.  A k-contiguous operand is stored [row][64 + 8 pad]
// and read with ds_read_b128; an operand whose reduction dimension is the strided one is stored as
// it lies in memory, [k][256 + 32 pad], and read with ds_read_b64_tr_b16 (the LDS transpose read),
// so no operand is ever transposed in HBM.  Blocks are renumbered so that each XCD (own L2) works
// on a contiguous band of tiles, grouped 8 tiles tall.
#include "common.h"

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int NT = 256;
constexpr int LDK = BK + 8;     // row stride (elements) of a k-contiguous tile  [256][72]
constexpr int LDN = 256 + 32;   // row stride (elements) of a k-major tile       [64][288]
constexpr int TILE = 256 * LDK; // == 64 * LDN elements per operand per stage
static_assert(TILE == 64 * LDN, "both tile layouts must have the same footprint");

typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;

// ---- global -> register staging of one operand tile (8 x 128-bit per thread) -------------------
template <bool KC>
struct Stager {
    uint32_t off[8];  // element offsets of this thread's 8 chunks at k = 0
    int krow;         // (non-KC) k row of chunk 0 / (KC) k column of all chunks
    // dim = extent of the non-reduction dimension, first = first row/col of the block tile
    __device__ __forceinline__ void init(int tid, int first, int dim, int64_t ld) {
        if (KC) {
            krow = (tid & 7) * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                int r = first + (tid >> 3) + 32 * i;
                r = r < dim ? r : dim - 1;
                off[i] = (uint32_t)((int64_t)r * ld + krow);
            }
        } else {
            krow = tid >> 5;
            int c = first + (tid & 31) * 8;
            c = c + 8 <= dim ? c : dim - 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) off[i] = (uint32_t)((int64_t)(krow + 8 * i) * ld + c);
        }
    }
    // k0 = first k of the tile; kadv = element offset of that k (k0 for KC, k0 * ld otherwise)
    __device__ __forceinline__ void load(const bf16_t* __restrict__ base, int k0, int64_t kadv, int K, bf16x8* r) const {
        const bf16_t* p = base + kadv;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool ok = KC ? (k0 + krow < K) : (k0 + krow + 8 * i < K);
            bf16x8 z;
#pragma unroll
            for (int j = 0; j < 8; ++j) z[j] = (bf16_t)0.0f;
            r[i] = ok ? *reinterpret_cast<const bf16x8*>(p + off[i]) : z;
        }
    }
    __device__ __forceinline__ void store(bf16_t* __restrict__ s, int tid, const bf16x8* r) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (KC) *reinterpret_cast<bf16x8*>(s + ((tid >> 3) + 32 * i) * LDK + (tid & 7) * 8) = r[i];
            else *reinterpret_cast<bf16x8*>(s + ((tid >> 5) + 8 * i) * LDN + (tid & 31) * 8) = r[i];
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

template <bool A_KC, bool B_KC, typename OutT>
__global__ __launch_bounds__(NT) void gemm_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ B, OutT* __restrict__ C,
                                                  int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int accumulate,
                                                  int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(16))) bf16_t smem[4 * TILE];  // A0 B0 A1 B1
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

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

    Stager<A_KC> sa;
    Stager<B_KC> sb;
    sa.init(tid, m0, M, lda);
    sb.init(tid, n0, N, ldb);
    bf16x8 ra[8], rb[8];

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
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
        bf16_t* sA = smem + cur * 2 * TILE;
        bf16_t* sB = sA + TILE;
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
            bf16x8 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = frag<A_KC>(sA, wm * 128 + i * 32, ks, lane);
#pragma unroll
            for (int j = 0; j < 4; ++j) fb[j] = frag<B_KC>(sB, wn * 128 + j * 32, ks, lane);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // epilogue: lane holds column (lane & 31); register r is row 8*(r/4) + 4*(lane>>5) + r%4
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + wn * 128 + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * 128 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row < M && col < N) store_out<OutT>(C + (int64_t)row * ldc + col, acc[i][j][r], accumulate != 0);
            }
        }
    }
}

}  // namespace

// a_kc / b_kc: 1 if the operand's reduction index is its contiguous one
//   A: a_kc ? A[m * lda + k] : A[k * lda + m]        B: b_kc ? B[n * ldb + k] : B[k * ldb + n]
// out_dtype: 0 bf16, 1 fp32.  accumulate: C += A*B instead of C = A*B.
extern "C" int ezl_gemm_bf16(const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                             int64_t ldc, int a_kc, int b_kc, int out_dtype, int accumulate, void* stream) {
    EZL_REQUIRE(M >= 0 && N >= 0 && K >= 0, EZL_EINVAL, "ezl_gemm_bf16: negative size");
    EZL_REQUIRE(out_dtype == 0 || out_dtype == 1, EZL_EUNSUPPORTED, "ezl_gemm_bf16: out_dtype must be 0 (bf16) or 1 (fp32)");
    if (M == 0 || N == 0) return EZL_OK;
    EZL_REQUIRE(K > 0, EZL_EUNSUPPORTED, "ezl_gemm_bf16: K must be positive");
    EZL_REQUIRE(A && B && C, EZL_EINVAL, "ezl_gemm_bf16: null pointer");
    EZL_REQUIRE(ezl_aligned16(A) && ezl_aligned16(B) && lda % 8 == 0 && ldb % 8 == 0, EZL_EINVAL,
                "ezl_gemm_bf16: operands must be 16-byte aligned with leading dimensions that are multiples of 8");
    // every 128-bit chunk must lie wholly inside or wholly outside the matrix
    EZL_REQUIRE(a_kc ? (K % 8 == 0) : (M % 8 == 0), EZL_EUNSUPPORTED, "ezl_gemm_bf16: contiguous extent of A must be a multiple of 8");
    EZL_REQUIRE(b_kc ? (K % 8 == 0) : (N % 8 == 0), EZL_EUNSUPPORTED, "ezl_gemm_bf16: contiguous extent of B must be a multiple of 8");
    EZL_REQUIRE(lda >= (a_kc ? K : M) && ldb >= (b_kc ? K : N) && ldc >= N, EZL_EINVAL, "ezl_gemm_bf16: leading dimension too small");
    const int64_t a_rows = a_kc ? M : K, b_rows = b_kc ? N : K;
    EZL_REQUIRE(a_rows * lda < (1LL << 32) && b_rows * ldb < (1LL << 32) && M < (1LL << 31) && N < (1LL << 31) && K < (1LL << 31),
                EZL_EUNSUPPORTED, "ezl_gemm_bf16: operand larger than 2^32 elements");
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    EZL_REQUIRE((int64_t)tiles_m * tiles_n < (1LL << 31), EZL_EUNSUPPORTED, "ezl_gemm_bf16: too many tiles");
    const dim3 grid((unsigned)(tiles_m * tiles_n)), block(NT);
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(AK, BKC, OT)                                                                                         \
    hipLaunchKernelGGL((gemm_kernel<AK, BKC, OT>), grid, block, 0, st, (const bf16_t*)A, (const bf16_t*)B, (OT*)C, (int)M, \
                       (int)N, (int)K, lda, ldb, ldc, accumulate, tiles_m, tiles_n)
    if (out_dtype == 0) {
        if (a_kc && b_kc) LAUNCH(true, true, bf16_t);
        else if (a_kc && !b_kc) LAUNCH(true, false, bf16_t);
        else if (!a_kc && !b_kc) LAUNCH(false, false, bf16_t);
        else LAUNCH(false, true, bf16_t);
    } else {
        if (a_kc && b_kc) LAUNCH(true, true, float);
        else if (a_kc && !b_kc) LAUNCH(true, false, float);
        else if (!a_kc && !b_kc) LAUNCH(false, false, float);
        else LAUNCH(false, true, float);
    }
#undef LAUNCH
    EZL_LAUNCH_CHECK("ezl_gemm_bf16");
    return EZL_OK;
}
