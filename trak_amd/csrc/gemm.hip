// fp32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32) for the scoring path.
//
// Stands in for the three torch matmuls of BasicScoreComputer: `block.T @ block`
// (trak/score_computers.py:153), `block @ xtx_inv` (:176) and `features @ target_grads.t()`
// (trak/utils.py:131), and is the building block of the blocked SPD inverse (spd.hip).
//
//   C[M, N] = alpha * op(A) * op(B) + beta * C      (then row i *= row_scale[i])
//
// Each operand is described by how it is stored relative to the contraction index k:
//   "row-k"  (KMAJOR = false): element (x, k) at ptr[x * ld + k]   (k contiguous)
//   "k-row"  (KMAJOR = true):  element (x, k) at ptr[k * ld + x]   (x contiguous)
// NT = (row-k, row-k), TN = (k-row, k-row), NN = (row-k, k-row).
//
// Workgroup = 256 threads = 4 waves in a 2x2 grid, 128 x BN tile of C (BN = 128 or 256), k step
// 16, two LDS buffers.  A wave owns 64 x BN/2 of C = 2 x (2 or 4) MFMA tiles (64 or 128
// accumulator VGPRs); the wide tile does twice the multiply-adds per LDS round trip and barrier
// and is used when C has at least 256 columns.  The MFMA sums over k in any order, so lane half
// h (= lane / 32) is given k = 8*s + 4*h + t for the t-th MFMA of sub-step s: a row-k operand
// then needs ONE 16-byte LDS read per four MFMAs.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "short_k_tile.h"
#include "trakhip_internal.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BKT = 16;
constexpr int kThreads = 256;
constexpr int kRowKStride = BKT + 4;   // floats; 80 B rows keep 16-byte reads conflict free
// an operand tile has ROWS rows (128 or 256) and BKT k-values; k-row tiles use ROWS floats per k
template <int ROWS>
struct Tile {
    static constexpr int pieces = ROWS * BKT / 4 / kThreads;  // 16-byte pieces per thread
    static constexpr int floats = ROWS * kRowKStride;          // >= BKT * ROWS
};

// ---- global -> registers -------------------------------------------------------------------

template <bool KMAJOR, bool ALIGNED, int ROWS>
__device__ __forceinline__ void load_tile(const float* __restrict__ p, uint64_t ld, uint64_t x0, uint64_t X,
                                          uint64_t k0, uint64_t K, int tid, float4 (&r)[Tile<ROWS>::pieces]) {
#pragma unroll
    for (int i = 0; i < Tile<ROWS>::pieces; ++i) {
        const int id = tid + kThreads * i;
        float4 v = {0.f, 0.f, 0.f, 0.f};
        if (!KMAJOR) {
            const uint64_t x = x0 + (id >> 2), k = k0 + 4 * (id & 3);
            if (x < X && k < K) {
                const float* q = p + x * ld + k;
                if (ALIGNED && k + 4 <= K) {
                    v = *reinterpret_cast<const float4*>(q);
                } else {
                    v.x = q[0];
                    if (k + 1 < K) v.y = q[1];
                    if (k + 2 < K) v.z = q[2];
                    if (k + 3 < K) v.w = q[3];
                }
            }
        } else {
            const uint64_t k = k0 + id / (ROWS / 4), x = x0 + 4 * (id % (ROWS / 4));
            if (k < K && x < X) {
                const float* q = p + k * ld + x;
                if (ALIGNED && x + 4 <= X) {
                    v = *reinterpret_cast<const float4*>(q);
                } else {
                    v.x = q[0];
                    if (x + 1 < X) v.y = q[1];
                    if (x + 2 < X) v.z = q[2];
                    if (x + 3 < X) v.w = q[3];
                }
            }
        }
        r[i] = v;
    }
}

template <bool KMAJOR, int ROWS>
__device__ __forceinline__ void store_tile(float* lds, int tid, const float4 (&r)[Tile<ROWS>::pieces]) {
#pragma unroll
    for (int i = 0; i < Tile<ROWS>::pieces; ++i) {
        const int id = tid + kThreads * i;
        if (!KMAJOR)
            *reinterpret_cast<float4*>(lds + (id >> 2) * kRowKStride + 4 * (id & 3)) = r[i];
        else
            *reinterpret_cast<float4*>(lds + (id / (ROWS / 4)) * ROWS + 4 * (id % (ROWS / 4))) = r[i];
    }
}

// The 4 operand values (t = 0..3) of lane (x, h) for sub-step s.
template <bool KMAJOR, int ROWS>
__device__ __forceinline__ float4 read_frag(const float* lds, int x, int h, int s) {
    if (!KMAJOR) return *reinterpret_cast<const float4*>(lds + x * kRowKStride + 8 * s + 4 * h);
    const float* q = lds + (8 * s + 4 * h) * ROWS + x;
    float4 v;
    v.x = q[0];
    v.y = q[ROWS];
    v.z = q[2 * ROWS];
    v.w = q[3 * ROWS];
    return v;
}

// One 128 x BN tile of C, tile number `tile` of a row-major tile grid tiles_n wide.
template <bool AK, bool BK, bool ALIGNED, int WN>
__device__ __forceinline__ void gemm_tile(const float* __restrict__ A, uint64_t lda, const float* __restrict__ B,
                                          uint64_t ldb, float* __restrict__ C, uint64_t ldc, uint64_t M, uint64_t N,
                                          uint64_t K, float alpha, float beta, const float* __restrict__ row_scale,
                                          uint32_t tiles_n, uint32_t flags, uint32_t tile) {
    constexpr int BN = 64 * WN;  // two waves side by side, WN 32-column MFMA tiles each
    __shared__ __attribute__((aligned(16))) float lds[2][Tile<BM>::floats + Tile<BN>::floats];

    const uint32_t tile_m = tile / tiles_n, tile_n = tile % tiles_n;
    const uint64_t m0 = (uint64_t)tile_m * BM, n0 = (uint64_t)tile_n * BN;
    // tiles strictly above the diagonal are not needed by a caller that reads the lower triangle
    if ((flags & trakhip::kGemmLowerTilesOnly) && n0 > m0 + BM - 1) return;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int x = lane & 31, h = lane >> 5;

    floatx16 acc[2][WN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const uint64_t nk = (K + BKT - 1) / BKT;
    float4 ra[Tile<BM>::pieces], rb[Tile<BN>::pieces];
    load_tile<AK, ALIGNED, BM>(A, lda, m0, M, 0, K, tid, ra);
    load_tile<BK, ALIGNED, BN>(B, ldb, n0, N, 0, K, tid, rb);
    store_tile<AK, BM>(lds[0], tid, ra);
    store_tile<BK, BN>(lds[0] + Tile<BM>::floats, tid, rb);
    __syncthreads();

    for (uint64_t kt = 0; kt < nk; ++kt) {
        const int cur = (int)(kt & 1);
        if (kt + 1 < nk) {
            load_tile<AK, ALIGNED, BM>(A, lda, m0, M, (kt + 1) * BKT, K, tid, ra);
            load_tile<BK, ALIGNED, BN>(B, ldb, n0, N, (kt + 1) * BKT, K, tid, rb);
        }
        const float* as = lds[cur];
        const float* bs = lds[cur] + Tile<BM>::floats;
#pragma unroll
        for (int s = 0; s < BKT / 8; ++s) {
            float4 fa[2], fb[WN];
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[i] = read_frag<AK, BM>(as, wm * 64 + 32 * i + x, h, s);
#pragma unroll
            for (int j = 0; j < WN; ++j) fb[j] = read_frag<BK, BN>(bs, wn * (32 * WN) + 32 * j + x, h, s);
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < WN; ++j) {
                        const float av = t == 0 ? fa[i].x : (t == 1 ? fa[i].y : (t == 2 ? fa[i].z : fa[i].w));
                        const float bv = t == 0 ? fb[j].x : (t == 1 ? fb[j].y : (t == 2 ? fb[j].z : fb[j].w));
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                    }
        }
        if (kt + 1 < nk) {
            store_tile<AK, BM>(lds[cur ^ 1], tid, ra);
            store_tile<BK, BN>(lds[cur ^ 1] + Tile<BM>::floats, tid, rb);
        }
        __syncthreads();
    }

    // D[m][n] of a 32x32 MFMA: lane holds column n = lane % 32; register r holds row
    // 8*(r/4) + 4*(lane/32) + r%4.  When C is accumulated into, its old values are fetched for 32 rows
    // at a time before any of them is overwritten (loads and stores through one pointer would
    // otherwise alternate, one memory round trip per element).
    const uint64_t col0 = n0 + wn * (32 * WN) + x;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint64_t row0 = m0 + wm * 64 + 32 * i + 4 * h;
        floatx16 prev[WN];
        if (beta != 0.0f) {
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint64_t row = row0 + 8 * (r >> 2) + (r & 3), col = col0 + 32 * j;
                    prev[j][r] = (row < M && col < N) ? C[row * ldc + col] : 0.0f;
                }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint64_t row = row0 + 8 * (r >> 2) + (r & 3);
            if (row >= M) continue;
            const float rs = row_scale ? row_scale[row] : 1.0f;
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const uint64_t col = col0 + 32 * j;
                if (col >= N) continue;
                float v = alpha * acc[i][j][r];
                if (beta != 0.0f) v += beta * prev[j][r];
                C[row * ldc + col] = v * rs;
            }
        }
    }
}

template <bool AK, bool BK, bool ALIGNED, int WN>
__global__ __launch_bounds__(kThreads, 2) void gemm_kernel(const float* __restrict__ A, uint64_t lda,
                                                           const float* __restrict__ B, uint64_t ldb,
                                                           float* __restrict__ C, uint64_t ldc, uint64_t M,
                                                           uint64_t N, uint64_t K, float alpha, float beta,
                                                           const float* __restrict__ row_scale,
                                                           uint32_t tiles_n, uint32_t flags) {
    gemm_tile<AK, BK, ALIGNED, WN>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, row_scale, tiles_n, flags,
                                   blockIdx.x);
}

// Several independent products of one shape in one launch: product y = blockIdx.y works on
// A + batch.a[y], B + batch.b[y], C + batch.c[y] (element offsets).  NN operands, 128 x 128 tiles.
__global__ __launch_bounds__(kThreads, 2) void gemm_nn_batched_kernel(const float* __restrict__ A, uint64_t lda,
                                                                      const float* __restrict__ B, uint64_t ldb,
                                                                      float* __restrict__ C, uint64_t ldc, uint64_t M,
                                                                      uint64_t N, uint64_t K, float alpha, float beta,
                                                                      uint32_t tiles_n, trakhip::GemmBatch batch) {
    const uint32_t y = blockIdx.y;
    const uint64_t my = batch.m[y] ? batch.m[y] : M;
    if ((uint64_t)(blockIdx.x / tiles_n) * BM >= my) return;  // (the whole workgroup: the grid is sized for the call's M)
    gemm_tile<false, true, true, 2>(A + batch.a[y], lda, B + batch.b[y], ldb, C + batch.c[y], ldc, my, N, K, alpha,
                                    beta, nullptr, tiles_n, 0u, blockIdx.x);
}

// NT product with a short contraction (K <= 128, the panel width of the blocked factorization):
// C[M, N] = alpha * A[M, K] * B[N, K]^T + beta * C, ROWS x 128 tiles.  The general kernel walks k in
// steps of 16 with one global-memory round trip per step, which is all latency when there are
// only eight steps; here both operand tiles are loaded whole (one round trip, one barrier) and the
// MFMAs run back to back.  Needs 16-byte aligned rows and K a multiple of 8.
// ROWS = 128: 2 x 2 waves of 64 x 64, 135 KB of LDS, one workgroup per CU.  ROWS = 32: 1 x 4 waves of
// 32 x 32 for products with few rows of tiles (the panel: N = 128), four times as many workgroups.
template <int ROWS>
__global__ __launch_bounds__(kThreads, 1) void gemm_nt_short_k_kernel(const float* __restrict__ A, uint64_t lda,
                                                                      const float* __restrict__ B, uint64_t ldb,
                                                                      float* __restrict__ C, uint64_t ldc, uint64_t M,
                                                                      uint64_t N, uint32_t K, float alpha, float beta,
                                                                      uint32_t tiles_n, uint32_t flags) {
    __shared__ __attribute__((aligned(16))) float lds[short_k::lds_floats<ROWS>()];
    // With kGemmLowerTilesOnly (square tiles only) the grid holds the lower-triangle tiles alone, numbered
    // row by row (a workgroup that only returns would still wait for a CU with this much LDS free).
    uint32_t tile_m, tile_n;
    if (ROWS == BM && (flags & trakhip::kGemmLowerTilesOnly)) {
        short_k::triangle_tile(blockIdx.x, tile_m, tile_n);
    } else {
        tile_m = blockIdx.x / tiles_n;
        tile_n = blockIdx.x % tiles_n;
    }
    short_k::tile<ROWS>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, tile_m, tile_n, lds);
}

template <bool AK, bool BK, int WN>
int launch_tiles(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
                 uint64_t N, uint64_t K, float alpha, float beta, const float* row_scale, bool aligned,
                 uint32_t flags, hipStream_t s) {
    constexpr int BN = 64 * WN;
    const uint64_t tm = (M + BM - 1) / BM, tn = (N + BN - 1) / BN;
    if (tm * tn > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    const dim3 grid((uint32_t)(tm * tn)), block(kThreads);
    if (aligned)
        hipLaunchKernelGGL((gemm_kernel<AK, BK, true, WN>), grid, block, 0, s, A, lda, B, ldb, C, ldc, M, N, K, alpha,
                           beta, row_scale, (uint32_t)tn, flags);
    else
        hipLaunchKernelGGL((gemm_kernel<AK, BK, false, WN>), grid, block, 0, s, A, lda, B, ldb, C, ldc, M, N, K,
                           alpha, beta, row_scale, (uint32_t)tn, flags);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

template <bool AK, bool BK>
int launch(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
           uint64_t N, uint64_t K, float alpha, float beta, const float* row_scale, uint32_t flags, hipStream_t s) {
    if (M == 0 || N == 0) return TRAKHIP_OK;
    if (!A || !B || !C) return TRAKHIP_ERR_NULL;
    const uint64_t min_lda = AK ? M : K, min_ldb = BK ? N : K;
    if (lda < min_lda || ldb < min_ldb || ldc < N) return TRAKHIP_ERR_SHAPE;
    const bool aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
                         (lda % 4 == 0) && (ldb % 4 == 0);
    // the wide tile pays off once C has a few hundred 128 x 256 tiles; narrow C keeps 128 x 128
    const bool wide = N >= 256 && ((M + BM - 1) / BM) * ((N + 255) / 256) >= 256;
    if (wide)
        return launch_tiles<AK, BK, 4>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, row_scale, aligned, flags, s);
    return launch_tiles<AK, BK, 2>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, row_scale, aligned, flags, s);
}

}  // namespace

namespace trakhip {

int gemm_nt(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
            uint64_t N, uint64_t K, float alpha, float beta, const float* row_scale, hipStream_t s, uint32_t flags) {
    const bool aligned = A && B && (reinterpret_cast<uintptr_t>(A) % 16 == 0) &&
                         (reinterpret_cast<uintptr_t>(B) % 16 == 0) && (lda % 4 == 0) && (ldb % 4 == 0);
    if (M && N && C && aligned && !row_scale && K >= 8 && K <= short_k::kMaxK && K % 8 == 0 && lda >= K && ldb >= K &&
        ldc >= N) {
        const uint64_t tm = (M + BM - 1) / BM, tn = (N + BM - 1) / BM;
        // Lower tiles only: a square tile grid is launched as its triangle; otherwise the flag is dropped
        // (computing the upper tiles too is allowed, skipping them is an optimisation).
        const bool triangle = (flags & kGemmLowerTilesOnly) && tm == tn;
        const uint64_t working = triangle ? tm * (tm + 1) / 2 : tm * tn;
        const bool whole = triangle || !(flags & kGemmLowerTilesOnly);
        // too few 128-row tiles to occupy the CUs: 32-row tiles, four times as many workgroups
        if (whole && !triangle && working <= 64) {
            const uint64_t tm32 = (M + 31) / 32;
            hipLaunchKernelGGL(gemm_nt_short_k_kernel<32>, dim3((uint32_t)(tm32 * tn)), dim3(kThreads), 0, s, A, lda, B,
                               ldb, C, ldc, M, N, (uint32_t)K, alpha, beta, (uint32_t)tn, 0u);
            return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
        }
        // one workgroup per CU (its LDS) and no overlap inside it: worth it for up to two rounds
        if (whole && working <= 512) {
            hipLaunchKernelGGL(gemm_nt_short_k_kernel<BM>, dim3((uint32_t)working), dim3(kThreads), 0, s, A, lda, B, ldb,
                               C, ldc, M, N, (uint32_t)K, alpha, beta, (uint32_t)tn,
                               triangle ? kGemmLowerTilesOnly : 0u);
            return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
        }
    }
    return launch<false, false>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, row_scale, flags, s);
}

int gemm_tn(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
            uint64_t N, uint64_t K, float alpha, float beta, hipStream_t s, uint32_t flags) {
    return launch<true, true>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, nullptr, flags, s);
}

int gemm_nn(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
            uint64_t N, uint64_t K, float alpha, float beta, hipStream_t s, uint32_t flags) {
    return launch<false, true>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, nullptr, flags, s);
}

int gemm_nn_batched(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
                    uint64_t N, uint64_t K, float alpha, float beta, const GemmBatch& batch, hipStream_t s) {
    if (M == 0 || N == 0 || batch.count == 0) return TRAKHIP_OK;
    if (!A || !B || !C) return TRAKHIP_ERR_NULL;
    if (batch.count > kGemmBatchMax || lda < K || ldb < N || ldc < N) return TRAKHIP_ERR_SHAPE;
    // the batched kernel uses 16-byte loads: every operand start and pitch must allow them
    if ((reinterpret_cast<uintptr_t>(A) % 16) || (reinterpret_cast<uintptr_t>(B) % 16) || (lda % 4) || (ldb % 4))
        return TRAKHIP_ERR_ALIGN;
    for (uint32_t y = 0; y < batch.count; ++y) {
        if ((batch.a[y] % 4) || (batch.b[y] % 4)) return TRAKHIP_ERR_ALIGN;
        if (batch.m[y] > M) return TRAKHIP_ERR_SHAPE;
    }
    const uint64_t tm = (M + BM - 1) / BM, tn = (N + 127) / 128;
    if (tm * tn > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    hipLaunchKernelGGL(gemm_nn_batched_kernel, dim3((uint32_t)(tm * tn), batch.count), dim3(kThreads), 0, s, A, lda, B,
                       ldb, C, ldc, M, N, K, alpha, beta, (uint32_t)tn, batch);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

}  // namespace trakhip
