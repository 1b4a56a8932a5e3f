// One tile of an NT product with a short contraction (K <= 128), shared by the stand-alone kernel of
// gemm.hip and the fused factorization step of spd.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace short_k {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kCols = 128;                  // columns of C per tile
constexpr int kMaxK = 128;
constexpr int kStride = kMaxK + 4;          // floats; 528-byte rows keep 16-byte reads conflict free

template <int ROWS>
constexpr int lds_floats() { return (ROWS + kCols) * kStride; }

// Tile number t of the lower triangle numbered row by row: (0,0), (1,0), (1,1), (2,0), ...
__device__ __forceinline__ void triangle_tile(uint32_t t, uint32_t& tile_m, uint32_t& tile_n) {
    tile_m = (uint32_t)((sqrtf(8.0f * (float)t + 1.0f) - 1.0f) * 0.5f);
    while (tile_m * (tile_m + 1) / 2 > t) --tile_m;
    while ((tile_m + 1) * (tile_m + 2) / 2 <= t) ++tile_m;
    tile_n = t - tile_m * (tile_m + 1) / 2;
}

// C[ROWS x 128 tile (tile_m, tile_n)] = alpha * A[M, K] * B[N, K]^T + beta * C.  Both operand tiles are
// loaded whole (one global round trip, one barrier), the MFMAs run back to back, the old values of C
// are fetched under them.  16-byte aligned rows, K <= 128 and a multiple of 8; 256 threads;
// `lds` holds lds_floats<ROWS>() floats, 16-byte aligned.
// ROWS = 128: 2 x 2 waves of 64 x 64.  ROWS = 32: 1 x 4 waves of 32 x 32.
template <int ROWS>
__device__ __forceinline__ void tile(const float* __restrict__ A, uint64_t lda, const float* __restrict__ B,
                                     uint64_t ldb, float* __restrict__ C, uint64_t ldc, uint64_t M, uint64_t N,
                                     uint32_t K, float alpha, float beta, uint32_t tile_m, uint32_t tile_n,
                                     float* __restrict__ lds) {
    constexpr int BM = kCols, kShortK = kMaxK, kShortStride = kStride;
    constexpr int WM = ROWS >= 64 ? 2 : 1, WNV = 4 / WM;           // wave grid
    constexpr int IT = ROWS / WM / 32, JT = BM / WNV / 32;          // 32 x 32 MFMA tiles per wave
    const uint64_t m0 = (uint64_t)tile_m * ROWS, n0 = (uint64_t)tile_n * BM;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave / WNV, wn = wave % WNV;
    const int x = lane & 31, h = lane >> 5;

    // rows x 32 float4 per operand, all loads in flight at once
    constexpr int kPiecesA = ROWS * (kShortK / 4) / kThreads, kPiecesB = BM * (kShortK / 4) / kThreads;
    float4 ra[kPiecesA], rb[kPiecesB];
#pragma unroll
    for (int i = 0; i < kPiecesA; ++i) {
        const int id = tid + kThreads * i;
        const uint32_t row = id >> 5, k4 = 4 * (id & 31);
        ra[i] = (m0 + row < M && k4 < K) ? *reinterpret_cast<const float4*>(A + (m0 + row) * lda + k4)
                                         : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < kPiecesB; ++i) {
        const int id = tid + kThreads * i;
        const uint32_t row = id >> 5, k4 = 4 * (id & 31);
        rb[i] = (n0 + row < N && k4 < K) ? *reinterpret_cast<const float4*>(B + (n0 + row) * ldb + k4)
                                         : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float* as = lds;
    float* bs = lds + ROWS * kShortStride;
#pragma unroll
    for (int i = 0; i < kPiecesA; ++i) {
        const int id = tid + kThreads * i;
        *reinterpret_cast<float4*>(as + (id >> 5) * kShortStride + 4 * (id & 31)) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < kPiecesB; ++i) {
        const int id = tid + kThreads * i;
        *reinterpret_cast<float4*>(bs + (id >> 5) * kShortStride + 4 * (id & 31)) = rb[i];
    }
    __syncthreads();

    const uint64_t row_base = m0 + wm * (32 * IT) + 4 * h, col_base = n0 + wn * (32 * JT) + x;
    floatx16 acc[IT][JT];
#pragma unroll
    for (int i = 0; i < IT; ++i)
#pragma unroll
        for (int j = 0; j < JT; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    // the old values of C are fetched here, so that their latency passes under the MFMAs
    floatx16 prev[IT][JT];
    if (beta != 0.0f) {
#pragma unroll
        for (int i = 0; i < IT; ++i)
#pragma unroll
            for (int j = 0; j < JT; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint64_t row = row_base + 32 * i + 8 * (r >> 2) + (r & 3);
                    const uint64_t col = col_base + 32 * j;
                    prev[i][j][r] = (row < M && col < N) ? C[row * ldc + col] : 0.f;
                }
    }
    // lane half h takes k = 8 s + 4 h + t for the t-th MFMA of sub-step s, as in the general kernel
    for (uint32_t s = 0; s < K / 8; ++s) {
        float4 fa[IT], fb[JT];
#pragma unroll
        for (int i = 0; i < IT; ++i)
            fa[i] = *reinterpret_cast<const float4*>(as + (wm * (32 * IT) + 32 * i + x) * kShortStride + 8 * s + 4 * h);
#pragma unroll
        for (int j = 0; j < JT; ++j)
            fb[j] = *reinterpret_cast<const float4*>(bs + (wn * (32 * JT) + 32 * j + x) * kShortStride + 8 * s + 4 * h);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < IT; ++i)
#pragma unroll
                for (int j = 0; j < JT; ++j) {
                    const float av = t == 0 ? fa[i].x : (t == 1 ? fa[i].y : (t == 2 ? fa[i].z : fa[i].w));
                    const float bv = t == 0 ? fb[j].x : (t == 1 ? fb[j].y : (t == 2 ? fb[j].z : fb[j].w));
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                }
    }
#pragma unroll
    for (int i = 0; i < IT; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint64_t row = row_base + 32 * i + 8 * (r >> 2) + (r & 3);
            if (row >= M) continue;
#pragma unroll
            for (int j = 0; j < JT; ++j) {
                const uint64_t col = col_base + 32 * j;
                if (col >= N) continue;
                float* c = C + row * ldc + col;
                float v = alpha * acc[i][j][r];
                if (beta != 0.0f) v += beta * prev[i][j][r];
                *c = v;
            }
        }
    }
}

}  // namespace short_k
