// (A + lambda I)^-1 for a symmetric positive definite fp32 matrix on one GPU, plus the
// "divide by the mean absolute entry" step of the reference.
//
// Stands in for  xtx_inv = torch.linalg.inv(xtx + lambda_reg * eye);  xtx_inv /= xtx_inv.abs().mean()
// (trak/score_computers.py:160-166).  The reference inverts with LU; the matrix here is a Gram
// matrix plus a ridge, so this file uses a blocked Cholesky factorization instead:
//
//   1. W = A + lambda I, padded with an identity block up to a multiple of 128;
//   2. for every 128-block column j:  one workgroup factors the diagonal block in LDS
//      (L_jj) and inverts it; the panel below it is  W[j+1:, j] * L_jj^-T  and the trailing
//      matrix gets  W -= panel * panel^T   (MFMA products; the trailing update and the next
//      diagonal block share one launch, see spd_step_kernel);
//   3. L^-1 by recursive halving: inv([[A,0],[B,C]]) = [[A^-1,0],[-C^-1 B A^-1, C^-1]]
//      (two GEMMs per node of the recursion tree);
//   4. inverse = L^-T L^-1 (one GEMM), then the mean of |.| by a two-stage reduction in a
//      fixed order and a scaling pass.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>
#include <vector>

#include "short_k_tile.h"
#include "trakhip_internal.h"

namespace {

constexpr int NB = 128;
constexpr int kSumBlocks = 1024;

__global__ __launch_bounds__(256) void spd_init_kernel(const float* __restrict__ A, uint64_t lda, float lambda,
                                                       uint64_t n, uint64_t np, float* __restrict__ W,
                                                       float* __restrict__ Li, int32_t* __restrict__ status) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx == 0 && status) *status = 0;
    if (idx >= np * np) return;
    const uint64_t i = idx / np, j = idx % np;
    float v;
    if (i < n && j < n)
        v = A[i * lda + j] + (i == j ? lambda : 0.0f);
    else
        v = (i == j) ? 1.0f : 0.0f;
    W[idx] = v;
    Li[idx] = 0.0f;  // the blocks above the diagonal stay zero: the final product reads all of Li
    // (every block of L that is read later - diagonal blocks, panels - is written first)
}

// One workgroup of four waves: Cholesky of the 128x128 diagonal block at W (lower triangle used),
// L block to Lout (upper part zero), its inverse to Linv_out.
//
// The block is handled as 4 x 4 sub-blocks of 32 in LDS (row pitch 129 floats: conflict free by rows
// and by columns).  For sub-block column p:
//   - ONE WAVE factors the 32 x 32 diagonal sub-block and inverts the factor, registers only, values of
//     other lanes through v_readlane: no barriers and no LDS round trips inside this strictly
//     sequential part (see factor_sub_block);
//   - the sub-blocks below become L = A X^T and the trailing sub-blocks get A -= L L^T, both on
//     v_mfma_f32_32x32x2_f32, one 32 x 32 tile per wave at a time.
// The off-diagonal sub-blocks of the inverse follow by halving, [A 0; B C]^-1 = [A^-1 0; -C^-1 B A^-1 C^-1],
// two levels (32 -> 64 -> 128), again on the MFMA.  About 1200 vector instructions per sub-block on one
// wave and a dozen workgroup barriers, against 128 barriers (and an LDS round trip
// each) for a column-at-a-time loop over the whole block.
constexpr int kSub = 32;
constexpr int kPitch = NB + 1;
constexpr int kTPitch = 2 * kSub + 1;

typedef float floatx16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Row 8*(r/4) + 4*(lane/32) + r%4 of a 32x32 MFMA result is in register r; its column is lane % 32.
__device__ __forceinline__ int mfma_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// Factor and invert the 32 x 32 sub-block at (base, base) of As with one wave.  Lane x of the lower
// half-wave holds row x of A in v[0..31]; lane 32 + c of the upper half holds column c of X, which
// starts as the identity (v[j] = X[j][c]).  Step k scales v[k] by s = 1 / sqrt(A[k][k]) in every lane
// (lower half: column k of L; upper half: the finished row k of X = L^-1), then for j > k every lane
// does v[j] -= v[k] L[j][k] with L[j][k] read from lane j: the trailing update of A in the lower half,
// forward elimination of the identity in the upper half - one lane read and one multiply-add per (k, j).
__device__ __forceinline__ void factor_sub_block(float* As, float* Xs, int base, int lane, int32_t first_index,
                                                 int32_t* status) {
    const int x = lane & 31;
    const bool lower = lane < kSub;
    float v[kSub];
    int32_t bad = 0;  // 1 + index of the first pivot that is not positive
    // every lane reads its row (the upper half-wave the same one again): 32 loads in flight, no
    // branch per element around them
    float row[kSub];
#pragma unroll
    for (int j = 0; j < kSub; ++j) row[j] = As[(base + x) * kPitch + base + j];
#pragma unroll
    for (int j = 0; j < kSub; ++j) {
        asm volatile("" : "+v"(row[j]));
        v[j] = lower ? row[j] : (j == x ? 1.0f : 0.0f);
    }
#pragma unroll
    for (int k = 0; k < kSub; ++k) {
        float d = lane_value(v[k], k);
        // a pivot that is not positive is recorded and replaced, without a branch: the 32 steps stay one
        // straight line of code
        const bool ok = d > 0.0f;
        bad = (ok || bad != 0) ? bad : 1 + first_index + k;
        d = ok ? d : 1.0f;
        float s = __builtin_amdgcn_rsqf(d);
        s = s * __builtin_fmaf(-0.5f * d * s, s, 1.5f);  // one Newton step on the 1 ulp hardware value
        const float t = v[k] * s;
        v[k] = t;
        // All lane reads first, then the multiply-adds: a scalar register written by a vector
        // instruction cannot be read by the next one.  The empty volatile statement and the fences pin
        // each step between its neighbours (otherwise lane reads of later steps drift up here and
        // their scalar results spill).
        __builtin_amdgcn_sched_barrier(0);
        float lj[kSub];
#pragma unroll
        for (int j = k + 1; j < kSub; ++j) lj[j] = lane_value(t, j);
#pragma unroll
        for (int j = k + 1; j < kSub; ++j) v[j] = __builtin_fmaf(-t, lj[j], v[j]);
        if (k + 1 < kSub) asm volatile("" : "+v"(v[k + 1]));
        __builtin_amdgcn_sched_barrier(0);
    }
    if (bad != 0 && lane == 0 && status && *status == 0) *status = bad;
    // lower half: row x of L (zero above the diagonal); upper half: X[j][x], zero above the diagonal by
    // construction.  One store per j for the whole wave.
    float* dst = lower ? As + (base + x) * kPitch + base : Xs + base * kPitch + base + x;
    const int step = lower ? 1 : kPitch;
#pragma unroll
    for (int j = 0; j < kSub; ++j) dst[j * step] = (lower && j > x) ? 0.0f : v[j];
}

// acc += sign * A[32 x K] * op(B): A rows at `a` (pitch pa, k contiguous); B^T rows at `b` (B_T: pitch
// pb, k contiguous) or B rows at `b` (k down the rows, pitch pb).  LDS operands.
template <bool B_T>
__device__ __forceinline__ floatx16 tile_product(const float* a, int pa, const float* b, int pb, int K, float sign,
                                                 floatx16 acc, int lane) {
    const int x = lane & 31, h = lane >> 5;
    for (int k2 = 0; k2 < K; k2 += 2) {  // the half-wave h takes k2 + h
        const int k = k2 + h;
        const float av = sign * a[x * pa + k];
        const float bv = B_T ? b[x * pb + k] : b[k * pb + x];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
    }
    return acc;
}

__device__ __forceinline__ floatx16 tile_load(const float* c, int pc, int lane) {
    const int x = lane & 31, h = lane >> 5;
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = c[mfma_row(r, h) * pc + x];
    return acc;
}

__device__ __forceinline__ void tile_store(float* c, int pc, const floatx16& acc, int lane) {
    const int x = lane & 31, h = lane >> 5;
#pragma unroll
    for (int r = 0; r < 16; ++r) c[mfma_row(r, h) * pc + x] = acc[r];
}

__device__ __forceinline__ floatx16 tile_zero() {
    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    return acc;
}

constexpr int kDiagLdsFloats = 2 * NB * kPitch + 2 * kSub * kTPitch;  // 148 736 bytes

// `panel`, when not null, is the 128 x 128 block of the factor to the left of this diagonal block
// (row pitch ldp) whose contribution has not been taken off W yet: the block that is factored is
// W - panel panel^T (its lower triangle).
__device__ __forceinline__ void diag_block(const float* __restrict__ W, uint64_t ldw, float* __restrict__ Lout,
                                           float* __restrict__ Linv_out, uint64_t ldl, int32_t block_index,
                                           int32_t* __restrict__ status, const float* __restrict__ panel,
                                           uint64_t ldp, float* __restrict__ lds) {
    float* As = lds;                        // the block, overwritten by its factor
    float* Xs = As + NB * kPitch;           // the inverse of the factor
    float* Ts = Xs + NB * kPitch;           // B A^-1 of the halving steps
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;  // wave index in a scalar register

    // thread -> (row tid / 32 + 8 i, four columns from 4 (tid % 32)); all sixteen loads in flight at once
    // (the block starts at a multiple of 128 floats of a 16-byte aligned matrix with ldw % 128 == 0)
    {
        const int r0 = tid >> 5, c = 4 * (tid & 31);
        float4 v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = *reinterpret_cast<const float4*>(W + (uint64_t)(r0 + 8 * i) * ldw + c);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int r = r0 + 8 * i;
            float* a = As + r * kPitch + c;
            float* x = Xs + r * kPitch + c;
            a[0] = (c + 0 <= r) ? v[i].x : 0.0f;
            a[1] = (c + 1 <= r) ? v[i].y : 0.0f;
            a[2] = (c + 2 <= r) ? v[i].z : 0.0f;
            a[3] = (c + 3 <= r) ? v[i].w : 0.0f;
            x[0] = x[1] = x[2] = x[3] = 0.0f;
        }
    }
    constexpr int kBlocks = NB / kSub;
    if (panel) {
        // Xs borrows the panel block; the ten 32 x 32 sub-blocks on or under the diagonal get
        // A -= P P^T (what is left above the diagonal is never read); then Xs is cleared again
        const int r0 = tid >> 5, c = 4 * (tid & 31);
        float4 v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) v[i] = *reinterpret_cast<const float4*>(panel + (uint64_t)(r0 + 8 * i) * ldp + c);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float* x = Xs + (r0 + 8 * i) * kPitch + c;
            x[0] = v[i].x, x[1] = v[i].y, x[2] = v[i].z, x[3] = v[i].w;
        }
        __syncthreads();
        for (int t = wave; t < kBlocks * (kBlocks + 1) / 2; t += 4) {
            const int ti = t < 1 ? 0 : (t < 3 ? 1 : (t < 6 ? 2 : 3)), tj = t - ti * (ti + 1) / 2;
            float* tile = As + kSub * ti * kPitch + kSub * tj;
            const floatx16 acc = tile_product<true>(Xs + kSub * ti * kPitch, kPitch, Xs + kSub * tj * kPitch, kPitch, NB,
                                                    -1.0f, tile_load(tile, kPitch, lane), lane);
            tile_store(tile, kPitch, acc, lane);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float* x = Xs + (r0 + 8 * i) * kPitch + c;
            x[0] = x[1] = x[2] = x[3] = 0.0f;
        }
    }
    __syncthreads();

    for (int p = 0; p < kBlocks; ++p) {
        const int base = kSub * p;
        if (wave == 0) factor_sub_block(As, Xs, base, lane, block_index * NB + base, status);
        __syncthreads();
        const int below = kBlocks - 1 - p;  // sub-blocks under the diagonal one
        if (below == 0) break;
        // L[t][p] = A[t][p] X_pp^T, one sub-block per wave (at most three)
        if (wave < below) {
            float* tile = As + (base + kSub * (1 + wave)) * kPitch + base;
            const floatx16 acc = tile_product<true>(tile, kPitch, Xs + base * kPitch + base, kPitch, kSub, 1.0f,
                                                    tile_zero(), lane);
            tile_store(tile, kPitch, acc, lane);  // every read of the tile precedes this in the wave's LDS order
        }
        __syncthreads();
        // A[ti][tj] -= L[ti][p] L[tj][p]^T for the sub-blocks tj <= ti below and right of (p, p)
        const int tiles = below * (below + 1) / 2;
        for (int t = wave; t < tiles; t += 4) {
            const int ti = t < 1 ? 0 : (t < 3 ? 1 : 2), tj = t - ti * (ti + 1) / 2;
            const int ri = base + kSub * (1 + ti), rj = base + kSub * (1 + tj);
            float* tile = As + ri * kPitch + rj;
            const floatx16 acc = tile_product<true>(As + ri * kPitch + base, kPitch, As + rj * kPitch + base, kPitch,
                                                    kSub, -1.0f, tile_load(tile, kPitch, lane), lane);
            tile_store(tile, kPitch, acc, lane);
        }
        __syncthreads();
    }

    // halving, level 1: sub-block pairs (0, 1) and (2, 3) on waves 0 and 1
    if (wave < 2) {
        const int lo = 2 * kSub * wave, mid = lo + kSub;
        float* scratch = Ts + kSub * wave * kTPitch;
        const floatx16 t = tile_product<false>(As + mid * kPitch + lo, kPitch, Xs + lo * kPitch + lo, kPitch, kSub, 1.0f,
                                               tile_zero(), lane);
        tile_store(scratch, kTPitch, t, lane);
    }
    __syncthreads();
    if (wave < 2) {
        const int lo = 2 * kSub * wave, mid = lo + kSub;
        const float* scratch = Ts + kSub * wave * kTPitch;
        const floatx16 r = tile_product<false>(Xs + mid * kPitch + mid, kPitch, scratch, kTPitch, kSub, -1.0f,
                                               tile_zero(), lane);
        tile_store(Xs + mid * kPitch + lo, kPitch, r, lane);
    }
    __syncthreads();
    // level 2: the 64 x 64 block under the diagonal, one 32 x 32 tile per wave
    {
        const int ti = wave >> 1, tj = wave & 1, half = 2 * kSub;
        const floatx16 t = tile_product<false>(As + (half + kSub * ti) * kPitch, kPitch, Xs + kSub * tj, kPitch, half,
                                               1.0f, tile_zero(), lane);
        tile_store(Ts + kSub * ti * kTPitch + kSub * tj, kTPitch, t, lane);
        __syncthreads();
        const floatx16 r = tile_product<false>(Xs + (half + kSub * ti) * kPitch + half, kPitch, Ts + kSub * tj, kTPitch,
                                               half, -1.0f, tile_zero(), lane);
        tile_store(Xs + (half + kSub * ti) * kPitch + kSub * tj, kPitch, r, lane);
    }
    __syncthreads();

    {
        const int r0 = tid >> 5, c = 4 * (tid & 31);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int r = r0 + 8 * i;
            const float* a = As + r * kPitch + c;
            const float* x = Xs + r * kPitch + c;
            const float a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];  // read first, then select: no branches
            const float x0 = x[0], x1 = x[1], x2 = x[2], x3 = x[3];
            float4 l, li;
            l.x = (c + 0 <= r) ? a0 : 0.0f, li.x = (c + 0 <= r) ? x0 : 0.0f;
            l.y = (c + 1 <= r) ? a1 : 0.0f, li.y = (c + 1 <= r) ? x1 : 0.0f;
            l.z = (c + 2 <= r) ? a2 : 0.0f, li.z = (c + 2 <= r) ? x2 : 0.0f;
            l.w = (c + 3 <= r) ? a3 : 0.0f, li.w = (c + 3 <= r) ? x3 : 0.0f;
            *reinterpret_cast<float4*>(Lout + (uint64_t)r * ldl + c) = l;
            *reinterpret_cast<float4*>(Linv_out + (uint64_t)r * ldl + c) = li;
        }
    }
}

__global__ __launch_bounds__(256) void spd_diag_kernel(const float* __restrict__ W, uint64_t ldw,
                                                       float* __restrict__ Lout, float* __restrict__ Linv_out,
                                                       uint64_t ldl, int32_t block_index,
                                                       int32_t* __restrict__ status) {
    __shared__ __attribute__((aligned(16))) float lds[kDiagLdsFloats];
    diag_block(W, ldw, Lout, Linv_out, ldl, block_index, status, nullptr, 0, lds);
}

// One step of the factorization in one launch, after the panel below diagonal block j is known:
// workgroup 0 takes the next diagonal block (j+1, j+1) - its own trailing update, then factor and
// inverse - while workgroups 1 .. T-1 apply the trailing update W -= panel panel^T to the other
// lower-triangle tiles (tile numbers in the triangle's row-by-row order; number 0 is that diagonal
// block).  Nothing in the launch depends on anything else in it, and the 31 us of the sequential
// diagonal work no longer sit between two launches but beside the trailing update.
//   Wt    trailing matrix, block (j+1, j+1) at its origin;  panel  L[j+1:, j] (rows x 128, pitch np)
__global__ __launch_bounds__(256, 1) void spd_step_kernel(float* __restrict__ Wt, const float* __restrict__ panel,
                                                          uint64_t np, uint64_t rows, float* __restrict__ Lout,
                                                          float* __restrict__ Linv_out, int32_t block_index,
                                                          int32_t* __restrict__ status) {
    constexpr int kLds = kDiagLdsFloats > short_k::lds_floats<NB>() ? kDiagLdsFloats : short_k::lds_floats<NB>();
    __shared__ __attribute__((aligned(16))) float lds[kLds];
    if (blockIdx.x == 0) {
        diag_block(Wt, np, Lout, Linv_out, np, block_index, status, panel, np, lds);
    } else {
        uint32_t tile_m, tile_n;
        short_k::triangle_tile(blockIdx.x, tile_m, tile_n);
        short_k::tile<NB>(panel, np, panel, np, Wt, np, rows, rows, NB, -1.0f, 1.0f, tile_m, tile_n, lds);
    }
}

__global__ __launch_bounds__(256) void abs_sum_kernel(const float* __restrict__ M, uint64_t ld, uint64_t n,
                                                      float* __restrict__ partial) {
    __shared__ float red[256];
    const uint64_t total = n * n;
    const uint64_t per = (total + kSumBlocks - 1) / kSumBlocks;
    const uint64_t lo = (uint64_t)blockIdx.x * per;
    const uint64_t hi = lo + per < total ? lo + per : total;
    float s = 0.0f;
    for (uint64_t e = lo + threadIdx.x; e < hi; e += 256) s += fabsf(M[(e / n) * ld + (e % n)]);
    red[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
}

__global__ __launch_bounds__(256) void mean_kernel(const float* __restrict__ partial, uint64_t n,
                                                   float* __restrict__ mean_out, float* __restrict__ mean_user) {
    __shared__ float red[256];
    float s = 0.0f;
    for (int e = threadIdx.x; e < kSumBlocks; e += 256) s += partial[e];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float mean = red[0] / ((float)n * (float)n);
        *mean_out = mean;
        if (mean_user) *mean_user = mean;
    }
}

__global__ __launch_bounds__(256) void scale_kernel(float* __restrict__ M, uint64_t ld, uint64_t n,
                                                    const float* __restrict__ mean) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n * n) return;
    const float inv = 1.0f / *mean;
    M[(idx / n) * ld + (idx % n)] *= inv;
}

struct Ctx {
    float* W;
    float* L;
    float* Li;
    uint64_t np;
    hipStream_t s;
};

// Inverse of the block lower-triangular factor by recursive halving:
//   [A 0; B C]^-1 = [A^-1 0; -C^-1 B A^-1  C^-1],
// two products per node of the tree (T = B A^-1 into W, which is free once the factorization is
// done, then -C^-1 T into Li).  Diagonal blocks are already inverted.  Nodes of one depth are
// independent, so they are collected per depth and every group of equal shape goes out as one
// batched launch: a dozen launches instead of two per node.
struct Node {
    uint64_t lo, mid, hi;  // block units
};

void collect_nodes(uint64_t lo, uint64_t hi, size_t depth, std::vector<std::vector<Node>>& levels) {
    if (hi - lo <= 1) return;
    const uint64_t mid = lo + (hi - lo) / 2;
    if (levels.size() <= depth) levels.resize(depth + 1);
    levels[depth].push_back({lo, mid, hi});
    collect_nodes(lo, mid, depth + 1, levels);
    collect_nodes(mid, hi, depth + 1, levels);
}

int tri_inverse_impl(Ctx& c, uint64_t nblk) {
    std::vector<std::vector<Node>> levels;
    collect_nodes(0, nblk, 0, levels);
    const uint64_t np = c.np;
    for (size_t d = levels.size(); d-- > 0;) {  // children before parents
        std::vector<Node>& nodes = levels[d];
        std::vector<char> done(nodes.size(), 0);
        for (size_t first = 0; first < nodes.size(); ++first) {
            if (done[first]) continue;
            const uint64_t r = (nodes[first].hi - nodes[first].mid) * NB, q = (nodes[first].mid - nodes[first].lo) * NB;
            trakhip::GemmBatch t_of_b, out_of_t;  // T = B * Ainv;  out = -Cinv * T
            t_of_b.count = out_of_t.count = 0;
            for (size_t i = first; i < nodes.size() && t_of_b.count < trakhip::kGemmBatchMax; ++i) {
                const Node& n = nodes[i];
                if (done[i] || (n.hi - n.mid) * NB != r || (n.mid - n.lo) * NB != q) continue;
                done[i] = 1;
                const uint32_t y = t_of_b.count++;
                out_of_t.count = t_of_b.count;
                const uint64_t below = n.mid * NB * np + n.lo * NB;  // block (mid, lo)
                t_of_b.a[y] = below;                                // B      in L
                t_of_b.b[y] = n.lo * NB * np + n.lo * NB;           // A^-1   in Li
                t_of_b.c[y] = below;                                // T      in W
                out_of_t.a[y] = n.mid * NB * np + n.mid * NB;       // C^-1   in Li
                out_of_t.b[y] = below;                              // T      in W
                out_of_t.c[y] = below;                              // result in Li
            }
            int e = trakhip::gemm_nn_batched(c.L, np, c.Li, np, c.W, np, r, q, q, 1.0f, 0.0f, t_of_b, c.s);
            if (!e) e = trakhip::gemm_nn_batched(c.Li, np, c.W, np, c.Li, np, r, q, r, -1.0f, 0.0f, out_of_t, c.s);
            if (e) return e;
        }
    }
    return TRAKHIP_OK;
}

// The node lists live in host containers; nothing they throw (std::bad_alloc) may cross the C ABI.
int tri_inverse(Ctx& c, uint64_t nblk) {
    try {
        return tri_inverse_impl(c, nblk);
    } catch (...) {
        return TRAKHIP_ERR_HOST_MEMORY;
    }
}

}  // namespace

namespace trakhip {

// Workspace: three np x np matrices (W, L, Li), the reduction scratch, and for small n a tail for the
// split planes of Li^T (for np >= 384 they fit into W and L, which are free by then).
static size_t planes_tail_bytes(uint64_t n, uint64_t np) {
    const size_t planes = split_bytes(n, n, TRAKHIP_F32), free_front = (size_t)(2 * np * np) * sizeof(float);
    return planes > free_front ? planes : 0;
}

size_t spd_inverse_workspace_bytes(uint64_t n) {
    if (n == 0) return 0;
    const uint64_t np = (n + NB - 1) / NB * NB;
    return (size_t)(3 * np * np + kSumBlocks + 4) * sizeof(float) + planes_tail_bytes(n, np);
}

int spd_inverse(const float* A, uint64_t lda, float lambda, float* inv, uint64_t ldi, uint64_t n, int normalize,
                float* mean_abs, int32_t* status, void* ws, size_t ws_bytes, hipStream_t s) {
    if (n == 0) return TRAKHIP_OK;
    if (!A || !inv || !ws) return TRAKHIP_ERR_NULL;
    if (lda < n || ldi < n || n > 0x40000) return TRAKHIP_ERR_SHAPE;
    if (ws_bytes < spd_inverse_workspace_bytes(n)) return TRAKHIP_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(ws) % 16) return TRAKHIP_ERR_ALIGN;
    const uint64_t np = (n + NB - 1) / NB * NB, nblk = np / NB;
    float* W = static_cast<float*>(ws);
    float* L = W + np * np;
    float* Li = L + np * np;
    float* partial = Li + np * np;
    float* mean_dev = partial + kSumBlocks;

    const uint64_t total = np * np;
    hipLaunchKernelGGL(spd_init_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, s, A, lda, lambda, n,
                       np, W, Li, status);
    if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;

    // Diagonal block 0 alone; then per block column j: the panel below it, and one launch that holds both
    // the trailing update and the next diagonal block (spd_step_kernel).  Trailing updates of more than
    // 512 tiles (n > 4096) go through the general product, with the diagonal block in a launch of its own.
    hipLaunchKernelGGL(spd_diag_kernel, dim3(1), dim3(256), 0, s, W, np, L, Li, np, 0, status);
    if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
    for (uint64_t j = 0; j + 1 < nblk; ++j) {
        const uint64_t off = j * NB * np + j * NB;
        const uint64_t rows = np - (j + 1) * NB, blocks = rows / NB;
        const uint64_t below = (j + 1) * NB * np + j * NB;
        const uint64_t tr = (j + 1) * NB * np + (j + 1) * NB;
        // panel = W[j+1:, j] * (L_jj^-1)^T
        int e = gemm_nt(W + below, np, Li + off, np, L + below, np, rows, NB, NB, 1.0f, 0.0f, nullptr, s);
        if (e) return e;
        const uint64_t tiles = blocks * (blocks + 1) / 2;
        if (tiles <= 512) {
            hipLaunchKernelGGL(spd_step_kernel, dim3((uint32_t)tiles), dim3(256), 0, s, W + tr, L + below, np, rows,
                               L + tr, Li + tr, (int32_t)(j + 1), status);
            if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
            continue;
        }
        // trailing matrix -= panel * panel^T (only the lower triangle of W is ever read)
        e = gemm_nt(L + below, np, L + below, np, W + tr, np, rows, rows, NB, -1.0f, 1.0f, nullptr, s,
                    kGemmLowerTilesOnly);
        if (e) return e;
        hipLaunchKernelGGL(spd_diag_kernel, dim3(1), dim3(256), 0, s, W + tr, np, L + tr, Li + tr, np,
                           (int32_t)(j + 1), status);
        if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
    }

    Ctx c = {W, L, Li, np, s};
    int e = tri_inverse(c, nblk);
    if (e) return e;

    // inverse = Li^T * Li (rows of Li at or beyond n do not reach the leading n x n block): the
    // symmetric product of the split operand Li^T, lower-triangle tiles mirrored, so the result is
    // exactly symmetric.  The planes go where W and L were (or behind the scratch for small n).
    void* planes = planes_tail_bytes(n, np) ? static_cast<void*>(mean_dev + 4) : static_cast<void*>(W);
    e = split_rows(Li, TRAKHIP_F32, np, n, n, 1, planes, split_bytes(n, n, TRAKHIP_F32), s);
    if (!e) e = gram_split(planes, n, n, TRAKHIP_F32, inv, ldi, 1.0f, 0.0f, nullptr, 0, s);
    if (e) return e;

    if (normalize || mean_abs) {
        hipLaunchKernelGGL(abs_sum_kernel, dim3(kSumBlocks), dim3(256), 0, s, inv, ldi, n, partial);
        hipLaunchKernelGGL(mean_kernel, dim3(1), dim3(256), 0, s, partial, n, mean_dev, mean_abs);
        if (normalize)
            hipLaunchKernelGGL(scale_kernel, dim3((uint32_t)((n * n + 255) / 256)), dim3(256), 0, s, inv, ldi, n,
                               mean_dev);
        if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
    }
    return TRAKHIP_OK;
}

}  // namespace trakhip

namespace {

// ---- inverse of a general matrix: elimination with partial pivoting -----------------------------------------
//
// For the matrices the Cholesky route above refuses: a Gram matrix rounded to fp16, or one of deficient
// rank with lambda = 0, is symmetric but need not be positive definite.  The reference inverts every
// matrix with LU and partial pivoting (torch.linalg.inv, trak/score_computers.py:163); this is the same
// pivoting on the device.  The augmented matrix [A + lambda I | I] (np x 2 np, np = n padded with an
// identity block to a multiple of 128) is reduced to [I | A^-1] block of columns by block of columns.
// For a block J of OB columns starting at j0 (the rows above j0 are finished pivot rows of earlier blocks):
//   1. the block's columns are factored as in a right-looking LU, SP columns at a time: gj_panel_kernel
//      (ONE workgroup holds rows j.. of the SP panel columns in registers) eliminates them column by column
//      with row pivoting (largest magnitude, lowest row on ties), leaves the multipliers (|l| <= 1) in the
//      rows below, the pivot rows' numbers, where the rows they displace go, and the packed factors of the
//      SP x SP pivot block; gj_rows_kernel moves the rows of the block's columns into place and turns the
//      pivot rows right of the panel into L11^-1 * (pivot rows); a product with SP values of k updates the
//      block's columns further right in the rows below.  Afterwards rows j0.. of J hold L \ U of the block.
//   2. the rest of the matrix (all columns right of the block, the identity half included) gets the block's
//      OB eliminations at once: gj_block_rows_kernel (one thread per column) applies the row moves, computes
//      Y = L_J^-1 * (pivot rows) (kept aside) and R = U_J^-1 * Y, which replaces the pivot rows;
//          rows below the block:  W[r, rest] -= L[r, J] * Y        (the LU update, multipliers at most 1)
//          rows above the block:  W[r, rest] -= W[r, J] * R        (the Gauss-Jordan part: back substitution
//                                                                   folded into the elimination)
//      two products with OB values of k.  No permutation is left to undo at the end: the row moves act on
//      whole rows of [A | I].
// OB = 64 from np = 3072 on (four or eight panels per block: the products over the rest move 12 np^2 bytes per
// block instead of per panel); below that OB = SP = 16 (fewer launches per column, which is what small
// matrices pay for).
//
// (Updating the rows below with the panel's original entries times D^-1 * (pivot rows), D the pivot block, would
// be one product for all rows; it is not done because its rounding errors grow with the condition of D, where
// the multipliers are at most 1.)

constexpr int kGjThreads = 1024;
constexpr int kGjMaxSp = 16;

struct GjStep {
    int32_t piv[kGjMaxSp];   // the row that becomes row j + c
    int32_t from[kGjMaxSp];  // rows of the pivot positions that were not chosen ...
    int32_t to[kGjMaxSp];    // ... and the vacated positions they move to
    int32_t moves;
    int32_t pad[3];
    float lu[kGjMaxSp * kGjMaxSp];  // the pivot block as packed factors: unit lower L below the diagonal, U on and above
};

__global__ __launch_bounds__(256) void gj_init_kernel(const float* __restrict__ A, uint64_t lda, float lambda,
                                                      uint64_t n, uint64_t np, float* __restrict__ W,
                                                      int32_t* __restrict__ status) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx == 0 && status) *status = 0;
    if (idx >= np * 2 * np) return;
    const uint64_t i = idx / (2 * np), j = idx % (2 * np);
    float v;
    if (j >= np)
        v = (j - np == i) ? 1.0f : 0.0f;
    else if (i < n && j < n)
        v = A[i * lda + j] + (i == j ? lambda : 0.0f);
    else
        v = (i == j) ? 1.0f : 0.0f;
    W[idx] = v;
}

// larger magnitude wins; on equal magnitudes the lower row (what a sequential search finds first)
__device__ __forceinline__ void gj_better(uint32_t& key, uint32_t& row, uint32_t okey, uint32_t orow) {
    if (okey > key || (okey == key && orow < row)) {
        key = okey;
        row = orow;
    }
}

template <class F, int... S>
__device__ __forceinline__ void gj_for_each(F& f, std::integer_sequence<int, S...>) {
    (f(std::integral_constant<int, S>{}), ...);
}

template <int SP, int RPT>
__global__ __launch_bounds__(kGjThreads) void gj_panel_kernel(float* __restrict__ W, uint64_t ld, uint32_t np,
                                                              uint32_t j, GjStep* __restrict__ step,
                                                              int32_t* __restrict__ status) {
    __shared__ uint32_t cand_key[kGjThreads / 64], cand_row[kGjThreads / 64];
    __shared__ float lu[SP][SP + 1];  // row c: the pivot row of column c as it was when chosen (packed L \ U)
    __shared__ int32_t piv[SP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float a[RPT][SP];
    uint32_t live = 0;  // bit i: row i of this thread exists and has not been a pivot
    // row slots of a thread that hold rows at all at this j (the panel shrinks as j grows)
    const int slots = (int)((np - j + kGjThreads - 1) / kGjThreads);
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const uint32_t r = j + (uint32_t)tid + (uint32_t)kGjThreads * i;
        if (r < np) {
            live |= 1u << i;
            const float4* src = reinterpret_cast<const float4*>(W + (uint64_t)r * ld + j);
#pragma unroll
            for (int c4 = 0; c4 < SP / 4; ++c4) {
                const float4 v = src[c4];
                a[i][4 * c4] = v.x, a[i][4 * c4 + 1] = v.y, a[i][4 * c4 + 2] = v.z, a[i][4 * c4 + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int c = 0; c < SP; ++c) a[i][c] = 0.0f;
        }
    }
    // (the columns are written out through a compile-time sequence: `#pragma unroll` gives up on a body
    // of this size, and the register array would be indexed at run time, i.e. live in scratch memory)
    auto column = [&](auto c_const) __attribute__((always_inline)) {
        constexpr int c = decltype(c_const)::value;
        // the pivot of column c: largest |a| among the rows that have not been pivots
        uint32_t key = 0, row = 0xFFFFFFFFu;
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            if (i < slots) {  // the same for the whole workgroup: a scalar branch
                if (live & (1u << i))
                    gj_better(key, row, __float_as_uint(fabsf(a[i][c])), j + (uint32_t)tid + (uint32_t)kGjThreads * i);
            }
        }
#pragma unroll
        for (int d = 1; d < 64; d <<= 1)
            gj_better(key, row, (uint32_t)__shfl_xor((int)key, d, 64), (uint32_t)__shfl_xor((int)row, d, 64));
        if (lane == 0) cand_key[wave] = key, cand_row[wave] = row;
        __syncthreads();
        // the sixteen waves' candidates, one per lane of every group of sixteen lanes, reduced inside the group
        static_assert(kGjThreads / 64 == 16, "one candidate per lane of a group of sixteen");
        key = cand_key[lane & 15], row = cand_row[lane & 15];
#pragma unroll
        for (int d = 1; d < 16; d <<= 1)
            gj_better(key, row, (uint32_t)__shfl_xor((int)key, d, 64), (uint32_t)__shfl_xor((int)row, d, 64));
        // its owner - one thread, known to all: row = j + thread + 1024 * slot - publishes the row (multipliers of
        // earlier columns in front, the eliminated row behind)
        const uint32_t rel = __builtin_amdgcn_readfirstlane(row) - j;
        const int owner = (int)(rel % kGjThreads), owner_slot = (int)(rel / kGjThreads);
        if (tid == owner) {
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                if (i == owner_slot) {
                    live &= ~(1u << i);
#pragma unroll
                    for (int c2 = 0; c2 < SP; ++c2) lu[c][c2] = a[i][c2];
                    if (a[i][c] == 0.0f && status) *status = (int32_t)(j + c + 1);  // exactly singular
                }
            }
            piv[c] = (int32_t)(rel + j);
        }
        __syncthreads();
        // multipliers by the reciprocal of the pivot, as LAPACK's unblocked LU scales a column
        const float rpivot = 1.0f / lu[c][c];
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            if (i < slots) {
                if (live & (1u << i)) {
                    const float l = a[i][c] * rpivot;
                    a[i][c] = l;
#pragma unroll
                    for (int c2 = c + 1; c2 < SP; ++c2) a[i][c2] = fmaf(-l, lu[c][c2], a[i][c2]);
                }
            }
        }
    };
    gj_for_each(column, std::make_integer_sequence<int, SP>{});
    // the rows that were never pivots now hold their SP multipliers: back to the matrix, where the row moves and
    // the update of the other columns find them
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        if (i < slots && (live & (1u << i))) {
            float4* dst = reinterpret_cast<float4*>(W + (uint64_t)(j + (uint32_t)tid + (uint32_t)kGjThreads * i) * ld + j);
#pragma unroll
            for (int c4 = 0; c4 < SP / 4; ++c4)
                dst[c4] = make_float4(a[i][4 * c4], a[i][4 * c4 + 1], a[i][4 * c4 + 2], a[i][4 * c4 + 3]);
        }
    }
    // D = (rows piv[0..SP) of the panel as they were) = L U with the packed factors in lu
    if (tid < SP) {
#pragma unroll
        for (int q = 0; q < SP; ++q) step->lu[tid * SP + q] = lu[tid][q];
        step->piv[tid] = piv[tid];
    }
    if (tid == 0) {
        // rows at the pivot positions j .. j+SP-1 that were not chosen go to the positions that the chosen
        // rows from further down leave behind, both in ascending order
        int32_t moves = 0, to_n = 0;
        for (int q = 0; q < SP; ++q) {
            const int32_t pos = (int32_t)j + q;
            bool chosen = false;
            for (int c = 0; c < SP; ++c) chosen |= piv[c] == pos;
            if (!chosen) step->from[moves++] = pos;
        }
        // vacated positions below the pivot block, ascending (selection over at most SP values)
        int32_t last = (int32_t)j + SP - 1;
        for (int m = 0; m < moves; ++m) {
            int32_t best = 0x7FFFFFFF;
            for (int c = 0; c < SP; ++c)
                if (piv[c] > last && piv[c] < best) best = piv[c];
            step->to[to_n++] = best;
            last = best;
        }
        step->moves = moves;
    }
}

// One thread per column of [col_begin, col_end): the rows move into place (pivot rows to j.., the rows they
// displace to the vacated positions).  Left of the panel that is all (multipliers of earlier panels travel with
// their rows); in the panel's columns the pivot rows become the packed factors; right of it they become
// Y = L^-1 * (pivot rows).  With y_out (the one-panel blocks of small matrices, where "right of the panel" is the
// whole rest) Y goes to y_out[c * ld + col] and the pivot rows become R = U^-1 * Y.
template <int SP>
__global__ __launch_bounds__(256) void gj_rows_kernel(float* __restrict__ W, uint64_t ld, uint32_t j, uint32_t col_begin,
                                                      uint32_t col_end, const GjStep* __restrict__ step,
                                                      float* __restrict__ y_out) {
    __shared__ GjStep st;
    for (uint32_t i = threadIdx.x; i < sizeof(GjStep) / 4; i += 256)
        reinterpret_cast<uint32_t*>(&st)[i] = reinterpret_cast<const uint32_t*>(step)[i];
    __syncthreads();
    const uint64_t col = (uint64_t)col_begin + (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (col >= col_end) return;
    float v[SP], d[SP];
#pragma unroll
    for (int c = 0; c < SP; ++c) v[c] = W[(uint64_t)st.piv[c] * ld + col];
#pragma unroll
    for (int m = 0; m < SP; ++m) d[m] = m < st.moves ? W[(uint64_t)st.from[m] * ld + col] : 0.0f;
    if (col >= j && col < (uint64_t)j + SP) {
#pragma unroll
        for (int c = 0; c < SP; ++c) v[c] = st.lu[c * SP + (int)(col - j)];
    } else if (col >= (uint64_t)j + SP) {
        // forward substitution with the unit lower factor
#pragma unroll
        for (int r = 1; r < SP; ++r)
#pragma unroll
            for (int q = 0; q < r; ++q) v[r] = fmaf(-st.lu[r * SP + q], v[q], v[r]);
        if (y_out) {
#pragma unroll
            for (int c = 0; c < SP; ++c) y_out[(uint64_t)c * ld + col] = v[c];
            // back substitution with the upper one
#pragma unroll
            for (int r = SP - 1; r >= 0; --r) {
#pragma unroll
                for (int q = r + 1; q < SP; ++q) v[r] = fmaf(-st.lu[r * SP + q], v[q], v[r]);
                v[r] = v[r] / st.lu[r * SP + r];
            }
        }
    }
#pragma unroll
    for (int c = 0; c < SP; ++c) W[(uint64_t)(j + c) * ld + col] = v[c];
#pragma unroll
    for (int m = 0; m < SP; ++m)
        if (m < st.moves) W[(uint64_t)st.to[m] * ld + col] = d[m];
}

__global__ __launch_bounds__(256) void gj_copy_out_kernel(const float* __restrict__ W, uint64_t ld, uint64_t np,
                                                          uint64_t n, float* __restrict__ inv, uint64_t ldi) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n * n) return;
    const uint64_t i = idx / n, c = idx % n;
    inv[i * ldi + c] = W[i * ld + np + c];
}

constexpr int kGjOb = 64;  // columns of a block of the large-matrix route

// One thread per column of the rest (col >= j0 + kGjOb).  The block's panels' row moves are applied one panel
// after the other (the pivot rows collect in LDS, one column of v per thread); then, with the factors L \ U that
// rows j0.. of the block's columns hold (F, read with wave-uniform addresses), Y = L^-1 v goes to
// y_out[c * ld + col] and R = U^-1 Y to rows j0.. of the column.  The 64 values are worked on eight at a time.
template <int SP>
__global__ __launch_bounds__(256) void gj_block_rows_kernel(float* __restrict__ W, uint64_t ld, uint32_t np, uint32_t j0,
                                                            const float* __restrict__ F,
                                                            const GjStep* __restrict__ steps, float* __restrict__ y_out) {
    constexpr int T = 8, NB8 = kGjOb / T, PANELS = kGjOb / SP;
    __shared__ float v[kGjOb][256];
    const int tid = threadIdx.x;
    const uint64_t col = (uint64_t)j0 + kGjOb + (uint64_t)blockIdx.x * 256 + tid;
    if (col >= 2ull * np) return;  // (no barrier below: a thread only reads the column of v that it wrote)
    for (int p = 0; p < PANELS; ++p) {
        const GjStep* st = steps + p;
        const int moves = st->moves;
        float x[SP], d[SP];
#pragma unroll
        for (int c = 0; c < SP; ++c) x[c] = W[(uint64_t)st->piv[c] * ld + col];
#pragma unroll
        for (int m = 0; m < SP; ++m) d[m] = m < moves ? W[(uint64_t)st->from[m] * ld + col] : 0.0f;
#pragma unroll
        for (int c = 0; c < SP; ++c) v[p * SP + c][tid] = x[c];
        // (a position j0 + p SP + c is never a source of a later panel: those take rows from further down)
#pragma unroll
        for (int m = 0; m < SP; ++m)
            if (m < moves) W[(uint64_t)st->to[m] * ld + col] = d[m];
    }
    // forward substitution with the unit lower factor, block row by block row
    for (int rb = 0; rb < NB8; ++rb) {
        float x[T];
#pragma unroll
        for (int i = 0; i < T; ++i) x[i] = v[rb * T + i][tid];
        for (int cb = 0; cb < rb; ++cb) {
            float y[T];
#pragma unroll
            for (int q = 0; q < T; ++q) y[q] = v[cb * T + q][tid];
            const float* l = F + (uint64_t)(rb * T) * ld + cb * T;
#pragma unroll
            for (int i = 0; i < T; ++i)
#pragma unroll
                for (int q = 0; q < T; ++q) x[i] = fmaf(-l[(uint64_t)i * ld + q], y[q], x[i]);
        }
        const float* l = F + (uint64_t)(rb * T) * ld + rb * T;
#pragma unroll
        for (int i = 1; i < T; ++i)
#pragma unroll
            for (int q = 0; q < i; ++q) x[i] = fmaf(-l[(uint64_t)i * ld + q], x[q], x[i]);
#pragma unroll
        for (int i = 0; i < T; ++i) {
            v[rb * T + i][tid] = x[i];
            y_out[(uint64_t)(rb * T + i) * ld + col] = x[i];
        }
    }
    // back substitution with the upper factor
    for (int rb = NB8 - 1; rb >= 0; --rb) {
        float x[T];
#pragma unroll
        for (int i = 0; i < T; ++i) x[i] = v[rb * T + i][tid];
        for (int cb = rb + 1; cb < NB8; ++cb) {
            float y[T];
#pragma unroll
            for (int q = 0; q < T; ++q) y[q] = v[cb * T + q][tid];
            const float* u = F + (uint64_t)(rb * T) * ld + cb * T;
#pragma unroll
            for (int i = 0; i < T; ++i)
#pragma unroll
                for (int q = 0; q < T; ++q) x[i] = fmaf(-u[(uint64_t)i * ld + q], y[q], x[i]);
        }
        const float* u = F + (uint64_t)(rb * T) * ld + rb * T;
#pragma unroll
        for (int i = T - 1; i >= 0; --i) {
#pragma unroll
            for (int q = i + 1; q < T; ++q) x[i] = fmaf(-u[(uint64_t)i * ld + q], x[q], x[i]);
            x[i] = x[i] / u[(uint64_t)i * ld + i];
        }
#pragma unroll
        for (int i = 0; i < T; ++i) {
            v[rb * T + i][tid] = x[i];
            W[(uint64_t)(j0 + rb * T + i) * ld + col] = x[i];
        }
    }
}

// the two products that carry a block's eliminations to the columns right of it (OB values of k):
// rows above the block with their own entries of the block's columns times R (which now is rows j0.. of W),
// rows below with their multipliers times Y
int gj_update_rest(float* W, uint64_t ld, uint32_t np, uint32_t j0, uint32_t ob, const float* Y, hipStream_t s) {
    const uint32_t end = j0 + ob;
    const uint64_t rest = 2ull * np - end;
    if (ob < kGjOb && j0 > 0 && end < np) {
        // one-panel blocks (small matrices): both products in one launch, a launch being what they cost.
        // Y lies behind W in the same workspace, so one base pointer serves both B operands.
        trakhip::GemmBatch two;
        two.count = 2;
        two.a[0] = j0, two.b[0] = (uint64_t)j0 * ld + end, two.c[0] = end, two.m[0] = j0;
        two.a[1] = (uint64_t)end * ld + j0, two.b[1] = (uint64_t)(Y - W) + end, two.c[1] = (uint64_t)end * ld + end;
        two.m[1] = np - end;
        const uint64_t m = j0 > np - end ? j0 : np - end;
        return trakhip::gemm_nn_batched(W, ld, W, ld, W, ld, m, rest, ob, -1.0f, 1.0f, two, s);
    }
    if (j0 > 0) {
        const int e = trakhip::gemm_nn(W + j0, ld, W + (uint64_t)j0 * ld + end, ld, W + end, ld, j0, rest, ob, -1.0f, 1.0f,
                                       s, 0);
        if (e) return e;
    }
    if (end < np)
        return trakhip::gemm_nn(W + (uint64_t)end * ld + j0, ld, Y + end, ld, W + (uint64_t)end * ld + end, ld, np - end,
                                rest, ob, -1.0f, 1.0f, s, 0);
    return TRAKHIP_OK;
}

// blocks of one panel: the whole rest of the matrix after every SP columns
template <int SP, int RPT>
int gj_run_flat(float* W, float* Y, uint32_t np, GjStep* steps, int32_t* status, hipStream_t s) {
    const uint64_t ld = 2ull * np;
    for (uint32_t j = 0; j < np; j += SP) {
        GjStep* st = steps + (j / SP) % 2;  // two records in turn: the next panel never overwrites one still in use
        hipLaunchKernelGGL((gj_panel_kernel<SP, RPT>), dim3(1), dim3(kGjThreads), 0, s, W, ld, np, j, st, status);
        const uint32_t cols = 2 * np - j;
        hipLaunchKernelGGL((gj_rows_kernel<SP>), dim3((cols + 255) / 256), dim3(256), 0, s, W, ld, j, j, 2 * np, st, Y);
        if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
        const int e = gj_update_rest(W, ld, np, j, SP, Y, s);
        if (e) return e;
    }
    return TRAKHIP_OK;
}

// blocks of kGjOb columns, kGjOb / SP panels each
template <int SP, int RPT>
int gj_run(float* W, float* Y, uint32_t np, GjStep* steps, int32_t* status, hipStream_t s) {
    const uint64_t ld = 2ull * np;
    for (uint32_t j0 = 0; j0 < np; j0 += kGjOb) {
        const uint32_t end = j0 + kGjOb;
        for (uint32_t j = j0; j < end; j += SP) {
            GjStep* st = steps + (j - j0) / SP;
            hipLaunchKernelGGL((gj_panel_kernel<SP, RPT>), dim3(1), dim3(kGjThreads), 0, s, W, ld, np, j, st, status);
            hipLaunchKernelGGL((gj_rows_kernel<SP>), dim3(1), dim3(256), 0, s, W, ld, j, j0, end, st, (float*)nullptr);
            if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
            if (j + SP < end && j + SP < np) {
                // the block's columns right of the panel, rows below it
                const int e = trakhip::gemm_nn(W + (uint64_t)(j + SP) * ld + j, ld, W + (uint64_t)j * ld + j + SP, ld,
                                               W + (uint64_t)(j + SP) * ld + j + SP, ld, np - j - SP, end - j - SP, SP,
                                               -1.0f, 1.0f, s, 0);
                if (e) return e;
            }
        }
        const uint32_t rest = 2 * np - end;
        hipLaunchKernelGGL((gj_block_rows_kernel<SP>), dim3((rest + 255) / 256), dim3(256), 0, s, W, ld, np, j0,
                           W + (uint64_t)j0 * ld + j0, steps, Y);
        if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
        const int e = gj_update_rest(W, ld, np, j0, kGjOb, Y, s);
        if (e) return e;
    }
    return TRAKHIP_OK;
}

}  // namespace

namespace trakhip {

constexpr uint64_t kGeneralInverseMaxN = 12288;

size_t general_inverse_workspace_bytes(uint64_t n) {
    if (n == 0 || n > kGeneralInverseMaxN) return 0;
    const uint64_t np = (n + NB - 1) / NB * NB;
    return (size_t)(2 * np * np + 2 * np * kGjOb + kSumBlocks + 4) * sizeof(float) + (kGjOb / 8) * sizeof(GjStep);
}

int general_inverse(const float* A, uint64_t lda, float lambda, float* inv, uint64_t ldi, uint64_t n, int normalize,
                    float* mean_abs, int32_t* status, void* ws, size_t ws_bytes, hipStream_t s) {
    if (n == 0) return TRAKHIP_OK;
    if (!A || !inv || !ws) return TRAKHIP_ERR_NULL;
    if (lda < n || ldi < n || n > kGeneralInverseMaxN) return TRAKHIP_ERR_SHAPE;
    if (ws_bytes < general_inverse_workspace_bytes(n)) return TRAKHIP_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(ws) % 16) return TRAKHIP_ERR_ALIGN;
    const uint64_t np = (n + NB - 1) / NB * NB;
    float* W = static_cast<float*>(ws);
    float* Y = W + 2 * np * np;  // kGjOb x 2 np: L^-1 * (pivot rows) of the block at work
    float* partial = Y + 2 * np * kGjOb;
    float* mean_dev = partial + kSumBlocks;
    GjStep* steps = reinterpret_cast<GjStep*>(mean_dev + 4);
    hipLaunchKernelGGL(gj_init_kernel, dim3((uint32_t)((2 * np * np + 255) / 256)), dim3(256), 0, s, A, lda, lambda, n,
                       np, W, status);
    if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
    // the panel's rows live in the registers of one workgroup: 16 columns of up to 6144 rows, or 8 of up to 12288
    // the panel's rows live in the registers of one workgroup: 16 columns of up to 6144 rows, or 8 of up to 12288
    const int e = np < 3072      ? gj_run_flat<16, 6>(W, Y, (uint32_t)np, steps, status, s)
                  : np <= 6144   ? gj_run<16, 6>(W, Y, (uint32_t)np, steps, status, s)
                                 : gj_run<8, 12>(W, Y, (uint32_t)np, steps, status, s);
    if (e) return e;
    hipLaunchKernelGGL(gj_copy_out_kernel, dim3((uint32_t)((n * n + 255) / 256)), dim3(256), 0, s, W, 2 * np, np, n, inv,
                       ldi);
    if (normalize || mean_abs) {
        hipLaunchKernelGGL(abs_sum_kernel, dim3(kSumBlocks), dim3(256), 0, s, inv, ldi, n, partial);
        hipLaunchKernelGGL(mean_kernel, dim3(1), dim3(256), 0, s, partial, n, mean_dev, mean_abs);
        if (normalize)
            hipLaunchKernelGGL(scale_kernel, dim3((uint32_t)((n * n + 255) / 256)), dim3(256), 0, s, inv, ldi, n,
                               mean_dev);
    }
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

}  // namespace trakhip
