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
//      matrix gets  W -= panel * panel^T   (both MFMA GEMMs from gemm.hip);
//   3. L^-1 by recursive halving: inv([[A,0],[B,C]]) = [[A^-1,0],[-C^-1 B A^-1, C^-1]]
//      (two GEMMs per node of the recursion tree);
//   4. inverse = L^-T L^-1 (one GEMM), then the mean of |.| by a two-stage reduction in a
//      fixed order and a scaling pass.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

#include "trakhip_internal.h"

namespace {

constexpr int NB = 128;
constexpr int kLd = NB + 1;
constexpr int kSumBlocks = 1024;

__global__ __launch_bounds__(256) void spd_init_kernel(const float* __restrict__ A, uint64_t lda, float lambda,
                                                       uint64_t n, uint64_t np, float* __restrict__ W,
                                                       float* __restrict__ L, float* __restrict__ Li,
                                                       int32_t* __restrict__ status) {
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
    L[idx] = 0.0f;
    Li[idx] = 0.0f;
}

// One workgroup of 1024 threads: Cholesky of the 128x128 diagonal block at W (lower triangle
// used), L block to Lout (upper part zero), its inverse to Linv_out.
//
// Both matrices live in registers, 4 x 4 elements per thread each, cyclically distributed so that
// every thread stays busy as the active part shrinks (four waves per SIMD hide the issue latency of
// this strictly sequential algorithm).  One loop of 128 steps, one barrier per step, does both
// jobs: step k broadcasts the unscaled column k of the trailing matrix A (l_k = raw / sqrt(d),
// d = A[k][k]) and the unscaled row k of B (B starts as I; x_k = B[k, :] / L[k][k] is row k of
// L^-1) through LDS, then every thread applies
//     A[r][c] -= raw[r] raw[c] / d                         (right-looking Cholesky)
//     B[r][c] -= raw[r] Braw[c] / d    for r > k           (forward substitution on all columns)
// from registers.  Thread t holds A rows t % 32 + 32 i, columns t / 32 + 32 j, and the transpose of
// that for B, so the threads that publish column k of A and row k of B are the same half of ONE
// wave.  A updates are not masked: entries of rows or columns <= k are never read again once step
// k is over.  Rows <= k of B are finished rows of L^-1 and are kept.
constexpr int kDiagGrid = 32;              // threads per side
constexpr int kDiagTile = NB / kDiagGrid;  // 4 elements per side per thread

__global__ __launch_bounds__(1024) void spd_diag_kernel(const float* __restrict__ W, uint64_t ldw,
                                                        float* __restrict__ Lout, float* __restrict__ Linv_out,
                                                        uint64_t ldl, int32_t block_index,
                                                        int32_t* __restrict__ status) {
    constexpr int G = kDiagGrid, T = kDiagTile;
    __shared__ float Ls[NB * kLd];   // the finished factor, column k valid after step k
    // column k of A and row k of B, unscaled; entry x = t + 32 i is kept at slot 4 t + i, so the four
    // values a thread needs are one 16-byte LDS access (two buffers, so the steps can overlap safely)
    __shared__ __attribute__((aligned(16))) float vec[2][NB];
    __shared__ __attribute__((aligned(16))) float bvec[2][NB];
    __shared__ float pivot[2];
    const int tid = threadIdx.x;
    const int p = tid % G, q = tid / G;  // p varies inside a half-wave, q selects the half-wave

    float a[T][T], b[T][T];  // A: rows p + G i, columns q + G j;  B: rows q + G i, columns p + G j
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int j = 0; j < T; ++j) {
            const int r = p + G * i, c = q + G * j;
            a[i][j] = (c <= r) ? W[(uint64_t)r * ldw + c] : 0.0f;
            b[i][j] = (q + G * i == p + G * j) ? 1.0f : 0.0f;
        }

    for (int k = 0; k < NB; ++k) {
        const int buf = k & 1;
        const int ks = k / G, kt = k % G;  // column k of A and row k of B: threads with q == kt, slot ks
        if (q == kt) {                     // one half-wave
            float col[T], row[T];
#pragma unroll
            for (int i = 0; i < T; ++i) {
                col[i] = 0.0f;
                row[i] = 0.0f;
#pragma unroll
                for (int j = 0; j < T; ++j)
                    if (j == ks) {
                        col[i] = a[i][j];
                        row[i] = b[j][i];
                    }
            }
            if (p == kt) {  // the diagonal element (k, k) is in slot [ks][ks] of this thread
                float d = 0.0f;
#pragma unroll
                for (int i = 0; i < T; ++i)
                    if (i == ks) d = col[i];
                if (!(d > 0.0f)) {
                    if (status && *status == 0) *status = 1 + block_index * NB + k;
                    d = 1.0f;
                }
                pivot[buf] = d;
            }
            *reinterpret_cast<float4*>(&vec[buf][T * p]) = make_float4(col[0], col[1], col[2], col[3]);
            *reinterpret_cast<float4*>(&bvec[buf][T * p]) = make_float4(row[0], row[1], row[2], row[3]);
        }
        __syncthreads();
        const float d = pivot[buf];
        // hardware reciprocal (1 ulp): it only scales the rank-1 updates; the factor itself below
        // is scaled with the correctly rounded 1 / sqrt(d)
        const float inv_d = __builtin_amdgcn_rcpf(d);
        const float4 vp = *reinterpret_cast<const float4*>(&vec[buf][T * p]);
        const float4 vq = *reinterpret_cast<const float4*>(&vec[buf][T * q]);
        const float4 bp = *reinterpret_cast<const float4*>(&bvec[buf][T * p]);
        const float lr[T] = {vp.x, vp.y, vp.z, vp.w};
        const float xc[T] = {bp.x, bp.y, bp.z, bp.w};
        const float rq[T] = {vq.x, vq.y, vq.z, vq.w};
        if (q == kt) {  // finished column k of L and row k of L^-1, off the critical path of the other waves
            const float inv_sd = 1.0f / sqrtf(d);
#pragma unroll
            for (int i = 0; i < T; ++i) {
                const int r = p + G * i;
                Ls[r * kLd + k] = (r >= k) ? lr[i] * inv_sd : 0.0f;  // L[k][k] = d / sqrt(d)
                const float x = xc[i] * inv_sd;
#pragma unroll
                for (int j = 0; j < T; ++j)
                    if (j == ks) b[j][i] = x;
            }
        }
        float lc[T], br[T];
#pragma unroll
        for (int j = 0; j < T; ++j) {
            const float v = rq[j] * inv_d;
            lc[j] = v;
            br[j] = (q + G * j > k) ? v : 0.0f;  // rows <= k of B are finished
        }
#pragma unroll
        for (int i = 0; i < T; ++i)
#pragma unroll
            for (int j = 0; j < T; ++j) {
                a[i][j] -= lr[i] * lc[j];
                b[i][j] -= br[i] * xc[j];
            }
    }
    __syncthreads();

#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int j = 0; j < T; ++j) {
            const int r = q + G * i, c = p + G * j;
            Lout[(uint64_t)r * ldl + c] = (c <= r) ? Ls[r * kLd + c] : 0.0f;
            Linv_out[(uint64_t)r * ldl + c] = (c <= r) ? b[i][j] : 0.0f;
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

int tri_inverse(Ctx& c, uint64_t nblk) {
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
                       np, W, L, Li, status);
    if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;

    for (uint64_t j = 0; j < nblk; ++j) {
        const uint64_t off = j * NB * np + j * NB;
        hipLaunchKernelGGL(spd_diag_kernel, dim3(1), dim3(1024), 0, s, W + off, np, L + off, Li + off, np,
                           (int32_t)j, status);
        if (hipGetLastError() != hipSuccess) return TRAKHIP_ERR_LAUNCH;
        if (j + 1 == nblk) break;
        const uint64_t rows = np - (j + 1) * NB;
        const uint64_t below = (j + 1) * NB * np + j * NB;
        // panel = W[j+1:, j] * (L_jj^-1)^T
        int e = gemm_nt(W + below, np, Li + off, np, L + below, np, rows, NB, NB, 1.0f, 0.0f, nullptr, s);
        if (e) return e;
        // trailing matrix -= panel * panel^T
        const uint64_t tr = (j + 1) * NB * np + (j + 1) * NB;
        e = gemm_nt(L + below, np, L + below, np, W + tr, np, rows, rows, NB, -1.0f, 1.0f, nullptr, s,
                    kGemmLowerTilesOnly);  // only the lower triangle of W is ever read
        if (e) return e;
    }

    Ctx c = {W, L, Li, np, s};
    int e = tri_inverse(c, nblk);
    if (e) return e;

    // inverse = Li^T * Li (rows of Li at or beyond n do not reach the leading n x n block): the
    // symmetric product of the split operand Li^T, lower-triangle tiles mirrored, so the result is
    // exactly symmetric.  The planes go where W and L were (or behind the scratch for small n).
    void* planes = planes_tail_bytes(n, np) ? static_cast<void*>(mean_dev + 4) : static_cast<void*>(W);
    e = split_rows(Li, TRAKHIP_F32, np, n, n, 1, planes, split_bytes(n, n, TRAKHIP_F32), s);
    if (!e) e = gram_split(planes, n, n, TRAKHIP_F32, inv, ldi, 1.0f, 0.0f, s);
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
