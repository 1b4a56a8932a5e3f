// fp32-accurate GEMM on the 16-bit matrix cores: C[M, N] = alpha * A * B^T + beta * C (row i *= row_scale[i]).
//
// The scoring GEMMs of BasicScoreComputer (trak/score_computers.py:153, :176, trak/utils.py:131)
// multiply fp32 matrices (or fp16 ones when TRAKer runs with use_half_precision, its default).
// v_mfma_f32_32x32x2_f32 runs at 157 TFLOP/s; v_mfma_f32_32x32x16_{bf16,f16} at 2.5 PFLOP/s,
// sixteen times the rate, with exact products and fp32 accumulation.
//
// fp32 operands: every fp32 value is the exact sum of three bf16 values (24 significand bits =
// 3 x 8), x = x1 + x2 + x3 with |x2| <= 2^-8 |x1|, |x3| <= 2^-16 |x1|, so
//     a * b = a1 b1 + (a1 b2 + a2 b1) + (a1 b3 + a2 b2 + a3 b1) + O(2^-24 |a b|)
// and six bf16 MFMAs give the product sum with the error of an fp32 dot product at 6/16 of the
// cost of the fp32 instruction.  The three terms left out are each below 2^-24 |a b|, the rounding
// a single fp32 multiplication makes.
// fp16 or bf16 operands (both of the same type): one plane, one MFMA, nothing left out.
// An opt-in cheaper variant for fp32 operands ("two fp16 planes"): every row is scaled by a power of two
// that brings its largest magnitude to [2^14, 2^15), then x = h1 + h2 with fp16 terms (22 significand
// bits for entries within 2^-18 of the row's largest, fewer below), and
//     a * b = a1 b1 + (a1 b2 + a2 b1) + O(2^-22 |a b|)
// with three fp16 MFMAs; the powers of two are taken out again in the epilogue.  Half the MFMAs of the
// three-plane product at four times its operand error bound.
//
// Operands are brought once, outside the GEMM, into "planes": plane p, k-octet o (8 consecutive k),
// row r is one 16-byte piece at ((p * K8 + o) * Rp + r) * 16 bytes, rows padded with zeros to a
// multiple of 256 and octets to a multiple of 8.  A 16-byte piece is exactly what one lane feeds to
// the MFMA (8 consecutive k of one row), consecutive rows are consecutive pieces, so global loads,
// LDS writes and LDS reads are all linear and conflict free, and the GEMM kernel moves 16-bit data
// only.
//
// Workgroup = 512 threads = 8 waves (4 x 2), 256 x 256 tile of C, a wave owns 64 x 128 of C (128
// accumulator VGPRs).  A step covers 16 S values of k (S = 1 for three planes, 4 for one plane):
// two LDS buffers of 48 or 64 KB filled by LDS-direct loads, one barrier per step, 48 or 32 MFMAs
// per wave and step.  Measured against this for three planes: 128 x 256 tiles with two workgroups
// per CU (9 % slower), 64 x 64 wave tiles at four waves per SIMD, three LDS buffers, register-staged
// loads, super-tile orders per XCD (all slower or equal).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "short_k_tile.h"
#include "trakhip_internal.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef uint32_t piece __attribute__((ext_vector_type(4)));  // 16 bytes = 8 x 16 bit = one lane's MFMA operand

constexpr int kWavesM = 4, kWavesN = 2;            // 4 x 2 waves, each owns 64 x 128 of C
constexpr int BM = 64 * kWavesM, BN = 128 * kWavesN;
constexpr int kWaves = kWavesM * kWavesN;
constexpr uint32_t kGemmTriangleGrid = 2u;          // kernel flag: the grid lists the lower-triangle tiles only
constexpr int kRowPad = 256;                       // rows of an operand are padded to this
constexpr int kOctetPad = 8;                       // octets (64 values of k) are padded to this

// ---- bringing operands into planes ---------------------------------------------------------

// binary32 -> nearest bf16 (ties to even) as a binary32 value; finite inputs
__device__ __forceinline__ float bf16_round(float x) {
    const uint32_t b = __float_as_uint(x);
    return __uint_as_float((b + 0x7FFFu + ((b >> 16) & 1u)) & 0xFFFF0000u);
}

// x = t[0] + t[1] + t[2] exactly (up to underflow of the last term), bf16 bit patterns
__device__ __forceinline__ void split3(float x, uint32_t (&t)[3]) {
    const float x1 = bf16_round(x);
    const float r1 = x - x1;
    const float x2 = bf16_round(r1);
    const float r2 = r1 - x2;
    t[0] = __float_as_uint(x1) >> 16;
    t[1] = __float_as_uint(x2) >> 16;
    t[2] = __float_as_uint(bf16_round(r2)) >> 16;
}

// One thread per (row r, octet o): reads 8 consecutive k of the row, writes its pieces.
// TRANS = false: src[r * ld + k];  TRANS = true: src[k * ld + r].  Rows >= rows and k >= K give
// zeros (the padding is rewritten on every call).  Threads of a workgroup cover 64 rows x 4 octets.
template <bool TRANS, bool ALIGNED>
__global__ __launch_bounds__(256) void split_kernel(const float* __restrict__ src, uint64_t ld, uint64_t rows,
                                                    uint64_t K, uint64_t Rp, uint64_t K8, uint32_t row_blocks,
                                                    uint4* __restrict__ planes) {
    const uint64_t r = (uint64_t)(blockIdx.x % row_blocks) * 64 + (threadIdx.x & 63);
    const uint64_t o = (uint64_t)(blockIdx.x / row_blocks) * 4 + (threadIdx.x >> 6);
    if (r >= Rp || o >= K8) return;
    float v[8];
    if (!TRANS && ALIGNED && r < rows && 8 * o + 8 <= K) {
        // the four waves of a workgroup read the four octets of a 128-byte line of each row
        const float4* q = reinterpret_cast<const float4*>(src + r * ld + 8 * o);
        const float4 lo = q[0], hi = q[1];
        v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w;
        v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint64_t k = 8 * o + i;
            v[i] = (r < rows && k < K) ? (TRANS ? src[k * ld + r] : src[r * ld + k]) : 0.0f;
        }
    }
    uint32_t w[3][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t lo[3], hi[3];
        split3(v[2 * i], lo);
        split3(v[2 * i + 1], hi);
#pragma unroll
        for (int p = 0; p < 3; ++p) w[p][i] = lo[p] | (hi[p] << 16);
    }
#pragma unroll
    for (int p = 0; p < 3; ++p) planes[((uint64_t)p * K8 + o) * Rp + r] = make_uint4(w[p][0], w[p][1], w[p][2], w[p][3]);
}

// The same for a 16-bit source (fp16 or bf16 bit patterns): one plane, the values themselves.
template <bool TRANS, bool ALIGNED>
__global__ __launch_bounds__(256) void relayout16_kernel(const uint16_t* __restrict__ src, uint64_t ld, uint64_t rows,
                                                         uint64_t K, uint64_t Rp, uint64_t K8, uint32_t row_blocks,
                                                         uint4* __restrict__ planes) {
    const uint64_t r = (uint64_t)(blockIdx.x % row_blocks) * 64 + (threadIdx.x & 63);
    const uint64_t o = (uint64_t)(blockIdx.x / row_blocks) * 4 + (threadIdx.x >> 6);
    if (r >= Rp || o >= K8) return;
    uint4 w;
    if (!TRANS && ALIGNED && r < rows && 8 * o + 8 <= K) {
        w = *reinterpret_cast<const uint4*>(src + r * ld + 8 * o);
    } else {
        uint32_t v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint64_t k = 8 * o + i;
            v[i] = (r < rows && k < K) ? (uint32_t)(TRANS ? src[k * ld + r] : src[r * ld + k]) : 0u;
        }
        w = make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
    }
    planes[o * Rp + r] = w;
}

// ---- two fp16 planes with a power-of-two scale per row ------------------------------------------

// Largest magnitude of every operand row as binary32 bits (non-negative floats order like unsigned
// integers).  Row-major operand: one wave per row.
__global__ __launch_bounds__(256) void absmax_rows_kernel(const float* __restrict__ src, uint64_t ld, uint64_t rows,
                                                          uint64_t K, uint32_t* __restrict__ maxbits) {
    const uint64_t r = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const int lane = threadIdx.x & 63;
    uint32_t m = 0;
    for (uint64_t k = lane; k < K; k += 64) {
        const uint32_t b = __float_as_uint(src[r * ld + k]) & 0x7FFFFFFFu;
        m = b > m ? b : m;
    }
#pragma unroll
    for (int w = 32; w > 0; w >>= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)m, w);
        m = o > m ? o : m;
    }
    if (lane == 0) maxbits[r] = m;
}

// Transposed operand (row r of the operand is column r of src[K, rows]): a thread walks one column over
// one chunk of k and merges with an atomic maximum (order independent); maxbits starts at zero.
constexpr int kColChunks = 64;
__global__ __launch_bounds__(256) void absmax_cols_kernel(const float* __restrict__ src, uint64_t ld, uint64_t rows,
                                                          uint64_t K, uint32_t* __restrict__ maxbits) {
    const uint64_t r = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    const uint64_t per = (K + kColChunks - 1) / kColChunks;
    const uint64_t k0 = (uint64_t)blockIdx.y * per, k1 = k0 + per < K ? k0 + per : K;
    uint32_t m = 0;
    for (uint64_t k = k0; k < k1; ++k) {
        const uint32_t b = __float_as_uint(src[k * ld + r]) & 0x7FFFFFFFu;
        m = b > m ? b : m;
    }
    if (m) atomicMax(maxbits + r, m);
}

__global__ __launch_bounds__(256) void zero_u32_kernel(uint32_t* __restrict__ p, uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// Power of two that brings a row whose largest magnitude has these bits into [2^14, 2^15) (fp16 tops
// out at 65504), and its inverse.  A row of zeros, or one that holds an infinity or a NaN, is left alone.
__device__ __forceinline__ void row_factors(uint32_t maxbits, float& scale, float& unscale) {
    int sh = 0;
    if (maxbits != 0u && maxbits < 0x7F800000u) {
        sh = 14 - ((int)(maxbits >> 23) - 127);
        sh = sh > 126 ? 126 : sh;
    }
    scale = __uint_as_float((uint32_t)(127 + sh) << 23);
    unscale = __uint_as_float((uint32_t)(127 - sh) << 23);
}

// One thread per (row r, octet o), as split_kernel: x * scale = h1 + h2 with fp16 terms, planes 0 and 1.
template <bool TRANS, bool ALIGNED>
__global__ __launch_bounds__(256) void split2_kernel(const float* __restrict__ src, uint64_t ld, uint64_t rows,
                                                     uint64_t K, uint64_t Rp, uint64_t K8, uint32_t row_blocks,
                                                     const uint32_t* __restrict__ maxbits, uint4* __restrict__ planes,
                                                     float* __restrict__ unscale_out) {
    const uint64_t r = (uint64_t)(blockIdx.x % row_blocks) * 64 + (threadIdx.x & 63);
    const uint64_t o = (uint64_t)(blockIdx.x / row_blocks) * 4 + (threadIdx.x >> 6);
    if (r >= Rp || o >= K8) return;
    float scale = 1.0f, unscale = 1.0f;
    if (r < rows) row_factors(maxbits[r], scale, unscale);
    if (o == 0 && r < rows) unscale_out[r] = unscale;
    float v[8];
    if (!TRANS && ALIGNED && r < rows && 8 * o + 8 <= K) {
        const float4* q = reinterpret_cast<const float4*>(src + r * ld + 8 * o);
        const float4 lo = q[0], hi = q[1];
        v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w;
        v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint64_t k = 8 * o + i;
            v[i] = (r < rows && k < K) ? (TRANS ? src[k * ld + r] : src[r * ld + k]) : 0.0f;
        }
    }
    uint32_t w[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t t[2][2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float x = v[2 * i + e] * scale;  // exact: a power of two, no overflow by construction
            const _Float16 h1 = (_Float16)x;       // round to nearest even
            const _Float16 h2 = (_Float16)(x - (float)h1);
            t[0][e] = (uint32_t)__builtin_bit_cast(uint16_t, h1);
            t[1][e] = (uint32_t)__builtin_bit_cast(uint16_t, h2);
        }
        w[0][i] = t[0][0] | (t[0][1] << 16);
        w[1][i] = t[1][0] | (t[1][1] << 16);
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) planes[((uint64_t)p * K8 + o) * Rp + r] = make_uint4(w[p][0], w[p][1], w[p][2], w[p][3]);
}

// ---- GEMM ----------------------------------------------------------------------------------

template <bool F16>
__device__ __forceinline__ floatx16 mfma16(const piece& a, const piece& b, floatx16 c) {
    if constexpr (F16)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c,
                                                      0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                       c, 0, 0, 0);
}

typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));

// 4 x 4 transpose inside every quad of lanes: lane q of a quad holds M[a][q] in v[a] and ends up with
// M[q][c] in v[c].  Two exchanges, over lane distance 2 and 1: (register r, lane q) trades places with
// (register r ^ d, lane q ^ d) where bit d of r and q differ.
__device__ __forceinline__ void quad_transpose(float (&v)[4], int lane) {
    const bool b1 = lane & 2, b0 = lane & 1;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const float send = b1 ? v[r] : v[r + 2];
        const float recv = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, send), 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
        if (b1) v[r] = recv; else v[r + 2] = recv;
    }
#pragma unroll
    for (int r = 0; r < 4; r += 2) {
        const float send = b0 ? v[r] : v[r + 1];
        const float recv = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, send), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
        if (b0) v[r] = recv; else v[r + 1] = recv;
    }
}

// Epilogue of a wave's 64 x (32 JT) part of C.  D[m][n] of a 32x32 MFMA: lane holds column
// n = lane % 32; register r holds row 8*(r/4) + 4*(lane/32) + r%4.  When C is accumulated into (ACCUM),
// its old values are fetched for 32 rows at a time before any of them is overwritten (loads and stores
// through one pointer would otherwise alternate, one memory round trip per element).
// SCALED: the accumulators are products of operands whose rows were multiplied by powers of two;
// a_unscale[row] and b_unscale[col] are the inverse factors (applied one after the other, so that no
// intermediate leaves the binary32 range when the result does not).
//
// A wave whose part of C lies wholly inside the matrix (all but the last row and column of tiles) takes
// the path without bounds tests and with 16-byte stores: a store instruction costs the texture path about
// 32 cycles whatever it carries, and with one 4-byte store per accumulator register (1024 per tile and
// CU) the epilogue of a tile took 33 000 cycles, a seventh of a product with 4096 values of k.  Four
// registers of a lane are four rows of one column; a 4 x 4 transpose inside every quad of lanes (DPP
// quad_perm, 16 vector instructions) turns them into four columns of one row, i.e. one 16-byte store,
// and a store instruction then writes eight whole 128-byte lines.
template <bool ACCUM, int JT, bool SCALED = false>
__device__ __forceinline__ void store_c(const floatx16 (&acc)[2][JT], float* __restrict__ C, uint64_t ldc, uint64_t M,
                                        uint64_t N, uint64_t row_base, uint64_t col0, int h, float alpha, float beta,
                                        const float* __restrict__ row_scale,
                                        const float* __restrict__ a_unscale = nullptr,
                                        const float* __restrict__ b_unscale = nullptr) {
    // wave-uniform: col0 = first column of the wave's part + lane % 32
    const bool inside = row_base + 64 <= M && col0 - (threadIdx.x & 31) + 32 * JT <= N;
    if (!SCALED && inside) {
        const int lane = threadIdx.x & 63, q = lane & 3;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // registers 4g .. 4g+3 are rows 8g + 4h + (0..3) of the lane's column; after the transpose inside
                // the quad the lane holds row 8g + 4h + q, columns 4 (x / 4) .. + 3 of every 32-column group
                const uint64_t row = row_base + 32 * i + 8 * g + 4 * h + q;
                const float rs = row_scale ? row_scale[row] : 1.0f;
                float* p = C + row * ldc + (col0 - q);
                float4u prev[ACCUM ? JT : 1];
                if constexpr (ACCUM) {
#pragma unroll
                    for (int j = 0; j < JT; ++j) prev[j] = *reinterpret_cast<const float4u*>(p + 32 * j);
                }
#pragma unroll
                for (int j = 0; j < JT; ++j) {
                    float v[4] = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    quad_transpose(v, lane);
                    float4u o;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        if constexpr (ACCUM)
                            o[c] = (alpha * v[c] + beta * prev[j][c]) * rs;
                        else
                            o[c] = alpha * v[c] * rs;
                    }
                    // streaming store: C is written once and is far larger than L2, where the operand panels
                    // that other workgroups are about to read should stay
                    __builtin_nontemporal_store(o, reinterpret_cast<float4u*>(p + 32 * j));
                }
            }
        }
        return;
    }
    float ub[JT];
#pragma unroll
    for (int j = 0; j < JT; ++j) ub[j] = (SCALED && col0 + 32 * j < N) ? b_unscale[col0 + 32 * j] : 1.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint64_t row0 = row_base + 32 * i + 4 * h;
        float ua[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint64_t row = row0 + 8 * (r >> 2) + (r & 3);
            ua[r] = (SCALED && row < M) ? a_unscale[row] : 1.0f;
        }
        // old values of C: fetched for a group of columns before any of them is overwritten (all four
        // 32-column groups at once, two at a time when the unscale factors take registers as well)
        constexpr int JG = (ACCUM && SCALED) ? (JT + 1) / 2 : JT;
#pragma unroll
        for (int j0 = 0; j0 < JT; j0 += JG) {
            floatx16 prev[ACCUM ? JG : 1];
            if constexpr (ACCUM) {
#pragma unroll
                for (int j = 0; j < JG; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint64_t row = row0 + 8 * (r >> 2) + (r & 3), col = col0 + 32 * (j0 + j);
                        prev[j][r] = (j0 + j < JT && row < M && col < N) ? C[row * ldc + col] : 0.0f;
                    }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint64_t row = row0 + 8 * (r >> 2) + (r & 3);
                if (row >= M) continue;
                const float rs = row_scale ? row_scale[row] : 1.0f;
#pragma unroll
                for (int j = 0; j < JG; ++j) {
                    const uint64_t col = col0 + 32 * (j0 + j);
                    if (j0 + j >= JT || col >= N) continue;
                    float v = acc[i][j0 + j][r];
                    if constexpr (SCALED) v = (v * ua[r]) * ub[j0 + j];
                    if constexpr (ACCUM)
                        C[row * ldc + col] = (alpha * v + beta * prev[j][r]) * rs;
                    else
                        C[row * ldc + col] = alpha * v * rs;
                }
            }
        }
    }
}

// A step of a tile is S sub-steps (two octets = one MFMA depth each); sub-step u holds
// [A: plane][half][256 rows] followed by [B: plane][half][256 rows].  The pieces are moved in chunks
// of 64 consecutive ones by the load unit straight into LDS (global_load_lds_dwordx4): the 64
// lanes of a wave fetch 64 consecutive rows of one (plane, octet), which land at 64 consecutive
// 16-byte slots starting at a wave-uniform LDS address; no staging registers, no LDS store
// instructions.  Wave w moves chunks w, w + 8, ...
//
// A chunk's 64 pieces are consecutive in memory as well (64 rows of one plane and octet), so its address
// is a wave-uniform base plus 16 bytes per lane, and the base moves by a fixed number of bytes from step
// to step: the bases live in scalar registers and a load costs two scalar additions.  (Computing the
// piece address per lane from plane, octet and row took about thirty instructions per load, in front of
// the MFMAs of every step.)
template <int P, int S>
struct StepMover {
    static constexpr int kAChunks = P * 2 * BM / 64, kBChunks = P * 2 * BN / 64;
    static constexpr int kSubChunks = kAChunks + kBChunks, kChunks = S * kSubChunks;
    // the first kLoaders waves move the chunks: wave w chunks w, w + kLoaders, ...  (all eight: leaving the loads
    // to four waves, so that the other four start their MFMAs at once, measured 1 % faster on the three-plane
    // product and is not worth a second code path)
    static constexpr int kLoaders = kWaves;
    static_assert(kChunks % kLoaders == 0, "every loading wave moves the same number of chunks");
    static_assert(BM % 64 == 0 && BN % 64 == 0, "a chunk lies in one (plane, half)");
    static constexpr int kPerWave = kChunks / kLoaders;
    const char* base[kPerWave];  // of this wave's chunks at the next step to load (wave-uniform)
    uint64_t step_a, step_b;     // bytes from one step to the next

    __device__ __forceinline__ void init(const piece* A, uint64_t Rpa, const piece* B, uint64_t Rpb, uint64_t K8,
                                         uint64_t m0, uint64_t n0, uint64_t s, int wave) {
        step_a = 2 * S * Rpa * sizeof(piece);
        step_b = 2 * S * Rpb * sizeof(piece);
#pragma unroll
        for (int i = 0; i < kPerWave; ++i) {
            const int c = wave % kLoaders + kLoaders * i;  // wave-uniform
            const int u = c / kSubChunks, cc = c % kSubChunks;
            if (cc < kAChunks) {
                const int e = 64 * cc, row = e % BM, ph = e / BM;  // ph = plane * 2 + half
                base[i] = reinterpret_cast<const char*>(A + ((uint64_t)(ph >> 1) * K8 + 2 * (s * S + u) + (ph & 1)) * Rpa + m0 + row);
            } else {
                const int e = 64 * (cc - kAChunks), row = e % BN, ph = e / BN;
                base[i] = reinterpret_cast<const char*>(B + ((uint64_t)(ph >> 1) * K8 + 2 * (s * S + u) + (ph & 1)) * Rpb + n0 + row);
            }
        }
    }
    // chunk i of the wave for the step the bases point at; then the base moves on to the step after
    __device__ __forceinline__ void move(int i, int wave, uint32_t lane_bytes, piece* lds) {
        const int c = wave % kLoaders + kLoaders * i;
        __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(base[i] + lane_bytes),
                                         (void __attribute__((address_space(3)))*)(lds + 64 * c), 16, 0, 0);
        // kAChunks is a multiple of kLoaders: which operand chunk i belongs to does not depend on the wave
        base[i] += ((kLoaders * i) % kSubChunks) < kAChunks ? step_a : step_b;
    }
    static_assert(kAChunks % kLoaders == 0 && kSubChunks % kLoaders == 0, "operand of a chunk: the same for all waves");
    __device__ __forceinline__ void move_all(int wave, uint32_t lane_bytes, piece* lds) {
        if (wave >= kLoaders) return;
#pragma unroll
        for (int i = 0; i < kPerWave; ++i) move(i, wave, lane_bytes, lds);
    }
};

// P planes per operand (3: split fp32, 1: a 16-bit type), F16 selects the fp16 MFMA, S sub-steps
// per barrier.
template <int P, bool F16, int S, bool ACCUM>
__global__ __launch_bounds__(64 * kWaves, 2) void gemm_split_kernel(
    const piece* __restrict__ A, uint64_t Rpa, const piece* __restrict__ B, uint64_t Rpb, uint64_t K8,
    float* __restrict__ C, uint64_t ldc, uint64_t M, uint64_t N, float alpha, float beta,
    const float* __restrict__ row_scale, uint32_t tiles_n, uint32_t flags, const float* __restrict__ a_unscale,
    const float* __restrict__ b_unscale, uint32_t parts, uint64_t part_stride) {
    constexpr int JT = BN / kWavesN / 32;            // 32-column MFMA tiles per wave
    constexpr int kAPieces = P * 2 * BM;             // [plane][half][row]
    constexpr int kSubPieces = P * 2 * (BM + BN);    // three planes: 3072 pieces = 48 KB
    constexpr int kBufPieces = S * kSubPieces;
    __shared__ piece lds[2][kBufPieces];

    // parts > 1: the grid is `parts` copies of the tile list; copy p multiplies the p-th share of the k
    // steps and writes its sums to the p-th matrix at C (a later pass adds the shares in order)
    uint32_t tile_id = blockIdx.x, part = 0;
    if (parts > 1) {
        const uint32_t per_part = gridDim.x / parts;
        part = blockIdx.x / per_part;
        tile_id = blockIdx.x % per_part;
        C += (uint64_t)part * part_stride;
    }
    uint32_t tile_m, tile_n;
    if (flags & kGemmTriangleGrid) {  // the tile list is the lower triangle, row by row
        short_k::triangle_tile(tile_id, tile_m, tile_n);
    } else {
        tile_m = tile_id / tiles_n;
        tile_n = tile_id % tiles_n;
    }
    const uint64_t m0 = (uint64_t)tile_m * BM, n0 = (uint64_t)tile_n * BN;
    // a symmetric product needs only the tiles that touch the lower triangle
    if ((flags & trakhip::kGemmLowerTilesOnly) && n0 > m0 + BM - 1) return;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;  // the wave number as a scalar
    const int wm = wave / kWavesN, wn = wave % kWavesN;
    const int x = lane & 31, h = lane >> 5;

    floatx16 acc[2][JT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < JT; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const uint64_t all_steps = K8 / (2 * S);
    const uint64_t first = all_steps * part / parts, steps = all_steps * (part + 1) / parts;  // [first, steps)
    StepMover<P, S> mover;
    mover.init(A, Rpa, B, Rpb, K8, m0, n0, first, wave);
    const uint32_t lane_bytes = (uint32_t)lane * (uint32_t)sizeof(piece);
    mover.move_all(wave, lane_bytes, lds[0]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // piece index of this lane's operand for plane p: A rows wm*64 + 32*i + x, B rows wn*128 + 32*j + x
    const int a_lane = h * BM + wm * 64 + x;
    const int b_lane = kAPieces + h * BN + wn * (32 * JT) + x;

    for (uint64_t s = first; s < steps; ++s) {
        const int cur = (int)((s - first) & 1);
        // the other buffer was last read before the barrier that ended the previous step
        if (s + 1 < steps) mover.move_all(wave, lane_bytes, lds[cur ^ 1]);
#pragma unroll
        for (int u = 0; u < S; ++u) {
            const piece* l = lds[cur] + u * kSubPieces;
            piece fa[2][P];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int p = 0; p < P; ++p) fa[i][p] = l[a_lane + p * 2 * BM + 32 * i];
#pragma unroll
            for (int j = 0; j < JT; ++j) {
                piece fb[P];
#pragma unroll
                for (int p = 0; p < P; ++p) fb[p] = l[b_lane + p * 2 * BN + 32 * j];
                if constexpr (P == 3) {
                    // the six plane pairs (pa, pb) with pa + pb <= 2, smallest terms first
                    constexpr int kPa[6] = {0, 1, 2, 0, 1, 0};
                    constexpr int kPb[6] = {2, 1, 0, 1, 0, 0};
#pragma unroll
                    for (int t6 = 0; t6 < 6; ++t6)
#pragma unroll
                        for (int i = 0; i < 2; ++i)
                            acc[i][j] = mfma16<F16>(fa[i][kPa[t6]], fb[kPb[t6]], acc[i][j]);
                } else if constexpr (P == 2) {
                    // the three plane pairs with pa + pb <= 1, smaller terms first
                    constexpr int kPa[3] = {0, 1, 0};
                    constexpr int kPb[3] = {1, 0, 0};
#pragma unroll
                    for (int t3 = 0; t3 < 3; ++t3)
#pragma unroll
                        for (int i = 0; i < 2; ++i)
                            acc[i][j] = mfma16<F16>(fa[i][kPa[t3]], fb[kPb[t3]], acc[i][j]);
                } else {
#pragma unroll
                    for (int i = 0; i < 2; ++i) acc[i][j] = mfma16<F16>(fa[i][0], fb[0], acc[i][j]);
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's pieces of the next step are in LDS
        __syncthreads();
    }

    store_c<ACCUM, JT, P == 2>(acc, C, ldc, M, N, m0 + wm * 64, n0 + wn * (32 * JT) + x, h, alpha, beta, row_scale,
                               a_unscale, b_unscale);
}

// ---- 16-bit operands read in place -----------------------------------------------------------
//
// Row-major fp16 / bf16 operands A[M, K], B[N, K] with K a multiple of 64 and 16-byte aligned rows need
// no planes.  A step is 64 values of k = one 128-byte line of every row: chunk c of a step is the
// lines of rows 8c .. 8c+7 of [256 rows of A | 256 rows of B], lane l of the moving wave fetches
// the 16-byte piece of row r = 8c + l/8 that belongs in slot l % 8, i.e. LDS holds each row's eight
// octets permuted: octet o sits in slot o ^ ((r / 2) % 8).  A wave's load instruction reads eight full
// lines; LDS serves a ds_read_b128 sixteen lanes at a time from 64 banks (256 bytes), and the sixteen
// lanes of a group (sixteen consecutive rows, one octet) land on sixteen different 16-byte columns
// of those 256 bytes - rows of equal parity share a 128-byte half and differ in r / 2.  Linear global
// reads, conflict-free LDS reads (XOR with r % 8 instead leaves a two-way conflict), and the same MFMA loop as
// the one-plane kernel.  Rows past M or N are fetched from the last row (their results are not stored).
template <bool F16, bool ACCUM>
__global__ __launch_bounds__(64 * kWaves, 2) void gemm_nt16_kernel(
    const piece* __restrict__ A, uint64_t lda8, const piece* __restrict__ B, uint64_t ldb8, uint64_t steps,
    float* __restrict__ C, uint64_t ldc, uint64_t M, uint64_t N, float alpha, float beta,
    const float* __restrict__ row_scale, uint32_t tiles_n, uint32_t tiles) {
    constexpr int JT = BN / kWavesN / 32;
    constexpr int kBufPieces = 8 * (BM + BN);  // 64 KB
    constexpr int kMoves = (BM + BN) / 8 / kWaves, kMovesA = BM / 8 / kWaves;  // chunks per wave and step
    __shared__ piece lds[2][kBufPieces];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;  // the wave number as a scalar
    const int wm = wave / kWavesN, wn = wave % kWavesN;
    const int x = lane & 31, h = lane >> 5;
    const int a_row = (wm * 64 + x) * 8, b_row = (BM + wn * (32 * JT) + x) * 8;  // first piece of the lane's rows

    // The workgroups are persistent: workgroup w computes tiles w, w + gridDim.x, ...  A load's address is a
    // scalar base (first row of the tile, advanced by one 128-byte line per step) plus this lane's byte offset
    // inside the tile's rows.
    const char* a_tile;
    const char* b_tile;
    uint32_t voff[kMoves];
    auto set_tile = [&](uint32_t t) {
        const uint64_t m0 = (uint64_t)(t / tiles_n) * BM, n0 = (uint64_t)(t % tiles_n) * BN;
        a_tile = reinterpret_cast<const char*>(A + m0 * lda8);
        b_tile = reinterpret_cast<const char*>(B + n0 * ldb8);
        // rows 8c + sub of chunk c = wave + 8 i': (row >> 1) % 8 = 4 (wave % 2) + sub / 2
        const int sub = lane >> 3, oct = (lane & 7) ^ ((4 * (wave & 1) + (sub >> 1)) & 7);
#pragma unroll
        for (int i = 0; i < kMoves; ++i) {
            const uint32_t row = 8 * (wave + kWaves * (i % kMovesA)) + sub;
            if (i < kMovesA) {
                const uint64_t last = M - 1 - m0;
                voff[i] = (uint32_t)(((row < last ? row : last) * lda8 + oct) * 16);
            } else {
                const uint64_t last = N - 1 - n0;
                voff[i] = (uint32_t)(((row < last ? row : last) * ldb8 + oct) * 16);
            }
        }
    };
    auto dma = [&](uint64_t s, piece* buf) {
#pragma unroll
        for (int i = 0; i < kMoves; ++i) {
            const int c = (i < kMovesA ? 0 : BM / 8) + wave + kWaves * (i % kMovesA);  // scalar
            const char* base = (i < kMovesA ? a_tile : b_tile) + s * 128;
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(base + voff[i]),
                                             (void __attribute__((address_space(3)))*)(buf + 64 * c), 16, 0, 0);
        }
    };

    // A step is four sub-steps of eight MFMAs (two A fragments x four B fragments).  The six fragments of
    // sub-step u + 1 are requested before the MFMAs of sub-step u are issued, so an LDS read has eight MFMAs
    // (256 cycles) to arrive instead of stalling the wave; the per-step barrier sits in front of the last
    // sub-step, whose MFMAs then cover the first reads from the other buffer.  Two register sets, alternating.
    piece fa[2][2], fb[2][JT];
    auto fetch = [&](int buf, int u, int set) {
        const piece* l = lds[buf] + ((2 * u + h) ^ ((x >> 1) & 7));
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[set][i] = l[a_row + 256 * i];
#pragma unroll
        for (int j = 0; j < JT; ++j) fb[set][j] = l[b_row + 256 * j];
    };

    uint32_t tile = blockIdx.x;
    if (tile >= tiles) return;
    set_tile(tile);
    int first = 0;  // buffer that holds step 0 of the current tile
    dma(0, lds[0]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (;;) {
        floatx16 acc[2][JT];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < JT; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        const uint64_t m0 = (uint64_t)(tile / tiles_n) * BM, n0 = (uint64_t)(tile % tiles_n) * BN;
        const uint32_t next = tile + gridDim.x;

        fetch(first, 0, 0);
        for (uint64_t s = 0; s < steps; ++s) {
            const int cur = (int)((s + first) & 1);
            const bool last_step = s + 1 == steps;
            if (!last_step) {
                dma(s + 1, lds[cur ^ 1]);
            } else if (next < tiles) {
                // step 0 of the next tile arrives under the last MFMAs and the stores of this one
                set_tile(next);
                dma(0, lds[cur ^ 1]);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int set = u & 1;
                // Wait for this sub-step's fragments HERE, while they are the only LDS reads in flight: the
                // compiler waits for all outstanding LDS reads at once (it cannot order them against the
                // LDS-direct loads), so the next reads are issued after this point and stay in flight under
                // the MFMAs.
                asm volatile("" ::"v"(fa[set][0]), "v"(fa[set][1]), "v"(fb[set][0]), "v"(fb[set][1]), "v"(fb[set][2]),
                             "v"(fb[set][3]));
                __builtin_amdgcn_sched_barrier(0);
                if (u < 3) {
                    fetch(cur, u + 1, set ^ 1);
                } else {
                    // every read of this buffer has completed; wait for this wave's part of the next buffer,
                    // meet the other waves, then start on the next buffer
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                    if (!last_step) fetch(cur ^ 1, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < JT; ++j)
#pragma unroll
                    for (int i = 0; i < 2; ++i) acc[i][j] = mfma16<F16>(fa[set][i], fb[set][j], acc[i][j]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        store_c<ACCUM, JT>(acc, C, ldc, M, N, m0 + wm * 64, n0 + wn * (32 * JT) + x, h, alpha, beta, row_scale);
        if (next >= tiles) break;
        first = (int)((steps + first) & 1);
        tile = next;
    }
}

// C[i][j] = C[j][i] for j > i: completes a symmetric matrix whose lower triangle was computed.
__global__ __launch_bounds__(256) void mirror_lower_kernel(float* __restrict__ C, uint64_t ldc, uint64_t n) {
    __shared__ float t[32][33];
    // 32 x 32 blocks strictly above or on the diagonal, read from their mirror image
    const uint32_t bi = blockIdx.y, bj = blockIdx.x;
    if (bj < bi) return;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const uint64_t src_row = (uint64_t)bj * 32 + r, src_col = (uint64_t)bi * 32 + tx;  // block (bj, bi), lower
        t[r][tx] = (src_row < n && src_col < n) ? C[src_row * ldc + src_col] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const uint64_t row = (uint64_t)bi * 32 + r, col = (uint64_t)bj * 32 + tx;
        if (row < n && col < n && col > row) C[row * ldc + col] = t[tx][r];
    }
}

// C = alpha * (P_0 + P_1 + ... in this order) + beta * C on the lower triangle, mirrored into the upper
// one: closes a symmetric product whose k range was shared out over `parts` matrices at P.
__global__ __launch_bounds__(256) void gram_combine_kernel(const float* __restrict__ P, uint64_t part_stride,
                                                           uint32_t parts, float* __restrict__ C, uint64_t ldc,
                                                           uint64_t n, float alpha, float beta) {
    __shared__ float t[32][33];
    const uint32_t bi = blockIdx.y, bj = blockIdx.x;  // 32 x 32 block (bi, bj) on or under the diagonal
    if (bj > bi) return;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const uint64_t row = (uint64_t)bi * 32 + r, col = (uint64_t)bj * 32 + tx;
        float v = 0.0f;
        if (row < n && col <= row) {
            for (uint32_t p = 0; p < parts; ++p) v += P[(uint64_t)p * part_stride + row * n + col];
            v *= alpha;
            if (beta != 0.0f) v += beta * C[row * ldc + col];
            C[row * ldc + col] = v;
        }
        t[r][tx] = v;
    }
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8) {
        const uint64_t row = (uint64_t)bj * 32 + r, col = (uint64_t)bi * 32 + tx;  // the mirror image
        if (row < n && col < n && col > row) C[row * ldc + col] = t[tx][r];
    }
}

uint64_t padded_rows(uint64_t rows) { return (rows + kRowPad - 1) / kRowPad * kRowPad; }
uint64_t octets(uint64_t K) { return (K + 8 * kOctetPad - 1) / (8 * kOctetPad) * kOctetPad; }
int planes_of(int dtype) { return dtype == TRAKHIP_F32 ? 3 : 1; }
bool known_dtype(int dtype) { return dtype == TRAKHIP_F16 || dtype == TRAKHIP_BF16 || dtype == TRAKHIP_F32; }

}  // namespace

namespace trakhip {

size_t split_bytes(uint64_t rows, uint64_t K, int dtype) {
    if (rows == 0 || K == 0 || !known_dtype(dtype)) return 0;
    return (size_t)(planes_of(dtype) * octets(K) * padded_rows(rows) * 16);
}

int split_rows(const void* src, int dtype, uint64_t ld, uint64_t rows, uint64_t K, int transposed, void* planes,
               size_t planes_bytes, hipStream_t s) {
    if (!known_dtype(dtype)) return TRAKHIP_ERR_DTYPE;
    if (rows == 0 || K == 0) return TRAKHIP_ERR_SHAPE;
    if (ld < (transposed ? rows : K)) return TRAKHIP_ERR_SHAPE;
    if (!src || !planes) return TRAKHIP_ERR_NULL;
    if (planes_bytes < split_bytes(rows, K, dtype)) return TRAKHIP_ERR_WORKSPACE;
    const size_t esz = dtype == TRAKHIP_F32 ? 4 : 2;
    if ((reinterpret_cast<uintptr_t>(src) % esz) || (reinterpret_cast<uintptr_t>(planes) % 16)) return TRAKHIP_ERR_ALIGN;
    const uint64_t Rp = padded_rows(rows), K8 = octets(K);
    const uint64_t gx = Rp / 64, gy = (K8 + 3) / 4;
    if (gx * gy > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    const dim3 grid((uint32_t)(gx * gy)), block(256);
    uint4* out = static_cast<uint4*>(planes);
    // 16-byte loads of 8 (fp32: 4) consecutive values need the row starts aligned
    const bool aligned = reinterpret_cast<uintptr_t>(src) % 16 == 0 && (ld * esz) % 16 == 0;
    if (dtype == TRAKHIP_F32) {
        const float* f = static_cast<const float*>(src);
        if (transposed)
            hipLaunchKernelGGL((split_kernel<true, false>), grid, block, 0, s, f, ld, rows, K, Rp, K8, (uint32_t)gx, out);
        else if (aligned)
            hipLaunchKernelGGL((split_kernel<false, true>), grid, block, 0, s, f, ld, rows, K, Rp, K8, (uint32_t)gx, out);
        else
            hipLaunchKernelGGL((split_kernel<false, false>), grid, block, 0, s, f, ld, rows, K, Rp, K8, (uint32_t)gx, out);
    } else {
        const uint16_t* h = static_cast<const uint16_t*>(src);
        if (transposed)
            hipLaunchKernelGGL((relayout16_kernel<true, false>), grid, block, 0, s, h, ld, rows, K, Rp, K8, (uint32_t)gx, out);
        else if (aligned)
            hipLaunchKernelGGL((relayout16_kernel<false, true>), grid, block, 0, s, h, ld, rows, K, Rp, K8, (uint32_t)gx, out);
        else
            hipLaunchKernelGGL((relayout16_kernel<false, false>), grid, block, 0, s, h, ld, rows, K, Rp, K8, (uint32_t)gx, out);
    }
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

}  // namespace trakhip

namespace {

// completes a symmetric matrix whose lower-triangle tiles were computed
int mirror_lower(float* C, uint64_t ldc, uint64_t N, hipStream_t s) {
    const uint64_t blocks = (N + 31) / 32;
    if (blocks > 65535) return TRAKHIP_ERR_SHAPE;
    hipLaunchKernelGGL(mirror_lower_kernel, dim3((uint32_t)blocks, (uint32_t)blocks), dim3(256), 0, s, C, ldc, N);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

// sub-steps per barrier of each operand format
int sub_steps(int dtype, bool two_planes) { return two_planes ? 2 : (dtype == TRAKHIP_F32 ? 1 : 4); }

// parts > 1 (symmetric products only): the k steps are shared out over `parts` launches' worth of
// workgroups that write plain sums into `parts` N x N matrices at C; see gram_combine_kernel.
int launch_split(const void* A_planes, uint64_t M, const void* B_planes, uint64_t N, uint64_t K, int dtype, float* C,
                 uint64_t ldc, float alpha, float beta, const float* row_scale, hipStream_t s, uint32_t flags,
                 const float* a_unscale, const float* b_unscale, uint32_t parts = 1) {
    if (M == 0 || N == 0) return TRAKHIP_OK;
    if (K == 0 || ldc < N) return TRAKHIP_ERR_SHAPE;
    if (!A_planes || !B_planes || !C) return TRAKHIP_ERR_NULL;
    if ((reinterpret_cast<uintptr_t>(A_planes) % 16) || (reinterpret_cast<uintptr_t>(B_planes) % 16) ||
        (reinterpret_cast<uintptr_t>(C) % 4))
        return TRAKHIP_ERR_ALIGN;
    const uint64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    uint64_t workgroups = tiles_m * tiles_n;
    if (parts > 1) {
        flags = kGemmTriangleGrid;
        workgroups = tiles_m * (tiles_m + 1) / 2 * parts;
    }
    const dim3 grid((uint32_t)workgroups), block(64 * kWaves);
    const piece* a = static_cast<const piece*>(A_planes);
    const piece* b = static_cast<const piece*>(B_planes);
    const uint64_t Rpa = padded_rows(M), Rpb = padded_rows(N), K8 = octets(K);
    // ACCUM (beta != 0) fetches the old C in the epilogue; kept out of the plain kernel
    void (*kernel)(const piece*, uint64_t, const piece*, uint64_t, uint64_t, float*, uint64_t, uint64_t, uint64_t, float,
                   float, const float*, uint32_t, uint32_t, const float*, const float*, uint32_t, uint64_t);
    const bool accum = beta != 0.0f;
    if (a_unscale)
        kernel = accum ? gemm_split_kernel<2, true, 2, true> : gemm_split_kernel<2, true, 2, false>;
    else if (dtype == TRAKHIP_F32)
        kernel = accum ? gemm_split_kernel<3, false, 1, true> : gemm_split_kernel<3, false, 1, false>;
    else if (dtype == TRAKHIP_F16)
        kernel = accum ? gemm_split_kernel<1, true, 4, true> : gemm_split_kernel<1, true, 4, false>;
    else
        kernel = accum ? gemm_split_kernel<1, false, 4, true> : gemm_split_kernel<1, false, 4, false>;
    hipLaunchKernelGGL(kernel, grid, block, 0, s, a, Rpa, b, Rpb, K8, C, ldc, M, N, alpha, beta, row_scale,
                       (uint32_t)tiles_n, flags, a_unscale, b_unscale, parts, (uint64_t)N * N);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

// A symmetric product has (tiles + 1) tiles / 2 workgroups' worth of work; up to 170 of them leave a third of
// the CUs idle, and the k range is long enough to share out: three shares, a round and a half of
// workgroups of a third of the work each.
constexpr uint32_t kGramParts = 3;
uint32_t gram_parts(uint64_t N, uint64_t K, int dtype, bool two_planes) {
    const uint64_t tiles = (N + BM - 1) / BM, lower = tiles * (tiles + 1) / 2;
    const uint64_t steps = octets(K) / (2 * sub_steps(dtype, two_planes));
    return (lower <= 170 && steps >= 8 * kGramParts) ? kGramParts : 1;
}

int gram_impl(const void* A_planes, const float* a_scales, uint64_t N, uint64_t K, int dtype, float* C, uint64_t ldc,
              float alpha, float beta, void* ws, size_t ws_bytes, hipStream_t s) {
    if (N == 0) return TRAKHIP_OK;
    const bool two_planes = a_scales != nullptr;
    const uint32_t parts = gram_parts(N, K, dtype, two_planes);
    const size_t need = (size_t)parts * N * N * sizeof(float);
    if (parts > 1 && ws && ws_bytes >= need && reinterpret_cast<uintptr_t>(ws) % 16 == 0) {
        if (!C) return TRAKHIP_ERR_NULL;
        if (ldc < N) return TRAKHIP_ERR_SHAPE;
        float* shares = static_cast<float*>(ws);
        const int e = launch_split(A_planes, N, A_planes, N, K, dtype, shares, N, 1.0f, 0.0f, nullptr, s, 0u, a_scales,
                                   a_scales, parts);
        if (e) return e;
        const uint64_t blocks = (N + 31) / 32;
        if (blocks > 65535) return TRAKHIP_ERR_SHAPE;
        hipLaunchKernelGGL(gram_combine_kernel, dim3((uint32_t)blocks, (uint32_t)blocks), dim3(256), 0, s, shares,
                           (uint64_t)N * N, parts, C, ldc, N, alpha, beta);
        return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
    }
    const int e = launch_split(A_planes, N, A_planes, N, K, dtype, C, ldc, alpha, beta, nullptr, s, trakhip::kGemmLowerTilesOnly,
                               a_scales, a_scales);
    if (e) return e;
    return mirror_lower(C, ldc, N, s);
}

}  // namespace

namespace trakhip {

int gemm_nt_split(const void* A_planes, uint64_t M, const void* B_planes, uint64_t N, uint64_t K, int dtype, float* C,
                  uint64_t ldc, float alpha, float beta, const float* row_scale, hipStream_t s, uint32_t flags) {
    if (!known_dtype(dtype)) return TRAKHIP_ERR_DTYPE;
    return launch_split(A_planes, M, B_planes, N, K, dtype, C, ldc, alpha, beta, row_scale, s, flags, nullptr, nullptr);
}

size_t split2_bytes(uint64_t rows, uint64_t K) {
    if (rows == 0 || K == 0) return 0;
    return (size_t)(2 * octets(K) * padded_rows(rows) * 16);
}

int split2_rows(const float* src, uint64_t ld, uint64_t rows, uint64_t K, int transposed, void* planes,
                size_t planes_bytes, float* scales, hipStream_t s) {
    if (rows == 0 || K == 0) return TRAKHIP_ERR_SHAPE;
    if (ld < (transposed ? rows : K)) return TRAKHIP_ERR_SHAPE;
    if (!src || !planes || !scales) return TRAKHIP_ERR_NULL;
    if (planes_bytes < split2_bytes(rows, K)) return TRAKHIP_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(src) % 4) || (reinterpret_cast<uintptr_t>(planes) % 16) ||
        (reinterpret_cast<uintptr_t>(scales) % 4))
        return TRAKHIP_ERR_ALIGN;
    const uint64_t Rp = padded_rows(rows), K8 = octets(K);
    const uint64_t gx = Rp / 64, gy = (K8 + 3) / 4;
    if (gx * gy > 0x7FFFFFFFull || rows > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    // scales[0 .. rows) receives the inverse factors; scales[rows .. 2 rows) holds the row maxima meanwhile
    uint32_t* maxbits = reinterpret_cast<uint32_t*>(scales + rows);
    if (transposed) {
        hipLaunchKernelGGL(zero_u32_kernel, dim3((uint32_t)((rows + 255) / 256)), dim3(256), 0, s, maxbits, rows);
        hipLaunchKernelGGL(absmax_cols_kernel, dim3((uint32_t)((rows + 255) / 256), kColChunks), dim3(256), 0, s, src, ld,
                           rows, K, maxbits);
    } else {
        hipLaunchKernelGGL(absmax_rows_kernel, dim3((uint32_t)((rows + 3) / 4)), dim3(256), 0, s, src, ld, rows, K,
                           maxbits);
    }
    const dim3 grid((uint32_t)(gx * gy)), block(256);
    uint4* out = static_cast<uint4*>(planes);
    const bool aligned = reinterpret_cast<uintptr_t>(src) % 16 == 0 && (ld * 4) % 16 == 0;
    if (transposed)
        hipLaunchKernelGGL((split2_kernel<true, false>), grid, block, 0, s, src, ld, rows, K, Rp, K8, (uint32_t)gx, maxbits,
                           out, scales);
    else if (aligned)
        hipLaunchKernelGGL((split2_kernel<false, true>), grid, block, 0, s, src, ld, rows, K, Rp, K8, (uint32_t)gx, maxbits,
                           out, scales);
    else
        hipLaunchKernelGGL((split2_kernel<false, false>), grid, block, 0, s, src, ld, rows, K, Rp, K8, (uint32_t)gx,
                           maxbits, out, scales);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

int gemm_nt_split2(const void* A_planes, const float* a_scales, uint64_t M, const void* B_planes, const float* b_scales,
                   uint64_t N, uint64_t K, float* C, uint64_t ldc, float alpha, float beta, const float* row_scale,
                   hipStream_t s, uint32_t flags) {
    if ((M && !a_scales) || (N && !b_scales)) return TRAKHIP_ERR_NULL;
    return launch_split(A_planes, M, B_planes, N, K, TRAKHIP_F32, C, ldc, alpha, beta, row_scale, s, flags, a_scales,
                        b_scales);
}

size_t gram_split_workspace_bytes(uint64_t N, uint64_t K, int dtype, int two_planes) {
    if (N == 0 || K == 0 || !known_dtype(dtype)) return 0;
    const uint32_t parts = gram_parts(N, K, dtype, two_planes != 0);
    return parts > 1 ? (size_t)parts * N * N * sizeof(float) : 0;
}

int gram_split2(const void* A_planes, const float* a_scales, uint64_t N, uint64_t K, float* C, uint64_t ldc, float alpha,
                float beta, void* ws, size_t ws_bytes, hipStream_t s) {
    if (N && !a_scales) return TRAKHIP_ERR_NULL;
    return gram_impl(A_planes, a_scales, N, K, TRAKHIP_F32, C, ldc, alpha, beta, ws, ws_bytes, s);
}

int gemm_nt16(const void* A, uint64_t lda, const void* B, uint64_t ldb, int dtype, float* C, uint64_t ldc, uint64_t M,
              uint64_t N, uint64_t K, float alpha, float beta, const float* row_scale, hipStream_t s) {
    if (dtype != TRAKHIP_F16 && dtype != TRAKHIP_BF16) return TRAKHIP_ERR_DTYPE;
    if (M == 0 || N == 0) return TRAKHIP_OK;
    if (K == 0 || K % 64 || lda < K || ldb < K || ldc < N) return TRAKHIP_ERR_SHAPE;
    // a lane's byte offset inside the 256 rows of a tile is kept in 32 bits
    if (lda >= (1ull << 23) || ldb >= (1ull << 23)) return TRAKHIP_ERR_SHAPE;
    if (!A || !B || !C) return TRAKHIP_ERR_NULL;
    if ((reinterpret_cast<uintptr_t>(A) % 16) || (reinterpret_cast<uintptr_t>(B) % 16) || (lda % 8) || (ldb % 8) ||
        (reinterpret_cast<uintptr_t>(C) % 4))
        return TRAKHIP_ERR_ALIGN;
    const uint64_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    if (tiles_m * tiles_n > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    void (*kernel)(const piece*, uint64_t, const piece*, uint64_t, uint64_t, float*, uint64_t, uint64_t, uint64_t, float,
                   float, const float*, uint32_t, uint32_t);
    const bool accum = beta != 0.0f;
    if (dtype == TRAKHIP_F16)
        kernel = accum ? gemm_nt16_kernel<true, true> : gemm_nt16_kernel<true, false>;
    else
        kernel = accum ? gemm_nt16_kernel<false, true> : gemm_nt16_kernel<false, false>;
    const uint32_t tiles = (uint32_t)(tiles_m * tiles_n);
    // persistent workgroups, one per CU (128 KB of LDS each)
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    hipLaunchKernelGGL(kernel, dim3(tiles < (uint32_t)cus ? tiles : (uint32_t)cus), dim3(64 * kWaves), 0, s,
                       static_cast<const piece*>(A), lda / 8, static_cast<const piece*>(B), ldb / 8, K / 64, C, ldc, M, N,
                       alpha, beta, row_scale, (uint32_t)tiles_n, tiles);
    return hipGetLastError() == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

int gram_split(const void* A_planes, uint64_t N, uint64_t K, int dtype, float* C, uint64_t ldc, float alpha, float beta,
               void* ws, size_t ws_bytes, hipStream_t s) {
    if (!known_dtype(dtype)) return TRAKHIP_ERR_DTYPE;
    return gram_impl(A_planes, nullptr, N, K, dtype, C, ldc, alpha, beta, ws, ws_bytes, s);
}

}  // namespace trakhip
