/* C ABI of libtrakhip.so: JL gradient projection and attribution-scoring kernels for
 * AMD MI355X (gfx950).
 *
 * Conventions
 *   - every pointer named *_dev is device memory on the current HIP device; the caller owns
 *     all buffers, the library never allocates device memory and never synchronizes;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*; NULL = default stream);
 *   - return value 0 = success, negative = error (trakhip_strerror gives the text); nothing
 *     is thrown across this boundary;
 *   - matrices are row-major, leading dimensions are counted in elements.
 *
 * Each entry point names the reference code (MadryLab/trak) it stands in for.
 */
#ifndef TRAKHIP_H
#define TRAKHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* input element types of the projection */
#define TRAKHIP_F16 0
#define TRAKHIP_BF16 1
#define TRAKHIP_F32 2

/* projection types: enum ProjectionType of fast_jl/types.cuh:4-7 */
#define TRAKHIP_RADEMACHER 0
#define TRAKHIP_NORMAL 1

#define TRAKHIP_OK 0
#define TRAKHIP_ERR_PROJ_DIM -1  /* proj dim not a multiple of 512 (fast_jl/fast_jl_kernel.cuh:113-115) */
#define TRAKHIP_ERR_SHAPE -2     /* empty / oversized / inconsistent shape */
#define TRAKHIP_ERR_DTYPE -3     /* unknown element type (fast_jl/fast_jl.cu:26) */
#define TRAKHIP_ERR_PROJ_TYPE -4
#define TRAKHIP_ERR_NULL -5      /* null pointer */
#define TRAKHIP_ERR_WORKSPACE -6 /* workspace too small */
#define TRAKHIP_ERR_ALIGN -7     /* pointer not aligned as documented */
#define TRAKHIP_ERR_LAUNCH -8    /* HIP refused the launch (hipGetLastError != hipSuccess) */
#define TRAKHIP_ERR_NOT_SPD -9   /* matrix handed to the SPD inverse is not positive definite */
#define TRAKHIP_ERR_NO_DEVICE -10
#define TRAKHIP_ERR_POINTER -11  /* destination is neither device memory nor page-locked host memory */
#define TRAKHIP_ERR_STATIC_LIMIT -12 /* trakhip_project_static: shape needs more than its static scratch */
#define TRAKHIP_ERR_HOST_MEMORY -13  /* host-side bookkeeping of a call could not be allocated */

const char* trakhip_strerror(int code);

/* Version of this ABI (bumped on incompatible change). */
int trakhip_abi_version(void);

/* ---- JL projection -------------------------------------------------------------------- */

/* Bytes of scratch a caller should bring to trakhip_project for these sizes: room for passes of
 * trakhip_project_rows_per_pass() = 64 rows.  The size depends on the shape and on the number of compute
 * units of the current HIP device (the launch is cut into at most that many workgroups; 256 is assumed
 * when the process has no device), so ask with the device current that will run the projection.  Stands in for the torch::zeros({B_pad, T, N})
 * intermediate of fast_jl/fast_jl.cu:48-49.  trakhip_project_workspace_min: the least that
 * trakhip_project accepts (passes of 32 rows: half as much once B >= 64; the call then runs 32 rows
 * at a time, with the same results). */
size_t trakhip_project_workspace(uint64_t B, uint64_t P, uint32_t proj_dim, uint32_t num_feature_tiles);
size_t trakhip_project_workspace_min(uint64_t B, uint64_t P, uint32_t proj_dim, uint32_t num_feature_tiles);

/* Rows that one pass of the projection kernels takes: 64 for fp16 / bf16 gradients (two 32-row MFMA
 * blocks share every generated matrix entry, Rademacher or normal), 32 for fp32 gradients.  The
 * reference has passes of 8, 16 or 32 rows (fast_jl/fast_jl.cu:44-76). */
uint32_t trakhip_project_rows_per_pass(int in_dtype, int proj_type);

/* out[B, proj_dim] (fp32) = in[B, P] x S, S generated on the fly from (seed, proj_dim,
 * num_feature_tiles, P).  Stands in for the six functions project_{rademacher,normal}_{8,16,32}
 * of fast_jl/fast_jl.cu:81-110 (host loop over batches of rows at fast_jl/fast_jl.cu:44-76, kernel
 * fast_jl/fast_jl_kernel.cuh:24-105, cross-tile sum fast_jl/fast_jl.cu:78).
 *   in_dev      row-major [B, P] with row pitch ld_in >= P elements, aligned to its element size
 *   in_dtype    TRAKHIP_F16 | TRAKHIP_BF16 | TRAKHIP_F32
 *   out_dev     [B, proj_dim] fp32, contiguous, 16-byte aligned; fully overwritten
 *   workspace   >= trakhip_project_workspace_min(...) bytes, 16-byte aligned (trakhip_project_workspace(...)
 *               bytes for the fastest path)
 *   proj_dim    multiple of 512;  P < 2^32;  any B >= 1
 */
int trakhip_project(const void* in_dev, int in_dtype, uint64_t B, uint64_t P, uint64_t ld_in,
                    float* out_dev, void* workspace_dev, size_t workspace_bytes, uint32_t proj_dim,
                    uint32_t seed, uint32_t num_feature_tiles, int proj_type, void* stream);

/* trakhip_project for callers that cannot allocate or hand over a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference:
 * fast_jl allocates its intermediate with torch::zeros on every call (fast_jl/fast_jl.cu:48-49).
 * Same arguments, checks and results (bit for bit) as trakhip_project, minus the workspace: the
 * partial sums live in a static device array of trakhip_project_static_limit() bytes (36 MiB) that
 * each GPU the library runs on holds until the process ends (rows go 64 at a time when the partial
 * sums of a 64-row pass fit into the array, else 32 at a time; same results either way).  A shape whose
 * trakhip_project_workspace_min() exceeds that is refused with TRAKHIP_ERR_STATIC_LIMIT (every shape
 * with proj_dim <= 262144 fits: a launch never has more partial blocks of 1024 columns than the device
 * has compute units).  Calls no hipMalloc / hipFree or any allocating routine.  All calls
 * on one GPU share the one array: calls that overlap in time on the same GPU (different streams
 * or threads) race and give wrong results; calls that follow one another on a stream do not. */
size_t trakhip_project_static_limit(void);
int trakhip_project_static(const void* in_dev, int in_dtype, uint64_t B, uint64_t P, uint64_t ld_in,
                           float* out_dev, uint32_t proj_dim, uint32_t seed, uint32_t num_feature_tiles,
                           int proj_type, void* stream);

/* The two phases of trakhip_project as separate calls, for one pass of B <= trakhip_project_rows_per_pass()
 * rows (workspace >= trakhip_project_workspace(B, ...)): phase 1 writes partial
 * sums [G, B, proj_dim] over G runs of consecutive features to the workspace (the kernel of
 * fast_jl/fast_jl_kernel.cuh:24-105 writing `output[row][tile][col]`; G depends only on the shape),
 * phase 2 adds them up in order into out_dev (the `.sum(1)` of fast_jl/fast_jl.cu:78), multiplied by
 * `scale` (1.0f for the plain sum; 1/sqrt(P) gives the `grads /= normalize_factor` of
 * trak/traker.py:426 for free).  A caller can time the phases or put its own epilogue between. */
int trakhip_project_partials(const void* in_dev, int in_dtype, uint64_t B, uint64_t P, uint64_t ld_in,
                             void* workspace_dev, size_t workspace_bytes, uint32_t proj_dim, uint32_t seed,
                             uint32_t num_feature_tiles, int proj_type, void* stream);
int trakhip_project_reduce(const void* workspace_dev, uint64_t B, uint64_t P, uint32_t proj_dim,
                           uint32_t num_feature_tiles, float scale, float* out_dev, void* stream);

/* Phase 2 with the rest of TRAKer.featurize's epilogue folded in: out[b, c] = cast((sum of the
 * partials) * scale), i.e. `grads /= normalize_factor; grads.to(dtype)` of trak/traker.py:426-428
 * (torch divides by a scalar as a multiplication by its fp32 reciprocal, so scale = 1.0f / sqrt(P)
 * gives the same bits), written with row pitch ld_out (elements) either to device memory or
 * straight into page-locked host memory (hipHostMalloc / torch pin_memory) - the staging buffer
 * of the `grads` store rows of trak/savers.py:406-410, which replaces the `.cpu()` copy.
 *   out_dtype   TRAKHIP_F16 | TRAKHIP_BF16 | TRAKHIP_F32 (round to nearest even)
 *   out         aligned to four elements, ld_out >= proj_dim and a multiple of 4; pageable host
 *               memory is refused with TRAKHIP_ERR_POINTER */
int trakhip_project_reduce_store(const void* workspace_dev, uint64_t B, uint64_t P, uint32_t proj_dim,
                                 uint32_t num_feature_tiles, float scale, int out_dtype, void* out,
                                 uint64_t ld_out, void* stream);

/* One piece of a gradient that is stored as a list of tensors (one per model parameter): features
 * [first, first + numel) of every row live at ptr[row * ld + (feature - first)]. */
typedef struct trakhip_segment {
    const void* ptr; /* device memory, aligned to the element size */
    uint64_t first;  /* first feature index of this piece */
    uint64_t numel;  /* features in this piece (>= 1) */
    uint64_t ld;     /* row pitch in elements (>= numel) */
} trakhip_segment;

/* Phase 1 of the projection reading the [B, P] gradient through a table of segments instead of one
 * dense matrix: the flatten-and-copy of trak.utils.vectorize (trak/utils.py:80-110) and the chunk
 * packing of ChunkedCudaProjector.project (trak/projectors.py:479-503) disappear.  segs_dev is a
 * device array of n_segs segments, sorted by `first`, contiguous (first[i+1] = first[i] + numel[i])
 * and covering [0, P); all of element type in_dtype; B <= trakhip_project_rows_per_pass().  Result and workspace as for
 * trakhip_project_partials; finish with trakhip_project_reduce. */
int trakhip_project_gather_partials(const trakhip_segment* segs_dev, uint32_t n_segs, int in_dtype, uint64_t B,
                                    uint64_t P, void* workspace_dev, size_t workspace_bytes, uint32_t proj_dim,
                                    uint32_t seed, uint32_t num_feature_tiles, int proj_type, void* stream);

/* Writes the block S[f0 : f0+nf, c0 : c0+nc] of the projection matrix that trakhip_project uses
 * for (seed, num_feature_tiles, P) as fp32, row-major [nf, nc].  The reference never stores S
 * (it exists only inside fast_jl/random.cuh:27-60); this is the hook that lets a caller check
 * the stream.  on_device != 0: out is device memory and a kernel on `stream` writes it;
 * on_device == 0: out is host memory, filled by host code before returning. */
int trakhip_materialize(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f0, uint64_t nf,
                        uint32_t c0, uint32_t nc, int proj_type, float* out, int on_device, void* stream);

/* ---- scoring (BasicScoreComputer) ---------------------------------------------------------- */

/* C[M, N] = alpha * A[M, K] * B[N, K]^T + beta * C, then row i scaled by row_scale[i] when
 * row_scale_dev != NULL; all fp32.  Stands in for `block @ xtx_inv` (trak/score_computers.py:176,
 * xtx_inv symmetric) and `features @ target_grads.t()` (trak/utils.py:131); the optional row scale
 * is the out_to_loss factor of trak/traker.py:670-678. */
int trakhip_gemm_nt(const float* A_dev, uint64_t lda, const float* B_dev, uint64_t ldb, float* C_dev,
                    uint64_t ldc, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta,
                    const float* row_scale_dev, void* stream);

/* C[M, N] = alpha * A[K, M]^T * B[K, N] + beta * C; fp32.  With A == B this is the
 * `block.T @ block` accumulation of trak/score_computers.py:145-155. */
int trakhip_gemm_tn(const float* A_dev, uint64_t lda, const float* B_dev, uint64_t ldb, float* C_dev,
                    uint64_t ldc, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta,
                    void* stream);

/* The same products on the 16-bit matrix cores (sixteen times the fp32 MFMA rate) without giving
 * up fp32 accuracy.  An operand is first brought into "planes" (trakhip_split_rows, one pass):
 * an fp32 matrix becomes three bf16 planes whose sum is the fp32 value exactly, and the product
 * uses six bf16 MFMAs per k step with fp32 accumulation (the terms left out are below 2^-24 of each
 * product, the rounding of one fp32 multiplication); an fp16 or bf16 matrix (what TRAKer stores
 * with use_half_precision) is one plane and one MFMA, with exact products.
 *   src_dtype                      TRAKHIP_F32 | TRAKHIP_F16 | TRAKHIP_BF16; both operands of a
 *                                  product must come from the same type
 *   trakhip_split_bytes            bytes of the planes of a [rows, K] operand
 *   trakhip_split_rows             src_dev is [rows, K] with row pitch ld (transposed == 0), or
 *                                  [K, rows] with row pitch ld (transposed != 0: the operand is
 *                                  the transpose of what is stored, as X^T in X^T X)
 *   trakhip_gemm_nt_split          C[M, N] = alpha * A * B^T + beta * C, row i *= row_scale[i];
 *                                  A_planes from a [M, K] operand, B_planes from a [N, K] one
 *   trakhip_gram_split             C[N, N] = alpha * A * A^T + beta * C: only the tiles that touch
 *                                  the lower triangle are computed, then the strict upper triangle
 *                                  is overwritten with the mirror image, so C is exactly
 *                                  symmetric; with beta != 0, C must have been produced this way.
 *                                  workspace_dev (may be NULL): trakhip_gram_split_workspace bytes,
 *                                  16-byte aligned.  A product with few tiles (N up to 4608) leaves
 *                                  CUs idle; with the workspace its k range is shared out over three
 *                                  sets of workgroups whose sums are added in a fixed order
 *   trakhip_gram_split_workspace   bytes that trakhip_gram_split (two_planes == 0) or
 *                                  trakhip_gram_split2 (two_planes != 0) can use for these sizes; 0
 *                                  when they would not use any
 * Stand in, like trakhip_gemm_nt / trakhip_gemm_tn, for trak/score_computers.py:153 (the Gram
 * product, A = the planes of block^T), :176 and trak/utils.py:131. */
size_t trakhip_split_bytes(uint64_t rows, uint64_t K, int src_dtype);
int trakhip_split_rows(const void* src_dev, int src_dtype, uint64_t ld, uint64_t rows, uint64_t K, int transposed,
                       void* planes_dev, size_t planes_bytes, void* stream);
int trakhip_gemm_nt_split(const void* A_planes_dev, uint64_t M, const void* B_planes_dev, uint64_t N, uint64_t K,
                          int src_dtype, float* C_dev, uint64_t ldc, float alpha, float beta,
                          const float* row_scale_dev, void* stream);
size_t trakhip_gram_split_workspace(uint64_t N, uint64_t K, int src_dtype, int two_planes);
int trakhip_gram_split(const void* A_planes_dev, uint64_t N, uint64_t K, int src_dtype, float* C_dev, uint64_t ldc,
                       float alpha, float beta, void* workspace_dev, size_t workspace_bytes, void* stream);

/* An opt-in cheaper form of the split products for fp32 operands: two fp16 planes per operand and
 * three fp16 MFMAs per k step instead of three bf16 planes and six MFMAs (about 1.75 times the speed).
 * trakhip_split2_rows multiplies every operand row by the power of two that brings its largest
 * magnitude into [2^14, 2^15) and stores x * 2^s = h1 + h2 (fp16, round to nearest even): 22 significand
 * bits for entries within 2^-18 of the row's largest, fewer below (absolute error <= 2^-26 of the
 * row's largest magnitude), against all 24 bits of the three-plane split.  The product leaves out
 * h2 * h2' (below 2^-22 of a product); the powers of two are removed again in the epilogue (exact).
 * Not a replacement for the exact split where inputs may hold rows of very uneven magnitude.
 *   trakhip_split2_bytes    bytes of the planes of a [rows, K] fp32 operand
 *   trakhip_split2_rows     src_dev as for trakhip_split_rows; scales_dev: 2 * rows floats, the first
 *                           `rows` of them are the inverse row factors that the products take, the rest
 *                           is scratch
 *   trakhip_gemm_nt_split2, trakhip_gram_split2   as trakhip_gemm_nt_split / trakhip_gram_split, with
 *                           each operand's scales_dev
 * Stand in for the same three matmuls (trak/score_computers.py:153, :176, trak/utils.py:131). */
size_t trakhip_split2_bytes(uint64_t rows, uint64_t K);
int trakhip_split2_rows(const float* src_dev, uint64_t ld, uint64_t rows, uint64_t K, int transposed, void* planes_dev,
                        size_t planes_bytes, float* scales_dev, void* stream);
int trakhip_gemm_nt_split2(const void* A_planes_dev, const float* A_scales_dev, uint64_t M, const void* B_planes_dev,
                           const float* B_scales_dev, uint64_t N, uint64_t K, float* C_dev, uint64_t ldc, float alpha,
                           float beta, const float* row_scale_dev, void* stream);
int trakhip_gram_split2(const void* A_planes_dev, const float* A_scales_dev, uint64_t N, uint64_t K, float* C_dev,
                        uint64_t ldc, float alpha, float beta, void* workspace_dev, size_t workspace_bytes,
                        void* stream);

/* C[M, N] (fp32) = alpha * A[M, K] * B[N, K]^T + beta * C, row i *= row_scale[i], for fp16 or bf16
 * operands read where they are: no planes, no extra pass.  For the two products of a TRAKer that
 * stores half precision whose operands are row-major along the contraction: `block @ xtx_inv`
 * (trak/score_computers.py:176) and `features @ target_grads.t()` (trak/utils.py:131).
 *   dtype      TRAKHIP_F16 | TRAKHIP_BF16, both operands
 *   K          a multiple of 64 (TRAKHIP_ERR_SHAPE otherwise; proj_dim is a multiple of 512)
 *   A_dev, B_dev  16-byte aligned, lda and ldb multiples of 8 elements (TRAKHIP_ERR_ALIGN otherwise) and
 *              below 2^23 elements (TRAKHIP_ERR_SHAPE otherwise)
 * A caller whose operands do not qualify uses trakhip_split_rows + trakhip_gemm_nt_split; the results
 * are the same bits (same MFMAs in the same order). */
int trakhip_gemm_nt16(const void* A_dev, uint64_t lda, const void* B_dev, uint64_t ldb, int dtype, float* C_dev,
                      uint64_t ldc, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta,
                      const float* row_scale_dev, void* stream);

/* out[i, j] = cast((acc[i, j] / divisor) * row_factor[i]) for the [N, M] fp32 score sums that
 * trakhip_gemm_nt accumulated over checkpoints (beta = 1): the closing expression of
 * TRAKer.finalize_scores, `(_scores / n) * (_avg_out_to_losses / n)` (trak/traker.py:670-678), with
 * divisor = n and row_factor[i] = the second factor, two correctly rounded fp32 operations in that
 * order, then the cast to the store's type (TRAKHIP_F16 | TRAKHIP_BF16 | TRAKHIP_F32).  `out` is device
 * memory or page-locked host memory (pageable host memory: TRAKHIP_ERR_POINTER), so the score
 * matrix crosses PCIe once, after the last checkpoint.  row_factor_dev may be NULL (factor 1). */
int trakhip_scores_finalize(const float* acc_dev, uint64_t ld_acc, uint64_t N, uint64_t M, float divisor,
                            const float* row_factor_dev, int out_dtype, void* out, uint64_t ld_out,
                            void* stream);

/* Bytes of scratch trakhip_spd_inverse needs for an n x n matrix. */
size_t trakhip_spd_inverse_workspace(uint64_t n);

/* inv[n, n] = (A + lambda * I)^-1 for symmetric positive definite A + lambda*I (fp32), then
 * divided by mean(|inv|) when normalize != 0; *mean_abs_dev (device, 1 float, may be NULL)
 * receives that mean.  Stands in for torch.linalg.inv + `xtx_inv /= xtx_inv.abs().mean()` of
 * trak/score_computers.py:160-166.  A_dev is not modified; inv_dev may not alias it.
 * status_dev (device, 1 int32, may be NULL) is set to 0, or to 1 + the index of the first
 * non-positive pivot. */
int trakhip_spd_inverse(const float* A_dev, uint64_t lda, float lambda, float* inv_dev, uint64_t ldi,
                        uint64_t n, int normalize, float* mean_abs_dev, int32_t* status_dev,
                        void* workspace_dev, size_t workspace_bytes, void* stream);

/* The same result for ANY nonsingular fp32 matrix A + lambda * I, by elimination with partial (row)
 * pivoting on the device: the route for a matrix that trakhip_spd_inverse reports as not positive
 * definite (status != 0) - a Gram matrix rounded to fp16, or one of deficient rank with lambda = 0, is
 * symmetric but need not be positive definite, and the reference inverts every matrix with LU and partial
 * pivoting (torch.linalg.inv, trak/score_computers.py:163).  n <= 12288 (TRAKHIP_ERR_SHAPE beyond, and
 * trakhip_general_inverse_workspace returns 0).  Arguments as trakhip_spd_inverse; status_dev is set to 0, or to
 * 1 + the index of the first pivot that is exactly zero (a singular matrix: the result is then not finite). */
size_t trakhip_general_inverse_workspace(uint64_t n);
int trakhip_general_inverse(const float* A_dev, uint64_t lda, float lambda, float* inv_dev, uint64_t ldi,
                            uint64_t n, int normalize, float* mean_abs_dev, int32_t* status_dev,
                            void* workspace_dev, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRAKHIP_H */
