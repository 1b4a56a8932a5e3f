// Internal C++ interface between the C ABI (capi.hip) and the kernel files.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/trakhip.h"

namespace trakhip {

size_t project_workspace_bytes(uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles);
size_t project_workspace_min_bytes(uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles);
uint32_t project_rows_per_pass(int dtype, int proj_type);
int project(const void* in, int dtype, uint64_t B, uint64_t P, uint64_t ld, float* out, void* ws,
            size_t ws_bytes, uint32_t k, uint32_t seed, uint32_t num_feature_tiles, int proj_type,
            hipStream_t s);
// the same without a workspace argument: partial sums go to a per-device static array
size_t project_static_limit_bytes();
int project_static(const void* in, int dtype, uint64_t B, uint64_t P, uint64_t ld, float* out, uint32_t k,
                   uint32_t seed, uint32_t num_feature_tiles, int proj_type, hipStream_t s);
int project_partials(const void* in, int dtype, uint64_t B, uint64_t P, uint64_t ld, void* ws, size_t ws_bytes,
                     uint32_t k, uint32_t seed, uint32_t num_feature_tiles, int proj_type, hipStream_t s);
int project_gather_partials(const trakhip_segment* segs, uint32_t n_segs, int dtype, uint64_t B, uint64_t P,
                            void* ws, size_t ws_bytes, uint32_t k, uint32_t seed, uint32_t num_feature_tiles,
                            int proj_type, hipStream_t s);
int project_reduce(const void* ws, uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles, float scale,
                   float* out, hipStream_t s);
int project_reduce_store(const void* ws, uint64_t B, uint64_t P, uint32_t k, uint32_t num_feature_tiles,
                         float scale, int out_dtype, void* out, uint64_t ld_out, hipStream_t s,
                         bool check_destination);
int scores_finalize(const float* acc, uint64_t ld_acc, uint64_t N, uint64_t M, float divisor,
                    const float* row_factor, int out_dtype, void* out, uint64_t ld_out, hipStream_t s);
bool kernel_can_write(const void* p);
int materialize_device(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f0, uint64_t nf,
                       uint32_t c0, uint32_t nc, int proj_type, float* out, hipStream_t s);
int materialize_host(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f0, uint64_t nf,
                     uint32_t c0, uint32_t nc, int proj_type, float* out);

// internal GEMM option (symmetric results: spd.hip, gemm_split.hip)
constexpr uint32_t kGemmLowerTilesOnly = 1u;  // skip output tiles strictly above the diagonal

// up to kGemmBatchMax products of one shape in one launch: element offsets of each product's operands
constexpr uint32_t kGemmBatchMax = 32;
struct GemmBatch {
    uint32_t count;
    uint64_t a[kGemmBatchMax], b[kGemmBatchMax], c[kGemmBatchMax];
    uint64_t m[kGemmBatchMax] = {};  // rows of product y when not zero (at most the call's M); zero: the call's M
};
int gemm_nn_batched(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
                    uint64_t N, uint64_t K, float alpha, float beta, const GemmBatch& batch, hipStream_t s);

int gemm_nt(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
            uint64_t N, uint64_t K, float alpha, float beta, const float* row_scale, hipStream_t s,
            uint32_t flags = 0);
int gemm_tn(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
            uint64_t N, uint64_t K, float alpha, float beta, hipStream_t s, uint32_t flags = 0);
int gemm_nn(const float* A, uint64_t lda, const float* B, uint64_t ldb, float* C, uint64_t ldc, uint64_t M,
            uint64_t N, uint64_t K, float alpha, float beta, hipStream_t s, uint32_t flags = 0);
// dtype = element type of the source matrices (TRAKHIP_F32: three bf16 planes; F16 / BF16: one plane)
size_t split_bytes(uint64_t rows, uint64_t K, int dtype);
int split_rows(const void* src, int dtype, uint64_t ld, uint64_t rows, uint64_t K, int transposed, void* planes,
               size_t planes_bytes, hipStream_t s);
int gemm_nt_split(const void* A_planes, uint64_t M, const void* B_planes, uint64_t N, uint64_t K, int dtype, float* C,
                  uint64_t ldc, float alpha, float beta, const float* row_scale, hipStream_t s, uint32_t flags = 0);
// ws (may be null): gram_split_workspace_bytes() bytes that let a product with few tiles share its k range out
size_t gram_split_workspace_bytes(uint64_t N, uint64_t K, int dtype, int two_planes);
int gram_split(const void* A_planes, uint64_t N, uint64_t K, int dtype, float* C, uint64_t ldc, float alpha, float beta,
               void* ws, size_t ws_bytes, hipStream_t s);
size_t split2_bytes(uint64_t rows, uint64_t K);
int split2_rows(const float* src, uint64_t ld, uint64_t rows, uint64_t K, int transposed, void* planes,
                size_t planes_bytes, float* scales, hipStream_t s);
int gemm_nt_split2(const void* A_planes, const float* a_scales, uint64_t M, const void* B_planes, const float* b_scales,
                   uint64_t N, uint64_t K, float* C, uint64_t ldc, float alpha, float beta, const float* row_scale,
                   hipStream_t s, uint32_t flags = 0);
int gram_split2(const void* A_planes, const float* a_scales, uint64_t N, uint64_t K, float* C, uint64_t ldc, float alpha,
                float beta, void* ws, size_t ws_bytes, hipStream_t s);
int gemm_nt16(const void* A, uint64_t lda, const void* B, uint64_t ldb, int dtype, float* C, uint64_t ldc, uint64_t M,
              uint64_t N, uint64_t K, float alpha, float beta, const float* row_scale, hipStream_t s);
size_t spd_inverse_workspace_bytes(uint64_t n);
int spd_inverse(const float* A, uint64_t lda, float lambda, float* inv, uint64_t ldi, uint64_t n,
                int normalize, float* mean_abs, int32_t* status, void* ws, size_t ws_bytes, hipStream_t s);
// the same for any nonsingular matrix (Gauss-Jordan elimination with partial pivoting)
size_t general_inverse_workspace_bytes(uint64_t n);
int general_inverse(const float* A, uint64_t lda, float lambda, float* inv, uint64_t ldi, uint64_t n,
                    int normalize, float* mean_abs, int32_t* status, void* ws, size_t ws_bytes, hipStream_t s);

}  // namespace trakhip
