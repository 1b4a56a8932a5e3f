// extern "C" surface of libtrakhip.so (declared in include/trakhip.h).
#include "trakhip_internal.h"

extern "C" {

const char* trakhip_strerror(int code) {
    switch (code) {
        case TRAKHIP_OK: return "success";
        case TRAKHIP_ERR_PROJ_DIM:
            return "Invalid Number of JL dimensions it has to be a multiple of 512";
        case TRAKHIP_ERR_SHAPE: return "invalid shape (empty, too large, or pitch smaller than row length)";
        case TRAKHIP_ERR_DTYPE: return "input must be fp16, bf16 or fp32";
        case TRAKHIP_ERR_PROJ_TYPE: return "unknown projection type";
        case TRAKHIP_ERR_NULL: return "null pointer argument";
        case TRAKHIP_ERR_WORKSPACE: return "workspace too small";
        case TRAKHIP_ERR_ALIGN: return "pointer not sufficiently aligned";
        case TRAKHIP_ERR_LAUNCH: return "HIP kernel launch failed";
        case TRAKHIP_ERR_NOT_SPD: return "matrix is not positive definite";
        case TRAKHIP_ERR_NO_DEVICE: return "no HIP device";
        case TRAKHIP_ERR_POINTER:
            return "destination is neither device memory nor page-locked host memory";
        case TRAKHIP_ERR_STATIC_LIMIT:
            return "shape needs more scratch than the static array of trakhip_project_static holds";
        case TRAKHIP_ERR_HOST_MEMORY: return "out of host memory while planning the call";
        default: return "unknown trakhip error";
    }
}

int trakhip_abi_version(void) { return 1; }

size_t trakhip_project_workspace(uint64_t B, uint64_t P, uint32_t proj_dim, uint32_t num_feature_tiles) {
    return trakhip::project_workspace_bytes(B, P, proj_dim, num_feature_tiles);
}

size_t trakhip_project_workspace_min(uint64_t B, uint64_t P, uint32_t proj_dim, uint32_t num_feature_tiles) {
    return trakhip::project_workspace_min_bytes(B, P, proj_dim, num_feature_tiles);
}

uint32_t trakhip_project_rows_per_pass(int in_dtype, int proj_type) {
    return trakhip::project_rows_per_pass(in_dtype, proj_type);
}

int trakhip_project(const void* in_dev, int in_dtype, uint64_t B, uint64_t P, uint64_t ld_in, float* out_dev,
                    void* workspace_dev, size_t workspace_bytes, uint32_t proj_dim, uint32_t seed,
                    uint32_t num_feature_tiles, int proj_type, void* stream) {
    return trakhip::project(in_dev, in_dtype, B, P, ld_in, out_dev, workspace_dev, workspace_bytes, proj_dim,
                            seed, num_feature_tiles, proj_type, static_cast<hipStream_t>(stream));
}

size_t trakhip_project_static_limit(void) { return trakhip::project_static_limit_bytes(); }

int trakhip_project_static(const void* in_dev, int in_dtype, uint64_t B, uint64_t P, uint64_t ld_in, float* out_dev,
                           uint32_t proj_dim, uint32_t seed, uint32_t num_feature_tiles, int proj_type,
                           void* stream) {
    return trakhip::project_static(in_dev, in_dtype, B, P, ld_in, out_dev, proj_dim, seed, num_feature_tiles,
                                   proj_type, static_cast<hipStream_t>(stream));
}

int trakhip_project_partials(const void* in_dev, int in_dtype, uint64_t B, uint64_t P, uint64_t ld_in,
                             void* workspace_dev, size_t workspace_bytes, uint32_t proj_dim, uint32_t seed,
                             uint32_t num_feature_tiles, int proj_type, void* stream) {
    return trakhip::project_partials(in_dev, in_dtype, B, P, ld_in, workspace_dev, workspace_bytes, proj_dim, seed,
                                     num_feature_tiles, proj_type, static_cast<hipStream_t>(stream));
}

int trakhip_project_gather_partials(const trakhip_segment* segs_dev, uint32_t n_segs, int in_dtype, uint64_t B,
                                    uint64_t P, void* workspace_dev, size_t workspace_bytes, uint32_t proj_dim,
                                    uint32_t seed, uint32_t num_feature_tiles, int proj_type, void* stream) {
    return trakhip::project_gather_partials(segs_dev, n_segs, in_dtype, B, P, workspace_dev, workspace_bytes,
                                            proj_dim, seed, num_feature_tiles, proj_type,
                                            static_cast<hipStream_t>(stream));
}

int trakhip_project_reduce(const void* workspace_dev, uint64_t B, uint64_t P, uint32_t proj_dim,
                           uint32_t num_feature_tiles, float scale, float* out_dev, void* stream) {
    return trakhip::project_reduce(workspace_dev, B, P, proj_dim, num_feature_tiles, scale, out_dev,
                                   static_cast<hipStream_t>(stream));
}

int trakhip_project_reduce_store(const void* workspace_dev, uint64_t B, uint64_t P, uint32_t proj_dim,
                                 uint32_t num_feature_tiles, float scale, int out_dtype, void* out,
                                 uint64_t ld_out, void* stream) {
    return trakhip::project_reduce_store(workspace_dev, B, P, proj_dim, num_feature_tiles, scale, out_dtype, out,
                                         ld_out, static_cast<hipStream_t>(stream), true);
}

int trakhip_scores_finalize(const float* acc_dev, uint64_t ld_acc, uint64_t N, uint64_t M, float divisor,
                            const float* row_factor_dev, int out_dtype, void* out, uint64_t ld_out,
                            void* stream) {
    return trakhip::scores_finalize(acc_dev, ld_acc, N, M, divisor, row_factor_dev, out_dtype, out, ld_out,
                                    static_cast<hipStream_t>(stream));
}

int trakhip_materialize(uint32_t seed, uint32_t num_feature_tiles, uint64_t P, uint64_t f0, uint64_t nf,
                        uint32_t c0, uint32_t nc, int proj_type, float* out, int on_device, void* stream) {
    if (on_device)
        return trakhip::materialize_device(seed, num_feature_tiles, P, f0, nf, c0, nc, proj_type, out,
                                           static_cast<hipStream_t>(stream));
    return trakhip::materialize_host(seed, num_feature_tiles, P, f0, nf, c0, nc, proj_type, out);
}

int trakhip_gemm_nt(const float* A_dev, uint64_t lda, const float* B_dev, uint64_t ldb, float* C_dev,
                    uint64_t ldc, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta,
                    const float* row_scale_dev, void* stream) {
    return trakhip::gemm_nt(A_dev, lda, B_dev, ldb, C_dev, ldc, M, N, K, alpha, beta, row_scale_dev,
                            static_cast<hipStream_t>(stream));
}

int trakhip_gemm_tn(const float* A_dev, uint64_t lda, const float* B_dev, uint64_t ldb, float* C_dev,
                    uint64_t ldc, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta, void* stream) {
    return trakhip::gemm_tn(A_dev, lda, B_dev, ldb, C_dev, ldc, M, N, K, alpha, beta,
                            static_cast<hipStream_t>(stream));
}

size_t trakhip_split_bytes(uint64_t rows, uint64_t K, int dtype) { return trakhip::split_bytes(rows, K, dtype); }

int trakhip_split_rows(const void* src_dev, int dtype, uint64_t ld, uint64_t rows, uint64_t K, int transposed,
                       void* planes_dev, size_t planes_bytes, void* stream) {
    return trakhip::split_rows(src_dev, dtype, ld, rows, K, transposed, planes_dev, planes_bytes,
                               static_cast<hipStream_t>(stream));
}

int trakhip_gemm_nt_split(const void* A_planes_dev, uint64_t M, const void* B_planes_dev, uint64_t N, uint64_t K,
                          int dtype, float* C_dev, uint64_t ldc, float alpha, float beta,
                          const float* row_scale_dev, void* stream) {
    return trakhip::gemm_nt_split(A_planes_dev, M, B_planes_dev, N, K, dtype, C_dev, ldc, alpha, beta, row_scale_dev,
                                  static_cast<hipStream_t>(stream));
}

size_t trakhip_gram_split_workspace(uint64_t N, uint64_t K, int dtype, int two_planes) {
    return trakhip::gram_split_workspace_bytes(N, K, dtype, two_planes);
}

int trakhip_gram_split(const void* A_planes_dev, uint64_t N, uint64_t K, int dtype, float* C_dev, uint64_t ldc,
                       float alpha, float beta, void* workspace_dev, size_t workspace_bytes, void* stream) {
    return trakhip::gram_split(A_planes_dev, N, K, dtype, C_dev, ldc, alpha, beta, workspace_dev, workspace_bytes,
                               static_cast<hipStream_t>(stream));
}

size_t trakhip_split2_bytes(uint64_t rows, uint64_t K) { return trakhip::split2_bytes(rows, K); }

int trakhip_split2_rows(const float* src_dev, uint64_t ld, uint64_t rows, uint64_t K, int transposed, void* planes_dev,
                        size_t planes_bytes, float* scales_dev, void* stream) {
    return trakhip::split2_rows(src_dev, ld, rows, K, transposed, planes_dev, planes_bytes, scales_dev,
                                static_cast<hipStream_t>(stream));
}

int trakhip_gemm_nt_split2(const void* A_planes_dev, const float* A_scales_dev, uint64_t M, const void* B_planes_dev,
                           const float* B_scales_dev, uint64_t N, uint64_t K, float* C_dev, uint64_t ldc, float alpha,
                           float beta, const float* row_scale_dev, void* stream) {
    return trakhip::gemm_nt_split2(A_planes_dev, A_scales_dev, M, B_planes_dev, B_scales_dev, N, K, C_dev, ldc, alpha,
                                   beta, row_scale_dev, static_cast<hipStream_t>(stream));
}

int trakhip_gram_split2(const void* A_planes_dev, const float* A_scales_dev, uint64_t N, uint64_t K, float* C_dev,
                        uint64_t ldc, float alpha, float beta, void* workspace_dev, size_t workspace_bytes,
                        void* stream) {
    return trakhip::gram_split2(A_planes_dev, A_scales_dev, N, K, C_dev, ldc, alpha, beta, workspace_dev,
                                workspace_bytes, static_cast<hipStream_t>(stream));
}

int trakhip_gemm_nt16(const void* A_dev, uint64_t lda, const void* B_dev, uint64_t ldb, int dtype, float* C_dev,
                      uint64_t ldc, uint64_t M, uint64_t N, uint64_t K, float alpha, float beta,
                      const float* row_scale_dev, void* stream) {
    return trakhip::gemm_nt16(A_dev, lda, B_dev, ldb, dtype, C_dev, ldc, M, N, K, alpha, beta, row_scale_dev,
                              static_cast<hipStream_t>(stream));
}

size_t trakhip_spd_inverse_workspace(uint64_t n) { return trakhip::spd_inverse_workspace_bytes(n); }

int trakhip_spd_inverse(const float* A_dev, uint64_t lda, float lambda, float* inv_dev, uint64_t ldi,
                        uint64_t n, int normalize, float* mean_abs_dev, int32_t* status_dev,
                        void* workspace_dev, size_t workspace_bytes, void* stream) {
    return trakhip::spd_inverse(A_dev, lda, lambda, inv_dev, ldi, n, normalize, mean_abs_dev, status_dev,
                                workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
}

size_t trakhip_general_inverse_workspace(uint64_t n) { return trakhip::general_inverse_workspace_bytes(n); }

int trakhip_general_inverse(const float* A_dev, uint64_t lda, float lambda, float* inv_dev, uint64_t ldi,
                            uint64_t n, int normalize, float* mean_abs_dev, int32_t* status_dev,
                            void* workspace_dev, size_t workspace_bytes, void* stream) {
    return trakhip::general_inverse(A_dev, lda, lambda, inv_dev, ldi, n, normalize, mean_abs_dev, status_dev,
                                    workspace_dev, workspace_bytes, static_cast<hipStream_t>(stream));
}

}  // extern "C"
