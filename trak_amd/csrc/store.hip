// Epilogue of the scoring path: turns the accumulated [N_train, M_targets] score sums into the
// stored scores, `(sum / n_models) * (avg_out_to_loss / n_models)` of trak/traker.py:670-678, cast
// to the store's element type and written to device memory or straight into page-locked host
// memory.  HBM / PCIe bound: 4 bytes read and 2 or 4 bytes written per score.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "store_cast.h"
#include "trakhip_internal.h"

namespace {

using trakhip::store4;

template <int OUT_DTYPE>
__device__ __forceinline__ void store1(void* dst, float v) {
    if constexpr (OUT_DTYPE == 2)
        *static_cast<float*>(dst) = v;
    else if constexpr (OUT_DTYPE == 0)
        *static_cast<uint16_t*>(dst) = trakhip::cast_f16_bits(v);
    else
        *static_cast<uint16_t*>(dst) = trakhip::cast_bf16_bits(v);
}

// one thread per four consecutive scores of a row; VEC = rows of both matrices keep four-element
// alignment, so a quad is one 16-byte load and one 8- or 16-byte store
template <int OUT_DTYPE, bool VEC>
__global__ __launch_bounds__(256) void scores_finalize_kernel(const float* __restrict__ acc, uint64_t ld_acc,
                                                              uint64_t N, uint64_t M, uint64_t quads,
                                                              float divisor,
                                                              const float* __restrict__ row_factor,
                                                              void* __restrict__ out, uint64_t ld_out) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= N * quads) return;
    const uint64_t row = i / quads, q = i - row * quads;
    const uint64_t c = q * 4;
    const float f = row_factor ? row_factor[row] : 1.0f;
    const float* src = acc + row * ld_acc + c;
    char* dst = static_cast<char*>(out) + (row * ld_out + c) * trakhip::out_elem_size(OUT_DTYPE);
    if (VEC || c + 4 <= M) {
        float4 v;
        if constexpr (VEC) {
            v = *reinterpret_cast<const float4*>(src);
        } else {
            v = {src[0], src[1], src[2], src[3]};
        }
        // two correctly rounded binary32 operations, in the order numpy evaluates the reference's
        // expression
        v.x = __fmul_rn(__fdiv_rn(v.x, divisor), f);
        v.y = __fmul_rn(__fdiv_rn(v.y, divisor), f);
        v.z = __fmul_rn(__fdiv_rn(v.z, divisor), f);
        v.w = __fmul_rn(__fdiv_rn(v.w, divisor), f);
        if constexpr (VEC) {
            store4<OUT_DTYPE>(dst, v);
        } else {
            const size_t es = trakhip::out_elem_size(OUT_DTYPE);
            store1<OUT_DTYPE>(dst, v.x);
            store1<OUT_DTYPE>(dst + es, v.y);
            store1<OUT_DTYPE>(dst + 2 * es, v.z);
            store1<OUT_DTYPE>(dst + 3 * es, v.w);
        }
    } else {
        const size_t es = trakhip::out_elem_size(OUT_DTYPE);
        for (uint64_t t = 0; c + t < M; ++t)
            store1<OUT_DTYPE>(dst + t * es, __fmul_rn(__fdiv_rn(src[t], divisor), f));
    }
}

template <int OUT_DTYPE>
hipError_t launch_finalize(bool vec, const float* acc, uint64_t ld_acc, uint64_t N, uint64_t M, float divisor,
                           const float* row_factor, void* out, uint64_t ld_out, hipStream_t s) {
    const uint64_t quads = (M + 3) / 4;
    const dim3 grid((uint32_t)((N * quads + 255) / 256)), block(256);
    if (vec)
        hipLaunchKernelGGL((scores_finalize_kernel<OUT_DTYPE, true>), grid, block, 0, s, acc, ld_acc, N, M, quads,
                           divisor, row_factor, out, ld_out);
    else
        hipLaunchKernelGGL((scores_finalize_kernel<OUT_DTYPE, false>), grid, block, 0, s, acc, ld_acc, N, M, quads,
                           divisor, row_factor, out, ld_out);
    return hipGetLastError();
}

}  // namespace

namespace trakhip {

bool kernel_can_write(const void* p) {
    if (!p) return false;
    hipPointerAttribute_t a;
    if (hipPointerGetAttributes(&a, p) != hipSuccess) {
        (void)hipGetLastError();  // pageable host memory is reported as an error: clear it
        return false;
    }
    return a.type == hipMemoryTypeDevice || a.type == hipMemoryTypeHost || a.type == hipMemoryTypeManaged;
}

int scores_finalize(const float* acc, uint64_t ld_acc, uint64_t N, uint64_t M, float divisor,
                    const float* row_factor, int out_dtype, void* out, uint64_t ld_out, hipStream_t s) {
    if (out_dtype != TRAKHIP_F16 && out_dtype != TRAKHIP_BF16 && out_dtype != TRAKHIP_F32) return TRAKHIP_ERR_DTYPE;
    if (ld_acc < M || ld_out < M || !(divisor != 0.0f)) return TRAKHIP_ERR_SHAPE;
    if (N == 0 || M == 0) return TRAKHIP_OK;
    if (!acc || !out) return TRAKHIP_ERR_NULL;
    const size_t es = out_elem_size(out_dtype);
    if ((reinterpret_cast<uintptr_t>(acc) % 4) || (reinterpret_cast<uintptr_t>(out) % es)) return TRAKHIP_ERR_ALIGN;
    const uint64_t quads = (M + 3) / 4;
    if ((N * quads + 255) / 256 > 0x7FFFFFFFull) return TRAKHIP_ERR_SHAPE;
    if (!kernel_can_write(out)) return TRAKHIP_ERR_POINTER;
    const bool vec = M % 4 == 0 && ld_acc % 4 == 0 && ld_out % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(acc) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % (4 * es) == 0;
    hipError_t e;
    if (out_dtype == TRAKHIP_F32)
        e = launch_finalize<TRAKHIP_F32>(vec, acc, ld_acc, N, M, divisor, row_factor, out, ld_out, s);
    else if (out_dtype == TRAKHIP_F16)
        e = launch_finalize<TRAKHIP_F16>(vec, acc, ld_acc, N, M, divisor, row_factor, out, ld_out, s);
    else
        e = launch_finalize<TRAKHIP_BF16>(vec, acc, ld_acc, N, M, divisor, row_factor, out, ld_out, s);
    return e == hipSuccess ? TRAKHIP_OK : TRAKHIP_ERR_LAUNCH;
}

}  // namespace trakhip
