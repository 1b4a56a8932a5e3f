// Output-side casts shared by the epilogue kernels: four fp32 results stored as fp32, fp16 or bf16
// (round to nearest even, the rounding of torch's Tensor.to and of numpy's astype).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace trakhip {

__device__ __forceinline__ uint16_t cast_f16_bits(float v) {
    // keep the binary32 value a separate, already rounded operand: without the empty asm the
    // compiler may fold the producing multiply into a mixed-precision FMA that rounds only once
    asm("" : "+v"(v));
    return __builtin_bit_cast(uint16_t, (_Float16)v);
}

__device__ __forceinline__ uint16_t cast_bf16_bits(float v) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x0040u);  // quiet NaN
    return (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}

// OUT_DTYPE: TRAKHIP_F16 (0), TRAKHIP_BF16 (1), TRAKHIP_F32 (2); dst is aligned to four elements
template <int OUT_DTYPE>
__device__ __forceinline__ void store4(void* dst, float4 r) {
    if constexpr (OUT_DTYPE == 2) {
        *reinterpret_cast<float4*>(dst) = r;
    } else if constexpr (OUT_DTYPE == 0) {
        uint2 w;
        w.x = (uint32_t)cast_f16_bits(r.x) | ((uint32_t)cast_f16_bits(r.y) << 16);
        w.y = (uint32_t)cast_f16_bits(r.z) | ((uint32_t)cast_f16_bits(r.w) << 16);
        *reinterpret_cast<uint2*>(dst) = w;
    } else {
        uint2 w;
        w.x = (uint32_t)cast_bf16_bits(r.x) | ((uint32_t)cast_bf16_bits(r.y) << 16);
        w.y = (uint32_t)cast_bf16_bits(r.z) | ((uint32_t)cast_bf16_bits(r.w) << 16);
        *reinterpret_cast<uint2*>(dst) = w;
    }
}

constexpr size_t out_elem_size(int out_dtype) { return out_dtype == 2 ? 4 : 2; }

// True when a kernel on the current device may write through p: device memory, or host memory
// that was allocated page-locked (hipHostMalloc, torch's pin_memory).  Pageable host memory is
// refused here, on the host, because a kernel that touches it faults the GPU.
bool kernel_can_write(const void* p);

}  // namespace trakhip
