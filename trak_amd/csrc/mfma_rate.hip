// Measurement aid, not part of the library's ABI: a loop of nothing but independent MFMAs on
// chosen operand data.  bench.py (--only mfma_rate) uses it to show what the matrix pipes
// sustain on this machine - the rate depends on the data because the clock is power limited -
// next to what the projection and GEMM kernels reach.  Built into its own shared object
// (libtrakhip_diag.so).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// operand kinds: 0 zeros; 1 gradient-like fp16 pairs (random sign and mantissa, exponent field
// 2..8); 2 fp16 +-1; 3 random fp16 below 2^15; 4 random bf16 (exponent field 100..139)
__device__ uint32_t make_operand(int kind, uint32_t r) {
    switch (kind) {
        case 0: return 0u;
        case 1:
            return ((r & 0x83FFu) | ((2u + ((r >> 10) % 7u)) << 10)) |
                   ((((r >> 16) & 0x83FFu) | ((2u + ((r >> 26) % 7u)) << 10)) << 16);
        case 2: return (r & 0x80008000u) | 0x3C003C00u;
        case 3: return r & 0xBFFFBFFFu;
        default:
            return ((r & 0x807Fu) | ((100u + ((r >> 7) % 40u)) << 7)) |
                   ((((r >> 16) & 0x807Fu) | ((100u + ((r >> 23) % 40u)) << 7)) << 16);
    }
}

// INSTR 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_32x32x16_bf16, 2: v_mfma_f32_32x32x2_f32
template <int INSTR>
__global__ __launch_bounds__(256) void mfma_rate_kernel(float* out, int iters, int kind_a, int kind_b, uint32_t seed) {
    uint32_t s = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + seed;
    auto rnd = [&]() {
        s ^= s << 13;
        s ^= s >> 17;
        s ^= s << 5;
        return s;
    };
    uint4 A[4], B[4];
    for (int i = 0; i < 4; ++i) {
        A[i] = {make_operand(kind_a, rnd()), make_operand(kind_a, rnd()), make_operand(kind_a, rnd()),
                make_operand(kind_a, rnd())};
        B[i] = {make_operand(kind_b, rnd()), make_operand(kind_b, rnd()), make_operand(kind_b, rnd()),
                make_operand(kind_b, rnd())};
    }
    floatx16 acc[4];
    for (int i = 0; i < 4; ++i)
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (INSTR == 0)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, A[i]),
                                                                __builtin_bit_cast(half8, B[i]), acc[i], 0, 0, 0);
            if (INSTR == 1)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, A[i]),
                                                                 __builtin_bit_cast(bf16x8, B[i]), acc[i], 0, 0, 0);
            if (INSTR == 2)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(A[i].x & 0xBF7FFFFFu),
                                                              __uint_as_float(B[i].x & 0xBF7FFFFFu), acc[i], 0, 0, 0);
        }
    }
    float r = 0;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 16; ++j) r += acc[i][j];
    out[blockIdx.x * 256 + threadIdx.x] = r;
}

}  // namespace

extern "C" {

// Floats that out_dev must hold.
size_t trakhip_diag_mfma_rate_out_floats(void) { return 512u * 256u; }

// Enqueues one dispatch of 512 workgroups x 256 threads (two waves per SIMD on 256 CUs), each wave
// issuing 4 * iters MFMAs on four independent accumulators.  Returns the flop of the dispatch
// (0 on bad arguments).
double trakhip_diag_mfma_rate(int instr, int kind_a, int kind_b, int iters, float* out_dev, void* stream) {
    if (instr < 0 || instr > 2 || iters <= 0 || !out_dev) return 0.0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (instr == 0) hipLaunchKernelGGL(mfma_rate_kernel<0>, dim3(512), dim3(256), 0, s, out_dev, iters, kind_a, kind_b, 1u);
    if (instr == 1) hipLaunchKernelGGL(mfma_rate_kernel<1>, dim3(512), dim3(256), 0, s, out_dev, iters, kind_a, kind_b, 1u);
    if (instr == 2) hipLaunchKernelGGL(mfma_rate_kernel<2>, dim3(512), dim3(256), 0, s, out_dev, iters, kind_a, kind_b, 1u);
    if (hipGetLastError() != hipSuccess) return 0.0;
    return 512.0 * 4.0 * iters * 4.0 * (instr == 2 ? 4096.0 : 32768.0);
}

}  // extern "C"
