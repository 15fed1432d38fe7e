// Rate probes: what the matrix pipe sustains by itself, on given operand values.
//
// The matrix kernels are measured against the published dense MFMA peak, which assumes the peak shader clock.  Under a
// matrix load the chip lowers its clock with the power the work draws, and that depends on the operand VALUES (zeros
// cost least).  These kernels issue nothing but MFMAs — four wavefronts per compute unit, one per SIMD, every
// accumulator register in use, operands loaded once from a caller-supplied buffer — so their rate is the ceiling for any
// kernel that also has to move data, on those values.  No counterpart in the reference; used by the benchmark only.
#include "gemm_tiles.hpp"

namespace th {

typedef float float4v __attribute__((ext_vector_type(4)));

// The accumulator is updated in place ("+a": the same AGPRs go in and come out), so that the loop holds nothing but MFMAs.
template <class T, int SHAPE, class Acc> __device__ inline void mfma_in_place(Acc& acc, const uint4v& a, const uint4v& b) {
    if constexpr (SHAPE == 0 && std::is_same_v<T, f16>) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    if constexpr (SHAPE == 0 && std::is_same_v<T, bf16>) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    if constexpr (SHAPE == 1 && std::is_same_v<T, f16>) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
    if constexpr (SHAPE == 1 && std::is_same_v<T, bf16>) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// SHAPE 0: v_mfma_f32_32x32x16, 16 accumulators of 16 registers; SHAPE 1: v_mfma_f32_16x16x32, 32 accumulators of 4;
// CHAIN: how many consecutive MFMAs update the same accumulator (a dependent MFMA takes its addend from the one before
// it, not from the register file: no slower, and cheaper in power).
// One iteration is 2^21 multiply-adds per wavefront either way (64 resp. 128 MFMAs); operands rotate through eight
// registers per side so that consecutive MFMAs see different values, as they do in a product.
template <class T, int SHAPE, int CHAIN = 1>
__global__ __launch_bounds__(256) void probe_mfma_kernel(const uint4v* operands, float* sink, uint32_t iterations) {
    uint4v a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = operands[i * 256 + threadIdx.x];
        b[i] = operands[(8 + i) * 256 + threadIdx.x];
    }
    float total = 0.0f;
    if constexpr (SHAPE == 0) {
        float16v acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
        for (uint32_t it = 0; it < iterations; ++it) {
#pragma unroll
            for (int m = 0; m < 64; ++m) mfma_in_place<T, 0>(acc[m % 16], b[(m + m / 16) % 8], a[(m / 4) % 8]);
        }
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMAs' results are read below
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) total += acc[i][v];
    } else {
        float4v acc[32];
#pragma unroll
        for (int i = 0; i < 32; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[i][v] = 0.0f;
        for (uint32_t it = 0; it < iterations; ++it) {
#pragma unroll
            for (int m = 0; m < 128; ++m) mfma_in_place<T, 1>(acc[(m / CHAIN) % 32], b[(m + m / 32) % 8], a[(m / 8) % 8]);
        }
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
        for (int i = 0; i < 32; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) total += acc[i][v];
    }
    sink[blockIdx.x * 256 + threadIdx.x] = total;
}

}  // namespace th

using namespace th;

extern "C" int tannic_hip_probe_mfma(int shape, int dtype, const void* operands, void* sink, uint32_t blocks, uint32_t iterations, tannic_stream_t stream) {
    if (!operands || !sink || blocks == 0 || shape < 0 || shape > 2) {
        set_error_text("probe_mfma: operands (64 KiB), sink (1 KiB per block) and a block count are required; shape is 0, 1 or 2");
        return TANNIC_ERROR;
    }
    hipStream_t s = as_stream(stream);
    const uint4v* ops = static_cast<const uint4v*>(operands);
    float* out = static_cast<float*>(sink);
    if (dtype == TANNIC_FLOAT16) {
        if (shape == 0) hipLaunchKernelGGL((probe_mfma_kernel<f16, 0>), dim3(blocks), dim3(256), 0, s, ops, out, iterations);
        else if (shape == 1) hipLaunchKernelGGL((probe_mfma_kernel<f16, 1>), dim3(blocks), dim3(256), 0, s, ops, out, iterations);
        else hipLaunchKernelGGL((probe_mfma_kernel<f16, 1, 2>), dim3(blocks), dim3(256), 0, s, ops, out, iterations);
    } else if (dtype == TANNIC_BFLOAT16) {
        if (shape == 0) hipLaunchKernelGGL((probe_mfma_kernel<bf16, 0>), dim3(blocks), dim3(256), 0, s, ops, out, iterations);
        else if (shape == 1) hipLaunchKernelGGL((probe_mfma_kernel<bf16, 1>), dim3(blocks), dim3(256), 0, s, ops, out, iterations);
        else hipLaunchKernelGGL((probe_mfma_kernel<bf16, 1, 2>), dim3(blocks), dim3(256), 0, s, ops, out, iterations);
    } else {
        return TANNIC_UNSUPPORTED_DTYPE;
    }
    return launch_status("probe_mfma_kernel");
}
