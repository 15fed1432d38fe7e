// Small fp32 products (a few hundred rows and columns): too few 64 x 128 tiles to give every compute unit one, and a
// tile that walks all of K alone pays the load latency of every step.  Here a workgroup owns a 32 x 32 tile of C and
// its four wavefronts split K; a lane loads its operand values straight from global memory (16 bytes along K where the
// operand is contiguous along K, single values otherwise: any strides, any alignment), several steps ahead of the
// v_mfma_f32_32x32x2f32 that use them, and the four partial tiles meet in LDS.  512 x 512 x 512 is 256 such workgroups:
// one per compute unit, each wavefront 64 MFMAs long.
// (C[m][n] = sum over k of A[m][k] * B[k][n] in fp32: src/cpu/matmul.cpp:60-124.)
#include "gemm_tiles.hpp"

namespace th {

typedef float float4_any __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kSmallWaves = 4;
constexpr int kSmallUnroll = 4;   // groups of 8 k whose loads are issued together

// the four values k .. k + 3 of one row (or column) of an operand: base + k * k_stride, zero from k_end on
template <bool K_CONTIGUOUS>
__device__ inline float4_any four_along_k(const float* base, int64_t k_stride, uint32_t k, uint32_t k_end) {
    if (K_CONTIGUOUS && k + 4 <= k_end) return *reinterpret_cast<const float4_any*>(base + k);
    float4_any v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = k + e < k_end ? base[static_cast<int64_t>(k + e) * k_stride] : 0.0f;
    return v;
}

template <bool A_K, bool B_K>
__global__ __launch_bounds__(64 * kSmallWaves) void gemm_small_f32_kernel(const float* A, const float* B, float* C, GemmProblem p, uint32_t tiles_n, uint32_t k_per_wave) {
    __shared__ float partial[kSmallWaves][16][64];
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.y, oa, ob, oc);
    const uint32_t tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64, r = lane % 32, h = lane / 32;
    // rows and columns past the end read the last one: they only feed results that are never stored
    const uint32_t m = tm * 32 + r < p.M ? tm * 32 + r : p.M - 1, n = tn * 32 + r < p.N ? tn * 32 + r : p.N - 1;
    const float* a_row = A + oa + static_cast<int64_t>(m) * p.a_rs;
    const float* b_col = B + ob + static_cast<int64_t>(n) * p.b_cs;
    const uint32_t k_begin = wave * k_per_wave < p.K ? wave * k_per_wave : p.K;
    const uint32_t k_end = k_begin + k_per_wave < p.K ? k_begin + k_per_wave : p.K;

    // MFMA e of a group of 8 k takes k + 4 * (lane / 32) + e from both operands.  The accumulator holds the tile
    // transposed (the column operand goes first): value v of a lane is row lane % 32, column 8 * (v / 4) + 4 * (lane / 32) + v % 4.
    float16v acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    for (uint32_t k0 = k_begin; k0 < k_end; k0 += 8 * kSmallUnroll) {
        float4_any fa[kSmallUnroll], fb[kSmallUnroll];
#pragma unroll
        for (int u = 0; u < kSmallUnroll; ++u) {
            const uint32_t k = k0 + 8 * u + 4 * h;
            fa[u] = four_along_k<A_K>(a_row, p.a_cs, k, k_end);
            fb[u] = four_along_k<B_K>(b_col, p.b_rs, k, k_end);
        }
#pragma unroll
        for (int u = 0; u < kSmallUnroll; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[u][e], fa[u][e], acc, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) partial[wave][v][lane] = acc[v];
    __syncthreads();
    // wavefront w adds up the values 4w .. 4w + 3 of every lane: four consecutive columns of one row
    float sum[4];
    const uint32_t row = tm * 32 + r, col = tn * 32 + 8 * wave + 4 * h;
    const float start = (p.row_bias && row < p.M) ? static_cast<const float*>(p.row_bias)[row] : 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        sum[e] = partial[0][4 * wave + e][lane];
#pragma unroll
        for (int w = 1; w < kSmallWaves; ++w) sum[e] += partial[w][4 * wave + e][lane];
        sum[e] += start;
    }
    if (row >= p.M || col >= p.N) return;
    store_piece_anywhere<float>(C + oc + static_cast<int64_t>(row) * p.c_rs + col, sum, p.N - col < 4 ? p.N - col : 4);
}

int gemm_small_f32(const GemmProblem& p, const float* a, const float* b, float* c, hipStream_t stream) {
    if (p.M == 0 || p.N == 0 || p.K == 0 || p.batches == 0 || p.batches > 65535 || p.c_group) return TANNIC_UNSUPPORTED_DTYPE;
    // Not when the tiles of the large kernels fill the chip, when K is too short to be worth splitting four ways, or when it
    // is long: a wavefront's share of K is one MFMA after the other, 64 clocks for two k, and the large kernels' blocks that
    // share K pass it (NT, us, this kernel against those: 512 x 512 x 512 8.1 / 14.5, 256^3 6.1 / 10.1, 1024 x 512 x 512
    // 11.9 / 16.2, 512 x 1024 x 1024 21.7 / 21.4, 512 x 512 x 2048 23.1 / 22.2, 384 x 384 x 4096 41 / 28).
    const uint64_t tiles_m = (p.M + 31) / 32, tiles_n = (p.N + 31) / 32, tiles = tiles_m * tiles_n * p.batches;
    if (tiles > 512 || p.K < 64 || p.K > 1024 || tiles * p.K > 512 * 512) return TANNIC_UNSUPPORTED_DTYPE;
    const uint32_t groups = (p.K + 7) / 8, k_per_wave = (groups + kSmallWaves - 1) / kSmallWaves * 8;
    const dim3 grid(static_cast<uint32_t>(tiles_m * tiles_n), p.batches), block(64 * kSmallWaves);
    const bool ak = p.a_cs == 1, bk = p.b_rs == 1;
    const uint32_t tn = static_cast<uint32_t>(tiles_n);
    if (ak && bk) hipLaunchKernelGGL((gemm_small_f32_kernel<true, true>), grid, block, 0, stream, a, b, c, p, tn, k_per_wave);
    else if (ak) hipLaunchKernelGGL((gemm_small_f32_kernel<true, false>), grid, block, 0, stream, a, b, c, p, tn, k_per_wave);
    else if (bk) hipLaunchKernelGGL((gemm_small_f32_kernel<false, true>), grid, block, 0, stream, a, b, c, p, tn, k_per_wave);
    else hipLaunchKernelGGL((gemm_small_f32_kernel<false, false>), grid, block, 0, stream, a, b, c, p, tn, k_per_wave);
    return launch_status("gemm_small_f32_kernel");
}

}  // namespace th
