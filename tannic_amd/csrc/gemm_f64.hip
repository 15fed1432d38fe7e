// float64 products on v_mfma_f64_16x16x4f64.
//
// The fp64 matrix instruction takes one double of each operand per lane and keeps the matrix pipe busy for 64 clocks, so
// there is nothing to stage: a lane loads its operand values straight from global memory (32 bytes along K where the
// operand is contiguous along K, single doubles otherwise: any strides, any alignment of whole doubles), several windows
// of 16 k ahead of the MFMAs that use them.  Every wavefront owns TM x TN tiles of 16 x 16; a workgroup is either four
// wavefronts side by side (2 x 2, each walking all of K), or, when that would leave most compute units without a block,
// four wavefronts that split K over one wavefront's tiles and add their partial sums up in LDS.
// (C[m][n] = sum over k of A[m][k] * B[k][n] in double: src/cpu/matmul.cpp:60-124.)
#include "gemm_common.hpp"

namespace th {

typedef double double4v __attribute__((ext_vector_type(4)));
typedef double double2_any __attribute__((ext_vector_type(2), aligned(8)));

// the four values k .. k + 3 of one row (or column) of an operand: base + k * k_stride, zero from k_end on
template <bool K_CONTIGUOUS>
__device__ inline void four_doubles_along_k(const double* base, int64_t k_stride, uint32_t k, uint32_t k_end, double (&v)[4]) {
    if (K_CONTIGUOUS && k + 4 <= k_end) {
        const double2_any lo = *reinterpret_cast<const double2_any*>(base + k), hi = *reinterpret_cast<const double2_any*>(base + k + 2);
        v[0] = lo[0];
        v[1] = lo[1];
        v[2] = hi[0];
        v[3] = hi[1];
        return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = k + e < k_end ? base[static_cast<int64_t>(k + e) * k_stride] : 0.0;
}

template <bool A_K, bool B_K, int TM, int TN, bool SPLIT, int DEPTH>
__global__ __launch_bounds__(256) void gemm_f64_kernel(const double* A, const double* B, double* C, GemmProblem p, uint32_t tiles_n, uint32_t k_per_wave) {
    constexpr int WM = 16 * TM, WN = 16 * TN, VALUES = TM * TN * 4;
    extern __shared__ double partial[];   // SPLIT: [4][VALUES][64]
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.y, oa, ob, oc);
    const uint32_t tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x % 64, r = lane % 16, g = lane / 16;
    uint32_t m0, n0, k_begin, k_end;
    if constexpr (SPLIT) {
        m0 = tm * WM;
        n0 = tn * WN;
        k_begin = wave * k_per_wave < p.K ? wave * k_per_wave : p.K;
        k_end = k_begin + k_per_wave < p.K ? k_begin + k_per_wave : p.K;
    } else {
        m0 = tm * 2 * WM + (wave / 2) * WM;
        n0 = tn * 2 * WN + (wave % 2) * WN;
        k_begin = 0;
        k_end = p.K;
    }
    // rows and columns past the end read the last one: they only feed results that are never stored
    const double* a_row[TM];
    const double* b_col[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const uint32_t m = m0 + 16 * i + r < p.M ? m0 + 16 * i + r : p.M - 1;
        a_row[i] = A + oa + static_cast<int64_t>(m) * p.a_rs;
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t n = n0 + 16 * j + r < p.N ? n0 + 16 * j + r : p.N - 1;
        b_col[j] = B + ob + static_cast<int64_t>(n) * p.b_cs;
    }

    // MFMA e of a window of 16 k takes k + 4 * (lane / 16) + e from both operands.  Value v of a lane's accumulator is
    // row 4 * v + lane / 16, column lane % 16 of the tile.
    double4v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = double4v{0.0, 0.0, 0.0, 0.0};
    // DEPTH windows are in flight: slot s is refilled with the window DEPTH further on as soon as its MFMAs are issued
    double fa[DEPTH][TM][4], fb[DEPTH][TN][4];
#pragma unroll
    for (int s = 0; s < DEPTH; ++s) {
#pragma unroll
        for (int i = 0; i < TM; ++i) four_doubles_along_k<A_K>(a_row[i], p.a_cs, k_begin + 16 * s + 4 * g, k_end, fa[s][i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) four_doubles_along_k<B_K>(b_col[j], p.b_rs, k_begin + 16 * s + 4 * g, k_end, fb[s][j]);
    }
    for (uint32_t k0 = k_begin; k0 < k_end; k0 += 16 * DEPTH) {
#pragma unroll
        for (int s = 0; s < DEPTH; ++s) {
            // (a window past k_end is all zeros: its MFMAs add nothing)
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[s][i][e], fb[s][j][e], acc[i][j], 0, 0, 0);
            const uint32_t k = k0 + 16 * (s + DEPTH) + 4 * g;
#pragma unroll
            for (int i = 0; i < TM; ++i) four_doubles_along_k<A_K>(a_row[i], p.a_cs, k, k_end, fa[s][i]);
#pragma unroll
            for (int j = 0; j < TN; ++j) four_doubles_along_k<B_K>(b_col[j], p.b_rs, k, k_end, fb[s][j]);
        }
    }

    // (sixteen lanes write sixteen consecutive doubles of a row)
    // With grouped columns (GemmProblem::c_group) column j of group q goes to C + q * c_group_stride + row * c_rs + j, and
    // the columns past a group's live ones nowhere; a per-row start value (row_bias) is added to the finished sum.
    auto store_tile = [&](int i, int j, const double4v& sum) {
        const uint32_t col = n0 + 16 * j + r;
        if (col >= p.N) return;
        int64_t at = oc + col;
        if (p.c_group) {
            uint32_t q, within;
            p.c_group_div.divmod(col, q, within);
            if (within >= p.c_group_live) return;
            at = static_cast<int64_t>(q) * p.c_group_stride + within;
        }
        const double* bias = static_cast<const double*>(p.row_bias);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint32_t row = m0 + 16 * i + 4 * v + g;
            if (row < p.M) C[at + static_cast<int64_t>(row) * p.c_rs] = bias ? sum[v] + bias[row] : sum[v];
        }
    };
    if constexpr (SPLIT) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 4; ++v) partial[(wave * VALUES + (i * TN + j) * 4 + v) * 64 + lane] = acc[i][j][v];
        __syncthreads();
        // wavefront w adds up the tiles w, w + 4, ...
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if ((i * TN + j) % 4 != static_cast<int>(wave)) continue;
                double4v sum;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    double s = partial[((i * TN + j) * 4 + v) * 64 + lane];
#pragma unroll
                    for (int w = 1; w < 4; ++w) s += partial[(w * VALUES + (i * TN + j) * 4 + v) * 64 + lane];
                    sum[v] = s;
                }
                store_tile(i, j, sum);
            }
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) store_tile(i, j, acc[i][j]);
    }
}

template <bool A_K, bool B_K, int TM, int TN, bool SPLIT, int DEPTH>
static int launch_f64_layout(const GemmProblem& p, const double* a, const double* b, double* c, hipStream_t stream, dim3 grid, uint32_t tiles_n, uint32_t k_per_wave) {
    constexpr size_t lds = SPLIT ? size_t(4) * TM * TN * 4 * 64 * sizeof(double) : 0;
    if constexpr (lds > 48 * 1024) {
        static std::atomic<uint64_t> raised{0};
        if (int rc = raise_lds_limit(reinterpret_cast<const void*>(&gemm_f64_kernel<A_K, B_K, TM, TN, SPLIT, DEPTH>), lds, raised)) return rc;
    }
    hipLaunchKernelGGL((gemm_f64_kernel<A_K, B_K, TM, TN, SPLIT, DEPTH>), grid, dim3(256), lds, stream, a, b, c, p, tiles_n, k_per_wave);
    return launch_status("gemm_f64_kernel");
}

template <int TM, int TN, bool SPLIT, int DEPTH>
static int launch_f64(const GemmProblem& p, const double* a, const double* b, double* c, hipStream_t stream) {
    constexpr uint32_t BM = SPLIT ? 16 * TM : 32 * TM, BN = SPLIT ? 16 * TN : 32 * TN;
    const uint64_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    if (tiles_m * tiles_n >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    const uint32_t windows = (p.K + 15) / 16, k_per_wave = (windows + 3) / 4 * 16;
    const dim3 grid(static_cast<uint32_t>(tiles_m * tiles_n), p.batches);
    const bool ak = p.a_cs == 1, bk = p.b_rs == 1;
    const uint32_t tn = static_cast<uint32_t>(tiles_n);
    if (ak && bk) return launch_f64_layout<true, true, TM, TN, SPLIT, DEPTH>(p, a, b, c, stream, grid, tn, k_per_wave);
    if (ak) return launch_f64_layout<true, false, TM, TN, SPLIT, DEPTH>(p, a, b, c, stream, grid, tn, k_per_wave);
    if (bk) return launch_f64_layout<false, true, TM, TN, SPLIT, DEPTH>(p, a, b, c, stream, grid, tn, k_per_wave);
    return launch_f64_layout<false, false, TM, TN, SPLIT, DEPTH>(p, a, b, c, stream, grid, tn, k_per_wave);
}

int gemm_mfma_f64(const GemmProblem& p, const double* a, const double* b, double* c, hipStream_t stream) {
    if (p.b_group_stride || (p.c_group && p.batches != 1)) return TANNIC_UNSUPPORTED_DTYPE;
    // (fewer than 17 rows under a long K stream through the kernels for few rows: they are bound by memory)
    if (p.M == 0 || p.N == 0 || p.K == 0 || p.batches == 0 || p.batches > 65535) return TANNIC_UNSUPPORTED_DTYPE;
    // (a product with grouped columns is a convolution's: no other kernel stores those, and it is taken whatever its extents)
    if (!p.c_group) {
        if (p.M < 8 || p.N < 8 || p.K < 16) return TANNIC_UNSUPPORTED_DTYPE;
        if (p.M <= 16 && p.a_cs == 1 && p.b_rs == 1 && p.K >= 256) return TANNIC_UNSUPPORTED_DTYPE;
    }
    // The matrix pipe bounds every shape of workgroup alike: what a choice costs is the rounds of 256 workgroups it
    // takes times the area of one.  Equal costs go to the larger tile, and a wavefront of 4 x 4 tiles loads half as much
    // per MFMA as one of 2 x 2 (the loads, not the matrix pipe, are what these kernels wait for).
    auto cost = [&](uint32_t bm, uint32_t bn) {
        const uint64_t blocks = static_cast<uint64_t>((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.batches;
        return static_cast<double>((blocks + 255) / 256) * bm * bn;
    };
    const double large = cost(128, 128), medium = cost(64, 64), small = cost(32, 32);
    if (large <= medium && large <= small) return launch_f64<4, 4, false, 2>(p, a, b, c, stream);
    if (medium <= small) return p.K >= 128 ? launch_f64<4, 4, true, 2>(p, a, b, c, stream) : launch_f64<2, 2, false, 4>(p, a, b, c, stream);
    return launch_f64<2, 2, true, 4>(p, a, b, c, stream);
}

}  // namespace th
