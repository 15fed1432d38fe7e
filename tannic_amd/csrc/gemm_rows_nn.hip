// At most eight rows (fp32; fp16 / bf16 where the tiles do badly) times a matrix that is contiguous along its columns: y[m][n] = sum over k of x[m][k] * W[k][n] with W[K,N]
// lying row by row (x . W as written, where a linear layer stores W^T).  The work is reading W once, and W's rows are
// the wrong way round for the matrix instructions (a fragment wants consecutive k of one column), so this is plain
// fused multiply-adds: a lane owns four consecutive columns, a wavefront 256, and walks its share of K reading whole
// rows of W (1 KB per wavefront and row of fp32, eight rows in flight); the rows of x it needs are staged once per
// workgroup in LDS as fp32 and read back as broadcasts.  Four wavefronts split a workgroup's rows of W and add up in
// LDS; the workgroups that share K leave fp32 partial sums that a second pass adds and rounds once.
// (C[m][n] = sum over k of A[m][k] * B[k][n] with fp32 sums for the 16-bit types: src/cpu/matmul.cpp:60-124.)
#include "gemm_common.hpp"

namespace th {

constexpr int kRowsNnWaves = 4;
constexpr int kRowsNnLdsFloats = 12288;   // 48 KB: the staged rows of x, then the wavefronts' sums

template <class T> struct FourOf;
template <> struct FourOf<float> { typedef float type __attribute__((ext_vector_type(4), aligned(4))); };
template <> struct FourOf<f16> { typedef _Float16 type __attribute__((ext_vector_type(4), aligned(2))); };
template <> struct FourOf<bf16> { typedef unsigned short type __attribute__((ext_vector_type(4), aligned(2))); };

template <class T> __device__ inline void widen_four(const typename FourOf<T>::type& v, float (&out)[4]) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if constexpr (std::is_same_v<T, bf16>) out[e] = to_float(bf16{v[e]});
        else out[e] = static_cast<float>(v[e]);
    }
}

// MR: rows of x a lane accumulates (a multiple of 4, at least M).  chunk: rows of W per wavefront (a multiple of 8).
// partial == nullptr: the workgroups do not share K and the result goes straight to c.
template <class T, int MR>
__global__ __launch_bounds__(64 * kRowsNnWaves) void gemm_rows_nn_kernel(const T* x, const T* w, float* partial, T* c, GemmProblem p, uint32_t groups, uint32_t chunk) {
    using Four = typename FourOf<T>::type;
    __shared__ __align__(16) float lds[kRowsNnLdsFloats];
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const uint32_t group = blockIdx.x % groups, share = blockIdx.x / groups;
    const uint32_t col = group * 256 + lane * 4;
    const bool active = col < p.N;   // (N is a multiple of 4)
    const uint32_t block_k = share * kRowsNnWaves * chunk, block_rows = kRowsNnWaves * chunk;

    // x[m][block_k + j] as fp32, [j][MR]; zero past the end of K and for the rows beyond M
    for (uint32_t i = threadIdx.x; i < block_rows * MR; i += 64 * kRowsNnWaves) {
        const uint32_t j = i / MR, m = i % MR, k = block_k + j;
        float v = 0.0f;
        if (m < p.M && k < p.K) v = static_cast<float>(widen(x[static_cast<int64_t>(m) * p.a_rs + static_cast<int64_t>(k) * p.a_cs]));
        lds[i] = v;
    }
    __syncthreads();

    float acc[MR][4];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[m][e] = 0.0f;
    const uint32_t k_begin = block_k + wave * chunk;
    const T* wp = w + col;
    for (uint32_t j0 = 0; j0 < chunk; j0 += 8) {
        Four rows[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const uint32_t k = k_begin + j0 + u;
            if (active && k < p.K) rows[u] = *reinterpret_cast<const Four*>(wp + static_cast<int64_t>(k) * p.b_rs);
            else rows[u] = Four{};
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            float wv[4];
            widen_four<T>(rows[u], wv);
            const float* xs = lds + (wave * chunk + j0 + u) * MR;
#pragma unroll
            for (int m4 = 0; m4 < MR; m4 += 4) {
                const float4 xv = *reinterpret_cast<const float4*>(xs + m4);
                const float xm[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[m4 + q][e] += xm[q] * wv[e];
            }
        }
    }
    // the other wavefronts' sums to LDS ([wave - 1][m][e][lane]), the first adds them to its own
    __syncthreads();
    if (wave != 0) {
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) lds[((wave - 1) * MR * 4 + m * 4 + e) * 64 + lane] = acc[m][e];
    }
    __syncthreads();
    if (wave != 0 || !active) return;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        if (static_cast<uint32_t>(m) >= p.M) break;
        float sum[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            sum[e] = acc[m][e];
#pragma unroll
            for (int v = 0; v < kRowsNnWaves - 1; ++v) sum[e] += lds[(v * MR * 4 + m * 4 + e) * 64 + lane];
        }
        if (partial) {
            *reinterpret_cast<float4*>(partial + (static_cast<size_t>(share) * p.M + m) * p.N + col) = float4{sum[0], sum[1], sum[2], sum[3]};
        } else {
            T* dst = c + static_cast<int64_t>(m) * p.c_rs + col;
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = narrow_result<T>(sum[e]);
        }
    }
}

// c[m][n] = sum over the shares of partial[share][m][n], rounded once.  A workgroup owns 64 quads of columns; its four
// wavefronts each add up every fourth share (eight loads in flight) and meet in LDS.
template <class T>
__global__ __launch_bounds__(256) void gemm_rows_nn_finish_kernel(const float* partial, T* c, uint32_t M, uint32_t N, int64_t c_rs, uint32_t shares, uint32_t total) {
    __shared__ float4 part[3][64];
    const uint32_t lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const uint32_t idx = blockIdx.x * 64 + lane;
    const bool live = idx < total;
    const uint32_t quads = N / 4, m = live ? idx / quads : 0, col = live ? (idx % quads) * 4 : 0;
    const float* src = partial + static_cast<size_t>(m) * N + col;
    const size_t step = static_cast<size_t>(M) * N;
    float4 sum = float4{0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t s0 = wave; s0 < shares; s0 += 32) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = (live && s0 + 4 * u < shares) ? *reinterpret_cast<const float4*>(src + (s0 + 4 * u) * step) : float4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            sum.x += v[u].x;
            sum.y += v[u].y;
            sum.z += v[u].z;
            sum.w += v[u].w;
        }
    }
    if (wave != 0) part[wave - 1][lane] = sum;
    __syncthreads();
    if (wave != 0 || !live) return;
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        sum.x += part[w][lane].x;
        sum.y += part[w][lane].y;
        sum.z += part[w][lane].z;
        sum.w += part[w][lane].w;
    }
    T* dst = c + static_cast<int64_t>(m) * c_rs + col;
    dst[0] = narrow_result<T>(sum.x);
    dst[1] = narrow_result<T>(sum.y);
    dst[2] = narrow_result<T>(sum.z);
    dst[3] = narrow_result<T>(sum.w);
}

template <class T, int MR>
static int launch_rows_nn(const GemmProblem& p, const T* x, const T* w, T* c, hipStream_t stream) {
    const uint32_t groups = (p.N + 255) / 256;
    // enough workgroups to keep every compute unit's loads going (fewer with more rows: every share of K costs a copy of the result)
    const uint32_t wanted = p.M <= 4 ? 1024 : 512;
    uint32_t shares = wanted / groups ? wanted / groups : 1;
    const uint32_t most = (p.K + 8 * kRowsNnWaves - 1) / (8 * kRowsNnWaves);   // at least eight rows of W per wavefront
    if (shares > most) shares = most;
    if (shares > 128) shares = 128;   // (every share is a row of partial sums the second pass has to add)
    uint32_t chunk = (p.K + shares * kRowsNnWaves - 1) / (shares * kRowsNnWaves);
    chunk = (chunk + 7) / 8 * 8;
    // the staged rows of x must fit (kRowsNnWaves * chunk * MR floats): more shares of K where they would not
    constexpr uint32_t longest = kRowsNnLdsFloats / (kRowsNnWaves * MR) / 8 * 8;
    if (chunk > longest) chunk = longest;
    shares = (p.K + kRowsNnWaves * chunk - 1) / (kRowsNnWaves * chunk);
    float* partial = nullptr;
    if (shares > 1 && scratch_acquire(reinterpret_cast<void**>(&partial), static_cast<size_t>(shares) * p.M * p.N * sizeof(float), stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
    hipLaunchKernelGGL((gemm_rows_nn_kernel<T, MR>), dim3(groups * shares), dim3(64 * kRowsNnWaves), 0, stream, x, w, partial, c, p, groups, chunk);
    int status = launch_status("gemm_rows_nn_kernel");
    if (partial) {
        if (status == TANNIC_SUCCESS) {
            const uint32_t total = p.M * (p.N / 4);
            hipLaunchKernelGGL((gemm_rows_nn_finish_kernel<T>), dim3((total + 63) / 64), dim3(256), 0, stream, partial, c, p.M, p.N, p.c_rs, shares, total);
            status = launch_status("gemm_rows_nn_finish_kernel");
        }
        scratch_release(partial, stream);
    }
    return status;
}

template <class T>
static int run_rows_nn(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    // (from nine rows on the multiply-adds, sixteen per loaded value and row block, take longer than W takes to arrive:
    // fp32 16 rows over 4096 x 4096 39 us against the tiles' 32)
    if (p.M == 0 || p.M > 8 || p.batches != 1 || p.row_bias || p.c_group || p.b_group_stride) return TANNIC_UNSUPPORTED_DTYPE;
    // W contiguous along its columns and not along K, whole quads of columns, enough of it that reading it is the work
    if (p.b_cs != 1 || p.b_rs == 1 || p.N % 4 != 0 || p.N < 256 || p.K < 64 || static_cast<uint64_t>(p.N) * p.K < (1u << 18)) return TANNIC_UNSUPPORTED_DTYPE;
    if (static_cast<uint64_t>(p.M) * p.N >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    if constexpr (sizeof(T) == 2) {
        // The 16-bit tiles that share K pass a wide W at this kernel's pace (fp16, one row over 4096 x 4096: 12 us either
        // way; 32000 x 512: 8 against 12 here).  What they do badly is a narrow W under a long K (512 x 16384: 16 against
        // 11 us) and an x that lies column by column with a number of rows no 16 bytes divide, which sends both operands
        // to the loaders for any alignment (four rows, 256 x 8192: 151 against 9 us).
        if (!(p.N <= 1024 || (p.a_cs != 1 && p.M % 8 != 0))) return TANNIC_UNSUPPORTED_DTYPE;
    }
    const T* x = static_cast<const T*>(a);
    const T* w = static_cast<const T*>(b);
    T* y = static_cast<T*>(c);
    if (p.M <= 4) return launch_rows_nn<T, 4>(p, x, w, y, stream);
    return launch_rows_nn<T, 8>(p, x, w, y, stream);
}

int gemm_rows_nn(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT32) return run_rows_nn<float>(p, a, b, c, stream);
    if (dtype == TANNIC_FLOAT16) return run_rows_nn<f16>(p, a, b, c, stream);
    if (dtype == TANNIC_BFLOAT16) return run_rows_nn<bf16>(p, a, b, c, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
