// Matrix product with very few rows (M <= 32; up to 64 over a small W), 16-bit types: y = x * W^T as the
// decoding step of a transformer runs it.  The work is reading W once; there is
// nothing to reuse, so nothing goes through LDS on the way in.
//
// v_mfma_f32_16x16x32: a block of 512 threads owns 16 columns of the result (16
// rows of W, which is K-contiguous); its eight wavefronts split K.  A lane loads
// its operand fragments straight from global memory — 16 bytes of a row of W
// (row lane % 16, k chunk lane / 16: four lanes cover 64 contiguous bytes of a
// row) and 16 bytes of a row of x — eight steps at a time, so that 8 KB per
// wavefront are in flight.  The eight partial 16x16 tiles meet in LDS, the
// first wavefront adds them, rounds once and stores four consecutive columns
// per lane.
#include "gemm_tiles.hpp"

namespace th {

typedef _Float16 half8y __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8y __attribute__((ext_vector_type(8)));
typedef float float4y __attribute__((ext_vector_type(4)));
typedef unsigned int uint4y __attribute__((ext_vector_type(4)));

template <class T> __device__ inline float4y skinny_mfma(uint4y a, uint4y b, float4y c) {
    if constexpr (std::is_same_v<T, f16>) {
        half8y x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, c, 0, 0, 0);
    } else {
        bfloat8y x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, c, 0, 0, 0);
    }
}

// fp32: element e of both 16-byte fragments is one k of the lane's four: four v_mfma_f32_16x16x4f32
template <> __device__ inline float4y skinny_mfma<float>(uint4y a, uint4y b, float4y c) {
    float x[4], y[4];
    __builtin_memcpy(x, &a, 16);
    __builtin_memcpy(y, &b, 16);
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(x[e], y[e], c, 0, 0, 0);
    return c;
}

// int8: 16 bytes are sixteen k of the lane's row, one v_mfma_i32_16x16x64_i8 per four chunks; sums and results are int32
typedef int int4y __attribute__((ext_vector_type(4)));
template <class T> struct SkinnyTypes { using Acc = float4y; using Out = T; };
template <> struct SkinnyTypes<int8_t> { using Acc = int4y; using Out = int32_t; };
template <class T> __device__ inline typename SkinnyTypes<T>::Acc skinny_step(uint4y a, uint4y b, typename SkinnyTypes<T>::Acc c) {
    if constexpr (std::is_same_v<T, int8_t>) {
        int4y x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_i32_16x16x64_i8(x, y, c, 0, 0, 0);
    } else {
        return skinny_mfma<T>(a, b, c);
    }
}

constexpr int kSkinnyWaves = 8;
constexpr int kSkinnyUnroll = 8;   // K steps of 32 whose loads are issued together

// what a chunk past the end of K reads instead: both operands, so that the product is an exact zero
__device__ const uint4y skinny_zeros = {0, 0, 0, 0};

// MB: blocks of 16 rows of x; NB: blocks of 16 columns per wavefront (a fragment of x then serves NB fragments of W)
template <class T, int MB, int NB>
__global__ __launch_bounds__(64 * kSkinnyWaves) void gemm_skinny_kernel(const T* x, const T* w, T* c, GemmProblem p, uint32_t k_per_wave) {
    __shared__ float4y partial[kSkinnyWaves][MB * NB][64];
    int64_t ox, ow, oc;
    batch_offsets(p, blockIdx.y, ox, ow, oc);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const uint32_t r = lane % 16, kc = lane / 16;
    const uint32_t n0 = blockIdx.x * 16 * NB;
    // rows past the end are read from the last row: they only feed results that are never stored
    const T* wrow[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const uint32_t n = n0 + nb * 16 + r < p.N ? n0 + nb * 16 + r : p.N - 1;
        wrow[nb] = w + ow + static_cast<int64_t>(n) * p.b_cs + kc * 8;
    }
    const T* xrow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const uint32_t m = mb * 16 + r < p.M ? mb * 16 + r : p.M - 1;
        xrow[mb] = x + ox + static_cast<int64_t>(m) * p.a_rs + kc * 8;
    }
    const uint32_t k_begin = wave * k_per_wave;
    const uint32_t k_end = k_begin + k_per_wave < p.K ? k_begin + k_per_wave : p.K;
    const T* zeros = reinterpret_cast<const T*>(&skinny_zeros) - kc * 8;

    float4y acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = float4y{0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t k0 = k_begin; k0 < k_end; k0 += 32 * kSkinnyUnroll) {
        uint4y fw[kSkinnyUnroll][NB], fx[kSkinnyUnroll][MB];
#pragma unroll
        for (int u = 0; u < kSkinnyUnroll; ++u) {
            const uint32_t k = k0 + 32 * u;
            const bool live = k + kc * 8 < k_end;   // K and the ranges are multiples of 8: a chunk is inside or outside
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) fw[u][nb] = *reinterpret_cast<const uint4y*>(live ? wrow[nb] + k : zeros + kc * 8);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) fx[u][mb] = *reinterpret_cast<const uint4y*>(live ? xrow[mb] + k : zeros + kc * 8);
        }
#pragma unroll
        for (int u = 0; u < kSkinnyUnroll; ++u)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = skinny_mfma<T>(fw[u][nb], fx[u][mb], acc[mb][nb]);
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) partial[wave][mb * NB + nb][lane] = acc[mb][nb];
    __syncthreads();
    if (wave != 0) return;
    // accumulator: lane -> row of x (m) lane % 16; value v -> column n0 + 4 * (lane / 16) + v
    T* cb = c + oc;
    const bool vector_ok = p.c_rs % 4 == 0 && p.N % 4 == 0 && reinterpret_cast<uintptr_t>(cb) % 8 == 0;
#pragma unroll
    for (int t = 0; t < MB * NB; ++t) {
        const int mb = t / NB, nb = t % NB;
        float4y sum = partial[0][t][lane];
#pragma unroll
        for (int v = 1; v < kSkinnyWaves; ++v) sum += partial[v][t][lane];
        const uint32_t m = mb * 16 + r, col = n0 + nb * 16 + 4 * kc;
        if (m >= p.M) continue;
        T out[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = narrow_result<T>(sum[e]);
        T* dst = cb + static_cast<int64_t>(m) * p.c_rs + col;
        if (vector_ok) {
            if (col < p.N) {
                uint2 bits;
                __builtin_memcpy(&bits, out, 8);
                *reinterpret_cast<uint2*>(dst) = bits;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < p.N) dst[e] = out[e];
        }
    }
}

// The same product with whole K windows of 64 (K a multiple of 64): the operands come in by direct global -> LDS loads.
//
// The kernel above asks for 16 bytes per lane with sixteen rows per instruction: 64 separate requests, and every
// 128-byte line of W is asked for eight times.  Each request is a tag lookup in the vector cache, and at one lookup a
// clock those lookups, not HBM, set the time.  Here a load instruction covers eight whole rows of a window (eight
// lanes per 128-byte line: eight requests), and LDS does the regrouping into MFMA fragments: a wavefront owns a ring
// of STAGES windows (per window 2 KB for each 16-row block of W and of x, rows XOR-swizzled like the tiles of the
// large kernels, on the global side), keeps STAGES - 1 windows on their way and waits, by vmcnt, for the oldest only.
// No barrier until the four wavefronts, which split K, add up their tiles.
typedef __attribute__((address_space(3))) void* skinny_lds_void;
constexpr int kStreamWaves = 4;
constexpr int kStreamBytesPerWave = 32 * 1024;

template <class T, int MB, int NB>
__global__ __launch_bounds__(64 * kStreamWaves) void gemm_skinny_stream_kernel(const T* x, const T* w, typename SkinnyTypes<T>::Out* c, GemmProblem p,
                                                                               uint32_t windows_per_wave) {
#if defined(__HIP_DEVICE_COMPILE__)
    using Acc = typename SkinnyTypes<T>::Acc;
    using Out = typename SkinnyTypes<T>::Out;
    constexpr int BLOCKS = MB + NB;                       // 16-row blocks per window: W's, then x's
    constexpr int STAGE_BYTES = BLOCKS * 2048, STAGES = kStreamBytesPerWave / STAGE_BYTES, LOADS = 2 * BLOCKS;
    static_assert(STAGES >= 3, "a ring of at least three windows");
    extern __shared__ __align__(16) unsigned char skinny_lds[];
    int64_t ox, ow, oc;
    batch_offsets(p, blockIdx.y, ox, ow, oc);
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const uint32_t r = lane % 16, kc = lane / 16;
    const uint32_t n0 = blockIdx.x * 16 * NB;
    unsigned char* ring = skinny_lds + wave * kStreamBytesPerWave;

    // buffer resources from the block's first row of W and from x: rows past the end read zeros
    auto records = [](uint64_t rows, int64_t pitch, uint32_t K) -> uint32_t {
        const uint64_t bytes = ((rows - 1) * static_cast<uint64_t>(pitch) + K) * sizeof(T);
        return bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(bytes);
    };
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(w + ow + static_cast<int64_t>(n0) * p.b_cs), 0, records(p.N - n0, p.b_cs, p.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(x + ox), 0, records(p.M, p.a_rs, p.K), 0x00020000);
    // load j of a window: rows 8 (j % 2) .. + 7 of block j / 2; the lane's row and its (swizzled) 16-byte chunk
    uint32_t voff[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
        const uint32_t row = (j % 2) * 8 + lane / 8, chunk = (lane % 8) ^ ((row >> 1) & 7u);
        const bool of_w = j / 2 < NB;
        const uint32_t block_row = (of_w ? j / 2 : j / 2 - NB) * 16 + row;
        voff[j] = block_row * static_cast<uint32_t>(of_w ? p.b_cs : p.a_rs) * sizeof(T) + chunk * 16;
    }
    auto issue = [&](uint32_t window, uint32_t stage) {
        const uint32_t k_bytes = window * 128;
#pragma unroll
        for (int j = 0; j < LOADS; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(j / 2 < NB ? rsrc_w : rsrc_x, (skinny_lds_void)(ring + stage * STAGE_BYTES + j * 1024), 16, voff[j], k_bytes, 0, 0);
    };
    const uint32_t all = p.K / kBKof<T>;   // windows of 128 bytes per row: 64 elements of 16 bits, 32 of fp32
    const uint32_t first = wave * windows_per_wave;
    const uint32_t count = first >= all ? 0 : (all - first < windows_per_wave ? all - first : windows_per_wave);

    Acc acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = Acc{0, 0, 0, 0};
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
        if (static_cast<uint32_t>(t) < count) issue(first + t, t);
    uint32_t stage = 0, fill = STAGES - 1;
    for (uint32_t i = 0; i < count; ++i) {
        if (i + STAGES - 1 < count) {
            issue(first + i + STAGES - 1, fill);
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 1) * LOADS) : "memory");    // loads complete in order: window i is in
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        const T* at = reinterpret_cast<const T*>(ring + stage * STAGE_BYTES);
        uint4y fw[2][NB], fx[2][MB];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) fw[half][nb] = *reinterpret_cast<const uint4y*>(at + nb * (2048 / sizeof(T)) + tile_offset<T>(r, half * 4 + kc));
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) fx[half][mb] = *reinterpret_cast<const uint4y*>(at + (NB + mb) * (2048 / sizeof(T)) + tile_offset<T>(r, half * 4 + kc));
        }
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = skinny_step<T>(fw[half][nb], fx[half][mb], acc[mb][nb]);
        stage = stage + 1 == STAGES ? 0 : stage + 1;
        fill = fill + 1 == STAGES ? 0 : fill + 1;
    }
    // the wavefronts' tiles meet in LDS (every wavefront's ring has been read: its own MFMAs needed the data)
    __syncthreads();
    Acc* partial = reinterpret_cast<Acc*>(skinny_lds);     // [wave][tile][lane]
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) partial[(wave * MB * NB + mb * NB + nb) * 64 + lane] = acc[mb][nb];
    __syncthreads();
    // accumulator: lane -> row of x (m) lane % 16; value v -> column n0 + 4 * (lane / 16) + v; wavefront t adds up tile t, t + 4, ..
    Out* cb = c + oc;
    const bool vector_ok = p.c_rs % 4 == 0 && p.N % 4 == 0 && reinterpret_cast<uintptr_t>(cb) % (4 * sizeof(Out)) == 0;
    for (int t = wave; t < MB * NB; t += kStreamWaves) {
        const int mb = t / NB, nb = t % NB;
        Acc sum = partial[t * 64 + lane];
#pragma unroll
        for (int v = 1; v < kStreamWaves; ++v) sum += partial[(v * MB * NB + t) * 64 + lane];
        const uint32_t m = mb * 16 + r, col = n0 + nb * 16 + 4 * kc;
        if (m >= p.M) continue;
        Out out[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (std::is_same_v<T, int8_t>) out[e] = sum[e];
            else out[e] = narrow_result<T>(sum[e]);
        }
        Out* dst = cb + static_cast<int64_t>(m) * p.c_rs + col;
        if (vector_ok) {
            if (col < p.N) {
                using Quad = std::conditional_t<sizeof(Out) == 2, uint2, uint4>;
                Quad bits;
                __builtin_memcpy(&bits, out, sizeof(Quad));
                *reinterpret_cast<Quad*>(dst) = bits;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < p.N) dst[e] = out[e];
        }
    }
#endif
}

template <class T, int MB, int NB>
static int launch_stream(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    auto kernel = gemm_skinny_stream_kernel<T, MB, NB>;
    constexpr size_t lds = kStreamWaves * kStreamBytesPerWave;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds, configured)) return rc;
    const uint32_t windows = p.K / kBKof<T>, per_wave = (windows + kStreamWaves - 1) / kStreamWaves;
    hipLaunchKernelGGL(kernel, dim3((p.N + 16 * NB - 1) / (16 * NB), p.batches), dim3(64 * kStreamWaves), lds, stream, static_cast<const T*>(a), static_cast<const T*>(b),
                       static_cast<typename SkinnyTypes<T>::Out*>(c), p, per_wave);
    return launch_status("gemm_skinny_stream_kernel");
}

template <class T>
int run_skinny(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    if (p.M == 0 || p.M > 64 || p.N == 0 || p.K == 0 || p.batches == 0 || p.batches > 65535 || p.row_bias || p.c_group) return TANNIC_UNSUPPORTED_DTYPE;
    // both operands K-contiguous; 16-byte chunks along K
    if (p.a_cs != 1 || p.b_rs != 1) return TANNIC_UNSUPPORTED_DTYPE;
    auto mult8 = [](int64_t v) { return v % kChunkOf<T> == 0; };   // whole 16-byte chunks
    if (!mult8(p.K) || !mult8(p.a_rs) || !mult8(p.b_cs)) return TANNIC_UNSUPPORTED_DTYPE;
    if (reinterpret_cast<uintptr_t>(a) % 16 || reinterpret_cast<uintptr_t>(b) % 16) return TANNIC_UNSUPPORTED_DTYPE;
    for (int d = 0; d < p.batch_rank; ++d)
        if (!mult8(p.a_bs[d]) || !mult8(p.b_bs[d])) return TANNIC_UNSUPPORTED_DTYPE;
    // whole windows of 64 and rows that do not overlap: the streaming kernel (offsets inside a block are 32-bit byte counts)
    if (p.K % kBKof<T> == 0 && p.a_rs >= static_cast<int64_t>(p.K) && p.b_cs >= static_cast<int64_t>(p.K) && p.a_rs < (1 << 22) && p.b_cs < (1 << 22)) {
        // Many small products under a short K (the scores of attention while decoding: one row against [4096, 128] per head):
        // a block's four wavefronts share K, two windows here, and a block moves 4 KB - the tiles do better (fp16, 256
        // heads: 73 against 173 us; 1024 x [512, 64]: 22 against 83; fp32 from 128 heads on: 64 against 95).  A single
        // product stays (one row against [32000, 256]: 7.5 against 13.7 us).
        if (sizeof(T) == 2 ? (p.batches >= 8 && p.K <= 512) : (p.batches >= 128 && p.K <= 128)) return TANNIC_UNSUPPORTED_DTYPE;
        // two column blocks per wavefront (half as many workgroups, x read half as often) while every compute unit still gets one
        const bool two = static_cast<uint64_t>((p.N + 31) / 32) * p.batches >= 400;
        if (p.M <= 16) return two ? launch_stream<T, 1, 2>(p, a, b, c, stream) : launch_stream<T, 1, 1>(p, a, b, c, stream);
        if (p.M <= 32) return two ? launch_stream<T, 2, 2>(p, a, b, c, stream) : launch_stream<T, 2, 1>(p, a, b, c, stream);
        // (fp32 stops here: with more row blocks its MFMAs, a sixteenth as fast, take longer than W takes to arrive; int8
        // beyond 32 rows has its tiles)
        if constexpr (sizeof(T) != 2) {
            return TANNIC_UNSUPPORTED_DTYPE;
        } else {
            // Up to 64 rows: every wavefront still brings its own windows of x, three or four 16-row blocks next to one of W, so
            // x comes out of the L2s N / 16 times.  That beats the tiles that share K while W is small (bf16, 64 rows, N x K =
            // 4096 x 4096: 10.0 against 14.1 us; 1024 x 4096: 7.5 against 12.1) and loses to them beyond (14336 x 4096: 33 against
            // 24 us).
            // (One product at a time: the many small products of an attention head - 64 x 64 x 64, a thousand of them - have one
            // window of K for four wavefronts and take 28 us here against 8 on tiles.)
            if (p.batches != 1 || p.K < 256 || static_cast<uint64_t>(p.N) * p.K > (20u << 20)) return TANNIC_UNSUPPORTED_DTYPE;
            if (p.M <= 48) return launch_stream<T, 3, 1>(p, a, b, c, stream);
            return launch_stream<T, 4, 1>(p, a, b, c, stream);
        }
    }
    if constexpr (sizeof(T) != 2) {
        return TANNIC_UNSUPPORTED_DTYPE;   // the kernel for other K is written for 16-bit fragments
    } else {
        if (p.M > 32) return TANNIC_UNSUPPORTED_DTYPE;
        // K is split evenly over the wavefronts, in whole steps of 32
        const uint32_t steps = (p.K + 31) / 32, per_wave = (steps + kSkinnyWaves - 1) / kSkinnyWaves;
        const uint32_t k_per_wave = per_wave * 32;
        // A single row costs almost nothing to load next to W; with more rows, two column blocks per wavefront halve
        // what x costs, as long as there are still blocks for every compute unit.
        const bool pairs = p.M > 4 && static_cast<uint64_t>((p.N + 31) / 32) * p.batches >= 224;
        const uint32_t blocks = pairs ? (p.N + 31) / 32 : (p.N + 15) / 16;
        const dim3 grid(blocks, p.batches), block(64 * kSkinnyWaves);
        const T* pa = static_cast<const T*>(a);
        const T* pb = static_cast<const T*>(b);
        T* pc = static_cast<T*>(c);
        if (p.M <= 16) {
            if (pairs) hipLaunchKernelGGL((gemm_skinny_kernel<T, 1, 2>), grid, block, 0, stream, pa, pb, pc, p, k_per_wave);
            else hipLaunchKernelGGL((gemm_skinny_kernel<T, 1, 1>), grid, block, 0, stream, pa, pb, pc, p, k_per_wave);
        } else {
            if (pairs) hipLaunchKernelGGL((gemm_skinny_kernel<T, 2, 2>), grid, block, 0, stream, pa, pb, pc, p, k_per_wave);
            else hipLaunchKernelGGL((gemm_skinny_kernel<T, 2, 1>), grid, block, 0, stream, pa, pb, pc, p, k_per_wave);
        }
        return launch_status("gemm_skinny_kernel");
    }
}

int gemm_skinny_f32(const GemmProblem& p, const float* a, const float* b, float* c, hipStream_t stream) { return run_skinny<float>(p, a, b, c, stream); }

// int8 x int8 -> int32, at most 32 rows over whole windows of 128 k: W goes by once where the 128-row tiles walk it at their own pace
int gemm_skinny_int8(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) { return run_skinny<int8_t>(p, a, b, c, stream); }

int gemm_skinny_16bit(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_skinny<f16>(p, a, b, c, stream);
    if (dtype == TANNIC_BFLOAT16) return run_skinny<bf16>(p, a, b, c, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
