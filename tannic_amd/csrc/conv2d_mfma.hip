// Implicit-GEMM conv2d on MFMA for gfx950.
//
// The convolution is the product  Y[co, p] = sum_k W[co, k] * X~[k, p]  with
//   p = (n, oh, ow) running over all output pixels, k = (ci, kh, kw) in the
//   weights' own memory order, and X~ the im2col matrix, which is never
//   materialised: a block of 256 threads owns a tile of BCO output channels x
//   128 pixels, walks K in steps of 32 and gathers its 128 x 32 slice of X~
//   straight from the NCHW signal into LDS (zero where a tap falls into the
//   padding), next to the BCO x 32 slice of the weights.  Lanes of a wavefront
//   gather consecutive pixels of one k, i.e. consecutive (stride 1) or evenly
//   strided addresses.  Both tiles sit in LDS as [row][32 k] with their four
//   16-byte chunks swizzled, exactly the operand layout of
//   v_mfma_f32_32x32x16_{f16,bf16}; accumulation is fp32, the bias seeds the
//   accumulator (src/cpu/conv2d.cpp:90) and the result is rounded once.
//   The MFMA's row operand is the weight tile and its column operand the pixel
//   tile, so that a lane ends up with one pixel column: the 32 lanes of a half
//   wavefront store 32 consecutive pixels of one output channel.
//
// fp32 signals take conv2d_gather32.hip, the same scheme on v_mfma_f32_32x32x2f32.
#include "conv_common.hpp"

namespace th {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

template <class T> struct ConvMfma;
template <> struct ConvMfma<f16> {
    __device__ static inline float16v run(uint4v a, uint4v b, float16v c) {
        half8 x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, c, 0, 0, 0);
    }
};
template <> struct ConvMfma<bf16> {
    __device__ static inline float16v run(uint4v a, uint4v b, float16v c) {
        bfloat8 x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, c, 0, 0, 0);
    }
};

constexpr int kConvThreads = 256;
constexpr int kConvBK = 32;   // k values per step
constexpr int kConvBP = 128;  // pixels per block
constexpr uint32_t kMaxTableK = 6144;  // entries of the k -> tap table kept in LDS

// One entry per k: element offset of tap (ci, kh, kw) relative to the window's
// origin, and (kh, kw) for the padding test.  k >= K gets kh = 0xFFFF, which
// fails every range test and so contributes zeros.
struct Tap {
    int32_t offset;
    uint16_t kh, kw;
};

// [rows][32] 16-bit tile, 64-byte rows, four 16-byte chunks per row.  Sixteen
// consecutive rows of one logical chunk fall into the sixteen 16-byte slots of
// the 256-byte LDS bank window.
__device__ inline uint32_t conv_tile_offset(uint32_t row, uint32_t chunk) { return row * kConvBK + ((chunk ^ ((row >> 2) & 3u)) * 8u); }

template <class T, int BCO, bool W_VECTOR>
__global__ __launch_bounds__(kConvThreads) void conv2d_mfma16_kernel(const T* x, const T* w, const T* bias, T* y, ConvProblem p,
                                                                      uint32_t K, uint32_t pixels, uint32_t co_tiles) {
    constexpr int BP = kConvBP, BK = kConvBK;
    constexpr int WCO = BCO / 2, WP = BP / 2;  // 2 x 2 wavefronts
    constexpr int TM = WCO / 32, TN = WP / 32;
    constexpr int W_CHUNKS = BCO * BK / 8 / kConvThreads;  // 16-byte weight chunks per thread and step
    extern __shared__ __align__(16) unsigned char conv_lds[];
    T* sW = reinterpret_cast<T*>(conv_lds);              // 2 x BCO x 32
    T* sX = sW + 2 * BCO * BK;                           // 2 x 128 x 32
    Tap* taps = reinterpret_cast<Tap*>(sX + 2 * BP * BK);
    const uint32_t ksteps = (K + BK - 1) / BK;

    // k -> tap table
    const uint32_t khw = p.KH * p.KW;
    for (uint32_t k = threadIdx.x; k < ksteps * BK; k += kConvThreads) {
        Tap t;
        if (k < K) {
            const uint32_t ci = k / khw, r = k % khw, kh = r / p.KW, kw = r % p.KW;
            t.offset = static_cast<int32_t>(ci * p.xs[1] + kh * p.xs[2] + kw * p.xs[3]);
            t.kh = static_cast<uint16_t>(kh);
            t.kw = static_cast<uint16_t>(kw);
        } else {
            t.offset = 0;
            t.kh = 0xFFFF;
            t.kw = 0;
        }
        taps[k] = t;
    }

    const uint32_t co0 = (blockIdx.x % co_tiles) * BCO;
    const uint32_t p0 = (blockIdx.x / co_tiles) * BP;

    // this thread's pixel (fixed for the whole kernel) and its half of each k step
    const uint32_t pc = threadIdx.x % BP;
    const uint32_t kq = __builtin_amdgcn_readfirstlane(threadIdx.x / BP);  // 0 or 1: k range [16*kq, 16*kq + 16)
    const uint32_t P = p0 + pc;
    const bool pixel_live = P < pixels;
    const uint32_t hw_out = p.HO * p.WO;
    const uint32_t n_img = pixel_live ? P / hw_out : 0;
    const uint32_t prem = pixel_live ? P % hw_out : 0;
    const int32_t base_h = static_cast<int32_t>((prem / p.WO) * p.stride_h) - static_cast<int32_t>(p.pad_h);
    const int32_t base_w = static_cast<int32_t>((prem % p.WO) * p.stride_w) - static_cast<int32_t>(p.pad_w);
    const T* xp = x + static_cast<int64_t>(n_img) * p.xs[0] + static_cast<int64_t>(base_h) * p.xs[2] + static_cast<int64_t>(base_w) * p.xs[3];
    const uint32_t H = pixel_live ? p.H : 0;  // a dead pixel fails every range test

    // weights: thread -> (row, chunk) of the BCO x 32 tile
    uint32_t w_row[W_CHUNKS], w_chunk[W_CHUNKS];
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
        const uint32_t id = threadIdx.x + kConvThreads * i;
        w_row[i] = id / 4;
        w_chunk[i] = id % 4;
    }

    // Values of the coming step.  Whether a value counts (tap inside the image,
    // k inside K) is recorded in bit masks and applied only when the registers
    // are written to LDS, so that nothing waits for the loads before the MFMAs
    // of the current step have been issued.
    uint16_t gx[16];
    uint32_t gx_live = 0;
    uint4v gw[W_CHUNKS];
    uint32_t gw_live = 0;     // one bit per weight element: chunk i, element q -> bit 8*i + q

    auto fetch = [&](uint32_t step) {
        const uint32_t kbase = step * BK + kq * 16;
        gx_live = 0;
        gw_live = 0;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const Tap t = taps[kbase + j];
            const uint32_t ih = static_cast<uint32_t>(base_h + static_cast<int32_t>(t.kh));
            const uint32_t iw = static_cast<uint32_t>(base_w + static_cast<int32_t>(t.kw));
            const bool ok = t.kh != 0xFFFF && ih < H && iw < p.W;  // unsigned: negative coordinates are huge
            // a tap outside the image reads the tensor's first element (valid memory) and is zeroed
            gx[j] = *reinterpret_cast<const uint16_t*>(ok ? xp + t.offset : x);
            gx_live |= static_cast<uint32_t>(ok) << j;
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const uint32_t co = co0 + w_row[i];
            const uint32_t k = step * BK + w_chunk[i] * 8;
            const uint32_t sco = co < p.O ? co : p.O - 1;
            const T* src = w + static_cast<int64_t>(sco) * K;
            if constexpr (W_VECTOR) {
                gw[i] = *reinterpret_cast<const uint4v*>(src + (k < K ? k : 0));
                gw_live |= (k < K ? 0xFFu : 0u) << (8 * i);
            } else {
                uint16_t e[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    e[q] = *reinterpret_cast<const uint16_t*>(src + (k + q < K ? k + q : 0));
                    gw_live |= static_cast<uint32_t>(k + q < K) << (8 * i + q);
                }
                __builtin_memcpy(&gw[i], e, 16);
            }
        }
    };
    auto commit = [&](uint32_t buf) {
        T* xt = sX + buf * BP * BK;
        T* wt = sW + buf * BCO * BK;
        uint16_t masked[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) masked[j] = (gx_live >> j) & 1u ? gx[j] : uint16_t(0);
        uint4v lo, hi;
        __builtin_memcpy(&lo, &masked[0], 16);
        __builtin_memcpy(&hi, &masked[8], 16);
        *reinterpret_cast<uint4v*>(xt + conv_tile_offset(pc, kq * 2)) = lo;
        *reinterpret_cast<uint4v*>(xt + conv_tile_offset(pc, kq * 2 + 1)) = hi;
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            uint16_t e[8];
            __builtin_memcpy(e, &gw[i], 16);
#pragma unroll
            for (int q = 0; q < 8; ++q) e[q] = (gw_live >> (8 * i + q)) & 1u ? e[q] : uint16_t(0);
            uint4v v;
            __builtin_memcpy(&v, e, 16);
            *reinterpret_cast<uint4v*>(wt + conv_tile_offset(w_row[i], w_chunk[i])) = v;
        }
    };

    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int wco = (wave / 2) * WCO, wp = (wave % 2) * WP;
    const uint32_t frag_row = lane % 32, frag_chunk = lane / 32;

    // accumulators start from the bias of their output channel: value v of a
    // 32x32 tile sits in row 8*(v/4) + 4*(lane/32) + v%4
    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t co = co0 + wco + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
            const float b = (p.has_bias && co < p.O) ? static_cast<float>(widen(bias[static_cast<int64_t>(co) * p.bs])) : 0.0f;
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j][v] = b;
        }

    __syncthreads();  // tap table complete
    fetch(0);
    commit(0);
    __syncthreads();

    for (uint32_t s = 0; s < ksteps; ++s) {
        const uint32_t cur = s & 1;
        if (s + 1 < ksteps) fetch(s + 1);
        const T* wt = sW + cur * BCO * BK;
        const T* xt = sX + cur * BP * BK;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            uint4v fw[TM], fx[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fw[i] = *reinterpret_cast<const uint4v*>(wt + conv_tile_offset(wco + i * 32 + frag_row, ks * 2 + frag_chunk));
#pragma unroll
            for (int j = 0; j < TN; ++j) fx[j] = *reinterpret_cast<const uint4v*>(xt + conv_tile_offset(wp + j * 32 + frag_row, ks * 2 + frag_chunk));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = ConvMfma<T>::run(fw[i], fx[j], acc[i][j]);
        }
        if (s + 1 < ksteps) commit(cur ^ 1);
        __syncthreads();
    }

    // store: the lane's pixel column, rows = output channels
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t Pj = p0 + wp + j * 32 + lane % 32;
        if (Pj >= pixels) continue;
        const uint32_t n = Pj / hw_out, r = Pj % hw_out;
        T* yp = y + static_cast<int64_t>(n) * p.ys[0] + static_cast<int64_t>(r / p.WO) * p.ys[2] + static_cast<int64_t>(r % p.WO) * p.ys[3];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t co = co0 + wco + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
                if (co < p.O) yp[static_cast<int64_t>(co) * p.ys[1]] = narrow<T>(acc[i][j][v]);
            }
    }
}

template <class T, int BCO, bool WV>
int launch_conv16(const ConvProblem& p, uint32_t K, uint32_t pixels, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    const uint32_t ksteps = (K + kConvBK - 1) / kConvBK;
    const size_t lds = sizeof(T) * 2 * (BCO + kConvBP) * kConvBK + sizeof(Tap) * ksteps * kConvBK;
    const uint32_t co_tiles = (p.O + BCO - 1) / BCO, p_tiles = (pixels + kConvBP - 1) / kConvBP;
    auto kernel = conv2d_mfma16_kernel<T, BCO, WV>;
    static std::atomic<uint64_t> configured{0};
    const size_t most = sizeof(T) * 2 * (BCO + kConvBP) * kConvBK + sizeof(Tap) * kMaxTableK;
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), most, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(co_tiles * p_tiles), dim3(kConvThreads), lds, stream, static_cast<const T*>(x), static_cast<const T*>(w),
                       static_cast<const T*>(bias), static_cast<T*>(y), p, K, pixels, co_tiles);
    return launch_status("conv2d_mfma16_kernel");
}

template <class T>
int run_conv16(const ConvProblem& p, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    const uint64_t K64 = static_cast<uint64_t>(p.C) * p.KH * p.KW;
    const uint64_t pixels64 = static_cast<uint64_t>(p.N) * p.HO * p.WO;
    if (K64 == 0 || pixels64 == 0 || p.O == 0) return TANNIC_SUCCESS;
    // kernel weights must be contiguous OIHW (k runs through memory in order)
    if (p.ws[3] != 1 || p.ws[2] != p.KW || p.ws[1] != static_cast<int64_t>(p.KH) * p.KW || p.ws[0] != static_cast<int64_t>(K64)) return TANNIC_UNSUPPORTED_DTYPE;
    if (K64 + kConvBK > kMaxTableK || pixels64 >= (1ull << 31) || p.KH >= 0xFFFF || p.KW >= 0xFFFF) return TANNIC_UNSUPPORTED_DTYPE;
    // tap offsets are kept as 32-bit element offsets
    const uint64_t reach = static_cast<uint64_t>(p.C) * static_cast<uint64_t>(p.xs[1] < 0 ? -p.xs[1] : p.xs[1]) +
                           static_cast<uint64_t>(p.KH) * static_cast<uint64_t>(p.xs[2] < 0 ? -p.xs[2] : p.xs[2]) +
                           static_cast<uint64_t>(p.KW) * static_cast<uint64_t>(p.xs[3] < 0 ? -p.xs[3] : p.xs[3]);
    if (reach >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    const uint32_t K = static_cast<uint32_t>(K64), pixels = static_cast<uint32_t>(pixels64);
    const bool wv = K % 8 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
    if (p.O > 64) return wv ? launch_conv16<T, 128, true>(p, K, pixels, x, w, bias, y, stream) : launch_conv16<T, 128, false>(p, K, pixels, x, w, bias, y, stream);
    return wv ? launch_conv16<T, 64, true>(p, K, pixels, x, w, bias, y, stream) : launch_conv16<T, 64, false>(p, K, pixels, x, w, bias, y, stream);
}

int conv2d_mfma(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_conv16<f16>(p, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_conv16<bf16>(p, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
