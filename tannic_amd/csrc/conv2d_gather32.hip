// Implicit-GEMM conv2d in fp32 on v_mfma_f32_32x32x2f32.
//
// The same product as conv2d_mfma.hip,  Y[co, p] = sum_k W[co, k] * X~[k, p]  with p over all output pixels and
// k = (ci, kh, kw) in the weights' own memory order, with the im2col matrix X~ never materialised: a block of 256
// threads owns BCO output channels x 128 pixels, walks K in steps of 16 and gathers its 128 x 16 slice of X~ from the
// NCHW signal into LDS (zero where a tap falls into the padding), next to the BCO x 16 slice of the weights.  A thread
// gathers eight k values of one pixel, so a wavefront reads consecutive (stride 1) or evenly strided addresses.
// The fp32 matrix instruction is sixteen times slower than the 16-bit one, which is what makes this the right
// structure here: the gathers hide behind the MFMAs, and the separate unfolding pass (a write and a read of the whole
// im2col matrix, as long as the product itself) disappears.
// LDS tiles are [row][16 k] floats, 64-byte rows whose four 16-byte chunks are swizzled by (row >> 2) & 3: sixteen
// consecutive rows of one chunk cover all banks.  A lane reads 16 bytes (k = 4 c .. 4 c + 3 of its row; lanes 0-31
// chunk c, lanes 32-63 chunk c + 1) and feeds element e of them to the e-th of four MFMAs: each MFMA multiplies two k
// values per row, and since both operands are read the same way every k meets its partner.
// Accumulation is fp32 from the bias (src/cpu/conv2d.cpp:90); a lane ends up with one pixel column, so the 32 lanes
// of a half wavefront store 32 consecutive pixels of one output channel.
#include "conv_common.hpp"

namespace th {

typedef float float16g __attribute__((ext_vector_type(16)));
typedef float float4g __attribute__((ext_vector_type(4)));

constexpr int kG32Threads = 256;
constexpr int kG32BK = 16;    // k values per step
constexpr int kG32BP = 128;   // pixels per block
constexpr uint32_t kG32MaxTableK = 6144;   // entries of the k -> tap table kept in LDS

// One entry per k: element offset of tap (ci, kh, kw) from the window's origin, and (kh, kw) for the padding test.
// k >= K gets kh = 0xFFFF, which fails every range test and so contributes zeros.
struct Tap32 {
    int32_t offset;
    uint16_t kh, kw;
};

template <int N, class F, int I = 0>
__device__ inline void g32_static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        g32_static_for<N, F, I + 1>(static_cast<F&&>(f));
    }
}

__device__ inline uint32_t g32_offset(uint32_t row, uint32_t chunk) { return row * kG32BK + ((chunk ^ ((row >> 2) & 3u)) * 4u); }

// MAPW: 32-bit words of the per-pixel map "tap (kh, kw) lies inside the image" (KH * KW <= 31: one, <= 63: two; the last
// bit stays clear and stands for "no such k").  0: larger kernels, every tap is range-tested as it is gathered.
template <int BCO, bool W_VECTOR, int MAPW>
__global__ __launch_bounds__(kG32Threads) void conv2d_gather32_kernel(const float* x, const float* w, const float* bias, float* y, ConvProblem p,
                                                                       uint32_t K, uint32_t pixels, uint32_t co_tiles) {
    constexpr int BP = kG32BP, BK = kG32BK;
    constexpr int WCO = BCO / 2, WP = BP / 2;   // 2 x 2 wavefronts
    constexpr int TM = WCO / 32, TN = WP / 32;
    constexpr int W_CHUNKS = BCO * BK / 4 / kG32Threads;   // 16-byte weight chunks per thread and step
    extern __shared__ __align__(16) unsigned char g32_lds[];
    float* sW = reinterpret_cast<float*>(g32_lds);   // 2 x BCO x 16
    float* sX = sW + 2 * BCO * BK;                   // 2 x 128 x 16
    Tap32* taps = reinterpret_cast<Tap32*>(sX + 2 * BP * BK);
    const uint32_t ksteps = (K + BK - 1) / BK;

    const uint32_t khw = p.KH * p.KW;
    for (uint32_t k = threadIdx.x; k < ksteps * BK; k += kG32Threads) {
        Tap32 t;
        if (k < K) {
            const uint32_t ci = k / khw, r = k % khw, kh = r / p.KW, kw = r % p.KW;
            t.offset = static_cast<int32_t>(ci * p.xs[1] + kh * p.xs[2] + kw * p.xs[3]);
            t.kh = static_cast<uint16_t>(MAPW ? r : kh);     // with a map: the tap's bit
            t.kw = static_cast<uint16_t>(kw);
        } else {
            t.offset = 0;
            t.kh = MAPW ? 32 * MAPW - 1 : 0xFFFF;
            t.kw = 0;
        }
        taps[k] = t;
    }

    const uint32_t co0 = (blockIdx.x % co_tiles) * BCO;
    const uint32_t p0 = (blockIdx.x / co_tiles) * BP;

    // this thread's pixel (fixed for the whole kernel) and its half of each k step
    const uint32_t pc = threadIdx.x % BP;
    const uint32_t kq = __builtin_amdgcn_readfirstlane(threadIdx.x / BP);   // k range [8 kq, 8 kq + 8) of the step
    const uint32_t P = p0 + pc;
    const bool pixel_live = P < pixels;
    const uint32_t hw_out = p.HO * p.WO;
    const uint32_t n_img = pixel_live ? P / hw_out : 0;
    const uint32_t prem = pixel_live ? P % hw_out : 0;
    const int32_t base_h = static_cast<int32_t>((prem / p.WO) * p.stride_h) - static_cast<int32_t>(p.pad_h);
    const int32_t base_w = static_cast<int32_t>((prem % p.WO) * p.stride_w) - static_cast<int32_t>(p.pad_w);
    const float* xp = x + static_cast<int64_t>(n_img) * p.xs[0] + static_cast<int64_t>(base_h) * p.xs[2] + static_cast<int64_t>(base_w) * p.xs[3];
    const uint32_t H = pixel_live ? p.H : 0;   // a dead pixel fails every range test
    // which taps of this pixel's window lie inside the image, and an offset that is always safe to read (the image's
    // first element) for those that do not
    uint64_t inside = 0;
    const int32_t safe = -static_cast<int32_t>(static_cast<int64_t>(base_h) * p.xs[2] + static_cast<int64_t>(base_w) * p.xs[3]);
    if constexpr (MAPW > 0) {
        // columns first (one bit per kw), then that pattern once per row of the window that lies inside
        uint32_t columns = 0;
        for (uint32_t kw = 0; kw < p.KW; ++kw) columns |= static_cast<uint32_t>(static_cast<uint32_t>(base_w + static_cast<int32_t>(kw)) < p.W) << kw;
        for (uint32_t kh = 0; kh < p.KH; ++kh)
            if (static_cast<uint32_t>(base_h + static_cast<int32_t>(kh)) < H) inside |= static_cast<uint64_t>(columns) << (kh * p.KW);
    }
    const uint32_t inside_low = static_cast<uint32_t>(inside);

    uint32_t w_row[W_CHUNKS], w_chunk[W_CHUNKS];
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
        const uint32_t id = threadIdx.x + kG32Threads * i;
        w_row[i] = id / 4;
        w_chunk[i] = id % 4;
    }

    // Values on their way, two sets: the set of step s + 1 was asked for during step s - 1 and goes to LDS during step s,
    // while the other set is asked for step s + 2.  Whether a value counts is recorded in bit masks and applied when the
    // registers are written to LDS.  All of this is issued BETWEEN the MFMAs of a step (see the loop), so that a
    // wavefront's address arithmetic, loads and LDS writes run while its own MFMAs occupy the matrix pipe.
    struct Fetched {
        float gx[8];
        uint32_t gx_live;
        float gw[W_CHUNKS][4];
        uint32_t gw_live;   // one bit per weight element: chunk i, element q -> bit 4 i + q
    };
    Fetched sets[2];
    Tap32 tap_of[8];       // the eight table entries of the step being asked for

    auto read_taps = [&](uint32_t step) {
        const uint32_t kbase = step * BK + kq * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) tap_of[j] = taps[kbase + j];
    };
    auto fetch_x = [&](Fetched& f, int j) {
        const Tap32 t = tap_of[j];
        if (j == 0) f.gx_live = 0;
        if constexpr (MAPW > 0) {
            // all ones when the tap's bit of the map is set; a tap outside reads the image's first element and is zeroed later
            const uint32_t all = MAPW == 1 ? static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int32_t>(inside_low), t.kh, 1u))
                                           : 0u - static_cast<uint32_t>((inside >> t.kh) & 1u);
            const int32_t offset = static_cast<int32_t>((static_cast<uint32_t>(t.offset) & all) | (static_cast<uint32_t>(safe) & ~all));
            f.gx[j] = xp[offset];
            f.gx_live |= all & (1u << j);
        } else {
            const uint32_t ih = static_cast<uint32_t>(base_h + static_cast<int32_t>(t.kh));
            const uint32_t iw = static_cast<uint32_t>(base_w + static_cast<int32_t>(t.kw));
            const bool ok = t.kh != 0xFFFF && ih < H && iw < p.W;   // unsigned: negative coordinates are huge
            // a tap outside the image reads the tensor's first element (valid memory) and is zeroed later
            f.gx[j] = *(ok ? xp + t.offset : x);
            f.gx_live |= static_cast<uint32_t>(ok) << j;
        }
    };
    auto fetch_w = [&](Fetched& f, uint32_t step, int i) {
        const uint32_t co = co0 + w_row[i];
        const uint32_t k = step * BK + w_chunk[i] * 4;
        const uint32_t sco = co < p.O ? co : p.O - 1;
        const float* src = w + static_cast<int64_t>(sco) * K;
        if (i == 0) f.gw_live = 0;
        if constexpr (W_VECTOR) {
            const float4g v = *reinterpret_cast<const float4g*>(src + (k < K ? k : 0));
            __builtin_memcpy(f.gw[i], &v, 16);
            f.gw_live |= (k < K ? 0xFu : 0u) << (4 * i);
        } else if (k + 4 <= K) {
            // rows of the weights start at any multiple of four bytes: one load of sixteen bytes all the same, which the
            // compiler splits where the hardware would not take it
            typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
            const float4u v = *reinterpret_cast<const float4u*>(src + k);
            __builtin_memcpy(f.gw[i], &v, 16);
            f.gw_live |= 0xFu << (4 * i);
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f.gw[i][q] = src[k + q < K ? k + q : 0];
                f.gw_live |= static_cast<uint32_t>(k + q < K) << (4 * i + q);
            }
        }
    };
    auto commit_x = [&](const Fetched& f, uint32_t buf) {
        float* xt = sX + buf * BP * BK;
        float masked[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t all = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int32_t>(f.gx_live), j, 1u));
            masked[j] = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, f.gx[j]) & all);
        }
        float4g lo, hi;
        __builtin_memcpy(&lo, &masked[0], 16);
        __builtin_memcpy(&hi, &masked[4], 16);
        *reinterpret_cast<float4g*>(xt + g32_offset(pc, kq * 2)) = lo;
        *reinterpret_cast<float4g*>(xt + g32_offset(pc, kq * 2 + 1)) = hi;
    };
    auto commit_w = [&](const Fetched& f, uint32_t buf, int i) {
        float* wt = sW + buf * BCO * BK;
        float e[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) e[q] = (f.gw_live >> (4 * i + q)) & 1u ? f.gw[i][q] : 0.0f;
        float4g v;
        __builtin_memcpy(&v, e, 16);
        *reinterpret_cast<float4g*>(wt + g32_offset(w_row[i], w_chunk[i])) = v;
    };
    auto fetch_all = [&](Fetched& f, uint32_t step) {
        read_taps(step);
#pragma unroll
        for (int j = 0; j < 8; ++j) fetch_x(f, j);
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) fetch_w(f, step, i);
    };
    auto commit_all = [&](const Fetched& f, uint32_t buf) {
        commit_x(f, buf);
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) commit_w(f, buf, i);
    };

    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int wco = (wave / 2) * WCO, wp = (wave % 2) * WP;
    const uint32_t frag_row = lane % 32, frag_chunk = lane / 32;

    // accumulators start from the bias of their output channel: value v of a 32 x 32 tile sits in row
    // 8 (v / 4) + 4 (lane / 32) + v % 4
    float16g acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t co = co0 + wco + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
            const float b = (p.has_bias && co < p.O) ? bias[static_cast<int64_t>(co) * p.bs] : 0.0f;
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j][v] = b;
        }

    __syncthreads();   // tap table complete
    const uint32_t last = ksteps - 1;
    fetch_all(sets[0], 0);
    commit_all(sets[0], 0);
    fetch_all(sets[1], last < 1 ? last : 1);
    __syncthreads();

    // One step: the MFMAs of LDS buffer PAR.  Between them: the fragments of the second half of the step are read, set
    // PAR is asked for step + 2 (past the end: the last step once more, never used), and set 1 - PAR (step + 1) goes
    // to the other buffer.  Every step issues the same operations, so that the waits for the loads count them exactly.
    constexpr int PER_E = TM * TN, MFMAS = (BK / 8) * 4 * PER_E;
    auto one_step = [&](auto par_, uint32_t step) {
        constexpr int PAR = decltype(par_)::value;
        const float* wt = sW + PAR * BCO * BK;
        const float* xt = sX + PAR * BP * BK;
        const uint32_t ask = step + 2 < ksteps ? step + 2 : last;
        float4g fw[2][TM], fx[2][TN];
        auto read_fragments = [&](int ks) {
#pragma unroll
            for (int i = 0; i < TM; ++i) fw[ks][i] = *reinterpret_cast<const float4g*>(wt + g32_offset(wco + i * 32 + frag_row, ks * 2 + frag_chunk));
#pragma unroll
            for (int j = 0; j < TN; ++j) fx[ks][j] = *reinterpret_cast<const float4g*>(xt + g32_offset(wp + j * 32 + frag_row, ks * 2 + frag_chunk));
        };
        read_fragments(0);
        read_taps(ask);
        __builtin_amdgcn_sched_barrier(0);
        g32_static_for<MFMAS>([&](auto m_) {
            constexpr int m = decltype(m_)::value;
            constexpr int ks = m / (4 * PER_E), e = (m / PER_E) % 4, i = (m % PER_E) / TN, j = m % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fw[ks][i][e], fx[ks][j][e], acc[i][j], 0, 0, 0);
            // the other work of the step, spread over its MFMAs: the loads of step + 2 first, the stores of step + 1
            // last (their loads went out early in the step before: they have had nearly two steps to arrive)
            constexpr int PIECES = 1 + 8 + W_CHUNKS + 1 + W_CHUNKS;    // fragments, taps, weights, commit x, commit w..
            constexpr int first = m * PIECES / MFMAS, end = (m + 1) * PIECES / MFMAS;
            g32_static_for<end - first>([&](auto o_) {
                constexpr int o = first + decltype(o_)::value;
                if constexpr (o == 0) read_fragments(1);
                else if constexpr (o < 1 + 8) fetch_x(sets[PAR], o - 1);
                else if constexpr (o < 1 + 8 + W_CHUNKS) fetch_w(sets[PAR], ask, o - 1 - 8);
                else if constexpr (o == 1 + 8 + W_CHUNKS) commit_x(sets[1 - PAR], 1 - PAR);
                else commit_w(sets[1 - PAR], 1 - PAR, o - 2 - 8 - W_CHUNKS);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
    };
    uint32_t step = 0;
    for (; step + 1 < ksteps; step += 2) {
        one_step(std::integral_constant<int, 0>{}, step);
        one_step(std::integral_constant<int, 1>{}, step + 1);
    }
    if (step < ksteps) one_step(std::integral_constant<int, 0>{}, step);

    // store: the lane's pixel column, rows = output channels
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t Pj = p0 + wp + j * 32 + lane % 32;
        if (Pj >= pixels) continue;
        const uint32_t n = Pj / hw_out, r = Pj % hw_out;
        float* yp = y + static_cast<int64_t>(n) * p.ys[0] + static_cast<int64_t>(r / p.WO) * p.ys[2] + static_cast<int64_t>(r % p.WO) * p.ys[3];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t co = co0 + wco + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
                if (co < p.O) yp[static_cast<int64_t>(co) * p.ys[1]] = acc[i][j][v];
            }
    }
}

template <int BCO, bool WV, int MAPW>
int launch_gather32_mapped(const ConvProblem& p, uint32_t K, uint32_t pixels, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    const uint32_t ksteps = (K + kG32BK - 1) / kG32BK;
    const size_t lds = sizeof(float) * 2 * (BCO + kG32BP) * kG32BK + sizeof(Tap32) * ksteps * kG32BK;
    const uint32_t co_tiles = (p.O + BCO - 1) / BCO, p_tiles = (pixels + kG32BP - 1) / kG32BP;
    auto kernel = conv2d_gather32_kernel<BCO, WV, MAPW>;
    static std::atomic<uint64_t> configured{0};
    const size_t most = sizeof(float) * 2 * (BCO + kG32BP) * kG32BK + sizeof(Tap32) * kG32MaxTableK;
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), most, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(co_tiles * p_tiles), dim3(kG32Threads), lds, stream, static_cast<const float*>(x), static_cast<const float*>(w),
                       static_cast<const float*>(bias), static_cast<float*>(y), p, K, pixels, co_tiles);
    return launch_status("conv2d_gather32_kernel");
}

template <int BCO, bool WV>
int launch_gather32(const ConvProblem& p, uint32_t K, uint32_t pixels, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    const uint64_t taps = static_cast<uint64_t>(p.KH) * p.KW;
    if (taps <= 31) return launch_gather32_mapped<BCO, WV, 1>(p, K, pixels, x, w, bias, y, stream);
    if (taps <= 63) return launch_gather32_mapped<BCO, WV, 2>(p, K, pixels, x, w, bias, y, stream);
    return launch_gather32_mapped<BCO, WV, 0>(p, K, pixels, x, w, bias, y, stream);
}

int conv2d_gather32(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype != TANNIC_FLOAT32) return TANNIC_UNSUPPORTED_DTYPE;
    const uint64_t K64 = static_cast<uint64_t>(p.C) * p.KH * p.KW;
    const uint64_t pixels64 = static_cast<uint64_t>(p.N) * p.HO * p.WO;
    if (K64 == 0 || pixels64 == 0 || p.O == 0) return TANNIC_SUCCESS;
    // kernel weights must be contiguous OIHW (k runs through memory in order)
    if (p.ws[3] != 1 || p.ws[2] != p.KW || p.ws[1] != static_cast<int64_t>(p.KH) * p.KW || p.ws[0] != static_cast<int64_t>(K64)) return TANNIC_UNSUPPORTED_DTYPE;
    if (K64 + kG32BK > kG32MaxTableK || pixels64 >= (1ull << 31) || p.KH >= 0xFFFF || p.KW >= 0xFFFF) return TANNIC_UNSUPPORTED_DTYPE;
    const uint64_t tiles = (pixels64 + kG32BP - 1) / kG32BP * ((p.O + 63) / 64);
    if (tiles >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    // tap offsets are kept as 32-bit element offsets
    const uint64_t reach = static_cast<uint64_t>(p.C) * static_cast<uint64_t>(p.xs[1] < 0 ? -p.xs[1] : p.xs[1]) +
                           static_cast<uint64_t>(p.KH) * static_cast<uint64_t>(p.xs[2] < 0 ? -p.xs[2] : p.xs[2]) +
                           static_cast<uint64_t>(p.KW) * static_cast<uint64_t>(p.xs[3] < 0 ? -p.xs[3] : p.xs[3]);
    if (reach >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    const uint32_t K = static_cast<uint32_t>(K64), pixels = static_cast<uint32_t>(pixels64);
    const bool wv = K % 4 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
    // 128 output channels per block only while that leaves a block for (nearly) every compute unit
    const uint64_t wide_blocks = (pixels64 + kG32BP - 1) / kG32BP * ((p.O + 127) / 128);
    if (p.O > 64 && wide_blocks >= 200) return wv ? launch_gather32<128, true>(p, K, pixels, x, w, bias, y, stream) : launch_gather32<128, false>(p, K, pixels, x, w, bias, y, stream);
    return wv ? launch_gather32<64, true>(p, K, pixels, x, w, bias, y, stream) : launch_gather32<64, false>(p, K, pixels, x, w, bias, y, stream);
}

}  // namespace th
