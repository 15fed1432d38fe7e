// conv2d with a 1x1 kernel on MFMA, 16-bit signals, up to 256 input channels, horizontal/vertical stride 1 or 2.
//
// The layer is a product  y[n] (O x pixels) = w (O x C) * x[n] (C x sampled pixels)  with a short inner dimension:
// a tiled matrix multiply spends as long filling and draining its tile as multiplying, and a strided layer would
// first need the sampled pixels gathered into a dense copy.  Here the weights never move: a multiplying wavefront
// keeps the 64 x C weights of its output channels in registers as MFMA fragments for the whole launch (C <= 256: at
// most 128 registers), and the block (256 output channels) walks over tiles of 64 pixels.
//
// A block is eight wavefronts, two on every SIMD, with different jobs, so that a wavefront held up by the memory
// pipeline does not hold up the matrix pipe:
//   * four MOVERS bring the signal in and the result out.  The C x 64 signal tile is read as 8 channels x 8 pixels
//     micro-blocks, one per thread; with stride 2 the eight pixels are the even elements of two 16-byte loads (four
//     pixels each; the two groups may sit on different rows).  A micro-block is transposed in registers and written
//     to LDS pixel-major, [64-channel panel][pixel][64 channels], 16-byte slots XOR-swizzled by the pixel number so
//     that fragment reads are bank-conflict free.  The loads of two tiles are in flight at any time (a tile's loads
//     are issued three tiles ahead of its product).  The staged result of the tile before is written out as whole
//     rows of the NCHW result, 16 bytes per lane.
//   * four MULTIPLIERS take the pixel fragments from LDS (the pixel fragment is the MFMA's first operand, so a
//     lane's accumulators are runs of four consecutive pixels of one output channel), multiply, round and stage the
//     result in LDS as [channel][pixel].
// Signal tiles and staged results have two LDS buffers each; one barrier per tile separates writers and readers.
// The weights are asked for as whole rows and regrouped into fragments through LDS.  HBM-bound: every sampled input
// row is read once per group of 256 output channels, the result written once.
#include "conv_common.hpp"

namespace th {

typedef _Float16 half8p __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8p __attribute__((ext_vector_type(8)));
typedef float float16p __attribute__((ext_vector_type(16)));
typedef unsigned int uint4p __attribute__((ext_vector_type(4)));
typedef unsigned int uint2p __attribute__((ext_vector_type(2)));

template <class T> __device__ inline float16p k1_mfma(uint4p a, uint4p b, float16p c) {
    if constexpr (std::is_same_v<T, f16>) {
        half8p x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, c, 0, 0, 0);
    } else {
        bfloat8p x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, c, 0, 0, 0);
    }
}

template <int N, class F, int I = 0>
__device__ inline void k1_static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        k1_static_for<N, F, I + 1>(static_cast<F&&>(f));
    }
}

constexpr int kK1Threads = 512;         // four multiplying and four moving wavefronts
constexpr int kK1Movers = 256;
constexpr int kK1Pixels = 64;          // pixels per tile
constexpr int kK1CoWave = 64;          // output channels per wavefront
constexpr int kK1CoBlock = 256;        // per block
constexpr int kK1Panel = 64 * 64;      // elements of one 64-channel panel of a tile
constexpr int kK1Pitch = kK1Pixels + 8;   // staged result rows, elements

struct K1Plan {
    uint32_t pixels;            // HO * WO
    uint32_t tiles, workers;    // (image, 64-pixel range) pairs; blocks per group of 256 output channels
    FastDiv div_wo, div_tiles_per_image;
};

// element offset of 16-byte slot `kc` of pixel `px` in a panel: rows of 128 bytes, slots swizzled so that both the
// fragment reads (16 consecutive pixels, one slot) and the transposing writes (8 pixel blocks x 2 channel blocks,
// odd pixel blocks one pixel ahead) of 16 lanes cover all 64 banks
__device__ inline uint32_t k1_offset(uint32_t px, uint32_t kc) { return px * 64u + ((kc ^ (((px >> 1) ^ (px >> 3)) & 7u)) * 8u); }

template <class T, int KSTEPS, int S>
__global__ __launch_bounds__(kK1Threads) void conv2d_k1_kernel(const T* x, const T* w, const T* bias, T* y, ConvProblem p, K1Plan q) {
    constexpr int C = KSTEPS * 16;
    constexpr int PANELS = C / 64;
        constexpr uint32_t BUFFER = PANELS * kK1Panel;             // elements of one signal tile in LDS
    constexpr uint32_t STAGE = 4 * kK1CoWave * kK1Pitch;       // elements of one staged result (four wavefronts' rows)
    extern __shared__ __align__(16) unsigned char k1_lds[];
    T* lds = reinterpret_cast<T*>(k1_lds);
    T* staged = lds + 2 * BUFFER;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
    const bool mover = wave >= 4;
    const int part = wave % 4;          // which 64 output channels a wavefront multiplies or writes out

    const uint32_t group = blockIdx.x / q.workers;
    // workgroups go round the eight dies in turn: consecutive workers (tiles that share cache lines of the signal
    // and of the result) are given to workgroups of one die, so that its L2 merges what they share
    uint32_t worker = blockIdx.x % q.workers;
    if (q.workers % 8 == 0) worker = (worker % 8) * (q.workers / 8) + worker / 8;
    const uint32_t co0 = group * kK1CoBlock + part * kK1CoWave;
    const uint32_t first = worker;
    if (first >= q.tiles) return;    // whole block: no barrier has been reached
    const uint32_t count = (q.tiles - first + q.workers - 1) / q.workers;    // tiles of this block: first + k * workers
    using Zero = std::integral_constant<int, 0>;
    using One = std::integral_constant<int, 1>;

    if (mover) {
        // ---- this thread's micro-blocks ---------------------------------------------------------------
        // Stride 1: one micro-block of 8 channels x 8 pixels (a 16-byte load per channel); C / 8 channel blocks x 8
        // pixel blocks.  Stride 2: a 16-byte load holds four pixels (its even elements), a micro-block is 8 channels
        // x 4 pixels, 16 pixel blocks x 16 channel blocks cover 128 channels and a thread has one micro-block per 128
        // channels: the lanes of a load instruction read consecutive pieces of a row, so that a cache line is asked
        // for by one instruction only (a line asked for again while it is on its way holds up the whole queue).
        // Threads without a micro-block of their own repeat another's loads and skip its writes, so that every
        // wavefront issues the same memory operations in every tile.
        const uint32_t tid = threadIdx.x - kK1Movers;
        constexpr int PXBS = S == 2 ? 16 : 8;                    // pixel blocks of a tile
        constexpr int BLOCKS = S == 2 ? (C / 8 + 15) / 16 : 1;    // micro-blocks per thread
        const uint32_t pxb = tid % PXBS;
        const uint32_t kb = S == 2 ? tid / 16 : (tid % C) / 8;    // channel block (of the first micro-block)
        const int64_t cstep = p.xs[1];
        const T* src = nullptr;
        uint4p raw[2][BLOCKS][8];   // two tiles on their way from HBM
        auto block_is_mine = [&](int b) { return S == 2 ? kb + 16 * b < C / 8 : tid < C; };

        auto locate = [&](uint32_t tile) {
            uint32_t n, pt;
            q.div_tiles_per_image.divmod(tile, n, pt);
            uint32_t pix = pt * kK1Pixels + pxb * (kK1Pixels / PXBS);
            if (pix >= q.pixels) pix = 0;                    // past the image: loads something valid, never stored
            uint32_t oh, ow;
            q.div_wo.divmod(pix, oh, ow);
            src = x + static_cast<int64_t>(n) * p.xs[0] + static_cast<int64_t>(oh * p.stride_h) * p.xs[2] + ow * S;
        };
        // tile number k of this block into register set `set`
        auto fetch = [&](auto set_, uint32_t k) {
            constexpr int set = decltype(set_)::value;
            // Never skipped: the count of memory operations between a tile's loads and their use is the same on every
            // path, which lets the wait before the use leave the younger loads and stores in flight.  Past the block's
            // last tile every lane loads the signal's first 16 bytes: one cache line an instruction, never used.
            const bool real = k < count;
            locate(first + (real ? k : 0) * q.workers);
            const int64_t step = real ? cstep : 0;
            if (!real) src = x;
#pragma unroll
            for (int b = 0; b < BLOCKS; ++b) {
                const uint32_t block = block_is_mine(b) ? kb + 16 * b : kb % (C / 8);
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) raw[set][b][kk] = *reinterpret_cast<const uint4p*>(src + static_cast<int64_t>(block * 8 + kk) * step);
            }
        };
        // The records of two pixels of a transposed micro-block (this thread's 8 channels each): two 16-byte LDS writes.
        // Threads of odd pixel blocks write the odd pixel first, which spreads a write over all banks.
        auto commit_pair = [&](auto set_, auto b_, auto m_, T* buffer) {
            constexpr int set = decltype(set_)::value, b = decltype(b_)::value, m = decltype(m_)::value;
            if (!block_is_mine(b)) return;
            uint32_t words[2][4];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int e = 2 * m + h;       // pixel of the micro-block
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t lo[4], hi[4];
                    __builtin_memcpy(lo, &raw[set][b][2 * j], 16);
                    __builtin_memcpy(hi, &raw[set][b][2 * j + 1], 16);
                    if (S == 2) words[h][j] = (lo[e] & 0xFFFFu) | (hi[e] << 16);        // even elements only
                    else if (e % 2 == 0) words[h][j] = (lo[e / 2] & 0xFFFFu) | (hi[e / 2] << 16);
                    else words[h][j] = (lo[e / 2] >> 16) | (hi[e / 2] & 0xFFFF0000u);
                }
            }
            const bool odd = pxb & 1;
            const uint32_t block = kb + 16 * b;
            T* panel = buffer + (block / 8) * kK1Panel;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                uint32_t out[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) out[j] = odd ? words[1 - h][j] : words[h][j];
                uint4p v;
                __builtin_memcpy(&v, out, 16);
                *reinterpret_cast<uint4p*>(panel + k1_offset(pxb * (kK1Pixels / PXBS) + 2 * m + (odd ? 1 - h : h), block % 8)) = v;
            }
        };
        auto commit = [&](auto set_, T* buffer) {
            k1_static_for<BLOCKS>([&](auto b_) { k1_static_for<kK1Pixels / PXBS / 2>([&](auto m_) { commit_pair(set_, b_, m_, buffer); }); });
        };
        // the staged rows of tile number k (those of multiplier `part`) written out whole.  A row of the tile is eight
        // 16-byte pieces; in the last tile of an image the lanes of the missing pieces repeat the last present one
        // (same bytes to the same address) instead of being switched off.
        auto write_rows = [&](uint32_t k) {
            const T* rows = staged + (k % 2) * STAGE + part * (kK1CoWave * kK1Pitch);
            uint32_t n, pt;
            q.div_tiles_per_image.divmod(first + k * q.workers, n, pt);
            const uint32_t present = (q.pixels - pt * kK1Pixels) / 8;     // >= 1
            const uint32_t piece = lane % 8 < present ? lane % 8 : present - 1;
            T* out = y + static_cast<int64_t>(n) * p.ys[0] + pt * kK1Pixels + piece * 8;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const uint32_t row = r * 8 + lane / 8;
                const uint4p v = *reinterpret_cast<const uint4p*>(rows + row * kK1Pitch + piece * 8);
                *reinterpret_cast<uint4p*>(out + static_cast<int64_t>(co0 + row) * p.ys[1]) = v;
            }
        };

        fetch(Zero{}, 0);
        fetch(One{}, 1);
        commit(Zero{}, lds);
        fetch(Zero{}, 2);
        __syncthreads();   // the first tile is in LDS, the multipliers have their weights
        // While the multipliers work on tile k: tile k + 1 (registers, set (k + 1) % 2) is transposed into the other
        // buffer, those registers start loading tile k + 3, and the staged result of tile k - 1 is written out.
        auto during = [&](auto par_, uint32_t k) {
            constexpr int PAR = decltype(par_)::value;     // k % 2
            using Next = std::integral_constant<int, 1 - PAR>;
            if (k + 1 < count) commit(Next{}, lds + (1 - PAR) * BUFFER);
            fetch(Next{}, k + 3);
            if (k >= 1) write_rows(k - 1);
            __syncthreads();
        };
        for (uint32_t k = 0; k < count; k += 2) {
            during(Zero{}, k);
            if (k + 1 < count) during(One{}, k + 1);
        }
        write_rows(count - 1);
        return;
    }

    // ---- a multiplier's weights, for the whole launch: 64 rows x C as MFMA fragments -----------------
    // Asked for as whole rows (a load instruction covers 1 KB of consecutive weights; taking the fragments straight
    // from global memory would touch 32 rows per instruction) and regrouped through this wavefront's share of the
    // staging area: 32 rows at a time, rows 16 bytes apart from a multiple of 128 so that the fragment reads of 16
    // lanes cover all banks.
    constexpr uint32_t PER_ROW = C / 8, WPITCH = C + 8;
    static_assert(32 * WPITCH <= 2 * kK1CoWave * kK1Pitch, "the regrouped rows fit a wavefront's two staging areas");
    uint4p afrag[2][KSTEPS];
    float start[2];
    {
        T* rows = staged + part * (2 * kK1CoWave * kK1Pitch);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint4p whole[KSTEPS];
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) {
                const uint32_t f = j * 64 + lane;
                whole[j] = *reinterpret_cast<const uint4p*>(w + static_cast<int64_t>(co0 + 32 * i + f / PER_ROW) * p.ws[0] + (f % PER_ROW) * 8);
            }
#pragma unroll
            for (int j = 0; j < KSTEPS; ++j) {
                const uint32_t f = j * 64 + lane;
                *reinterpret_cast<uint4p*>(rows + (f / PER_ROW) * WPITCH + (f % PER_ROW) * 8) = whole[j];
            }
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) afrag[i][ks] = *reinterpret_cast<const uint4p*>(rows + (lane % 32) * WPITCH + (2 * ks + lane / 32) * 8);
            const uint32_t co = co0 + 32 * i + lane % 32;
            start[i] = bias ? static_cast<float>(widen(bias[static_cast<int64_t>(co) * p.bs])) : 0.0f;
        }
    }
    // The fragments are in registers before the first barrier; said here so that no wait for them is placed in the loop.
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) asm volatile("" : "+v"(afrag[i][ks]));
    __syncthreads();

    // One tile: multiply from LDS buffer PAR, round, stage as [channel][pixel] in staging area PAR.
    auto one_tile = [&](auto par_) {
        constexpr int PAR = decltype(par_)::value;
        float16p acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = start[i];
        const T* buffer = lds + PAR * BUFFER;
        T* stage = staged + PAR * STAGE + part * (kK1CoWave * kK1Pitch);
        uint4p bfrag[2][2];   // [step parity][pixel tile]: the fragments of a step are read during the step before
        auto read_fragments = [&](auto ks_) {
            constexpr int ks = decltype(ks_)::value;
            const T* panel = buffer + (ks / 4) * kK1Panel;
            const uint32_t kc = (ks % 4) * 2 + lane / 32;
#pragma unroll
            for (int j = 0; j < 2; ++j) bfrag[ks % 2][j] = *reinterpret_cast<const uint4p*>(panel + k1_offset(32 * j + lane % 32, kc));
        };
        read_fragments(Zero{});
        k1_static_for<KSTEPS>([&](auto ks_) {
            constexpr int ks = decltype(ks_)::value;
            if constexpr (ks + 1 < KSTEPS) read_fragments(std::integral_constant<int, ks + 1>{});
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = k1_mfma<T>(bfrag[ks % 2][j], afrag[i][ks], acc[i][j]);
        });
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v4 = 0; v4 < 4; ++v4) {
                    T four[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) four[e] = narrow_result<T>(acc[i][j][4 * v4 + e]);
                    uint2p bits;
                    __builtin_memcpy(&bits, four, 8);
                    *reinterpret_cast<uint2p*>(stage + (32 * i + lane % 32) * kK1Pitch + 32 * j + 8 * v4 + 4 * (lane / 32)) = bits;
                }
        __syncthreads();   // staged rows complete; the next tile's buffer is complete; this tile's buffer is free
    };
    for (uint32_t k = 0; k < count; k += 2) {
        one_tile(Zero{});
        if (k + 1 < count) one_tile(One{});
    }
}

template <class T, int KSTEPS, int S>
int launch_k1(const ConvProblem& p, const K1Plan& q, uint32_t groups, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    constexpr int C = KSTEPS * 16;
    constexpr size_t lds = sizeof(T) * (2 * (C / 64) * kK1Panel + 2 * 4 * kK1CoWave * kK1Pitch);
    auto kernel = conv2d_k1_kernel<T, KSTEPS, S>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(groups * q.workers), dim3(kK1Threads), lds, stream, static_cast<const T*>(x), static_cast<const T*>(w),
                       static_cast<const T*>(bias), static_cast<T*>(y), p, q);
    return launch_status("conv2d_k1_kernel");
}

template <class T, int S>
int pick_k1(const ConvProblem& p, const K1Plan& q, uint32_t groups, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    switch (p.C) {
        case 64: return launch_k1<T, 4, S>(p, q, groups, x, w, bias, y, stream);
        case 128: return launch_k1<T, 8, S>(p, q, groups, x, w, bias, y, stream);
        case 192: return launch_k1<T, 12, S>(p, q, groups, x, w, bias, y, stream);
        case 256: return launch_k1<T, 16, S>(p, q, groups, x, w, bias, y, stream);
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
}

template <class T>
int run_k1(const ConvProblem& p, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (p.KH != 1 || p.KW != 1 || p.pad_h != 0 || p.pad_w != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.stride_h != p.stride_w || (p.stride_w != 1 && p.stride_w != 2)) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.C == 0 || p.C % 64 != 0 || p.C > 256 || p.O == 0 || p.O % kK1CoBlock != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.N == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    const uint64_t pixels = static_cast<uint64_t>(p.HO) * p.WO;
    if (pixels % 8 != 0 || pixels >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    // weights: rows of C contiguous channels, 16-byte fragments
    if (p.ws[1] != 1 || p.ws[0] % 8 != 0 || reinterpret_cast<uintptr_t>(w) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    // result: the pixels of a channel contiguous, rows written 16 bytes at a time
    if (p.ys[3] != 1 || p.ys[2] != static_cast<int64_t>(p.WO) || p.ys[1] % 8 != 0 || p.ys[0] % 8 != 0 || reinterpret_cast<uintptr_t>(y) % 16 != 0)
        return TANNIC_UNSUPPORTED_DTYPE;
    // signal: 16-byte loads along W
    if (p.xs[3] != 1 || p.xs[2] % 8 != 0 || p.xs[1] % 8 != 0 || p.xs[0] % 8 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.stride_w == 1) {
        // eight consecutive pixels are one load: a run must not cross a row
        if (p.WO % 8 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    } else {
        // four pixels are the even elements of one load of eight: the eighth must exist
        if (p.WO % 4 != 0 || static_cast<uint64_t>(p.WO) * 2 > p.W) return TANNIC_UNSUPPORTED_DTYPE;
    }
    K1Plan q{};
    q.pixels = static_cast<uint32_t>(pixels);
    const uint32_t tiles_per_image = (q.pixels + kK1Pixels - 1) / kK1Pixels;
    const uint64_t tiles = static_cast<uint64_t>(p.N) * tiles_per_image;
    if (tiles >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    q.tiles = static_cast<uint32_t>(tiles);
    const uint32_t groups = p.O / kK1CoBlock;
    // one block per compute unit (up to 138 KB of LDS, every register): as many workers per group as that allows
    const uint32_t per_group = groups >= 256 ? 1 : 256 / groups;
    q.workers = q.tiles < per_group ? q.tiles : per_group;
    q.div_wo = FastDiv(p.WO);
    q.div_tiles_per_image = FastDiv(tiles_per_image);
    if (p.stride_w == 1) return pick_k1<T, 1>(p, q, groups, x, w, bias, y, stream);
    return pick_k1<T, 2>(p, q, groups, x, w, bias, y, stream);
}

int conv2d_k1(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_k1<f16>(p, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_k1<bf16>(p, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
