// conv2d with a 3x3 (or 5x5) kernel on MFMA, 16-bit signals — the common ResNet-style layer.
//
// One block of 256 threads computes 64 output channels of R whole output rows
// of one image (up to 128 * TN pixels).  The input channels are walked in chunks
// of 32.  For every chunk the block holds in LDS
//   * the weights of its 64 output channels for all nine taps, [tap][channel out][32 channels in], and
//   * the input patch: the (R-1)*stride + 3 input rows the R output rows need,
//     channels-last, [row][column + padding][32 channels], with real zeros in the padding,
// in two stages: while the MFMAs of chunk c read one stage, the registers that
// hold chunk c+1 are written to the other stage and refilled with chunk c+2
// from global memory, one memory operation between MFMAs.  With ONE_STAGE the
// block has a single stage (chunk c+1 is written after the MFMAs of chunk c) and
// half the registers, so that two blocks fit a compute unit and cover each other;
// a 5x5 kernel's weights (100 KB a chunk) leave room for one stage of one block.
// Weights are read straight from the OIHW tensor: a thread loads the 8 channels x
// 9 taps of one output channel (72 consecutive elements) and regroups them in
// registers into nine 8-channel vectors.  The signal is read as 8 channels x 8
// columns micro-blocks (eight 16-byte loads along W) and transposed in registers.
// Every 64-byte LDS record (32 channels of one pixel or one output channel) has
// its four 16-byte slots XOR-swizzled by the record number, so fragment reads of
// 32 consecutive records are bank-conflict free.
// The pixel fragment is the MFMA's first operand: an accumulator holds, for the
// lane's output channel, runs of four consecutive pixels.  The block's result is
// rounded into LDS as [channel][pixel] and written out as whole rows, 16 bytes
// per lane (NCHW keeps the pixels of a channel contiguous).
#include "conv_common.hpp"

namespace th {

typedef _Float16 half8k __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8k __attribute__((ext_vector_type(8)));
typedef float float16k __attribute__((ext_vector_type(16)));
typedef unsigned int uint4k __attribute__((ext_vector_type(4)));
typedef unsigned int uint4k_any __attribute__((ext_vector_type(4), aligned(2)));   // 16 bytes at any element of a 16-bit tensor

template <class T> __device__ inline float16k k3_mfma(uint4k a, uint4k b, float16k c) {
    if constexpr (std::is_same_v<T, f16>) {
        half8k x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, c, 0, 0, 0);
    } else {
        bfloat8k x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, c, 0, 0, 0);
    }
}

template <int N, class F, int I = 0>
__device__ inline void k3_static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        k3_static_for<N, F, I + 1>(static_cast<F&&>(f));
    }
}

constexpr int kK3Threads = 256;
constexpr int kK3BCO = 64;     // output channels per block
constexpr int kK3CH = 32;      // input channels per chunk = elements per LDS record
constexpr int kK3Passes = 2;   // micro-blocks per thread and chunk (one where two blocks share a compute unit)

struct K3Plan {
    uint32_t R, IH, IWp, row_blocks, co_tiles;
    uint32_t patch_records;   // IH * IWp
    uint32_t stage_elems;     // elements of one LDS stage: weights + patch
    uint32_t microblocks;     // 4 * (W / 8) * IH
    uint32_t vector_store;    // rows of the result can be written 16 bytes at a time
    FastDiv div_colblocks, div_wo, div_row_blocks, div_co_tiles, div_pad, div_w, div_w4;   // the last two: W and 4 W (flat staging)
};

// what a micro-block outside the image reads: its eight loads all come from here
__device__ const uint4k k3_zeros = {0, 0, 0, 0};

__device__ inline uint32_t k3_offset(uint32_t rec, uint32_t slot) { return rec * kK3CH + ((slot ^ ((rec >> 2) & 3u)) * 8u); }

// KH x KW: the kernel's size; BPC: blocks that share a compute unit (2 only with ONE_STAGE).
// FLAT: rows of any width at any alignment.  The rows of the patch that lie inside the image are one contiguous run of a
// channel plane; it is cut into pieces of eight elements from its first element on (the last piece moved back so that
// it ends with the run), a micro-block is eight channels of a piece, loaded with 16-byte loads at whatever address that
// is, and its eight columns go to the records of their (row, column), which may be on two or three rows of the patch.
// Rows of the patch outside the image are zeroed once.  Without FLAT a micro-block is eight aligned columns of one row.
template <class T, int TN, bool ONE_STAGE, int KH, int KW, int BPC, bool FLAT>
__global__ __launch_bounds__(kK3Threads, BPC) void conv2d_k3_kernel(const T* x, const T* w, const T* bias, T* y, ConvProblem p, K3Plan q) {
    constexpr int TM = kK3BCO / 32;
    constexpr int kK3Taps = KH * KW;
    constexpr uint32_t kK3WeightElems = kK3Taps * kK3BCO * kK3CH;
    constexpr int PASSES = BPC == 2 ? 1 : kK3Passes;   // micro-blocks per thread and chunk
    extern __shared__ __align__(16) unsigned char k3_lds[];
    T* lds = reinterpret_cast<T*>(k3_lds);

    // workgroups go round the eight dies in turn: neighbouring tiles (which share rows of the signal and cache
    // lines of the result) are given to workgroups of one die, so that its L2 serves what they share
    uint32_t block = blockIdx.x;
    if (gridDim.x % 8 == 0) block = (block % 8) * (gridDim.x / 8) + block / 8;
    uint32_t tile, ct;
    q.div_co_tiles.divmod(block, tile, ct);
    uint32_t n, rb;
    q.div_row_blocks.divmod(tile, n, rb);
    const uint32_t oh0 = rb * q.R, co0 = ct * kK3BCO;
    const uint32_t chunks = p.C / kK3CH;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;

    // ---- per-thread constants of the staging ------------------------------------------------
    // weights: output channel threadIdx / 4, channels (threadIdx % 4) * 8 .. + 7 of the chunk
    const uint32_t w_co = threadIdx.x / 4, w_c8 = threadIdx.x % 4;
    const T* w_src = w + static_cast<int64_t>(co0 + w_co < p.O ? co0 + w_co : p.O - 1) * p.ws[0] + w_c8 * 8 * kK3Taps;
    const uint32_t w_dst = k3_offset(w_co, w_c8);   // + tap * 64 records; 64 is a multiple of 16, the swizzle stays
    // signal micro-blocks: index -> (row of the patch, block of 8 columns, block of 8 channels)
    const T* p_src[PASSES];
    int64_t p_cstep[PASSES];
    uint32_t p_dst[PASSES], p_slot[PASSES];
    uint32_t p_row[PASSES], p_col[PASSES];   // FLAT: patch row and column of the micro-block's first element
    bool p_mine[PASSES];
    // FLAT: the rows of the patch inside the image, [first_in, end_in) of IH
    const int32_t ih_first = static_cast<int32_t>(oh0 * p.stride_h) - static_cast<int32_t>(p.pad_h);
    const uint32_t row_lo = ih_first < 0 ? 0u : static_cast<uint32_t>(ih_first);
    const uint32_t row_hi = static_cast<uint32_t>(ih_first + static_cast<int32_t>(q.IH)) < p.H ? static_cast<uint32_t>(ih_first + static_cast<int32_t>(q.IH)) : p.H;
    const uint32_t first_in = row_lo - static_cast<uint32_t>(ih_first), end_in = row_hi - static_cast<uint32_t>(ih_first);
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
        const uint32_t mb = threadIdx.x + kK3Threads * ps;
        const uint32_t cb = mb % 4, t1 = mb / 4;
        p_slot[ps] = cb;
        if constexpr (FLAT) {
            const uint32_t run = (row_hi - row_lo) * p.W;           // elements; at least 8 (checked by the host)
            p_mine[ps] = t1 * 8 < run;
            const uint32_t e0 = !p_mine[ps] ? 0 : t1 * 8 + 8 <= run ? t1 * 8 : run - 8;
            uint32_t r0, c0;
            q.div_w.divmod(e0, r0, c0);
            p_row[ps] = first_in + r0;
            p_col[ps] = c0;
            p_dst[ps] = 0;
            p_src[ps] = x + static_cast<int64_t>(n) * p.xs[0] + static_cast<int64_t>(cb * 8) * p.xs[1] + static_cast<int64_t>(row_lo) * p.xs[2] + e0;
            p_cstep[ps] = p.xs[1];
        } else {
            uint32_t prow, colb;
            q.div_colblocks.divmod(t1, prow, colb);
            const int32_t ih = static_cast<int32_t>(oh0 * p.stride_h + prow) - static_cast<int32_t>(p.pad_h);
            p_mine[ps] = mb < q.microblocks;
            const bool live = p_mine[ps] && ih >= 0 && ih < static_cast<int32_t>(p.H);
            // rows outside the image are zeros in LDS: their micro-blocks load zeros
            p_src[ps] = live ? x + static_cast<int64_t>(n) * p.xs[0] + static_cast<int64_t>(cb * 8) * p.xs[1] + static_cast<int64_t>(ih) * p.xs[2] + colb * 8
                             : reinterpret_cast<const T*>(&k3_zeros);
            p_cstep[ps] = live ? p.xs[1] : 0;
            p_dst[ps] = prow * q.IWp + p.pad_w + colb * 8;   // first of the eight records
            p_row[ps] = p_col[ps] = 0;
        }
    }

    uint4k wreg[kK3Taps];
    uint4k preg[PASSES][8];
    auto fetch_w = [&](int k, uint32_t chunk) {
        wreg[k] = *reinterpret_cast<const uint4k*>(w_src + static_cast<int64_t>(chunk) * (kK3CH * kK3Taps) + k * 8);
    };
    auto fetch_p = [&](int ps, int cc, uint32_t chunk) {
        if constexpr (FLAT) preg[ps][cc] = *reinterpret_cast<const uint4k_any*>(p_src[ps] + (static_cast<int64_t>(chunk) * kK3CH + cc) * p_cstep[ps]);
        else preg[ps][cc] = *reinterpret_cast<const uint4k*>(p_src[ps] + (static_cast<int64_t>(chunk) * kK3CH + cc) * p_cstep[ps]);
    };
    // tap `tap` of the eight channels: elements cc * taps + tap of the 8 * taps loaded ones
    auto commit_w = [&](int tap, T* stage) {
        uint16_t all[8 * kK3Taps], out[8];
        __builtin_memcpy(all, wreg, 16 * kK3Taps);
#pragma unroll
        for (int cc = 0; cc < 8; ++cc) out[cc] = all[cc * kK3Taps + tap];
        uint4k v;
        __builtin_memcpy(&v, out, 16);
        *reinterpret_cast<uint4k*>(stage + w_dst + tap * (kK3BCO * kK3CH)) = v;
    };
    // column px of the micro-block: element px of each of the eight channel vectors
    auto commit_p = [&](int ps, int px, T* stage) {
        if (!p_mine[ps]) return;
        uint16_t out[8];
#pragma unroll
        for (int cc = 0; cc < 8; ++cc) {
            uint16_t in[8];
            __builtin_memcpy(in, &preg[ps][cc], 16);
            out[cc] = in[px];
        }
        uint4k v;
        __builtin_memcpy(&v, out, 16);
        uint32_t rec = p_dst[ps] + px;
        if constexpr (FLAT) {
            // column px of the piece: up to two rows further down (rows are at least four columns wide)
            uint32_t row = p_row[ps], col = p_col[ps] + px;
            if (col >= p.W) { col -= p.W; ++row; }
            if (col >= p.W) { col -= p.W; ++row; }
            rec = row * q.IWp + p.pad_w + col;
        }
        *reinterpret_cast<uint4k*>(stage + kK3WeightElems + k3_offset(rec, p_slot[ps])) = v;
    };

    // ---- prologue: chunk 0 into stage 0, chunk 1 into registers ------------------------------------
    // (the bias goes first: loads return in order, and the accumulators are seeded while the tiles are on their way)
    float bias_v[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const uint32_t co = co0 + i * 32 + lane % 32;
        bias_v[i] = (p.has_bias && co < p.O) ? static_cast<float>(widen(bias[static_cast<int64_t>(co) * p.bs])) : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < kK3Taps; ++k) fetch_w(k, 0);
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
        for (int cc = 0; cc < 8; ++cc) fetch_p(ps, cc, 0);
    // the padding columns of both stages are zero and no staging write ever touches them
    {
        const uint32_t per_row = 2 * p.pad_w * 4;   // 16-byte slots of padding per patch row
        const uint32_t total = per_row * q.IH;
        for (uint32_t i = threadIdx.x; i < (ONE_STAGE ? 1 : 2) * total; i += kK3Threads) {
            const uint32_t st = i >= total ? 1 : 0, r = i - st * total;
            uint32_t row, e;
            q.div_pad.divmod(r, row, e);
            const uint32_t slot = e % 4, side = e / 4;
            const uint32_t col = side < p.pad_w ? side : p.W + side;
            *reinterpret_cast<uint4k*>(lds + st * q.stage_elems + kK3WeightElems + k3_offset(row * q.IWp + col, slot)) = uint4k{0, 0, 0, 0};
        }
        if constexpr (FLAT) {
            // the rows of the patch above and below the image: no micro-block ever writes them
            const uint32_t outside = q.IH - (end_in - first_in), slots = outside * 4 * p.W;
            for (uint32_t i = threadIdx.x; i < (ONE_STAGE ? 1 : 2) * slots; i += kK3Threads) {
                const uint32_t st = i >= slots ? 1 : 0, r = i - st * slots;
                uint32_t k, e;
                q.div_w4.divmod(r, k, e);
                const uint32_t row = k < first_in ? k : end_in + (k - first_in);
                *reinterpret_cast<uint4k*>(lds + st * q.stage_elems + kK3WeightElems + k3_offset(row * q.IWp + p.pad_w + e / 4, e % 4)) = uint4k{0, 0, 0, 0};
            }
        }
    }
    // the lane's pixels: group wave + 4 * j, pixel lane % 32 of the group
    const uint32_t npix_tile = q.R * p.WO;
    uint32_t pbase[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t qp = (wave + 4 * j) * 32 + lane % 32;
        uint32_t r = 0, ow = 0;
        if (qp < npix_tile) q.div_wo.divmod(qp, r, ow);
        pbase[j] = r * p.stride_h * q.IWp + ow * p.stride_w;
    }
    float16k acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = bias_v[i];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < kK3Taps; ++k) commit_w(k, lds);
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
        for (int px = 0; px < 8; ++px) commit_p(ps, px, lds);
    if (chunks > 1) {
#pragma unroll
        for (int k = 0; k < kK3Taps; ++k) fetch_w(k, 1);
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
            for (int cc = 0; cc < 8; ++cc) fetch_p(ps, cc, 1);
    }
    __syncthreads();

    // ---- chunks ------------------------------------------------------------------------------------
    // fragment addresses: weights  wlane ^ (half * 16) + tap * 2048 + i * 1024   (elements)
    //                     patch    (xoff[j] ^ (half * 16)),  xoff from the record pbase[j] + kh * IWp + kw
    const uint32_t frag_slot = lane / 32;
    const uint32_t wlane = k3_offset(lane % 32, frag_slot);   // record i * 32 + lane % 32: same swizzle for every i and tap
    uint4k fw[2][2][TM], fx[2][2][TN];   // [buffer][half][...]
    auto read_fragments = [&](const T* stage, int tap, int into) {
        const uint32_t tap_rec = (tap / KW) * q.IWp + tap % KW;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t xoff = k3_offset(pbase[j] + tap_rec, frag_slot);
#pragma unroll
            for (int half = 0; half < 2; ++half) fx[into][half][j] = *reinterpret_cast<const uint4k*>(stage + kK3WeightElems + (xoff ^ (half * 16u)));
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int half = 0; half < 2; ++half)
                fw[into][half][i] = *reinterpret_cast<const uint4k*>(stage + (wlane ^ (half * 16u)) + tap * (kK3BCO * kK3CH) + i * 32 * kK3CH);
    };
    auto run_chunk = [&](uint32_t chunk, auto commit_tag, auto fetch_tag) {
        constexpr bool COMMIT = decltype(commit_tag)::value, FETCH = decltype(fetch_tag)::value;
        constexpr int PER_HALF = TM * TN, PER_TAP = 2 * PER_HALF, MFMAS = kK3Taps * PER_TAP;
        // memory operations of the chunk in order: weights out, weights in, then each pass of the signal out and in
        constexpr int OPS = 2 * kK3Taps + PASSES * 16;
        const T* stage = lds + (ONE_STAGE ? 0 : (chunk & 1) * q.stage_elems);
        T* next = lds + (ONE_STAGE ? 0 : ((chunk & 1) ^ 1) * q.stage_elems);
        read_fragments(stage, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        k3_static_for<MFMAS>([&](auto m_tag) {
            constexpr int m = decltype(m_tag)::value;
            constexpr int tap = m / PER_TAP, half = (m % PER_TAP) / PER_HALF, i = (m % PER_HALF) / TN, j = m % TN;
            if constexpr (m % PER_TAP == 0 && tap + 1 < kK3Taps) {
                read_fragments(stage, tap + 1, (tap + 1) & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            acc[i][j] = k3_mfma<T>(fx[tap & 1][half][j], fw[tap & 1][half][i], acc[i][j]);
            constexpr int first = ONE_STAGE ? 0 : m * OPS / MFMAS, last = ONE_STAGE ? 0 : (m + 1) * OPS / MFMAS;
            k3_static_for<last - first>([&](auto o_tag) {
                constexpr int o = first + decltype(o_tag)::value;
                if constexpr (o < kK3Taps) { if constexpr (COMMIT) commit_w(o, next); }
                else if constexpr (o < 2 * kK3Taps) { if constexpr (FETCH) fetch_w(o - kK3Taps, chunk + 2); }
                else {
                    constexpr int r = o - 2 * kK3Taps, ps = r / 16, e = r % 16;
                    if constexpr (e < 8) { if constexpr (COMMIT) commit_p(ps, e, next); }
                    else { if constexpr (FETCH) fetch_p(ps, e - 8, chunk + 2); }
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
        if constexpr (ONE_STAGE && COMMIT) {
            // the only stage is free now: the next chunk goes in, the one after it into the registers
#pragma unroll
            for (int k = 0; k < kK3Taps; ++k) commit_w(k, next);
#pragma unroll
            for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
                for (int px = 0; px < 8; ++px) commit_p(ps, px, next);
            if constexpr (FETCH) {
#pragma unroll
                for (int k = 0; k < kK3Taps; ++k) fetch_w(k, chunk + 2);
#pragma unroll
                for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
                    for (int cc = 0; cc < 8; ++cc) fetch_p(ps, cc, chunk + 2);
            }
            __syncthreads();
        }
    };
    using Yes = std::true_type;
    using No = std::false_type;
    uint32_t chunk = 0;
    for (; chunk + 2 < chunks; ++chunk) run_chunk(chunk, Yes{}, Yes{});
    if (chunk + 1 < chunks) { run_chunk(chunk, Yes{}, No{}); ++chunk; }
    run_chunk(chunk, No{}, No{});

    // ---- result: accumulators -> LDS [channel][pixel] -> global rows ----------------------------------
    // accumulator (i, j): lane -> channel i * 32 + lane % 32; value v -> pixel 8 * (v / 4) + 4 * (lane / 32) + v % 4 of group wave + 4 j
    constexpr int PITCH = 128 * TN + 8;
    T* out = lds;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                T r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = narrow_result<T>(acc[i][j][g * 4 + e]);
                uint2 bits;
                __builtin_memcpy(&bits, r, 8);
                *reinterpret_cast<uint2*>(out + (i * 32 + lane % 32) * PITCH + (wave + 4 * j) * 32 + g * 8 + 4 * (lane / 32)) = bits;
            }
    __syncthreads();
    const uint32_t rows_here = p.HO - oh0 < q.R ? p.HO - oh0 : q.R;
    const uint32_t npix = rows_here * p.WO;
    T* ybase = y + static_cast<int64_t>(n) * p.ys[0] + static_cast<int64_t>(oh0) * p.ys[2];
    // one loop per way of storing, so that each stays a plain loop over the wavefront's sixteen channels
    if (q.vector_store == 1) {
        // rows of the tile follow each other in memory: npix contiguous elements, a multiple of 8, 16-byte aligned
        for (uint32_t c = wave; c < kK3BCO; c += 4) {
            if (co0 + c >= p.O) break;
            T* yrow = ybase + static_cast<int64_t>(co0 + c) * p.ys[1];
            const T* srow = out + c * PITCH;
            for (uint32_t pix = lane * 8; pix < npix; pix += 64 * 8) *reinterpret_cast<uint4k*>(yrow + pix) = *reinterpret_cast<const uint4k*>(srow + pix);
        }
    } else if (q.vector_store == 2) {
        // the same at any alignment and length: whole pieces of eight, then the last few one by one
        for (uint32_t c = wave; c < kK3BCO; c += 4) {
            if (co0 + c >= p.O) break;
            T* yrow = ybase + static_cast<int64_t>(co0 + c) * p.ys[1];
            const T* srow = out + c * PITCH;
            for (uint32_t pix = lane * 8; pix < npix; pix += 64 * 8) {
                if (pix + 8 <= npix) *reinterpret_cast<uint4k_any*>(yrow + pix) = *reinterpret_cast<const uint4k*>(srow + pix);
                else for (uint32_t e = pix; e < npix; ++e) yrow[e] = srow[e];
            }
        }
    } else {
        for (uint32_t c = wave; c < kK3BCO; c += 4) {
            if (co0 + c >= p.O) break;
            T* yrow = ybase + static_cast<int64_t>(co0 + c) * p.ys[1];
            const T* srow = out + c * PITCH;
            for (uint32_t pix = lane; pix < npix; pix += 64) {
                uint32_t r, ow;
                q.div_wo.divmod(pix, r, ow);
                yrow[static_cast<int64_t>(r) * p.ys[2] + static_cast<int64_t>(ow) * p.ys[3]] = srow[pix];
            }
        }
    }
}

template <class T, int TN, bool ONE_STAGE, int KH, int KW, int BPC, bool FLAT>
int launch_k3_as(const ConvProblem& p, const K3Plan& q, size_t lds, uint32_t blocks, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    auto kernel = conv2d_k3_kernel<T, TN, ONE_STAGE, KH, KW, BPC, FLAT>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), 160 * 1024, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kK3Threads), lds, stream, static_cast<const T*>(x), static_cast<const T*>(w), static_cast<const T*>(bias),
                       static_cast<T*>(y), p, q);
    return launch_status("conv2d_k3_kernel");
}

template <class T, int TN, bool ONE_STAGE, int KH, int KW, int BPC>
int launch_k3(bool flat, const ConvProblem& p, const K3Plan& q, size_t lds, uint32_t blocks, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (flat) return launch_k3_as<T, TN, ONE_STAGE, KH, KW, BPC, true>(p, q, lds, blocks, x, w, bias, y, stream);
    return launch_k3_as<T, TN, ONE_STAGE, KH, KW, BPC, false>(p, q, lds, blocks, x, w, bias, y, stream);
}

template <class T, int KH, int KW>
int run_k3(const ConvProblem& p, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    constexpr uint32_t TAPS = KH * KW, WEIGHT_ELEMS = TAPS * kK3BCO * kK3CH;
    if (p.KH != KH || p.KW != KW) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.C == 0 || p.C % kK3CH != 0 || p.xs[3] != 1) return TANNIC_UNSUPPORTED_DTYPE;
    // 16-byte loads.  Aligned staging: rows a multiple of 8 wide, rows, channels and images starting at multiples of 8
    // elements.  Otherwise flat staging: rows that follow each other in memory (a channel plane is one run), at least four
    // columns, and at least eight elements of the image in every block's patch (its rows inside the image: KH - pad_h or more).
    const bool aligned = p.W % 8 == 0 && p.xs[2] % 8 == 0 && p.xs[1] % 8 == 0 && p.xs[0] % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
    const bool flat = !aligned;
    if (flat && (p.xs[2] != static_cast<int64_t>(p.W) || p.W < 4 || p.pad_h >= KH || p.H < KH - p.pad_h || static_cast<uint64_t>(KH - p.pad_h) * p.W < 8 ||
                 reinterpret_cast<uintptr_t>(x) % sizeof(T) != 0))
        return TANNIC_UNSUPPORTED_DTYPE;
    if (p.ws[3] != 1 || p.ws[2] != KW || p.ws[1] != static_cast<int64_t>(TAPS) || p.ws[0] != static_cast<int64_t>(p.C) * TAPS || reinterpret_cast<uintptr_t>(w) % 16 != 0)
        return TANNIC_UNSUPPORTED_DTYPE;
    if (p.N == 0 || p.O == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    K3Plan q{};
    q.IWp = p.W + 2 * p.pad_w;
    const size_t budget = 158 * 1024;
    // the largest number of output rows whose tile fits: pixels, LDS, staging registers
    int tn = 0, mode = 0;   // mode 0: two stages; 1: one stage, two blocks per compute unit; 2: one stage, one block
    double best = 0.0;
    auto consider = [&](uint32_t R, int m, double weight) {
        const uint32_t IH = (R - 1) * p.stride_h + KH;
        const size_t stage = (static_cast<size_t>(WEIGHT_ELEMS) + static_cast<size_t>(IH) * q.IWp * kK3CH) * sizeof(T);
        const uint64_t microblocks = flat ? 4ull * ((static_cast<uint64_t>(p.W) * IH + 7) / 8) : 4ull * (p.W / 8) * IH;
        const int t = R * p.WO > 256 ? 4 : 2;
        const size_t out_bytes = static_cast<size_t>(kK3BCO) * (128 * t + 8) * sizeof(T);
        if (microblocks > (m == 1 ? 1 : kK3Passes) * kK3Threads) return;
        if (m == 0 && 2 * stage > budget) return;
        if (m == 1 && (stage > budget / 2 || out_bytes > budget / 2 || t != 2)) return;
        if (m == 2 && (stage > budget || out_bytes > budget)) return;
        const double fill = static_cast<double>(R * p.WO) / (128.0 * t);              // lanes with a pixel
        const double rows = static_cast<double>(p.HO) / (((p.HO + R - 1) / R) * R);    // rows of the last block that exist
        const double halo = static_cast<double>(R * p.stride_h) / IH;                  // input rows read once
        const double score = weight * fill * rows * (0.5 + 0.5 * halo);
        if (score >= best) { best = score; q.R = R; q.IH = IH; tn = t; mode = m; }
    };
    constexpr bool SMALL = TAPS <= 9;   // a larger kernel's chunk of weights leaves room for one stage of one block only
    if (SMALL)
        for (uint32_t R = 1; R <= p.HO && R * p.WO <= 512; ++R) consider(R, 0, 1.0);
    // Few chunks: one stage per block and tiles of at most 256 pixels, so that two blocks share a compute unit and
    // one block's loads, LDS writes and result rows run under the other's MFMAs.  With more than four chunks the
    // LDS writes between the chunks, which a single stage cannot hide inside a block, cost more than that gains.
    if (SMALL && p.C <= 4 * kK3CH)
        for (uint32_t R = 1; R <= p.HO && R * p.WO <= 256; ++R) consider(R, 1, 1.25);
    // 5x5: one stage, the whole LDS, tiles of at most 256 pixels (what the registers hold next to 25 taps of weights).
    if (!SMALL)
        for (uint32_t R = 1; R <= p.HO && R * p.WO <= 256; ++R) consider(R, 2, 1.0);
    if (best == 0.0) return TANNIC_UNSUPPORTED_DTYPE;
    q.row_blocks = (p.HO + q.R - 1) / q.R;
    q.co_tiles = (p.O + kK3BCO - 1) / kK3BCO;
    q.patch_records = q.IH * q.IWp;
    q.stage_elems = WEIGHT_ELEMS + q.patch_records * kK3CH;
    q.microblocks = 4 * (p.W / 8) * q.IH;
    q.div_colblocks = FastDiv(p.W / 8);
    q.div_wo = FastDiv(p.WO);
    q.div_row_blocks = FastDiv(q.row_blocks);
    q.div_co_tiles = FastDiv(q.co_tiles);
    q.div_pad = FastDiv(p.pad_w ? 8 * p.pad_w : 1);
    q.div_w = FastDiv(p.W);
    q.div_w4 = FastDiv(4 * p.W);
    const bool rows_follow = p.ys[3] == 1 && p.ys[2] == static_cast<int64_t>(p.WO);
    q.vector_store = rows_follow && p.ys[1] % 8 == 0 && p.ys[0] % 8 == 0 && (q.R * p.WO) % 8 == 0 && (static_cast<uint64_t>(p.HO) * p.WO) % 8 == 0 &&
                             reinterpret_cast<uintptr_t>(y) % 16 == 0 ? 1
                     : rows_follow && reinterpret_cast<uintptr_t>(y) % sizeof(T) == 0 ? 2 : 0;
    const uint64_t blocks = static_cast<uint64_t>(p.N) * q.row_blocks * q.co_tiles;
    if (blocks >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    const size_t stage_bytes = static_cast<size_t>(q.stage_elems) * sizeof(T);
    const size_t out_bytes = static_cast<size_t>(kK3BCO) * (128 * tn + 8) * sizeof(T);
    const size_t held = (mode == 0 ? 2 : 1) * stage_bytes;
    const size_t lds = held > out_bytes ? held : out_bytes;
    const uint32_t nb = static_cast<uint32_t>(blocks);
    if constexpr (SMALL) {
        if (mode == 1) return launch_k3<T, 2, true, KH, KW, 2>(flat, p, q, lds, nb, x, w, bias, y, stream);
        if (tn == 4) return launch_k3<T, 4, false, KH, KW, 1>(flat, p, q, lds, nb, x, w, bias, y, stream);
        return launch_k3<T, 2, false, KH, KW, 1>(flat, p, q, lds, nb, x, w, bias, y, stream);
    } else {
        return launch_k3<T, 2, true, KH, KW, 1>(flat, p, q, lds, nb, x, w, bias, y, stream);
    }
}

// This file is compiled in two parts (TH_K3_PART): 0 holds the 3x3 kernels and the entry point, 1 the 5x5 kernels.
#ifndef TH_K3_PART
#define TH_K3_PART 0
#endif

int conv2d_k5(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);

#if TH_K3_PART == 1
int conv2d_k5(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_k3<f16, 5, 5>(p, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_k3<bf16, 5, 5>(p, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}
#else
int conv2d_k3(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (p.KH == 5 && p.KW == 5) return conv2d_k5(p, dtype, x, w, bias, y, stream);
    if (dtype == TANNIC_FLOAT16) return run_k3<f16, 3, 3>(p, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_k3<bf16, 3, 3>(p, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}
#endif

}  // namespace th
