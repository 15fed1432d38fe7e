// conv2d on MFMA with the input patch staged in LDS — the fast path for 16-bit
// signals whose channel count is a multiple of 32.
//
// A block of 256 threads produces, for one image, R full output rows x BCO
// output channels.  Input channels are taken 32 at a time.  For each such
// chunk the block copies the (R-1)*stride + KH input rows it needs from the
// NCHW signal into LDS with 16-byte loads along W, transposing 8x8
// (channel x column) micro-blocks in registers so that LDS holds the patch
// channels-last: [row][column + padding][32 channels], 64 bytes per pixel.  The
// zero padding is real zeros in LDS, written once, so the inner loop has no
// range tests.  The chunk's weights come from a copy rearranged once per call to
// [tap][output channel][input channel] and land in LDS as [tap][BCO][32].
// Then, per tap (kh, kw) and per 16 channels, an MFMA operand is one 16-byte LDS
// read per lane on either side: v_mfma_f32_32x32x16_{f16,bf16} with the weight
// tile as row operand and 32 consecutive output pixels as column operand.  The
// 16-byte chunks of both LDS tiles are XOR-swizzled so that those reads are
// bank-conflict free.  LDS use is about 60 KB, so two blocks share a CU and one
// block's staging overlaps the other's MFMAs.
//
// Accumulation is fp32 from the bias (src/cpu/conv2d.cpp:90), one rounding at the
// end.  The order of summation is (channel chunk, kh, kw, channel) instead of the
// CPU path's (channel, kh, kw); with fp32 accumulation the difference is rounding
// noise.
#include "conv_common.hpp"

namespace th {

typedef _Float16 half8p __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8p __attribute__((ext_vector_type(8)));
typedef float float16p __attribute__((ext_vector_type(16)));
typedef unsigned int uint4p __attribute__((ext_vector_type(4)));

template <class T> __device__ inline float16p patch_mfma(uint4p a, uint4p b, float16p c) {
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

constexpr int kPatchThreads = 256;
constexpr int kCC = 32;  // input channels per chunk

struct PatchPlan {
    uint32_t R;            // output rows per block
    uint32_t IH;           // patch rows held in LDS
    uint32_t IWp;          // patch columns: W + 2 * pad_w
    uint32_t row_blocks;   // ceil(HO / R)
    uint32_t co_tiles;
    uint32_t groups;       // ceil(R * WO / 32)
    uint32_t rows_strided; // KH == 1: patch row r holds input row (oh0 + r) * stride_h - pad_h
};

// weights rearranged to [tap][O][C] (C fastest) for contiguous chunk loads
template <class T>
__global__ void conv_weights_tap_major_kernel(const T* w, T* out, ConvProblem p, uint32_t total) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const uint32_t c = i % p.C, o = (i / p.C) % p.O, tap = i / (p.C * p.O);
    const uint32_t kh = tap / p.KW, kw = tap % p.KW;
    out[i] = w[o * p.ws[0] + c * p.ws[1] + kh * p.ws[2] + kw * p.ws[3]];
}

// element offset of 16-byte chunk `chunk` (0..3) of record `rec` in a [records][32] tile
__device__ inline uint32_t rec_offset(uint32_t rec, uint32_t chunk) { return rec * kCC + ((chunk ^ ((rec >> 2) & 3u)) * 8u); }

template <class T, int BCO>
__global__ __launch_bounds__(kPatchThreads, 2) void conv2d_patch_kernel(const T* x, const T* wt, const T* bias, T* y, ConvProblem p, PatchPlan q) {
    constexpr int TM = BCO / 32;
    extern __shared__ __align__(16) unsigned char patch_lds[];
    T* patch = reinterpret_cast<T*>(patch_lds);
    const uint32_t patch_records = q.IH * q.IWp;
    T* wl = patch + patch_records * kCC;
    const uint32_t taps = p.KH * p.KW;

    uint32_t b = blockIdx.x;
    const uint32_t ct = b % q.co_tiles; b /= q.co_tiles;
    const uint32_t rb = b % q.row_blocks;
    const uint32_t n = b / q.row_blocks;
    const uint32_t co0 = ct * BCO, oh0 = rb * q.R;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;

    // zero the whole patch once: padding columns and rows outside the image stay zero
    for (uint32_t i = threadIdx.x; i < patch_records * kCC / 8; i += kPatchThreads) reinterpret_cast<uint4p*>(patch)[i] = uint4p{0, 0, 0, 0};

    // the lane's output pixels: groups `wave` and `wave + 4` of 32 consecutive pixels of the R x WO block
    const uint32_t npix = q.R * p.WO;
    uint32_t pbase[2];   // patch record of the window origin (kh = kw = 0)
    bool group_live[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t g = wave + 4 * j;
        group_live[j] = g < q.groups;
        const uint32_t qp = g * 32 + lane % 32;
        const bool live = qp < npix && oh0 + qp / p.WO < p.HO;
        const uint32_t r = live ? qp / p.WO : 0, ow = live ? qp % p.WO : 0;
        pbase[j] = (q.rows_strided ? r : r * p.stride_h) * q.IWp + ow * p.stride_w;
    }

    float16p acc[TM][2];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t co = co0 + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
            const float bv = (p.has_bias && co < p.O) ? static_cast<float>(widen(bias[static_cast<int64_t>(co) * p.bs])) : 0.0f;
            acc[i][0][v] = bv;
            acc[i][1][v] = bv;
        }

    const uint32_t colblocks = p.W / 8;
    const uint32_t microblocks = 4 * colblocks * q.IH;
    const T* xn = x + static_cast<int64_t>(n) * p.xs[0];
    const uint32_t frag_chunk = lane / 32;

    for (uint32_t c0 = 0; c0 < p.C; c0 += kCC) {
        __syncthreads();  // everyone is done reading the previous chunk (and with the zero fill)
        // ---- signal chunk -> LDS, channels-last --------------------------------------
        for (uint32_t mb = threadIdx.x; mb < microblocks; mb += kPatchThreads) {
            const uint32_t cb = mb % 4, colb = (mb / 4) % colblocks, prow = mb / (4 * colblocks);
            const int32_t ih = q.rows_strided ? static_cast<int32_t>((oh0 + prow) * p.stride_h) - static_cast<int32_t>(p.pad_h)
                                              : static_cast<int32_t>(oh0 * p.stride_h + prow) - static_cast<int32_t>(p.pad_h);
            if (ih < 0 || ih >= static_cast<int32_t>(p.H)) continue;
            const T* src = xn + static_cast<int64_t>(c0 + cb * 8) * p.xs[1] + static_cast<int64_t>(ih) * p.xs[2] + colb * 8;
            uint16_t in[8][8];
#pragma unroll
            for (int cc = 0; cc < 8; ++cc) {
                const uint4p v = *reinterpret_cast<const uint4p*>(src + static_cast<int64_t>(cc) * p.xs[1]);
                __builtin_memcpy(in[cc], &v, 16);
            }
            const uint32_t rec0 = prow * q.IWp + p.pad_w + colb * 8;
#pragma unroll
            for (int px = 0; px < 8; ++px) {
                uint16_t out[8];
#pragma unroll
                for (int cc = 0; cc < 8; ++cc) out[cc] = in[cc][px];
                uint4p v;
                __builtin_memcpy(&v, out, 16);
                *reinterpret_cast<uint4p*>(patch + rec_offset(rec0 + px, cb)) = v;
            }
        }
        // ---- weight chunk -> LDS [tap][BCO][32] ------------------------------------------
        for (uint32_t id = threadIdx.x; id < taps * BCO * 4; id += kPatchThreads) {
            const uint32_t ch = id % 4, row = (id / 4) % BCO, tap = id / (4 * BCO);
            const uint32_t co = co0 + row < p.O ? co0 + row : p.O - 1;
            const uint4p v = *reinterpret_cast<const uint4p*>(wt + (static_cast<int64_t>(tap) * p.O + co) * p.C + c0 + ch * 8);
            *reinterpret_cast<uint4p*>(wl + rec_offset(tap * BCO + row, ch)) = v;
        }
        __syncthreads();
        // ---- MFMAs: taps x two 16-channel slices -----------------------------------------------
        for (uint32_t tap = 0; tap < taps; ++tap) {
            const uint32_t kh = tap / p.KW, kw = tap % p.KW;
            const uint32_t tap_rec = (q.rows_strided ? 0 : kh) * q.IWp + kw;
#pragma unroll
            for (int ks = 0; ks < kCC / 16; ++ks) {
                uint4p fw[TM], fx[2];
#pragma unroll
                for (int i = 0; i < TM; ++i) fw[i] = *reinterpret_cast<const uint4p*>(wl + rec_offset(tap * BCO + i * 32 + lane % 32, ks * 2 + frag_chunk));
#pragma unroll
                for (int j = 0; j < 2; ++j) fx[j] = *reinterpret_cast<const uint4p*>(patch + rec_offset(pbase[j] + tap_rec, ks * 2 + frag_chunk));
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    acc[i][0] = patch_mfma<T>(fw[i], fx[0], acc[i][0]);
                    if (group_live[1]) acc[i][1] = patch_mfma<T>(fw[i], fx[1], acc[i][1]);
                }
            }
        }
    }

    // store: the lane's pixel column, rows = output channels; 32 lanes write 32 consecutive pixels
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t qp = (wave + 4 * j) * 32 + lane % 32;
        if (!group_live[j] || qp >= npix) continue;
        const uint32_t oh = oh0 + qp / p.WO, ow = qp % p.WO;
        if (oh >= p.HO) continue;
        T* yp = y + static_cast<int64_t>(n) * p.ys[0] + static_cast<int64_t>(oh) * p.ys[2] + static_cast<int64_t>(ow) * p.ys[3];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t co = co0 + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
                if (co < p.O) yp[static_cast<int64_t>(co) * p.ys[1]] = narrow<T>(acc[i][j][v]);
            }
    }
}

template <class T, int BCO>
int launch_patch(const ConvProblem& p, const PatchPlan& q, size_t lds, const void* x, const T* wt, const void* bias, void* y, hipStream_t stream) {
    auto kernel = conv2d_patch_kernel<T, BCO>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), 160 * 1024, configured)) return rc;
    const uint32_t grid = p.N * q.row_blocks * q.co_tiles;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kPatchThreads), lds, stream, static_cast<const T*>(x), wt, static_cast<const T*>(bias),
                       static_cast<T*>(y), p, q);
    return launch_status("conv2d_patch_kernel");
}

template <class T>
int run_patch(const ConvProblem& p, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    // conditions of this path: channel chunks of 32, rows of the signal readable with aligned 16-byte loads
    if (p.C == 0 || p.C % kCC != 0 || p.W % 8 != 0 || p.xs[3] != 1 || p.xs[2] % 8 != 0 || p.xs[1] % 8 != 0 || p.xs[0] % 8 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (reinterpret_cast<uintptr_t>(x) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.N == 0 || p.O == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    const uint32_t taps = p.KH * p.KW;
    const int BCO = p.O > 64 ? 128 : 64;
    PatchPlan q{};
    q.rows_strided = p.KH == 1 ? 1 : 0;
    q.IWp = p.W + 2 * p.pad_w;
    q.co_tiles = (p.O + BCO - 1) / BCO;
    // rows per block: as many as keep 256 pixels and ~64 KB of LDS, scored by how well they fill the block
    const size_t w_bytes = static_cast<size_t>(taps) * BCO * kCC * sizeof(T);
    double best = 0.0;
    size_t best_lds = 0;
    for (uint32_t R = 1; R <= p.HO && R * p.WO <= 256; ++R) {
        const uint32_t IH = q.rows_strided ? R : (R - 1) * p.stride_h + p.KH;
        const size_t lds = static_cast<size_t>(IH) * q.IWp * kCC * sizeof(T) + w_bytes;
        if (lds > 150 * 1024) break;
        const uint32_t groups = (R * p.WO + 31) / 32;
        const double fill = static_cast<double>(R * p.WO) / (((groups + 3) / 4) * 128.0);
        const double rows = static_cast<double>(p.HO) / (((p.HO + R - 1) / R) * R);
        const double score = fill * rows * (lds <= 80 * 1024 ? 1.0 : 0.7);
        if (score >= best) { best = score; q.R = R; q.IH = IH; q.groups = groups; best_lds = lds; }
    }
    if (best == 0.0) return TANNIC_UNSUPPORTED_DTYPE;
    q.row_blocks = (p.HO + q.R - 1) / q.R;
    if (static_cast<uint64_t>(p.N) * q.row_blocks * q.co_tiles >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    // weights, rearranged once per call
    const uint64_t wcount = static_cast<uint64_t>(taps) * p.O * p.C;
    if (wcount >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    T* wt = nullptr;
    if (scratch_acquire(reinterpret_cast<void**>(&wt), wcount * sizeof(T), stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
    hipLaunchKernelGGL((conv_weights_tap_major_kernel<T>), dim3((wcount + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(w), wt, p,
                       static_cast<uint32_t>(wcount));
    int status = launch_status("conv_weights_tap_major_kernel");
    if (status == TANNIC_SUCCESS) {
        status = BCO == 128 ? launch_patch<T, 128>(p, q, best_lds, x, wt, bias, y, stream) : launch_patch<T, 64>(p, q, best_lds, x, wt, bias, y, stream);
    }
    scratch_release(wt, stream);
    return status;
}

int conv2d_patch(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_patch<f16>(p, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_patch<bf16>(p, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
