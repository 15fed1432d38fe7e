// conv2d with a 1x1 kernel, fp16 / bf16 / fp32 signals: a matrix product per image.
//
// y[n] (O x HO*WO) = w (O x C) * x[n] (C x HO*WO): the kernel tensor is the
// K-contiguous operand, an NCHW image is the row-major one (pixels contiguous for
// each channel) and NCHW output is the plain row-major result, so the batched
// MFMA matrix-multiply kernel runs it as it stands, with the bias as its per-row
// start value.  With a stride the pixels the product needs are first gathered
// into a dense [N][C][HO*WO] copy (the only extra traffic: one write and one
// read of a quarter of the image for stride 2).
#include "conv_common.hpp"
#include "gemm_common.hpp"

namespace th {

// out[row][ow] = x[n][c][oh * stride_h][ow * stride_w], row = (n * C + c) * HO + oh; four outputs per thread.
// PAIRS: horizontal stride 2 over contiguous, aligned rows: the eight columns the four outputs come from are one load.
template <class T, bool PAIRS>
__global__ __launch_bounds__(256) void conv_subsample4_kernel(const T* x, T* out, ConvProblem p, FastDiv div_quads, FastDiv div_ho, FastDiv div_c, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    uint32_t row, quad, nc, oh, n, c;
    div_quads.divmod(idx, row, quad);
    div_ho.divmod(row, nc, oh);
    div_c.divmod(nc, n, c);
    const T* src = x + static_cast<int64_t>(n) * p.xs[0] + static_cast<int64_t>(c) * p.xs[1] + static_cast<int64_t>(oh * p.stride_h) * p.xs[2] +
                   static_cast<int64_t>(quad * 4 * p.stride_w) * p.xs[3];
    T v[4];
    if constexpr (PAIRS) {
        using Eight = std::conditional_t<sizeof(T) == 2, uint4, ulonglong4>;
        T in[8];
        const Eight bits8 = *reinterpret_cast<const Eight*>(src);
        __builtin_memcpy(in, &bits8, sizeof(Eight));
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = in[2 * e];
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = src[static_cast<int64_t>(e * p.stride_w) * p.xs[3]];
    }
    using Quad = std::conditional_t<sizeof(T) == 2, uint2, uint4>;
    Quad bits;
    __builtin_memcpy(&bits, v, sizeof(Quad));
    *reinterpret_cast<Quad*>(out + static_cast<int64_t>(row) * p.WO + quad * 4) = bits;
}

// Pixel counts that are not a multiple of 16 bytes (14 x 14, 7 x 7 ...): ONE product O x C . C x (N * pitch), pitch the
// count rounded up to 16 bytes, does the whole batch on whole tiles (a product per image would have 200 or 56 columns) and
// stores its columns image by image (GemmProblem::c_group), straight into y.  Without a stride it also reads the images
// where they lie (GemmProblem::b_group_stride).  With one, or when a channel's pixels are not one run of memory, the
// sampled pixels of every (image, channel) first go to rows of `pitch` elements (the rest zeros), channel by channel with
// the images side by side:
// out[(c * N + n) * pitch + pix] = x[n][c][oh * stride_h][ow * stride_w], pix = oh * WO + ow; 16 bytes per thread.
template <class T, bool PLANE>
__global__ __launch_bounds__(256) void conv_repitch_kernel(const T* x, T* out, ConvProblem p, uint32_t pixels, uint32_t pitch, FastDiv div_groups, FastDiv div_c,
                                                           FastDiv div_wo, uint32_t total) {
    constexpr int E = 16 / sizeof(T);
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    uint32_t row, group, n, c, oh, ow;
    div_groups.divmod(idx, row, group);
    div_c.divmod(row, n, c);
    const T* plane = x + static_cast<int64_t>(n) * p.xs[0] + static_cast<int64_t>(c) * p.xs[1];
    uint4 bits;
    if (PLANE && group * E + E <= pixels) {
        // no stride, rows that follow each other: the pixels of a channel are one run of memory
        typedef unsigned int uint4_any __attribute__((ext_vector_type(4), aligned(2)));   // 16 bytes at any element
        const uint4_any run = *reinterpret_cast<const uint4_any*>(plane + group * E);
        __builtin_memcpy(&bits, &run, 16);
    } else {
        div_wo.divmod(group * E, oh, ow);
        T v[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const bool live = group * E + e < pixels;
            v[e] = live ? plane[static_cast<int64_t>(oh * p.stride_h) * p.xs[2] + static_cast<int64_t>(ow * p.stride_w) * p.xs[3]] : T{};
            if (++ow == p.WO) { ow = 0; ++oh; }
        }
        __builtin_memcpy(&bits, v, 16);
    }
    *reinterpret_cast<uint4*>(out + (static_cast<size_t>(c) * p.N + n) * pitch + group * E) = bits;
}

template <class T>
int product(const GemmProblem& g, int dtype, const void* a, const void* b, void* c, hipStream_t stream) {
    if constexpr (std::is_same_v<T, float>) return gemm_mfma_f32(g, static_cast<const float*>(a), static_cast<const float*>(b), static_cast<float*>(c), stream);
    else return gemm_mfma_16bit(g, dtype, a, b, c, stream);
}

template <class T>
int run_pointwise(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (p.KH != 1 || p.KW != 1 || p.pad_h != 0 || p.pad_w != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.has_bias && p.bs != 1 && p.O > 1) return TANNIC_UNSUPPORTED_DTYPE;   // the product reads its row bias as a dense vector
    if (p.N == 0 || p.O == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    if (p.C == 0) return TANNIC_UNSUPPORTED_DTYPE;
    // the kernel tensor as a K-contiguous O x C matrix; the result as row-major O x (HO*WO) per image
    if (p.ws[1] != 1) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.ys[3] != 1 || p.ys[2] != static_cast<int64_t>(p.WO)) return TANNIC_UNSUPPORTED_DTYPE;
    const uint64_t pixels = static_cast<uint64_t>(p.HO) * p.WO;
    if (pixels >= (1ull << 31) || p.N > 65535) return TANNIC_UNSUPPORTED_DTYPE;
    GemmProblem g{};
    g.M = p.O;
    g.N = static_cast<uint32_t>(pixels);
    g.K = p.C;
    g.a_rs = p.ws[0];
    g.a_cs = 1;
    g.b_cs = 1;
    g.c_rs = p.ys[1];
    g.batch_rank = 1;
    g.batches = p.N;
    for (int d = 0; d < 6; ++d) {
        g.batch_extent[d] = 1;
        g.a_bs[d] = g.b_bs[d] = g.c_bs[d] = 0;
    }
    g.batch_extent[0] = p.N;
    g.c_bs[0] = p.ys[0];
    g.row_bias = bias;
    const bool dense = p.stride_h == 1 && p.stride_w == 1;
    constexpr int E = 16 / sizeof(T);   // elements per 16 bytes
    if (pixels % E != 0) {
        // rows of pixels that do not start at multiples of 16 bytes: through rows of a rounded-up pitch (see conv_repitch_kernel)
        if (p.ws[0] % E != 0 || p.C % E != 0 || reinterpret_cast<uintptr_t>(w) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
        const uint32_t pitch = static_cast<uint32_t>((pixels + E - 1) / E * E), groups = pitch / E;
        const uint64_t in_rows = static_cast<uint64_t>(p.N) * p.C, out_rows = static_cast<uint64_t>(p.N) * p.O;
        if (in_rows * groups >= (1ull << 31) || out_rows * groups >= (1ull << 31) || static_cast<uint64_t>(p.N) * pitch >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
        const bool plane = dense && p.xs[3] == 1 && p.xs[2] == static_cast<int64_t>(p.W) && reinterpret_cast<uintptr_t>(x) % sizeof(T) == 0;
        const uint64_t columns = static_cast<uint64_t>(p.N) * pitch;
        // one product O x C . C x (N * pitch) for the whole batch; the columns of image n go to y[n], rows p.ys[1] apart
        g.N = static_cast<uint32_t>(columns);
        g.batch_rank = 0;
        g.batches = 1;
        g.batch_extent[0] = 1;
        g.b_bs[0] = g.c_bs[0] = 0;
        g.c_rs = p.ys[1];
        g.c_group = pitch;
        g.c_group_live = static_cast<uint32_t>(pixels);
        g.c_group_stride = p.ys[0];
        g.c_group_div = FastDiv(pitch);
        if (plane && p.C <= 256) {
            // The pixels of a channel are one run of memory and there are few channels: the product reads the images where
            // they lie, its loaders taking 16-byte pieces at whatever address they start.  (Those loads are slower than
            // aligned ones and the kernel that knows them walks all of K in one block; batch 32, fp16: 256 -> 1024 over
            // 14 x 14 16.6 against 18.4 us through re-pitched rows, but 1024 -> 256 28 against 22 us, 2048 -> 512 over
            // 7 x 7 53 against 26 us.)
            g.b_rs = p.xs[1];
            g.b_group_stride = p.xs[0];
            const int direct = product<T>(g, dtype, w, x, y, stream);
            if (direct != TANNIC_UNSUPPORTED_DTYPE) return direct;
            g.b_group_stride = 0;
        }
        T* dense_x = nullptr;
        if (scratch_acquire(reinterpret_cast<void**>(&dense_x), in_rows * pitch * sizeof(T), stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
        const uint32_t total_in = static_cast<uint32_t>(in_rows * groups);
        if (plane)
            hipLaunchKernelGGL((conv_repitch_kernel<T, true>), dim3((total_in + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(x), dense_x, p,
                               static_cast<uint32_t>(pixels), pitch, FastDiv(groups), FastDiv(p.C), FastDiv(p.WO), total_in);
        else
            hipLaunchKernelGGL((conv_repitch_kernel<T, false>), dim3((total_in + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(x), dense_x, p,
                               static_cast<uint32_t>(pixels), pitch, FastDiv(groups), FastDiv(p.C), FastDiv(p.WO), total_in);
        int status = launch_status("conv_repitch_kernel");
        if (status == TANNIC_SUCCESS) {
            g.b_rs = static_cast<int64_t>(columns);
            status = product<T>(g, dtype, w, dense_x, y, stream);
            if (status == TANNIC_UNSUPPORTED_DTYPE) {
                set_error_text("conv2d: internal: the 1x1 product refused a problem its caller had checked");
                status = TANNIC_ERROR;
            }
        }
        scratch_release(dense_x, stream);
        return status;
    }
    if (dense) {
        if (p.xs[3] != 1 || p.xs[2] != static_cast<int64_t>(p.W)) return TANNIC_UNSUPPORTED_DTYPE;
        g.b_rs = p.xs[1];
        g.b_bs[0] = p.xs[0];
        return product<T>(g, dtype, w, x, y, stream);
    }
    // strided: gather first.  The product's own conditions are checked before any work is queued.
    if (p.WO % 4 != 0 || pixels % E != 0 || p.ws[0] % E != 0 || p.C % E != 0 || reinterpret_cast<uintptr_t>(w) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    const uint64_t rows = static_cast<uint64_t>(p.N) * p.C * p.HO, quads = rows * (p.WO / 4);
    if (quads >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    T* dense_x = nullptr;
    if (scratch_acquire(reinterpret_cast<void**>(&dense_x), rows * p.WO * sizeof(T), stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
    // eight source columns per thread in one load: they must exist (the last group may reach one column past the last
    // sampled one) and start at a multiple of the load size
    const bool pairs = p.stride_w == 2 && p.xs[3] == 1 && static_cast<uint64_t>(p.WO) * 2 <= p.W && p.xs[2] % 8 == 0 &&
                       p.xs[1] % 8 == 0 && p.xs[0] % 8 == 0 && reinterpret_cast<uintptr_t>(x) % (8 * sizeof(T)) == 0;
    if (pairs)
        hipLaunchKernelGGL((conv_subsample4_kernel<T, true>), dim3((quads + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(x), dense_x, p, FastDiv(p.WO / 4),
                           FastDiv(p.HO), FastDiv(p.C), static_cast<uint32_t>(quads));
    else
        hipLaunchKernelGGL((conv_subsample4_kernel<T, false>), dim3((quads + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(x), dense_x, p, FastDiv(p.WO / 4),
                           FastDiv(p.HO), FastDiv(p.C), static_cast<uint32_t>(quads));
    int status = launch_status("conv_subsample4_kernel");
    if (status == TANNIC_SUCCESS) {
        g.b_rs = static_cast<int64_t>(pixels);
        g.b_bs[0] = static_cast<int64_t>(p.C) * static_cast<int64_t>(pixels);
        status = product<T>(g, dtype, w, dense_x, y, stream);
        // the conditions above are the product's: a refusal here would leave the result unwritten
        if (status == TANNIC_UNSUPPORTED_DTYPE) {
            set_error_text("conv2d: internal: the 1x1 product refused a problem its caller had checked");
            status = TANNIC_ERROR;
        }
    }
    scratch_release(dense_x, stream);
    return status;
}

int conv2d_pointwise(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run_pointwise<f16>(p, dtype, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_pointwise<bf16>(p, dtype, x, w, bias, y, stream);
    if (dtype == TANNIC_FLOAT32) return run_pointwise<float>(p, dtype, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
