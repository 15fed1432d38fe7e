// conv2d for fp16 / bf16 / fp32 signals with few output pixels per image and many channels (the last stages of a ResNet:
// 3x3 over 7 x 7 with 512 channels): unfold the whole batch, then ONE matrix product.
//
// A tile of the patch kernels (conv2d_k3.hip) is one image's pixels, 49 of them in a tile made for 256, and every block
// regroups the weights of its 64 output channels again, 590 KB for 512 channels.  With so few pixels the unfolded
// operand is small instead (K x N x pixels: 16.5 MB for the layer above at batch 32), so it is written out,
//   col[k][n * pitch + pix] = x[n][c][oh * stride_h + kh - pad_h][ow * stride_w + kw - pad_w]   (zero in the padding),
// k = (c, kh, kw) in the kernel tensor's own order, pitch = pixels rounded up to 16 bytes, images side by side, and
// (O x N * pitch) = w (O x K) . col runs on the matrix-multiply kernels with the bias as per-row start value and its
// columns stored image by image, straight into y (GemmProblem::c_group).  Sums run over k in the reference's order
// (src/cpu/conv2d.cpp:45-60).
#include "conv_common.hpp"
#include "gemm_common.hpp"

namespace th {

// 16 bytes (eight or four pixels of one k and image) per thread
template <class T>
__global__ __launch_bounds__(256) void conv_unfold_batch_kernel(const T* x, T* col, ConvProblem p, uint32_t pixels, uint32_t pitch, FastDiv div_groups, FastDiv div_n,
                                                            FastDiv div_wo, FastDiv div_taps, FastDiv div_kw, uint32_t total) {
    constexpr int E = 16 / sizeof(T);
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    // neighbouring threads: the pixel groups, then the taps of one (channel, image) — they all read the same few rows of one plane
    uint32_t rest, plane_id, group, n, c, tap, kh, kw, oh, ow;
    div_groups.divmod(idx, rest, group);
    div_taps.divmod(rest, plane_id, tap);
    div_n.divmod(plane_id, c, n);
    div_kw.divmod(tap, kh, kw);
    const uint32_t row = (c * div_taps.d + tap) * p.N + n;   // k * N + n
    const T* plane = x + static_cast<int64_t>(n) * p.xs[0] + static_cast<int64_t>(c) * p.xs[1];
    div_wo.divmod(group * E, oh, ow);
    T v[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const uint32_t ih = oh * p.stride_h + kh - p.pad_h, iw = ow * p.stride_w + kw - p.pad_w;   // unsigned: above and left of the image are huge
        const bool inside = group * E + e < pixels && ih < p.H && iw < p.W;
        v[e] = inside ? plane[static_cast<int64_t>(ih) * p.xs[2] + static_cast<int64_t>(iw) * p.xs[3]] : T{};
        if (++ow == p.WO) { ow = 0; ++oh; }
    }
    uint4 bits;
    __builtin_memcpy(&bits, v, 16);
    *reinterpret_cast<uint4*>(col + static_cast<size_t>(row) * pitch + group * E) = bits;
}

// dst[o][k] = k < K ? src[o][k] : 0 for rows of K and of Kp elements
template <class T>
__global__ __launch_bounds__(256) void conv_pad_rows_kernel(const T* src, T* dst, uint32_t K, uint32_t Kp, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const uint32_t o = idx / Kp, k = idx % Kp;
    dst[idx] = k < K ? src[static_cast<size_t>(o) * K + k] : T{};
}

template <class T>
__global__ __launch_bounds__(256) void conv_zero_kernel(T* dst, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx < total) dst[idx] = T{};
}

// ANY_SIZE: as the last kernel before the general ones, for whatever the specialised kernels have refused, as long as
// the unfolded operand stays small enough to be worth writing out.
template <class T, bool ANY_SIZE>
static int run_unfold_batch(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (p.has_bias && p.bs != 1 && p.O > 1) return TANNIC_UNSUPPORTED_DTYPE;   // the product reads its row bias as a dense vector
    if (p.N == 0 || p.O == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    constexpr int E = 16 / sizeof(T);
    const uint64_t K = static_cast<uint64_t>(p.C) * p.KH * p.KW, pixels = static_cast<uint64_t>(p.HO) * p.WO;
    // Where this pays: few pixels per image (a tile of the patch kernels would be mostly empty), a long K, and enough
    // columns in all for whole tiles of the product.
    // (ANY_SIZE, fp16, us against the general tile kernel: K = 2352 49 / 104, 648 13 / 38, 600 22 / 31, 360 23 / 26, but 216 20 / 15,
    // 144 33 / 25, 72 25 / 16: with a short K the unfolded operand is as large as the work)
    // More pixels per image, but few in the whole batch, leave the patch kernels with a handful of blocks that each walk
    // all of K, where the product shares K between blocks; signals one row high (conv1d) also fill their patches badly.
    // (fp16, us patches / unfolded: batch 8 256 -> 256 1x7 over 256 75 / 23, batch 32 512 -> 128 1x3 over 256 76 / 33,
    // batch 1 512 -> 512 5x5 over 28 x 28 119 / 42, batch 8 256 -> 128 5x5 over 14 x 14 63 / 37; but batch 8 over 28 x 28,
    // 6272 pixels, 64 / 67 and 139 / 207; with a stride of 2 and 512 channels, batch 32 over 28 x 28, 136 / 80)
    const uint64_t batch_pixels = p.N * pixels;
    const bool few = pixels <= 100 ? K >= 512
                                   : (K >= 768 && (batch_pixels <= 2048 || (p.HO == 1 && batch_pixels <= 8192))) || (K >= 2304 && batch_pixels <= 4096) ||
                                         (K >= 4608 && batch_pixels <= 8192 && p.stride_h > 1 && p.stride_w > 1);
    // (float64: the alternative is the scalar kernel, one thread per result walking K alone.  Six output channels sharing an
    // unfolded column already beat it at full occupancy, and with few results in all it is bound by that walk: 4 images
    // 349 -> 8 channels 7x7 over 8 x 8, 32 results under a K of 17101, 2202 us.  The float64 product reads single doubles
    // and asks nothing of K or of where the weights lie.)
    constexpr bool f64 = std::is_same_v<T, double>;
    if (f64 ? (p.O < 6 && batch_pixels * p.O >= 65536) : (ANY_SIZE ? K < 320 : !few)) return TANNIC_UNSUPPORTED_DTYPE;
    if (K >= (1u << 24) || pixels >= (1u << 24)) return TANNIC_UNSUPPORTED_DTYPE;
    const uint32_t pitch = static_cast<uint32_t>((pixels + E - 1) / E * E);
    // (fewer columns than two tiles are wide stay with the patch kernels, unless the results are so few that the product
    // runs a workgroup per 4 x 4 of them: one image 672 -> 8 4x4 over 8 x 8, 200 results under a K of 10752, 197 us on patches)
    if (!ANY_SIZE && static_cast<uint64_t>(p.N) * pitch < 256 && static_cast<uint64_t>(p.O) * p.N * pitch > 8192) return TANNIC_UNSUPPORTED_DTYPE;
    // The unfolded operand is kept small: ANY_SIZE takes the images in runs whose unfolded operand stays within the
    // limit (one image's may reach four times that), one product per run, all through the same buffer.
    const uint64_t limit = (ANY_SIZE ? 256ull : 512ull) << 20, image_bytes = K * pitch * sizeof(T);
    uint32_t run = p.N;
    if (image_bytes * p.N > limit) {
        if (!ANY_SIZE || image_bytes > 4 * limit) return TANNIC_UNSUPPORTED_DTYPE;
        run = static_cast<uint32_t>(limit / image_bytes);
        if (run == 0) run = 1;
    }
    const uint64_t columns = static_cast<uint64_t>(run) * pitch;
    if (columns >= (1ull << 31) || K * run * (pitch / E) >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    // the kernel tensor as a K-contiguous O x K matrix, the result as pixel-contiguous rows
    if (p.ws[3] != 1 || p.ws[2] != static_cast<int64_t>(p.KW) || p.ws[1] != static_cast<int64_t>(p.KH) * p.KW || p.ws[0] != static_cast<int64_t>(K) ||
        (!f64 && K % E == 0 && reinterpret_cast<uintptr_t>(w) % 16 != 0))
        return TANNIC_UNSUPPORTED_DTYPE;
    if (p.ys[3] != 1 || p.ys[2] != static_cast<int64_t>(p.WO)) return TANNIC_UNSUPPORTED_DTYPE;
    // A K that no 16 bytes divide would leave the rows of the weights misaligned and the product on the tiles for operands
    // at any address, which do not share K: the weights are copied into rows of Kp elements, zeros at their ends, and the
    // unfolded operand gets Kp - K rows of zeros (fp32 405 -> 32 7x7 s3 over 126 x 126, K = 19845: 1523 us on those tiles).
    const uint32_t Kp = f64 ? static_cast<uint32_t>(K) : static_cast<uint32_t>((K + E - 1) / E * E);
    if (static_cast<uint64_t>(p.O) * Kp >= (1ull << 31) || static_cast<uint64_t>(Kp - K) * columns >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    T* padded = nullptr;
    if (Kp != K) {
        if (scratch_acquire(reinterpret_cast<void**>(&padded), static_cast<size_t>(p.O) * Kp * sizeof(T), stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
        const uint32_t total = p.O * Kp;
        hipLaunchKernelGGL((conv_pad_rows_kernel<T>), dim3((total + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(w), padded, static_cast<uint32_t>(K), Kp, total);
        if (launch_status("conv_pad_rows_kernel") != TANNIC_SUCCESS) {
            scratch_release(padded, stream);
            return TANNIC_ERROR;
        }
    }
    const void* weights = padded ? static_cast<const void*>(padded) : w;
    T* col = nullptr;
    if (scratch_acquire(reinterpret_cast<void**>(&col), static_cast<size_t>(Kp) * columns * sizeof(T), stream) != TANNIC_SUCCESS) {
        if (padded) scratch_release(padded, stream);
        return TANNIC_ERROR;
    }
    int status = TANNIC_SUCCESS;
    for (uint32_t n0 = 0; n0 < p.N && status == TANNIC_SUCCESS; n0 += run) {
        ConvProblem part = p;
        part.N = p.N - n0 < run ? p.N - n0 : run;
        const T* x_part = static_cast<const T*>(x) + static_cast<int64_t>(n0) * p.xs[0];
        T* y_part = static_cast<T*>(y) + static_cast<int64_t>(n0) * p.ys[0];
        const uint64_t part_columns = static_cast<uint64_t>(part.N) * pitch;
        const uint32_t groups = pitch / E, total = static_cast<uint32_t>(K * part.N * groups);
        hipLaunchKernelGGL((conv_unfold_batch_kernel<T>), dim3((total + 255) / 256), dim3(256), 0, stream, x_part, col, part, static_cast<uint32_t>(pixels), pitch,
                           FastDiv(groups), FastDiv(part.N), FastDiv(p.WO), FastDiv(p.KH * p.KW), FastDiv(p.KW), total);
        status = launch_status("conv_unfold_batch_kernel");
        if (status != TANNIC_SUCCESS) break;
        if (Kp != K) {
            const uint32_t tail = static_cast<uint32_t>((Kp - K) * part_columns);
            hipLaunchKernelGGL((conv_zero_kernel<T>), dim3((tail + 255) / 256), dim3(256), 0, stream, col + static_cast<size_t>(K) * part_columns, tail);
            status = launch_status("conv_zero_kernel");
            if (status != TANNIC_SUCCESS) break;
        }
        GemmProblem g{};
        g.M = p.O;
        g.N = static_cast<uint32_t>(part_columns);
        g.K = Kp;
        g.a_rs = padded ? static_cast<int64_t>(Kp) : p.ws[0];
        g.a_cs = 1;
        g.b_rs = static_cast<int64_t>(part_columns);
        g.b_cs = 1;
        // the columns of image n go to y[n]: rows p.ys[1] apart, images p.ys[0]
        g.c_rs = p.ys[1];
        g.c_group = pitch;
        g.c_group_live = static_cast<uint32_t>(pixels);
        g.c_group_stride = p.ys[0];
        g.c_group_div = FastDiv(pitch);
        g.batch_rank = 0;
        g.batches = 1;
        for (int d = 0; d < 6; ++d) {
            g.batch_extent[d] = 1;
            g.a_bs[d] = g.b_bs[d] = g.c_bs[d] = 0;
        }
        g.row_bias = bias;
        // few results under a long K (a handful of pixels in all): a workgroup per 4 x 4 of them instead of one tile walking K
        status = gemm_few_results(g, dtype, weights, col, y_part, stream);
        if (status != TANNIC_UNSUPPORTED_DTYPE) continue;
        if constexpr (f64) status = gemm_mfma_f64(g, static_cast<const double*>(weights), reinterpret_cast<const double*>(col), static_cast<double*>(y_part), stream);
        else if constexpr (std::is_same_v<T, float>) status = gemm_mfma_f32(g, static_cast<const float*>(weights), reinterpret_cast<const float*>(col), static_cast<float*>(y_part), stream);
        else status = gemm_mfma_16bit(g, dtype, weights, col, y_part, stream);
        if (status == TANNIC_UNSUPPORTED_DTYPE && n0 != 0) {
            // (the first run of images decides: a refusal there leaves the convolution to the next kernel, nothing stored yet)
            set_error_text("conv2d: internal: the unfolded product refused a run of images after it had taken the first");
            status = TANNIC_ERROR;
        }
    }
    scratch_release(col, stream);
    if (padded) scratch_release(padded, stream);
    return status;
}

int conv2d_unfold_batch(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    // float64 has this path and the scalar kernel only (a 1x1 kernel's "unfolding" is a copy of the signal)
    if (dtype == TANNIC_FLOAT64) return run_unfold_batch<double, true>(p, dtype, x, w, bias, y, stream);
    if (p.KH == 1 && p.KW == 1) return TANNIC_UNSUPPORTED_DTYPE;   // conv2d_pointwise.hip: no unfolding needed
    if (dtype == TANNIC_FLOAT16) return run_unfold_batch<f16, false>(p, dtype, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_unfold_batch<bf16, false>(p, dtype, x, w, bias, y, stream);
    if (dtype == TANNIC_FLOAT32) {
        const int status = run_unfold_batch<float, false>(p, dtype, x, w, bias, y, stream);
        if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
        // fp32 has no patch kernels, and the gathering tiles (conv2d_gather32.hip) are few when the whole batch has few pixels:
        // each walks all of K alone, where the product over the unfolded batch shares K between blocks
        // (batch 8, us gathered / unfolded: 64 -> 64 7x7 over 14 x 14 175 / 34, 256 -> 128 3x3 124 / 38, 64 -> 64 3x3 over
        // 28 x 28 35 / 27; at batch 32 over 28 x 28, 25088 pixels, 38 / 53 and 186 / 269)
        if (static_cast<uint64_t>(p.N) * p.HO * p.WO <= 8192) return run_unfold_batch<float, true>(p, dtype, x, w, bias, y, stream);
        return TANNIC_UNSUPPORTED_DTYPE;
    }
    return TANNIC_UNSUPPORTED_DTYPE;
}

int conv2d_unfold_batch_any(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (p.KH == 1 && p.KW == 1) return TANNIC_UNSUPPORTED_DTYPE;
    if (dtype == TANNIC_FLOAT16) return run_unfold_batch<f16, true>(p, dtype, x, w, bias, y, stream);
    if (dtype == TANNIC_BFLOAT16) return run_unfold_batch<bf16, true>(p, dtype, x, w, bias, y, stream);
    // (fp32 comes here after its gathering tiles and its own unfolding have refused: a K beyond the tiles' table)
    if (dtype == TANNIC_FLOAT32) return run_unfold_batch<float, true>(p, dtype, x, w, bias, y, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

}  // namespace th
