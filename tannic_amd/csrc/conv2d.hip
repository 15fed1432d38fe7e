// conv2d entry points: checks, dtype table, direct kernel.
//
// Status rules follow src/cpu/conv2d.cpp:116-197 (ERROR on rank or shape
// mismatch), the table :221-253 (same dtype for signal and kernel).  fp16, bf16
// and fp32 problems with contiguous operands go to the implicit-GEMM MFMA
// kernel (conv2d_mfma.hip); everything else runs the direct kernel below, which
// honours arbitrary strides and walks the taps in the CPU path's order
// (ci, kh, kw).  16-bit types accumulate in fp32 and round once.
#include "conv_common.hpp"

namespace th {

template <class T>
__global__ __launch_bounds__(256) void conv2d_direct_kernel(const T* x, const T* w, const T* bias, T* y, ConvProblem p, uint32_t total) {
    using Acc = std::conditional_t<is_16bit<T>::value, float, std::conditional_t<std::is_integral_v<T>, std::make_unsigned_t<std::conditional_t<std::is_integral_v<T>, T, int>>, T>>;
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    uint32_t rem = idx;
    const uint32_t ow = rem % p.WO; rem /= p.WO;
    const uint32_t oh = rem % p.HO; rem /= p.HO;
    const uint32_t co = rem % p.O;
    const uint32_t n = rem / p.O;
    Acc acc = p.has_bias ? static_cast<Acc>(widen(bias[static_cast<int64_t>(co) * p.bs])) : Acc(0);
    const int64_t bh = static_cast<int64_t>(oh) * p.stride_h - p.pad_h;
    const int64_t bw = static_cast<int64_t>(ow) * p.stride_w - p.pad_w;
    for (uint32_t ci = 0; ci < p.C; ++ci)
        for (uint32_t kh = 0; kh < p.KH; ++kh) {
            const int64_t ih = bh + kh;
            if (ih < 0 || ih >= p.H) continue;
            for (uint32_t kw = 0; kw < p.KW; ++kw) {
                const int64_t iw = bw + kw;
                if (iw < 0 || iw >= p.W) continue;
                const T xv = x[n * p.xs[0] + ci * p.xs[1] + ih * p.xs[2] + iw * p.xs[3]];
                const T wv = w[co * p.ws[0] + ci * p.ws[1] + kh * p.ws[2] + kw * p.ws[3]];
                acc += static_cast<Acc>(widen(xv)) * static_cast<Acc>(widen(wv));
            }
        }
    y[n * p.ys[0] + co * p.ys[1] + oh * p.ys[2] + ow * p.ys[3]] = narrow<T>(acc);
}

template <class T>
int run_direct(const ConvProblem& p, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    const size_t total = static_cast<size_t>(p.N) * p.O * p.HO * p.WO;
    if (total == 0) return TANNIC_SUCCESS;
    if (total >= (1ull << 31)) {
        set_error_text("conv2d: output of 2^31 elements or more is not supported");
        return TANNIC_ERROR;
    }
    hipLaunchKernelGGL((conv2d_direct_kernel<T>), dim3((total + 255) / 256), dim3(256), 0, stream, static_cast<const T*>(x),
                       static_cast<const T*>(w), static_cast<const T*>(bias), static_cast<T*>(y), p, static_cast<uint32_t>(total));
    return launch_status("conv2d_direct_kernel");
}

static int conv2d_entry(const tannic_tensor_t* x, const tannic_tensor_t* w, const tannic_tensor_t* bias, tannic_tensor_t* y,
                        tannic_stream_t stream, const size_t pad[2], const size_t stride[2]) {
    if (!x || !w || !y || !pad || !stride) return TANNIC_ERROR;
    if (!have_storage(x, w, bias, y)) return TANNIC_ERROR;
    // dispatch on (signal, kernel) dtype first: unsupported pairs report
    // UNSUPPORTED_DTYPE before any shape check, as the table lookup does
    if (x->dtype != w->dtype) return TANNIC_UNSUPPORTED_DTYPE;
    switch (x->dtype) {
        case TANNIC_INT8: case TANNIC_INT16: case TANNIC_INT32: case TANNIC_INT64:
        case TANNIC_FLOAT16: case TANNIC_BFLOAT16: case TANNIC_FLOAT32: case TANNIC_FLOAT64: break;
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
    if (x->rank != 4 || w->rank != 4 || y->rank != 4 || (bias && bias->rank != 1)) return TANNIC_ERROR;
    if (!destination_is(y, x->dtype, "conv2d: the result's dtype is not the signal's")) return TANNIC_ERROR;
    if (bias && bias->dtype != x->dtype) {
        set_error_text("conv2d: the bias's dtype is not the signal's");
        return TANNIC_ERROR;
    }
    if (stride[0] == 0 || stride[1] == 0) return TANNIC_ERROR;
    const size_t N = x->shape.sizes[0], C = x->shape.sizes[1], H = x->shape.sizes[2], W = x->shape.sizes[3];
    const size_t O = w->shape.sizes[0], KC = w->shape.sizes[1], KH = w->shape.sizes[2], KW = w->shape.sizes[3];
    if (C != KC || (bias && bias->shape.sizes[0] != O)) return TANNIC_ERROR;
    if (H + 2 * pad[0] < KH || W + 2 * pad[1] < KW) return TANNIC_ERROR;
    const size_t HO = (H + 2 * pad[0] - KH) / stride[0] + 1;
    const size_t WO = (W + 2 * pad[1] - KW) / stride[1] + 1;
    if (y->shape.sizes[0] != N || y->shape.sizes[1] != O || y->shape.sizes[2] != HO || y->shape.sizes[3] != WO) return TANNIC_ERROR;
    const size_t limit = 1ull << 31;
    if (N >= limit || C >= limit || H >= limit || W >= limit || O >= limit || KH >= limit || KW >= limit || pad[0] >= limit ||
        pad[1] >= limit || stride[0] >= limit || stride[1] >= limit) {
        set_error_text("conv2d: dimension of 2^31 or more");
        return TANNIC_ERROR;
    }
    ConvProblem p{};
    p.N = N; p.C = C; p.H = H; p.W = W; p.O = O; p.KH = KH; p.KW = KW; p.HO = HO; p.WO = WO;
    p.pad_h = pad[0]; p.pad_w = pad[1]; p.stride_h = stride[0]; p.stride_w = stride[1];
    for (int d = 0; d < 4; ++d) {
        p.xs[d] = x->strides.sizes[d];
        p.ws[d] = w->strides.sizes[d];
        p.ys[d] = y->strides.sizes[d];
    }
    p.has_bias = bias != nullptr;
    // the bias is read through its stride (a column of a matrix is a valid bias; the CPU path reads b[co], src/cpu/conv2d.cpp:86)
    p.bs = bias ? bias->strides.sizes[0] : 0;
    const void* pb = bias ? bias->address : nullptr;
    hipStream_t s = as_stream(stream);
    // Kernels in order of preference.  A 1x1 kernel has no tap to amortise a staged patch over: its weights stay in
    // registers when they fit (conv2d_k1.hip), otherwise it is a matrix product per image (conv2d_pointwise.hip).
    int status = TANNIC_UNSUPPORTED_DTYPE;
    const bool pointwise = p.KH == 1 && p.KW == 1;
    if (pointwise) status = conv2d_k1(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (pointwise && status == TANNIC_UNSUPPORTED_DTYPE) status = conv2d_pointwise(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    if (!pointwise) status = conv2d_stem(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    // few pixels per image under many channels: the unfolded batch as one product (before the patch kernels, whose tile would be mostly empty)
    if (!pointwise || x->dtype == TANNIC_FLOAT64) status = conv2d_unfold_batch(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    if (!pointwise) status = conv2d_k3(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    if (!pointwise) status = conv2d_resident(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    if (!pointwise) status = conv2d_patch(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    status = conv2d_gather32(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    status = conv2d_unfold(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    // 16-bit shapes none of the above takes: unfolded and multiplied, or the general tile kernel.  Large images go to
    // the tile kernel first: their unfolded operand is hundreds of megabytes under few output channels
    // (fp16, batch 8, 7x7, us unfolded / tiles: 64 -> 64 over 112 x 112 468 / 303, 24 -> 48 168 / 123, over 56 x 56 110 / 139, 48 / 56).
    const bool large_images = static_cast<uint64_t>(p.HO) * p.WO > 8192;
    if (large_images) status = conv2d_mfma(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    status = conv2d_unfold_batch_any(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    if (!large_images) status = conv2d_mfma(p, x->dtype, x->address, w->address, pb, y->address, s);
    if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    switch (x->dtype) {
        case TANNIC_INT8: return run_direct<int8_t>(p, x->address, w->address, pb, y->address, s);
        case TANNIC_INT16: return run_direct<int16_t>(p, x->address, w->address, pb, y->address, s);
        case TANNIC_INT32: return run_direct<int32_t>(p, x->address, w->address, pb, y->address, s);
        case TANNIC_INT64: return run_direct<int64_t>(p, x->address, w->address, pb, y->address, s);
        case TANNIC_FLOAT16: return run_direct<f16>(p, x->address, w->address, pb, y->address, s);
        case TANNIC_BFLOAT16: return run_direct<bf16>(p, x->address, w->address, pb, y->address, s);
        case TANNIC_FLOAT32: return run_direct<float>(p, x->address, w->address, pb, y->address, s);
        case TANNIC_FLOAT64: return run_direct<double>(p, x->address, w->address, pb, y->address, s);
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
}

// conv1d (src/cpu/conv1d.cpp:17-125) is conv2d on signals one row high: x[N,C,L] as [N,C,1,L], w[O,C,K] as
// [O,C,1,K], same loops in the same order (channel, tap), same status rules with rank 3 in place of 4.
static int conv1d_entry(const tannic_tensor_t* x, const tannic_tensor_t* w, tannic_tensor_t* y, tannic_stream_t stream, size_t pad, size_t stride) {
    if (!x || !w || !y) return TANNIC_ERROR;
    if (!have_storage(x, w, y)) return TANNIC_ERROR;
    if (x->dtype != w->dtype) return TANNIC_UNSUPPORTED_DTYPE;
    switch (x->dtype) {
        case TANNIC_INT8: case TANNIC_INT16: case TANNIC_INT32: case TANNIC_INT64:
        case TANNIC_FLOAT16: case TANNIC_BFLOAT16: case TANNIC_FLOAT32: case TANNIC_FLOAT64: break;
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
    if (x->rank != 3 || w->rank != 3 || y->rank != 3) return TANNIC_ERROR;
    if (!destination_is(y, x->dtype, "conv1d: the result's dtype is not the signal's")) return TANNIC_ERROR;
    auto with_row = [](const tannic_tensor_t* t) {
        tannic_tensor_t r = *t;
        r.rank = 4;
        r.shape.sizes[3] = t->shape.sizes[2];
        r.strides.sizes[3] = t->strides.sizes[2];
        r.shape.sizes[2] = 1;
        r.strides.sizes[2] = static_cast<int64_t>(t->shape.sizes[2]) * t->strides.sizes[2];
        return r;
    };
    const tannic_tensor_t x4 = with_row(x), w4 = with_row(w);
    tannic_tensor_t y4 = with_row(y);
    const size_t pad2[2] = {0, pad}, stride2[2] = {1, stride};
    return conv2d_entry(&x4, &w4, nullptr, &y4, stream, pad2, stride2);
}

}  // namespace th

extern "C" {
int tannic_hip_conv1d(const tannic_tensor_t* x, const tannic_tensor_t* w, tannic_tensor_t* y, tannic_stream_t stream, size_t pad, size_t stride) {
    return th::conv1d_entry(x, w, y, stream, pad, stride);
}
int tannic_hip_conv2d(const tannic_tensor_t* x, const tannic_tensor_t* w, tannic_tensor_t* y, tannic_stream_t stream,
                      const size_t pad[2], const size_t stride[2]) {
    return th::conv2d_entry(x, w, nullptr, y, stream, pad, stride);
}
int tannic_hip_conv2d_biased(const tannic_tensor_t* x, const tannic_tensor_t* w, const tannic_tensor_t* bias, tannic_tensor_t* y,
                             tannic_stream_t stream, const size_t pad[2], const size_t stride[2]) {
    if (!bias) return TANNIC_ERROR;
    return th::conv2d_entry(x, w, bias, y, stream, pad, stride);
}
}
