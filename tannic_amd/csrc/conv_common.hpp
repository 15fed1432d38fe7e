// Problem description shared by the convolution kernels.
#pragma once

#include "common.hpp"

namespace th {

// NCHW signal, OIHW kernel, cross-correlation with zero padding
// (src/cpu/conv2d.cpp:17-64).  Strides are element strides of each operand.
struct ConvProblem {
    uint32_t N, C, H, W;       // signal
    uint32_t O, KH, KW;        // kernel: O x C x KH x KW
    uint32_t HO, WO;           // output spatial size
    uint32_t pad_h, pad_w, stride_h, stride_w;
    int64_t xs[4], ws[4], ys[4];
    int64_t bs;                // element stride of the bias (the CPU path reads it as 1, src/cpu/conv2d.cpp:86)
    bool has_bias;
};

// Each returns TANNIC_UNSUPPORTED_DTYPE when the problem does not meet its
// conditions, so that the caller can try the next, more general kernel.
int conv2d_k1(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_pointwise(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_stem(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_k3(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_resident(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_patch(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_gather32(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_unfold(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
// few output pixels per image under many channels (fp16, bf16, fp32): the whole batch unfolded side by side, one product
int conv2d_unfold_batch(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_unfold_batch_any(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);
int conv2d_mfma(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream);

}  // namespace th
