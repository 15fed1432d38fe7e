// conv2d for fp32 signals with kernels larger than 1x1: unfold, then multiply.
//
// The signal is unfolded into col[n][k][pixel], k = (channel, kernel row, kernel
// column) in the kernel tensor's own order and pixels contiguous, which is the
// row-major operand of a matrix product; y[n] (O x pixels) = w (O x K) * col[n]
// then runs on the fp32 MFMA matrix-multiply kernel with the bias as its per-row
// start value.  K is padded to a multiple of 4 with zero rows (and the kernel
// tensor copied into rows of that length when it needs it), so that every row of
// both operands starts at a 16-byte boundary.  Images are processed in groups
// that keep the unfolded copy below a fixed size.
#include "conv_common.hpp"
#include "gemm_common.hpp"

namespace th {

// col[(n * Kp + k) * P + pixel], four consecutive pixels per thread
__global__ __launch_bounds__(256) void conv_unfold_kernel(const float* x, float* col, ConvProblem p, uint32_t n_first, uint32_t Kp, uint32_t K, uint32_t P, FastDiv div_quads,
                                                          FastDiv div_kp, FastDiv div_wo, FastDiv div_taps, FastDiv div_kw, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    uint32_t row, quad, n, k;
    div_quads.divmod(idx, row, quad);
    div_kp.divmod(row, n, k);
    float4 out = float4{0.0f, 0.0f, 0.0f, 0.0f};
    if (k < K) {
        uint32_t c, tap, kh, kw;
        div_taps.divmod(k, c, tap);
        div_kw.divmod(tap, kh, kw);
        const float* src = x + static_cast<int64_t>(n_first + n) * p.xs[0] + static_cast<int64_t>(c) * p.xs[1];
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            uint32_t oh, ow;
            div_wo.divmod(quad * 4 + e, oh, ow);
            const int32_t ih = static_cast<int32_t>(oh * p.stride_h + kh) - static_cast<int32_t>(p.pad_h);
            const int32_t iw = static_cast<int32_t>(ow * p.stride_w + kw) - static_cast<int32_t>(p.pad_w);
            const bool inside = ih >= 0 && ih < static_cast<int32_t>(p.H) && iw >= 0 && iw < static_cast<int32_t>(p.W);
            v[e] = inside ? src[static_cast<int64_t>(ih) * p.xs[2] + static_cast<int64_t>(iw) * p.xs[3]] : 0.0f;
        }
        out = float4{v[0], v[1], v[2], v[3]};
    }
    *reinterpret_cast<float4*>(col + static_cast<size_t>(row) * P + quad * 4) = out;
}

// rows of Kp elements: w[o][c][kh][kw] followed by zeros
__global__ __launch_bounds__(256) void conv_pad_weights_kernel(const float* w, float* out, ConvProblem p, uint32_t Kp, uint32_t K, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const uint32_t o = idx / Kp, k = idx % Kp;
    float v = 0.0f;
    if (k < K) {
        const uint32_t taps = p.KH * p.KW, c = k / taps, tap = k % taps;
        v = w[static_cast<int64_t>(o) * p.ws[0] + static_cast<int64_t>(c) * p.ws[1] + static_cast<int64_t>(tap / p.KW) * p.ws[2] + static_cast<int64_t>(tap % p.KW) * p.ws[3]];
    }
    out[idx] = v;
}

int conv2d_unfold(const ConvProblem& p, int dtype, const void* x, const void* w, const void* bias, void* y, hipStream_t stream) {
    if (dtype != TANNIC_FLOAT32) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.has_bias && p.bs != 1 && p.O > 1) return TANNIC_UNSUPPORTED_DTYPE;   // the product reads its row bias as a dense vector
    if (p.N == 0 || p.O == 0 || p.HO == 0 || p.WO == 0) return TANNIC_SUCCESS;
    const uint64_t K64 = static_cast<uint64_t>(p.C) * p.KH * p.KW, P64 = static_cast<uint64_t>(p.HO) * p.WO;
    // the product's conditions, checked before anything is queued: whole 16-byte groups of pixels, dense result rows
    if (K64 == 0 || K64 >= (1u << 24) || P64 >= (1u << 28) || P64 % 4 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.ys[3] != 1 || p.ys[2] != static_cast<int64_t>(p.WO)) return TANNIC_UNSUPPORTED_DTYPE;
    const uint32_t K = static_cast<uint32_t>(K64), P = static_cast<uint32_t>(P64), Kp = (K + 3) / 4 * 4;
    const bool plain_weights = K == Kp && p.ws[3] == 1 && p.ws[2] == static_cast<int64_t>(p.KW) && p.ws[1] == static_cast<int64_t>(p.KH) * p.KW &&
                               p.ws[0] % 4 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
    // images per group: the unfolded copy stays below 512 MiB (one image at least)
    const uint64_t per_image = static_cast<uint64_t>(Kp) * P * sizeof(float);
    uint64_t group = (512ull << 20) / per_image;
    if (group == 0) group = 1;
    if (group > p.N) group = p.N;
    if (group > 65535) group = 65535;
    if (group * Kp * (P / 4) >= (1ull << 31)) group = ((1ull << 31) - 1) / (static_cast<uint64_t>(Kp) * (P / 4));
    if (group == 0) return TANNIC_UNSUPPORTED_DTYPE;
    const size_t weight_bytes = plain_weights ? 0 : (static_cast<size_t>(p.O) * Kp * sizeof(float) + 255) & ~size_t(255);
    unsigned char* scratch = nullptr;
    if (scratch_acquire(reinterpret_cast<void**>(&scratch), weight_bytes + group * per_image, stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
    float* col = reinterpret_cast<float*>(scratch + weight_bytes);
    const float* wk = static_cast<const float*>(w);
    int64_t w_ld = p.ws[0];
    int status = TANNIC_SUCCESS;
    if (!plain_weights) {
        const uint64_t total = static_cast<uint64_t>(p.O) * Kp;
        if (total >= (1ull << 31)) status = TANNIC_UNSUPPORTED_DTYPE;
        if (status == TANNIC_SUCCESS) {
            hipLaunchKernelGGL(conv_pad_weights_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, static_cast<const float*>(w), reinterpret_cast<float*>(scratch), p, Kp, K,
                               static_cast<uint32_t>(total));
            status = launch_status("conv_pad_weights_kernel");
            wk = reinterpret_cast<const float*>(scratch);
            w_ld = Kp;
        }
    }
    for (uint32_t n0 = 0; n0 < p.N && status == TANNIC_SUCCESS; n0 += static_cast<uint32_t>(group)) {
        const uint32_t count = p.N - n0 < group ? p.N - n0 : static_cast<uint32_t>(group);
        const uint32_t total = static_cast<uint32_t>(static_cast<uint64_t>(count) * Kp * (P / 4));
        hipLaunchKernelGGL(conv_unfold_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, static_cast<const float*>(x), col, p, n0, Kp, K, P, FastDiv(P / 4), FastDiv(Kp),
                           FastDiv(p.WO), FastDiv(p.KH * p.KW), FastDiv(p.KW), total);
        status = launch_status("conv_unfold_kernel");
        if (status != TANNIC_SUCCESS) break;
        GemmProblem g{};
        g.M = p.O;
        g.N = P;
        g.K = Kp;
        g.a_rs = w_ld;
        g.a_cs = 1;
        g.b_rs = P;
        g.b_cs = 1;
        g.c_rs = p.ys[1];
        g.batch_rank = 1;
        g.batches = count;
        for (int d = 0; d < 6; ++d) {
            g.batch_extent[d] = 1;
            g.a_bs[d] = g.b_bs[d] = g.c_bs[d] = 0;
        }
        g.batch_extent[0] = count;
        g.b_bs[0] = static_cast<int64_t>(Kp) * P;
        g.c_bs[0] = p.ys[0];
        g.row_bias = bias;
        status = gemm_mfma_f32(g, wk, col, static_cast<float*>(y) + static_cast<int64_t>(n0) * p.ys[0], stream);
        if (status == TANNIC_UNSUPPORTED_DTYPE) {
            set_error_text("conv2d: internal: the unfolded product refused a problem its caller had checked");
            status = TANNIC_ERROR;
        }
    }
    scratch_release(scratch, stream);
    return status;
}

}  // namespace th
