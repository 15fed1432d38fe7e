// Implicit-GEMM convolution on MFMA (placeholder body is replaced below).
#include "conv_common.hpp"

namespace th {
int conv2d_mfma(const ConvProblem&, int, const void*, const void*, const void*, void*, hipStream_t) { return TANNIC_UNSUPPORTED_DTYPE; }
}  // namespace th
