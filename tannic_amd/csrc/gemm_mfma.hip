// MFMA matrix-multiply kernels (placeholder bodies are replaced below).
#include "gemm_common.hpp"

namespace th {
int gemm_mfma_16bit(const GemmProblem&, int, const void*, const void*, void*, hipStream_t) { return TANNIC_UNSUPPORTED_DTYPE; }
int gemm_mfma_f32(const GemmProblem&, const float*, const float*, float*, hipStream_t) { return TANNIC_UNSUPPORTED_DTYPE; }
}  // namespace th
