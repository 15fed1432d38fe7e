/*
 * ref_shim.cpp — C entry points onto the REAL reference CPU backend.  TEST
 * INFRASTRUCTURE ONLY.  Compiled only where /root/reference is mounted, together
 * with the reference's own src/cpu sources (read in place, never copied), into
 * oracle/_ref/libtannic_ref.so.  It forwards to the reference's cpu:: functions
 * so that the restatement in oracle.cpp can be compared with the real thing.
 * It includes the reference's public headers; the struct layouts are asserted
 * to equal the ones of include/tannic_hip.h so that one descriptor serves both.
 *
 * The reference's 16-bit float kernels need <stdfloat> (GCC >= 13), which this
 * image lacks, so they are compiled out of this build (HAS_FLOAT16 = 0) and
 * fp16/bf16 calls return UNSUPPORTED_DTYPE here.
 */
#include <cstddef>
#include "cpu/ops.hpp"
#include "cpu/matmul.hpp"
#include "cpu/conv.hpp"
#include "cpu/argred.hpp"
#include "cpu/cmps.hpp"
#include "cpu/complex.hpp"
#include "cpu/cpy.hpp"
#include "cpu/reps.hpp"
#include "cpu/concat.hpp"
#include "cpu/outer.hpp"
#include "cpu/triang.hpp"
#include "cpu/val.hpp"

static_assert(sizeof(tensor_t) == 176 && offsetof(tensor_t, rank) == 8 && offsetof(tensor_t, shape) == 16 &&
              offsetof(tensor_t, strides) == 80 && offsetof(tensor_t, dtype) == 144 &&
              offsetof(tensor_t, environment) == 148 && offsetof(tensor_t, size) == 160 &&
              offsetof(tensor_t, layout) == 168, "reference tensor_t layout differs from tannic_hip.h");
static_assert(sizeof(scalar_t) == 16 && offsetof(scalar_t, dtype) == 8, "reference scalar_t layout");
static_assert(TYPES == 13 && float16 == 6 && bfloat16 == 7 && float32 == 8 && complex128 == 11, "reference type enum");
static_assert(SUCCESS == 0 && ERROR == 1 && UNSUPPORTED_DTYPE == 2 && INCOMPATIBLE_DEVICES == 4, "reference status enum");
static_assert(SINGLETON == 0 && CONTIGUOUS == 1 && STRIDED == 2, "reference layout enum");

#define UNARY(name) int ref_##name(const tensor_t* s, tensor_t* d) { return cpu::name(s, d); }
#define BINARY(name) int ref_##name(const tensor_t* a, const tensor_t* b, tensor_t* d) { return cpu::name(a, b, d); }
#define REDUCE(name) int ref_##name(const tensor_t* s, tensor_t* d, uint8_t ax) { return cpu::name(s, d, ax); }

extern "C" {
UNARY(neg) UNARY(repack) UNARY(log) UNARY(exp) UNARY(sqrt) UNARY(abs) UNARY(sin) UNARY(cos) UNARY(tan)
UNARY(sinh) UNARY(cosh) UNARY(tanh)
int ref_rsqrt(const tensor_t* s, tensor_t* d, float eps) { return cpu::rsqrt(s, d, eps); }
BINARY(add) BINARY(sub) BINARY(mul) BINARY(pow)
BINARY(eq) BINARY(ne) BINARY(gt) BINARY(ge) BINARY(lt) BINARY(le)
BINARY(view_as_cartesian) BINARY(view_as_polar) BINARY(gemm)
int ref_scale(const tensor_t* s, const scalar_t* k, tensor_t* d) { return cpu::scale(s, k, d); }
REDUCE(argsum) REDUCE(argmean) REDUCE(argmax) REDUCE(argmin)
int ref_conv2d(const tensor_t* x, const tensor_t* w, tensor_t* y, const size_t pad[2], const size_t stride[2]) {
    return cpu::conv2d(x, w, y, pad, stride);
}
int ref_conv2d_biased(const tensor_t* x, const tensor_t* w, const tensor_t* b, tensor_t* y, const size_t pad[2], const size_t stride[2]) {
    return cpu::conv2d(x, w, b, y, pad, stride);
}
int ref_conv1d(const tensor_t* x, const tensor_t* w, tensor_t* y, size_t pad, size_t stride) { return cpu::conv1d(x, w, y, pad, stride); }
int ref_cpy(const tensor_t* s, tensor_t* d) { return cpu::cpy(s, d); }
int ref_repeat(const tensor_t* s, tensor_t* d, int axis, int reps) { return cpu::repeat(s, d, axis, reps); }
int ref_concat(const tensor_t* a, const tensor_t* b, tensor_t* d, int axis) { return cpu::concat(a, b, d, axis); }
int ref_outer(const tensor_t* a, const tensor_t* b, tensor_t* d) { return cpu::outer(a, b, d); }
int ref_triu(const tensor_t* s, tensor_t* d, int k) { return cpu::triu(s, d, k); }
int ref_tril(const tensor_t* s, tensor_t* d, int k) { return cpu::tril(s, d, k); }
int ref_allclose(const tensor_t* a, const tensor_t* b, double rtol, double atol) {
    try { return cpu::allclose(a, b, rtol, atol) ? 1 : 0; } catch (...) { return -1; }
}
}
