// Unary elementwise entry points: neg, repack, log, exp, sqrt, rsqrt, abs,
// sin, cos, tan, sinh, cosh, tanh.
// Semantics follow the reference CPU path: dst[i] = D(op(src[i])) evaluated in
// the source precision, 16-bit values through float with one rounding
// (src/cpu/ops-unary.cpp:106-198); the source may be strided, the destination
// is written contiguously in logical order (src/cpu/ops-unary.cpp:61-104).
#include "elementwise.hpp"

namespace th {

enum UnaryKind { U_NEG, U_CPY, U_LOG, U_EXP, U_SQRT, U_RSQRT, U_ABS, U_SIN, U_COS, U_TAN, U_SINH, U_COSH, U_TANH };

template <int K> __device__ inline float math(float x) {
    if constexpr (K == U_LOG) return logf(x);
    else if constexpr (K == U_EXP) return expf(x);
    else if constexpr (K == U_SQRT) return sqrtf(x);
    else if constexpr (K == U_ABS) return fabsf(x);
    else if constexpr (K == U_SIN) return sinf(x);
    else if constexpr (K == U_COS) return cosf(x);
    else if constexpr (K == U_TAN) return tanf(x);
    else if constexpr (K == U_SINH) return sinhf(x);
    else if constexpr (K == U_COSH) return coshf(x);
    else return tanhf(x);
}

template <int K> __device__ inline double math(double x) {
    if constexpr (K == U_LOG) return log(x);
    else if constexpr (K == U_EXP) return exp(x);
    else if constexpr (K == U_SQRT) return sqrt(x);
    else if constexpr (K == U_ABS) return fabs(x);
    else if constexpr (K == U_SIN) return sin(x);
    else if constexpr (K == U_COS) return cos(x);
    else if constexpr (K == U_TAN) return tan(x);
    else if constexpr (K == U_SINH) return sinh(x);
    else if constexpr (K == U_COSH) return cosh(x);
    else return tanh(x);
}

template <class T, int K>
struct UnaryF {
    using S0 = T;
    using S1 = uint8_t;
    using D = T;
    static constexpr int sources = 1;
    const T* a;
    const uint8_t* b;
    T* out;
    double eps;

    __device__ inline T operator()(T x, uint8_t) const {
        if constexpr (K == U_CPY) {
            return x;
        } else if constexpr (K == U_NEG) {
            if constexpr (std::is_same_v<T, c64> || std::is_same_v<T, c128>) return T{-x.re, -x.im};
            else if constexpr (std::is_same_v<T, bf16>) return bf16{static_cast<uint16_t>(x.bits ^ 0x8000u)};
            else if constexpr (std::is_integral_v<T>) {
                using U = std::make_unsigned_t<T>;
                return static_cast<T>(static_cast<U>(0) - static_cast<U>(x));
            } else return -x;
        } else if constexpr (K == U_RSQRT) {
            // evaluated in double whatever the element type (src/cpu/ops-unary.cpp:141-149).  For a 16-bit result the
            // hardware's reciprocal square root (1 ulp in fp32) gives the same value except where the exact one lies within
            // 2^-24 of a rounding boundary of the 16-bit type, and runs at the memory stream's speed, which double does not.
            // A sum below the smallest normal float (a bfloat16 subnormal with eps = 0) is one the instruction reads as zero:
            // it is scaled by 2^24 first and the result by 2^12.
            if constexpr (is_16bit<T>::value) {
                const float t = widen(x) + static_cast<float>(eps);
                const bool tiny = t > 0.0f && t < 1.17549435e-38f;
                const float r = __builtin_amdgcn_rsqf(tiny ? t * 16777216.0f : t);
                return narrow<T>(tiny ? r * 4096.0f : r);
            } else return narrow<T>(1.0 / sqrt(static_cast<double>(widen(x)) + eps));
        } else if constexpr (K == U_ABS && std::is_integral_v<T>) {
            using U = std::make_unsigned_t<T>;
            return x < 0 ? static_cast<T>(static_cast<U>(0) - static_cast<U>(x)) : x;
        } else if constexpr (is_16bit<T>::value) {
            // exp of a 16-bit value: the hardware exponential is ~2 ulp in fp32, far inside half an ulp of the
            // 16-bit result, and keeps eight exponentials per lane off the critical path of the memory stream
            if constexpr (K == U_EXP) return narrow<T>(__expf(widen(x)));
            else return narrow<T>(math<K>(widen(x)));
        } else {
            return math<K>(x);
        }
    }
};

template <class T, int K>
int run_unary(const tannic_tensor_t* src, tannic_tensor_t* dst, hipStream_t stream, double eps) {
    if (!same_extents(src, dst)) return shape_mismatch("unary op: source and destination shapes differ");
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = dst->rank;
    contiguous_strides(rank, dst->shape.sizes, strides[2]);
    if (src->layout == TANNIC_STRIDED) {
        // walk dst's shape over the source's strides, size-1 dims pinned to 0
        for (int d = 0; d < rank; ++d) strides[0][d] = dst->shape.sizes[d] == 1 ? 0 : src->strides.sizes[d];
    } else {
        // SINGLETON and CONTIGUOUS sources are read linearly
        contiguous_strides(rank, dst->shape.sizes, strides[0]);
    }
    Plan plan;
    size_t one = 1;
    const bool scalar = rank == 0;
    if (!build_plan(plan, scalar ? 1 : rank, scalar ? &one : dst->shape.sizes, strides, 3)) {
        set_error_text("elementwise: tensors of 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    if constexpr (K == U_CPY) {
        // a source that is contiguous along another dimension than the last: tiles through LDS
        const int tiled = transposed_copy<typename BitsOf<sizeof(T)>::type>(plan, src->address, dst->address, stream);
        if (tiled != TANNIC_UNSUPPORTED_DTYPE) return tiled;
    }
    // operand 1 is unused: give it the source's strides so that it never blocks merging
    UnaryF<T, K> f{static_cast<const T*>(src->address), nullptr, static_cast<T*>(dst->address), eps};
    return launch_elementwise(f, plan, stream);
}

template <int K>
int unary(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, double eps = 0.0) {
    if (!src || !dst) return TANNIC_ERROR;
    if (!have_storage(src, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    with_type(src->dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        constexpr bool cplx = std::is_same_v<T, c64> || std::is_same_v<T, c128>;
        constexpr bool flt = std::is_floating_point_v<T> || is_16bit<T>::value;
        // coverage per function: src/cpu/ops-unary.cpp:202-370
        constexpr bool ok = (K == U_NEG || K == U_CPY) ? true
                          : K == U_ABS ? (flt || std::is_same_v<T, int32_t> || std::is_same_v<T, int64_t>)
                          : (flt && !cplx);
        if constexpr (ok) {
            if (!destination_is(dst, dtype_code<T>(), "unary op: the destination's dtype is not the source's")) status = TANNIC_ERROR;
            else status = run_unary<T, K>(src, dst, as_stream(stream), eps);
        }
    });
    return status;
}

}  // namespace th

using namespace th;

extern "C" {
int tannic_hip_neg(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_NEG>(s, d, st); }
int tannic_hip_repack(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_CPY>(s, d, st); }
int tannic_hip_log(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_LOG>(s, d, st); }
int tannic_hip_exp(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_EXP>(s, d, st); }
int tannic_hip_sqrt(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_SQRT>(s, d, st); }
int tannic_hip_rsqrt(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st, float eps) {
    return unary<U_RSQRT>(s, d, st, static_cast<double>(eps));
}
int tannic_hip_abs(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_ABS>(s, d, st); }
int tannic_hip_sin(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_SIN>(s, d, st); }
int tannic_hip_cos(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_COS>(s, d, st); }
int tannic_hip_tan(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_TAN>(s, d, st); }
int tannic_hip_sinh(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_SINH>(s, d, st); }
int tannic_hip_cosh(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_COSH>(s, d, st); }
int tannic_hip_tanh(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st) { return unary<U_TANH>(s, d, st); }
}
