// Elementwise operators the reference does not have: quotient, dtype change, SwiGLU gate.
// A Tannic program writes them today as chains (x * rsqrt(y) * rsqrt(y), a product with a tensor of the wanted
// type, g * rsqrt(exp(-g) + 1)^2 * u); here each is one pass over its operands.  They run on the same streaming
// engine as the reference-defined operators, with the same broadcasting (src/cpu/ops-binary.cpp:79-105).
//   div    : dst = a / b.  Floating pairs of the multiplication table (src/cpu/ops-binary.cpp:286-360), same
//            destination type; 16-bit pairs are divided in float and rounded once.
//   cast   : dst[i] = value of src[i] in dst's type, between any two real types.  Float to integer truncates
//            toward zero; values outside the integer range give its nearest end and NaN gives 0.
//   swiglu : dst = gate / (1 + exp(-gate)) * up for two tensors of one floating type, evaluated in float
//            (double for float64) and rounded once.
#include <limits>

#include "elementwise.hpp"

namespace th {

template <class T> constexpr bool is_real_float_v = std::is_floating_point_v<T> || is_16bit<T>::value;

template <class A, class B>
struct QuotientType {
    static auto pick() {
        if constexpr (!is_real_float_v<A> || !is_real_float_v<B>) return type_tag<void>{};
        else if constexpr (is_16bit<A>::value && is_16bit<B>::value) {
            if constexpr (std::is_same_v<A, B>) return type_tag<A>{}; else return type_tag<void>{};
        } else if constexpr (is_16bit<A>::value) return type_tag<B>{};
        else if constexpr (is_16bit<B>::value) return type_tag<A>{};
        else if constexpr (std::is_same_v<A, double> || std::is_same_v<B, double>) return type_tag<double>{};
        else return type_tag<float>{};
    }
    using type = typename decltype(pick())::type;
};

template <class A, class B, class R>
struct DivF {
    using S0 = A;
    using S1 = B;
    using D = R;
    static constexpr int sources = 2;
    const A* a;
    const B* b;
    R* out;
    __device__ inline R operator()(A x, B y) const {
        using CT = std::conditional_t<is_16bit<R>::value, float, R>;
        return narrow<R>(static_cast<CT>(widen(x)) / static_cast<CT>(widen(y)));
    }
};

template <class T>
struct SwigluF {
    using S0 = T;
    using S1 = T;
    using D = T;
    static constexpr int sources = 2;
    const T* a;
    const T* b;
    T* out;
    __device__ inline T operator()(T g, T u) const {
        if constexpr (std::is_same_v<T, double>) {
            return g / (1.0 + exp(-g)) * u;
        } else {
            const float x = widen(g);
            // 16-bit results: the hardware exponential's error is far below half an ulp of the result
            const float e = is_16bit<T>::value ? __expf(-x) : expf(-x);
            return narrow<T>(x / (1.0f + e) * static_cast<float>(widen(u)));
        }
    }
};

template <class A, class B>
struct CastF {
    using S0 = A;
    using S1 = uint8_t;
    using D = B;
    static constexpr int sources = 1;
    const A* a;
    const uint8_t* b;
    B* out;
    __device__ inline B operator()(A x, uint8_t) const {
        if constexpr (std::is_same_v<A, B>) return x;
        else if constexpr (std::is_integral_v<A> && std::is_integral_v<B>) return static_cast<B>(x);
        else if constexpr (std::is_integral_v<B>) {
            // float -> integer: truncation toward zero, the ends of the range for anything beyond them, 0 for NaN
            const auto v = widen(x);
            using V = std::remove_const_t<decltype(v)>;
            constexpr V top = sizeof(B) == 8 ? static_cast<V>(9223372036854775808.0) : static_cast<V>(1ull << (8 * sizeof(B) - 1));
            if (!(v == v)) return static_cast<B>(0);
            if (v >= top) return std::numeric_limits<B>::max();
            if (v <= -top) return std::numeric_limits<B>::min();
            return static_cast<B>(v);
        } else if constexpr (std::is_integral_v<A>) {
            if constexpr (is_16bit<B>::value) return narrow<B>(static_cast<float>(x));
            else return static_cast<B>(x);
        } else if constexpr (is_16bit<B>::value) {
            if constexpr (std::is_same_v<A, double>) {
                // one rounding: going through float would round twice, so the float keeps a sticky last bit
                // (magnitude truncated, last bit set when anything was dropped) and the 16-bit rounding decides
                float f = static_cast<float>(x);
                if (x == x && static_cast<double>(f) != x) {
                    uint32_t bits;
                    __builtin_memcpy(&bits, &f, 4);
                    if (fabs(static_cast<double>(f)) > fabs(x)) bits -= 1;
                    bits |= 1u;
                    __builtin_memcpy(&f, &bits, 4);
                }
                return narrow<B>(f);
            } else {
                return narrow<B>(static_cast<float>(widen(x)));
            }
        } else {
            return static_cast<B>(widen(x));
        }
    }
};

template <class F, class A, class B, class R>
int run_pair(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, hipStream_t stream) {
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = dst->rank;
    Plan plan;
    size_t one = 1;
    if (rank == 0) {
        if (!build_plan(plan, 1, &one, strides, 3)) return TANNIC_ERROR;
    } else {
        if (!broadcasts_to(a, dst) || !broadcasts_to(b, dst)) {
            set_error_text("binary op: an operand's shape does not broadcast to the destination's");
            return TANNIC_ERROR;
        }
        aligned_strides(a, rank, strides[0]);
        aligned_strides(b, rank, strides[1]);
        for (int d = 0; d < rank; ++d) strides[2][d] = dst->strides.sizes[d];
        if (!build_plan(plan, rank, dst->shape.sizes, strides, 3)) {
            set_error_text("elementwise: tensors of 2^31 elements or more are not supported");
            return TANNIC_ERROR;
        }
    }
    F f{static_cast<const A*>(a->address), static_cast<const B*>(b->address), static_cast<R*>(dst->address)};
    return launch_elementwise(f, plan, stream);
}

template <class A, class B>
int run_cast(const tannic_tensor_t* src, tannic_tensor_t* dst, hipStream_t stream) {
    if (!same_extents(src, dst)) return shape_mismatch("cast: source and destination shapes differ");
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = dst->rank;
    contiguous_strides(rank, dst->shape.sizes, strides[2]);
    if (src->layout == TANNIC_STRIDED) {
        for (int d = 0; d < rank; ++d) strides[0][d] = dst->shape.sizes[d] == 1 ? 0 : src->strides.sizes[d];
    } else {
        contiguous_strides(rank, dst->shape.sizes, strides[0]);
    }
    Plan plan;
    size_t one = 1;
    const bool scalar = rank == 0;
    if (!build_plan(plan, scalar ? 1 : rank, scalar ? &one : dst->shape.sizes, strides, 3)) {
        set_error_text("elementwise: tensors of 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    CastF<A, B> f{static_cast<const A*>(src->address), nullptr, static_cast<B*>(dst->address)};
    return launch_elementwise(f, plan, stream);
}

template <class F> inline bool with_real_type(int dtype, F&& f) {
    if (dtype == TANNIC_COMPLEX64 || dtype == TANNIC_COMPLEX128) return false;
    return with_type(dtype, f);
}

}  // namespace th

using namespace th;

extern "C" {

#if !defined(TH_EXTENDED_ONLY) || TH_EXTENDED_ONLY == 0
int tannic_hip_div(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!a || !b || !dst) return TANNIC_ERROR;
    if (!have_storage(a, b, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    with_real_type(a->dtype, [&](auto ta) {
        with_real_type(b->dtype, [&](auto tb) {
            using A = typename decltype(ta)::type;
            using B = typename decltype(tb)::type;
            if constexpr (!std::is_same_v<A, c64> && !std::is_same_v<A, c128> && !std::is_same_v<B, c64> && !std::is_same_v<B, c128>) {
                using R = typename QuotientType<A, B>::type;
                if constexpr (!std::is_void_v<R>) {
                    if (!destination_is(dst, dtype_code<R>(), "div: the destination's dtype is not the pair's quotient type")) status = TANNIC_ERROR;
                    else status = run_pair<DivF<A, B, R>, A, B, R>(a, b, dst, as_stream(stream));
                }
            }
        });
    });
    return status;
}

int tannic_hip_swiglu(const tannic_tensor_t* gate, const tannic_tensor_t* up, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!gate || !up || !dst) return TANNIC_ERROR;
    if (!have_storage(gate, up, dst)) return TANNIC_ERROR;
    if (gate->dtype != up->dtype || gate->dtype != dst->dtype) return TANNIC_UNSUPPORTED_DTYPE;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    with_real_type(gate->dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        if constexpr (is_real_float_v<T>) status = run_pair<SwigluF<T>, T, T, T>(gate, up, dst, as_stream(stream));
    });
    return status;
}
#endif

#if !defined(TH_EXTENDED_ONLY) || TH_EXTENDED_ONLY == 1
int tannic_hip_cast(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!src || !dst) return TANNIC_ERROR;
    if (!have_storage(src, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    with_real_type(src->dtype, [&](auto ta) {
        with_real_type(dst->dtype, [&](auto tb) {
            using A = typename decltype(ta)::type;
            using B = typename decltype(tb)::type;
            if constexpr (!std::is_same_v<A, c64> && !std::is_same_v<A, c128> && !std::is_same_v<B, c64> && !std::is_same_v<B, c128>)
                status = run_cast<A, B>(src, dst, as_stream(stream));
        });
    });
    return status;
}
#endif

}  // extern "C"
