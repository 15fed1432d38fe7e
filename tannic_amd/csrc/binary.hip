// Broadcasting binary elementwise entry points: add, sub, mul, pow.
// The operand pair selects the destination type exactly as the reference's
// tables do (src/cpu/ops-binary.cpp:168-430); the arithmetic is C++'s usual
// conversion of the pair, 16-bit pairs being evaluated in float and rounded
// once.  Broadcasting follows src/cpu/ops-binary.cpp:79-105: operands are
// right-aligned on the destination and size-1 dims get stride 0.
//
// Pairs the reference's tables hold that are NOT offered here, on purpose:
//   - 16-bit float with an integer operand, and pow of two 16-bit operands:
//     the reference kernels write 4-byte results while its front end sizes the
//     destination for 2-byte ones (include/tannic/operations.hpp:133-135 vs
//     src/cpu/ops-binary.cpp:199-206,388) — on a device that is an
//     out-of-bounds write, so these return UNSUPPORTED_DTYPE.
#include "elementwise.hpp"

namespace th {

enum BinaryKind { B_ADD, B_SUB, B_MUL, B_POW };

template <class T> constexpr bool is_cplx_v = std::is_same_v<T, c64> || std::is_same_v<T, c128>;
template <class T> constexpr bool is_16_v = is_16bit<T>::value;

// Destination type of a pair; void = unsupported.
template <class A, class B, int K>
struct BinaryResult {
    static auto pick() {
        if constexpr (is_cplx_v<A> || is_cplx_v<B>) {
            if constexpr (std::is_same_v<A, B> && K != B_POW) return type_tag<A>{}; else return type_tag<void>{};
        } else if constexpr (std::is_integral_v<A> && std::is_integral_v<B>) {
            if constexpr (K == B_POW) return type_tag<void>{};
            else if constexpr (sizeof(A) >= sizeof(B)) return type_tag<A>{};
            else return type_tag<B>{};
        } else if constexpr (is_16_v<A> && is_16_v<B>) {
            if constexpr (std::is_same_v<A, B> && K != B_POW) return type_tag<A>{}; else return type_tag<void>{};
        } else if constexpr (is_16_v<A> || is_16_v<B>) {
            using O = std::conditional_t<is_16_v<A>, B, A>;
            if constexpr (std::is_floating_point_v<O>) return type_tag<O>{}; else return type_tag<void>{};
        } else if constexpr (std::is_integral_v<A> || std::is_integral_v<B>) {
            using I = std::conditional_t<std::is_integral_v<A>, A, B>;
            using F = std::conditional_t<std::is_integral_v<A>, B, A>;
            if constexpr (std::is_same_v<I, int32_t>) return type_tag<F>{}; else return type_tag<void>{};
        } else {
            if constexpr (std::is_same_v<A, double> || std::is_same_v<B, double>) return type_tag<double>{};
            else return type_tag<float>{};
        }
    }
    using type = typename decltype(pick())::type;
};

template <class A, class B, class R, int K>
struct BinaryF {
    using S0 = A;
    using S1 = B;
    using D = R;
    static constexpr int sources = 2;
    const A* a;
    const B* b;
    R* out;

    __device__ inline R operator()(A x, B y) const {
        if constexpr (is_cplx_v<R>) {
            if constexpr (K == B_ADD) return R{x.re + y.re, x.im + y.im};
            else if constexpr (K == B_SUB) return R{x.re - y.re, x.im - y.im};
            else return R{x.re * y.re - x.im * y.im, x.re * y.im + x.im * y.re};
        } else if constexpr (std::is_integral_v<R>) {
            // wrap-around arithmetic in the destination width
            using U = std::make_unsigned_t<R>;
            const U u = static_cast<U>(static_cast<R>(x)), v = static_cast<U>(static_cast<R>(y));
            if constexpr (K == B_ADD) return static_cast<R>(u + v);
            else if constexpr (K == B_SUB) return static_cast<R>(u - v);
            else return static_cast<R>(u * v);
        } else {
            using CT = std::conditional_t<is_16_v<R>, float, R>;
            if constexpr (K == B_POW) {
                // std::pow with an integer argument is evaluated in double
                if constexpr (std::is_integral_v<A> || std::is_integral_v<B> || std::is_same_v<CT, double>)
                    return narrow<R>(pow(static_cast<double>(widen(x)), static_cast<double>(widen(y))));
                else
                    return narrow<R>(powf(static_cast<float>(widen(x)), static_cast<float>(widen(y))));
            } else {
                const CT u = static_cast<CT>(widen(x)), v = static_cast<CT>(widen(y));
                if constexpr (K == B_ADD) return narrow<R>(u + v);
                else if constexpr (K == B_SUB) return narrow<R>(u - v);
                else return narrow<R>(u * v);
            }
        }
    }
};

template <class A, class B, class R, int K>
int run_binary(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, hipStream_t stream) {
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = dst->rank;
    Plan plan;
    size_t one = 1;
    if (dst->layout == TANNIC_SINGLETON || rank == 0) {
        // one element: *dst = op(*a, *b) (src/cpu/ops-binary.cpp:67-73)
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
    BinaryF<A, B, R, K> f{static_cast<const A*>(a->address), static_cast<const B*>(b->address), static_cast<R*>(dst->address)};
    return launch_elementwise(f, plan, stream);
}

template <int K>
int binary(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!a || !b || !dst) return TANNIC_ERROR;
    if (!have_storage(a, b, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    with_type(a->dtype, [&](auto ta) {
        with_type(b->dtype, [&](auto tb) {
            using A = typename decltype(ta)::type;
            using B = typename decltype(tb)::type;
            using R = typename BinaryResult<A, B, K>::type;
            if constexpr (!std::is_void_v<R>) {
                if (!destination_is(dst, dtype_code<R>(), "binary op: the destination's dtype is not the pair's result type")) status = TANNIC_ERROR;
                else status = run_binary<A, B, R, K>(a, b, dst, as_stream(stream));
            }
        });
    });
    return status;
}

}  // namespace th

using namespace th;

extern "C" {
#if !defined(TH_BINARY_ONLY) || TH_BINARY_ONLY == 0
int tannic_hip_add(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return binary<B_ADD>(a, b, d, s); }
#endif
#if !defined(TH_BINARY_ONLY) || TH_BINARY_ONLY == 1
int tannic_hip_sub(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return binary<B_SUB>(a, b, d, s); }
#endif
#if !defined(TH_BINARY_ONLY) || TH_BINARY_ONLY == 2
int tannic_hip_mul(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return binary<B_MUL>(a, b, d, s); }
#endif
#if !defined(TH_BINARY_ONLY) || TH_BINARY_ONLY == 3
int tannic_hip_pow(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return binary<B_POW>(a, b, d, s); }
#endif
}
