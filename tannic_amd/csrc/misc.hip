// scale, cpy, complex construction, comparisons, allclose.
#include "elementwise.hpp"

namespace th {

// ------------------------------------------------------------------------
// scale: dst = src * k, k given in the tensor's dtype on the HOST
// (src/cpu/ops-scale.cpp:59-84; integers multiply as unsigned, :103-116)
// ------------------------------------------------------------------------
template <class T>
struct ScaleF {
    using S0 = T;
    using S1 = uint8_t;
    using D = T;
    static constexpr int sources = 1;
    const T* a;
    const uint8_t* b;
    T* out;
    T k;
    __device__ inline T operator()(T x, uint8_t) const {
        if constexpr (is_16bit<T>::value) return narrow<T>(widen(x) * widen(k));
        else return static_cast<T>(x * k);
    }
};

template <class T>
int run_scale(const tannic_tensor_t* src, const tannic_scalar_t* sc, tannic_tensor_t* dst, hipStream_t stream) {
    if (!same_extents(src, dst)) return shape_mismatch("scale: source and destination shapes differ");
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = dst->rank;
    contiguous_strides(rank, dst->shape.sizes, strides[2]);
    if (src->layout == TANNIC_CONTIGUOUS) contiguous_strides(rank, dst->shape.sizes, strides[0]);
    else for (int d = 0; d < rank; ++d) strides[0][d] = dst->shape.sizes[d] == 1 ? 0 : src->strides.sizes[d];
    Plan plan;
    size_t one = 1;
    if (!build_plan(plan, rank == 0 ? 1 : rank, rank == 0 ? &one : dst->shape.sizes, strides, 3)) {
        set_error_text("elementwise: tensors of 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    ScaleF<T> f{static_cast<const T*>(src->address), nullptr, static_cast<T*>(dst->address), T{}};
    std::memcpy(&f.k, sc->address, sizeof(T));
    return launch_elementwise(f, plan, stream);
}

// ------------------------------------------------------------------------
// cpy: strided -> strided, size-1 dims of either side pinned to index 0
// (src/cpu/cpy.cpp:18-80).  Elements are moved as opaque bit patterns.
// ------------------------------------------------------------------------
struct alignas(16) Bits128 { uint64_t lo, hi; };

template <class T>
struct CopyF {
    using S0 = T;
    using S1 = uint8_t;
    using D = T;
    static constexpr int sources = 1;
    const T* a;
    const uint8_t* b;
    T* out;
    __device__ inline T operator()(T x, uint8_t) const { return x; }
};

template <class T>
int run_cpy(const tannic_tensor_t* src, tannic_tensor_t* dst, hipStream_t stream) {
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = src->rank;
    // the copy walks the destination's index space: a source dim must have that extent or 1 (pinned to index 0)
    if (dst->rank != rank) return shape_mismatch("cpy: source and destination differ in rank");
    for (int d = 0; d < rank; ++d)
        if (src->shape.sizes[d] != 1 && src->shape.sizes[d] != dst->shape.sizes[d])
            return shape_mismatch("cpy: a source extent is neither 1 nor the destination's");
    for (int d = 0; d < rank; ++d) {
        strides[0][d] = src->shape.sizes[d] == 1 ? 0 : src->strides.sizes[d];
        strides[2][d] = dst->shape.sizes[d] == 1 ? 0 : dst->strides.sizes[d];
    }
    Plan plan;
    size_t one = 1;
    if (!build_plan(plan, rank == 0 ? 1 : rank, rank == 0 ? &one : dst->shape.sizes, strides, 3)) {
        set_error_text("elementwise: tensors of 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    const int tiled = transposed_copy<typename BitsOf<sizeof(T)>::type>(plan, src->address, dst->address, stream);
    if (tiled != TANNIC_UNSUPPORTED_DTYPE) return tiled;
    CopyF<T> f{static_cast<const T*>(src->address), nullptr, static_cast<T*>(dst->address)};
    return launch_elementwise(f, plan, stream);
}

// ------------------------------------------------------------------------
// view_as_cartesian / view_as_polar (src/cpu/complex.cpp:28-99, tables :152-219)
// ------------------------------------------------------------------------
template <class A, class B>
struct ComplexResult {
    static auto pick() {
        constexpr bool ia = std::is_integral_v<A>, ib = std::is_integral_v<B>;
        constexpr bool fa = std::is_floating_point_v<A>, fb = std::is_floating_point_v<B>;
        if constexpr (ia && ib) return type_tag<float>{};
        else if constexpr (ia && fb) { if constexpr (std::is_same_v<A, int32_t>) return type_tag<B>{}; else return type_tag<void>{}; }
        else if constexpr (fa && ib) { if constexpr (std::is_same_v<B, int32_t>) return type_tag<A>{}; else return type_tag<void>{}; }
        else if constexpr (fa && fb) {
            if constexpr (std::is_same_v<A, double> || std::is_same_v<B, double>) return type_tag<double>{};
            else return type_tag<float>{};
        } else return type_tag<void>{};
    }
    using type = typename decltype(pick())::type;
};

template <class A, class B, class C, bool POLAR>
struct ComplexF {
    using S0 = A;
    using S1 = B;
    using D = cplx<C>;
    static constexpr int sources = 2;
    const A* a;
    const B* b;
    D* out;
    // cos/sin in the angle's own precision (double for integer angles), then
    // the product under the usual arithmetic conversions, as the CPU path's
    // `rho * std::cos(theta)` evaluates (src/cpu/complex.cpp:84-85)
    __device__ static inline auto cosine(B v) {
        if constexpr (std::is_same_v<B, float>) return cosf(v); else return cos(static_cast<double>(v));
    }
    __device__ static inline auto sine(B v) {
        if constexpr (std::is_same_v<B, float>) return sinf(v); else return sin(static_cast<double>(v));
    }
    __device__ inline D operator()(A u, B v) const {
        if constexpr (!POLAR) return D{static_cast<C>(u), static_cast<C>(v)};
        else return D{static_cast<C>(u * cosine(v)), static_cast<C>(u * sine(v))};
    }
};

template <class A, class B, class C, bool POLAR>
int run_complex(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, hipStream_t stream) {
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = dst->rank;
    if (rank != 0 && (a->rank != rank || b->rank != rank)) {
        set_error_text("complex: operands must have the destination's rank");
        return TANNIC_ERROR;
    }
    // both parts are indexed by the destination's coordinates: an extent must be the destination's or 1
    for (int d = 0; d < rank; ++d)
        for (const tannic_tensor_t* t : {a, b})
            if (t->shape.sizes[d] != 1 && t->shape.sizes[d] != dst->shape.sizes[d])
                return shape_mismatch("complex: an operand extent is neither 1 nor the destination's");
    for (int d = 0; d < rank; ++d) {
        strides[0][d] = a->shape.sizes[d] == 1 ? 0 : a->strides.sizes[d];
        strides[1][d] = b->shape.sizes[d] == 1 ? 0 : b->strides.sizes[d];
    }
    contiguous_strides(rank, dst->shape.sizes, strides[2]);
    Plan plan;
    size_t one = 1;
    if (!build_plan(plan, rank == 0 ? 1 : rank, rank == 0 ? &one : dst->shape.sizes, strides, 3)) {
        set_error_text("elementwise: tensors of 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    ComplexF<A, B, C, POLAR> f{static_cast<const A*>(a->address), static_cast<const B*>(b->address),
                               static_cast<cplx<C>*>(dst->address)};
    return launch_elementwise(f, plan, stream);
}

template <bool POLAR>
int complex_entry(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!a || !b || !dst) return TANNIC_ERROR;
    if (!have_storage(a, b, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    with_type(a->dtype, [&](auto ta) {
        with_type(b->dtype, [&](auto tb) {
            using A = typename decltype(ta)::type;
            using B = typename decltype(tb)::type;
            constexpr bool plain = (std::is_integral_v<A> || std::is_floating_point_v<A>) &&
                                   (std::is_integral_v<B> || std::is_floating_point_v<B>);
            if constexpr (plain) {
                using C = typename ComplexResult<A, B>::type;
                if constexpr (!std::is_void_v<C>) {
                    if (!destination_is(dst, dtype_code<cplx<C>>(), "complex: the destination's dtype is not the pair's complex type")) status = TANNIC_ERROR;
                    else status = run_complex<A, B, C, POLAR>(a, b, dst, as_stream(stream));
                }
            }
        });
    });
    return status;
}

// ------------------------------------------------------------------------
// Comparisons -> bit-packed booleans, LSB first in logical row-major order
// (src/cpu/cmps.cpp:16-41, :85-105).  A thread produces one output byte from
// eight consecutive elements.
// ------------------------------------------------------------------------
enum CmpKind { C_EQ, C_NE, C_GT, C_GE, C_LT, C_LE };

template <int K, class T>
__device__ inline bool compare(T x, T y) {
    if constexpr (std::is_same_v<T, bf16>) return compare<K>(to_float(x), to_float(y));
    else if constexpr (K == C_EQ) return x == y;
    else if constexpr (K == C_NE) return x != y;
    else if constexpr (K == C_GT) return x > y;
    else if constexpr (K == C_GE) return x >= y;
    else if constexpr (K == C_LT) return x < y;
    else return x <= y;
}

// Strided operands: a thread produces one output byte from eight consecutive elements.
template <class T, int K>
__global__ __launch_bounds__(kBlock) void compare_kernel(const T* a, const T* b, uint8_t* out, uint32_t ne, Plan p) {
    const uint32_t byte = blockIdx.x * kBlock + threadIdx.x;
    const uint32_t first = byte * 8;
    if (first >= ne) return;
    uint32_t bits = 0;
    const uint32_t n = ne - first < 8 ? ne - first : 8;
    for (uint32_t i = 0; i < n; ++i) {
        const Offsets o = decode<1>(p, first + i);
        bits |= static_cast<uint32_t>(compare<K>(a[o.o0], b[o.o1])) << i;
    }
    out[byte] = static_cast<uint8_t>(bits);
}

// Contiguous operands: every lane reads ONE 16-byte vector per operand (fully coalesced) and turns it
// into N = 16 / sizeof(T) result bits; lanes that hold less than a byte pass their bits down to the
// first lane of their byte.
template <class T, int K>
__global__ __launch_bounds__(kBlock) void compare_flat_kernel(const T* a, const T* b, uint8_t* out, uint32_t ne) {
    constexpr int N = 16 / sizeof(T);
    const uint32_t t = blockIdx.x * kBlock + threadIdx.x;
    const uint32_t first = t * N;
    uint32_t bits = 0;
    if (first + N <= ne) {
        const Pack<T, N> x = load_pack<T, N>(a + first);
        const Pack<T, N> y = load_pack<T, N>(b + first);
#pragma unroll
        for (int i = 0; i < N; ++i) bits |= static_cast<uint32_t>(compare<K>(x.v[i], y.v[i])) << i;
    } else if (first < ne) {
        for (uint32_t i = 0; first + i < ne; ++i) bits |= static_cast<uint32_t>(compare<K>(a[first + i], b[first + i])) << i;
    }
    if constexpr (N >= 8) {
        // N = 8: one byte; N = 16: two bytes
        if (first < ne) {
            out[first / 8] = static_cast<uint8_t>(bits);
            if (N == 16 && first + 8 < ne) out[first / 8 + 1] = static_cast<uint8_t>(bits >> 8);
        }
    } else {
        // 8 / N consecutive lanes make one byte (a wavefront never splits a byte: 64 * N is a multiple of 8)
        constexpr int LANES = 8 / N;
#pragma unroll
        for (int s = 1; s < LANES; ++s) bits |= __shfl_down(bits & ((1u << N) - 1u), s) << (s * N);
        if (t % LANES == 0 && first < ne) out[first / 8] = static_cast<uint8_t>(bits);
    }
}

template <class T, int K>
int run_compare(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, hipStream_t stream) {
    if (!same_extents(a, dst) || !same_extents(b, dst)) return shape_mismatch("compare: operand and destination shapes differ");
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = dst->rank;
    // each source is walked with its own strides over the destination's shape
    for (int d = 0; d < rank; ++d) {
        strides[0][d] = a->strides.sizes[d];
        strides[1][d] = b->strides.sizes[d];
    }
    contiguous_strides(rank, dst->shape.sizes, strides[2]);
    Plan plan;
    size_t one = 1;
    if (dst->size >= (1ull << 31) || !build_plan(plan, rank == 0 ? 1 : rank, rank == 0 ? &one : dst->shape.sizes, strides, 3)) {
        set_error_text("compare: tensors of 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    const uint32_t ne = rank == 0 ? 1u : static_cast<uint32_t>(dst->size);
    if (ne == 0) return TANNIC_SUCCESS;
    const int last = plan.rank - 1;
    plan.row_vectors = plan.extent[last];
    plan.row_div = FastDiv(plan.row_vectors);
    plan.total_vectors = ne;
    const T* pa = static_cast<const T*>(a->address);
    const T* pb = static_cast<const T*>(b->address);
    const bool flat = plan.rank == 1 && plan.stride[0][0] == 1 && plan.stride[1][0] == 1 &&
                      reinterpret_cast<uintptr_t>(pa) % 16 == 0 && reinterpret_cast<uintptr_t>(pb) % 16 == 0;
    const uint32_t bytes = (ne + 7) / 8;
    const uint32_t grid = (bytes + kBlock - 1) / kBlock;
    constexpr uint32_t PER_THREAD = 16 / sizeof(T);
    const uint32_t flat_grid = ((ne + PER_THREAD - 1) / PER_THREAD + kBlock - 1) / kBlock;
    // The CPU path ORs a true result into a rank-0 destination and leaves a false
    // one untouched (src/cpu/cmps.cpp:87-93), which reads memory nobody wrote.
    // Here the byte is always written: 1 or 0.
    if (flat) hipLaunchKernelGGL((compare_flat_kernel<T, K>), dim3(flat_grid), dim3(kBlock), 0, stream, pa, pb,
                                 static_cast<uint8_t*>(dst->address), ne);
    else hipLaunchKernelGGL((compare_kernel<T, K>), dim3(grid), dim3(kBlock), 0, stream, pa, pb,
                            static_cast<uint8_t*>(dst->address), ne, plan);
    return launch_status("compare_kernel");
}

template <int K>
int compare_entry(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!a || !b || !dst) return TANNIC_ERROR;
    if (!have_storage(a, b, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    // The CPU path dispatches on the first source only and reads the second as the same type (src/cpu/cmps.cpp:108-202),
    // which runs past the end of a narrower second operand: operands of different dtypes are refused here.
    if (a->dtype != b->dtype) {
        set_error_text("comparison: operands of different dtypes");
        return TANNIC_UNSUPPORTED_DTYPE;
    }
    if (!destination_is(dst, TANNIC_BOOLEAN, "comparison: the destination is not boolean")) return TANNIC_ERROR;
    with_type(a->dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        if constexpr (!std::is_same_v<T, c64> && !std::is_same_v<T, c128>)
            status = run_compare<T, K>(a, b, dst, as_stream(stream));
    });
    return status;
}

// ------------------------------------------------------------------------
// allclose: false iff some element has |a-b| > atol + rtol*|b|, in double
// (src/cpu/val.cpp:17-70).  NaN differences never trip the test, as there.
// ------------------------------------------------------------------------
__global__ void fill_flag_kernel(int* flag, int value) { *flag = value; }

template <class T>
__global__ __launch_bounds__(kBlock) void allclose_kernel(const T* a, const T* b, uint32_t ne, Plan p, double rtol, double atol, int* differs) {
    bool bad = false;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < ne; i += gridDim.x * kBlock) {
        const Offsets o = decode<1>(p, i);
        const double x = static_cast<double>(widen(a[o.o0]));
        const double y = static_cast<double>(widen(b[o.o1]));
        if (fabs(x - y) > atol + rtol * fabs(y)) bad = true;
    }
    if (bad) *differs = 1;
}

template <class T>
int run_allclose(const tannic_tensor_t* a, const tannic_tensor_t* b, hipStream_t stream, double rtol, double atol) {
    if (refuses_while_recording(stream, "allclose")) return -1;
    if (!same_extents(a, b)) {
        set_error_text("allclose: operand shapes differ");
        return -1;
    }
    int64_t strides[kMaxOperands][TANNIC_DIMENSIONS] = {};
    const int rank = a->rank;
    for (int d = 0; d < rank; ++d) {
        strides[0][d] = a->strides.sizes[d];
        strides[1][d] = b->strides.sizes[d];
    }
    Plan plan;
    size_t one = 1;
    if (a->size >= (1ull << 31) || !build_plan(plan, rank == 0 ? 1 : rank, rank == 0 ? &one : a->shape.sizes, strides, 3)) {
        set_error_text("allclose: tensors of 2^31 elements or more are not supported");
        return -1;
    }
    const uint32_t ne = rank == 0 ? 1u : static_cast<uint32_t>(a->size);
    plan.row_vectors = plan.extent[plan.rank - 1];
    plan.row_div = FastDiv(plan.row_vectors);
    plan.total_vectors = ne;
    int* flag = nullptr;
    if (scratch_acquire(reinterpret_cast<void**>(&flag), sizeof(int), stream) != TANNIC_SUCCESS) return -1;
    hipLaunchKernelGGL(fill_flag_kernel, dim3(1), dim3(1), 0, stream, flag, 0);
    if (ne) {
        uint32_t grid = (ne + kBlock - 1) / kBlock;
        if (grid > 4096) grid = 4096;
        hipLaunchKernelGGL((allclose_kernel<T>), dim3(grid), dim3(kBlock), 0, stream, static_cast<const T*>(a->address),
                           static_cast<const T*>(b->address), ne, plan, rtol, atol, flag);
    }
    int differs = 1;
    hipError_t err = hipMemcpyAsync(&differs, flag, sizeof(int), hipMemcpyDeviceToHost, stream);
    if (err == hipSuccess) err = hipStreamSynchronize(stream);
    scratch_release(flag, stream);
    if (err != hipSuccess) {
        set_error("allclose", __FILE__, __LINE__, err);
        return -1;
    }
    return differs ? 0 : 1;
}

}  // namespace th

using namespace th;

extern "C" {

int tannic_hip_scale(const tannic_tensor_t* src, const tannic_scalar_t* sc, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!src || !sc || !dst || !sc->address) return TANNIC_ERROR;
    if (!have_storage(src, dst)) return TANNIC_ERROR;
    if (src->dtype != sc->dtype) return TANNIC_UNSUPPORTED_DTYPE;
    if (!destination_is(dst, src->dtype, "scale: the destination's dtype is not the source's")) return TANNIC_ERROR;
    hipStream_t s = as_stream(stream);
    switch (src->dtype) {
        case TANNIC_INT8: return run_scale<uint8_t>(src, sc, dst, s);
        case TANNIC_INT16: return run_scale<uint16_t>(src, sc, dst, s);
        case TANNIC_INT32: return run_scale<uint32_t>(src, sc, dst, s);
        case TANNIC_INT64: return run_scale<uint64_t>(src, sc, dst, s);
        case TANNIC_FLOAT16: return run_scale<f16>(src, sc, dst, s);
        case TANNIC_BFLOAT16: return run_scale<bf16>(src, sc, dst, s);
        case TANNIC_FLOAT32: return run_scale<float>(src, sc, dst, s);
        case TANNIC_FLOAT64: return run_scale<double>(src, sc, dst, s);
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
}

int tannic_hip_cpy(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!src || !dst) return TANNIC_ERROR;
    if (!have_storage(src, dst)) return TANNIC_ERROR;
    if (dtype_size(dst->dtype) != dtype_size(src->dtype)) {   // elements move as bits of the source's width
        set_error_text("cpy: source and destination elements differ in size");
        return TANNIC_ERROR;
    }
    hipStream_t s = as_stream(stream);
    switch (dtype_size(src->dtype)) {
        case 1: return run_cpy<uint8_t>(src, dst, s);
        case 2: return run_cpy<uint16_t>(src, dst, s);
        case 4: return run_cpy<uint32_t>(src, dst, s);
        case 8: return run_cpy<uint64_t>(src, dst, s);
        case 16: return run_cpy<Bits128>(src, dst, s);
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
}

int tannic_hip_view_as_cartesian(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) {
    return complex_entry<false>(a, b, d, s);
}
int tannic_hip_view_as_polar(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) {
    return complex_entry<true>(a, b, d, s);
}

int tannic_hip_eq(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return compare_entry<C_EQ>(a, b, d, s); }
int tannic_hip_ne(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return compare_entry<C_NE>(a, b, d, s); }
int tannic_hip_gt(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return compare_entry<C_GT>(a, b, d, s); }
int tannic_hip_ge(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return compare_entry<C_GE>(a, b, d, s); }
int tannic_hip_lt(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return compare_entry<C_LT>(a, b, d, s); }
int tannic_hip_le(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* d, tannic_stream_t s) { return compare_entry<C_LE>(a, b, d, s); }

int tannic_hip_allclose(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_stream_t stream, double rtol, double atol) {
    if (!a || !b || !have_storage(a, b)) return -1;
    if (a->dtype != b->dtype) {   // the second operand would be read as the first's type (src/cpu/val.cpp:73-83 does)
        set_error_text("allclose: operands of different dtypes");
        return -1;
    }
    hipStream_t s = as_stream(stream);
    switch (a->dtype) {
        case TANNIC_FLOAT16: return run_allclose<f16>(a, b, s, rtol, atol);
        case TANNIC_BFLOAT16: return run_allclose<bf16>(a, b, s, rtol, atol);
        case TANNIC_FLOAT32: return run_allclose<float>(a, b, s, rtol, atol);
        case TANNIC_FLOAT64: return run_allclose<double>(a, b, s, rtol, atol);
        default: return -1;
    }
}

}  // extern "C"
