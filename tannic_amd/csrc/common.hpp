// Shared definitions of the gfx950 device library: element types, error
// reporting, launch helpers.  Internal to csrc/; the public surface is
// include/tannic_hip.h.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <type_traits>

#include "../../include/tannic_hip.h"

namespace th {

// ---- error reporting ------------------------------------------------------
// The reference terminates the process on a runtime failure
// (src/cuda/exc.cuh:8-16).  A C ABI that is also loaded into foreign hosts
// must not do that: failures are recorded here and surface as TANNIC_ERROR.
void set_error(const char* what, const char* file, int line, hipError_t code);
void set_error_text(const char* text);

#define TH_TRY(expr)                                               \
    do {                                                           \
        hipError_t th_err_ = (expr);                               \
        if (th_err_ != hipSuccess) {                               \
            ::th::set_error(#expr, __FILE__, __LINE__, th_err_);   \
            return TANNIC_ERROR;                                   \
        }                                                          \
    } while (0)

inline hipStream_t as_stream(tannic_stream_t s) { return reinterpret_cast<hipStream_t>(s.address); }

// Raises a kernel's dynamic LDS limit, once per device: the attribute belongs to the device's copy of the code.
inline int raise_lds_limit(const void* kernel, size_t bytes, std::atomic<uint64_t>& done) {
    int device = 0;
    TH_TRY(hipGetDevice(&device));
    const uint64_t bit = uint64_t(1) << (device & 63);
    if (done.load(std::memory_order_acquire) & bit) return TANNIC_SUCCESS;
    TH_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    done.fetch_or(bit, std::memory_order_release);
    return TANNIC_SUCCESS;
}

// Result of the launch that was just enqueued.
inline int launch_status(const char* what) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        set_error(what, __FILE__, __LINE__, err);
        return TANNIC_ERROR;
    }
    return TANNIC_SUCCESS;
}

// ---- element types --------------------------------------------------------
using f16 = _Float16;

// bfloat16 as raw bits; conversions are explicit so that every rounding is
// visible: widening is exact, narrowing rounds to nearest even.
struct bf16 {
    uint16_t bits;
};

__host__ __device__ inline float to_float(bf16 v) {
    union { uint32_t u; float f; } c;
    c.u = static_cast<uint32_t>(v.bits) << 16;
    return c.f;
}

__host__ __device__ inline bf16 to_bf16(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    bf16 r;
    if ((c.u & 0x7FFFFFFFu) > 0x7F800000u) {
        r.bits = static_cast<uint16_t>((c.u >> 16) | 0x40u);  // quiet NaN
    } else {
        r.bits = static_cast<uint16_t>((c.u + 0x7FFFu + ((c.u >> 16) & 1u)) >> 16);
    }
    return r;
}

template <class T>
struct cplx {
    T re, im;
};
using c64 = cplx<float>;
using c128 = cplx<double>;

template <class T> struct is_16bit { static constexpr bool value = false; };
template <> struct is_16bit<f16> { static constexpr bool value = true; };
template <> struct is_16bit<bf16> { static constexpr bool value = true; };

// widen<T>: value of a 16-bit type as float, anything else unchanged
__host__ __device__ inline float widen(f16 v) { return static_cast<float>(v); }
__host__ __device__ inline float widen(bf16 v) { return to_float(v); }
template <class T> __host__ __device__ inline T widen(T v) { return v; }

// narrow<D>(x): x converted to D with one rounding
template <class D, class X> __host__ __device__ inline D narrow(X x) {
    if constexpr (std::is_same_v<D, bf16>) return to_bf16(static_cast<float>(x));
    else return static_cast<D>(x);
}

// narrow_result<D>(x): the rounding of an fp32 accumulator in the matrix kernels.  bf16 uses the hardware's
// round-to-nearest-even conversion there (the bit-level routine above stays for the elementwise kernels, whose
// results are compared bit for bit, NaN payloads included).
template <class D> __device__ inline D narrow_result(float x) {
    if constexpr (std::is_same_v<D, bf16>) {
        const __bf16 h = static_cast<__bf16>(x);
        bf16 r;
        __builtin_memcpy(&r.bits, &h, 2);
        return r;
    } else {
        return static_cast<D>(x);
    }
}

template <class T> struct type_tag { using type = T; };

// Calls f(type_tag<T>{}) for the element type of a dtype code.
template <class F> inline bool with_type(int dtype, F&& f) {
    switch (dtype) {
        case TANNIC_INT8: f(type_tag<int8_t>{}); return true;
        case TANNIC_INT16: f(type_tag<int16_t>{}); return true;
        case TANNIC_INT32: f(type_tag<int32_t>{}); return true;
        case TANNIC_INT64: f(type_tag<int64_t>{}); return true;
        case TANNIC_FLOAT16: f(type_tag<f16>{}); return true;
        case TANNIC_BFLOAT16: f(type_tag<bf16>{}); return true;
        case TANNIC_FLOAT32: f(type_tag<float>{}); return true;
        case TANNIC_FLOAT64: f(type_tag<double>{}); return true;
        case TANNIC_COMPLEX64: f(type_tag<c64>{}); return true;
        case TANNIC_COMPLEX128: f(type_tag<c128>{}); return true;
        default: return false;
    }
}

// The dtype code of an element type (the inverse of with_type).
template <class T> constexpr int dtype_code() {
    if constexpr (std::is_same_v<T, int8_t>) return TANNIC_INT8;
    else if constexpr (std::is_same_v<T, int16_t>) return TANNIC_INT16;
    else if constexpr (std::is_same_v<T, int32_t>) return TANNIC_INT32;
    else if constexpr (std::is_same_v<T, int64_t>) return TANNIC_INT64;
    else if constexpr (std::is_same_v<T, f16>) return TANNIC_FLOAT16;
    else if constexpr (std::is_same_v<T, bf16>) return TANNIC_BFLOAT16;
    else if constexpr (std::is_same_v<T, float>) return TANNIC_FLOAT32;
    else if constexpr (std::is_same_v<T, double>) return TANNIC_FLOAT64;
    else if constexpr (std::is_same_v<T, c64>) return TANNIC_COMPLEX64;
    else if constexpr (std::is_same_v<T, c128>) return TANNIC_COMPLEX128;
    else return -1;
}

// A kernel writes elements of one type; a destination described with another dtype would be over- or under-run.
// (The reference's kernels take the front end's word for it; here a descriptor that does not fit is refused.)
inline bool destination_is(const tannic_tensor_t* dst, int dtype, const char* who) {
    if (static_cast<int>(dst->dtype) == dtype) return true;
    set_error_text(who);
    return false;
}

inline size_t dtype_size(int dtype) {
    switch (dtype) {
        case TANNIC_INT8: return 1;
        case TANNIC_INT16: case TANNIC_FLOAT16: case TANNIC_BFLOAT16: return 2;
        case TANNIC_INT32: case TANNIC_FLOAT32: return 4;
        case TANNIC_INT64: case TANNIC_FLOAT64: case TANNIC_COMPLEX64: return 8;
        case TANNIC_COMPLEX128: return 16;
        default: return 0;
    }
}

// Elements a descriptor's shape spans (1 for rank 0).
inline size_t element_count(const tannic_tensor_t* t) {
    size_t n = 1;
    for (int d = 0; d < t->rank; ++d) n *= t->shape.sizes[d];
    return n;
}

// Every given tensor has at most TANNIC_DIMENSIONS dims and either storage or no elements (a kernel handed a null
// address faults the device; a rank beyond the descriptor's arrays would be read past them).
template <class... Ts> inline bool have_storage(const Ts*... t) {
    if (!((t == nullptr || t->rank <= TANNIC_DIMENSIONS) && ...)) {
        set_error_text("a tensor's rank is beyond what a descriptor holds");
        return false;
    }
    const bool ok = ((t == nullptr || t->address != nullptr || element_count(t) == 0) && ...);
    if (!ok) set_error_text("a tensor with elements has no storage (null address)");
    return ok;
}

// ---- 32-bit division by a launch-time constant ------------------------------
// q = n / d for n < 2^31 with one multiply-high, one add and one shift.
struct FastDiv {
    uint32_t d, magic, shift;
    __host__ __device__ FastDiv() : d(1), magic(1), shift(0) {}
    // the divisor 2^31: every n below it has quotient 0 and remainder n
    __host__ __device__ static FastDiv beyond_all() {
        FastDiv f;
        f.d = 1u << 31;
        f.magic = 1;
        f.shift = 31;
        return f;
    }
    // (a divisor of 0 only comes from an empty index space, where nothing is ever divided: it is taken as 1)
    explicit FastDiv(uint32_t divisor) : d(divisor ? divisor : 1) {
        for (shift = 0; shift < 32; ++shift)
            if ((1u << shift) >= d) break;
        const uint64_t one = 1;
        magic = static_cast<uint32_t>(((one << 32) * ((one << shift) - d)) / d + 1);
    }
    __device__ inline uint32_t div(uint32_t n) const { return (__umulhi(n, magic) + n) >> shift; }
    __device__ inline void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
        q = div(n);
        r = n - q * d;
    }
};

// What tannic_hip_counters reports (for tests that check what a call did, not only what it returned).
enum Counter { kCounterScratchAcquired = 0, kCounterMemoryCalls = 1, kCounterKShares = 2, kCounters = 3 };
void count(Counter which, uint64_t value, bool set = false);

// Work scratch obtained stream-ordered for the duration of one call.
int scratch_acquire(void** ptr, size_t nbytes, hipStream_t stream);
int scratch_release(void* ptr, hipStream_t stream);

// True while `stream` is being recorded into a graph: calls that wait for the stream refuse (and say why) instead of
// breaking the recording.  Sets the error text when it returns true.
bool refuses_while_recording(hipStream_t stream, const char* call);

}  // namespace th
