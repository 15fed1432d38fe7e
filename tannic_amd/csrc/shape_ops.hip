// repeat (interleaved repetition along an axis) and triu / tril.
//
// Both move elements as opaque bit patterns: no arithmetic, so every dtype of a
// given width shares a kernel.  repeat gathers from an arbitrarily strided
// source into the contiguous destination (src/cpu/reps.cpp:18-54); when the
// source's last dimension is contiguous and 16-byte friendly, groups of 16 bytes
// are moved as one element.  triu / tril are rank-2 only, like the reference
// (src/cpu/triang.cpp:24-105), and keep its index arithmetic: `i + k` is formed
// in unsigned 64-bit, so a negative k wraps for the rows i < -k.
#include "common.hpp"

namespace th {

struct RepeatPlan {
    int rank, axis;
    uint32_t reps;
    uint32_t total;              // destination elements (in units of the moved element)
    FastDiv div[8];              // destination extents, innermost last
    uint32_t extent[8];
    int64_t stride[8];           // source strides in units of the moved element
    FastDiv div_reps;
};

template <class U>
__global__ __launch_bounds__(256) void repeat_kernel(const U* src, U* dst, RepeatPlan q) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= q.total) return;
    uint32_t rest = idx;
    int64_t off = 0;
    for (int d = q.rank - 1; d >= 0; --d) {
        uint32_t next, coord;
        q.div[d].divmod(rest, next, coord);
        rest = next;
        if (d == q.axis) coord = q.div_reps.div(coord);
        off += static_cast<int64_t>(coord) * q.stride[d];
    }
    dst[idx] = src[off];
}

template <class U>
int launch_repeat(const void* src, void* dst, const RepeatPlan& q, hipStream_t stream) {
    hipLaunchKernelGGL((repeat_kernel<U>), dim3((q.total + 255) / 256), dim3(256), 0, stream, static_cast<const U*>(src), static_cast<U*>(dst), q);
    return launch_status("repeat_kernel");
}

int run_repeat(const tannic_tensor_t* src, tannic_tensor_t* dst, int axis, int reps, hipStream_t stream) {
    size_t esize;
    switch (dst->dtype) {
        case TANNIC_INT8: esize = 1; break;
        case TANNIC_INT16: case TANNIC_FLOAT16: case TANNIC_BFLOAT16: esize = 2; break;
        case TANNIC_INT32: case TANNIC_FLOAT32: esize = 4; break;
        case TANNIC_INT64: case TANNIC_FLOAT64: esize = 8; break;
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
    const int rank = src->rank;
    if (rank < 1 || rank > 8 || dst->rank != rank || axis < 0 || axis >= rank || reps < 1) {
        set_error_text("repeat: rank, axis or count out of range");
        return TANNIC_ERROR;
    }
    uint64_t total = 1;
    for (int d = 0; d < rank; ++d) {
        const size_t want = src->shape.sizes[d] * (d == axis ? static_cast<size_t>(reps) : 1);
        if (dst->shape.sizes[d] != want) {
            set_error_text("repeat: destination shape does not match");
            return TANNIC_ERROR;
        }
        total *= want;
    }
    if (total == 0) return TANNIC_SUCCESS;
    if (total >= (1ull << 31)) {
        set_error_text("repeat: destination of 2^31 elements or more is not supported");
        return TANNIC_ERROR;
    }
    RepeatPlan q{};
    q.rank = rank;
    q.axis = axis;
    q.reps = static_cast<uint32_t>(reps);
    q.div_reps = FastDiv(q.reps);
    // 16-byte groups along a contiguous last dimension that is not the repeated one
    const size_t group = 16 / esize;
    bool wide = rank >= 1 && axis != rank - 1 && src->strides.sizes[rank - 1] == 1 && src->shape.sizes[rank - 1] % group == 0 &&
                reinterpret_cast<uintptr_t>(src->address) % 16 == 0 && reinterpret_cast<uintptr_t>(dst->address) % 16 == 0;
    for (int d = 0; wide && d < rank - 1; ++d)
        if (src->strides.sizes[d] % static_cast<int64_t>(group) != 0) wide = false;
    const size_t unit = wide ? group : 1;
    for (int d = 0; d < rank; ++d) {
        const bool last = d == rank - 1;
        q.extent[d] = static_cast<uint32_t>(dst->shape.sizes[d] / (last ? unit : 1));
        q.div[d] = FastDiv(q.extent[d]);
        q.stride[d] = last ? src->strides.sizes[d] : src->strides.sizes[d] / static_cast<int64_t>(unit);
    }
    q.total = static_cast<uint32_t>(total / unit);
    if (wide) return launch_repeat<uint4>(src->address, dst->address, q, stream);
    switch (esize) {
        case 1: return launch_repeat<uint8_t>(src->address, dst->address, q, stream);
        case 2: return launch_repeat<uint16_t>(src->address, dst->address, q, stream);
        case 4: return launch_repeat<uint32_t>(src->address, dst->address, q, stream);
        default: return launch_repeat<uint64_t>(src->address, dst->address, q, stream);
    }
}

template <class U, bool UPPER>
__global__ __launch_bounds__(256) void triangular_kernel(const U* src, U* dst, uint32_t rows, uint32_t cols, int64_t ss0, int64_t ss1, int64_t ds0, int64_t ds1, int k, FastDiv div_cols) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= rows * cols) return;
    uint32_t i, j;
    div_cols.divmod(idx, i, j);
    // size_t arithmetic of the CPU path: i + k with k converted to unsigned 64-bit
    const uint64_t edge = static_cast<uint64_t>(i) + static_cast<uint64_t>(static_cast<int64_t>(k));
    const bool keep = UPPER ? static_cast<uint64_t>(j) >= edge : static_cast<uint64_t>(j) <= edge;
    dst[static_cast<int64_t>(i) * ds0 + static_cast<int64_t>(j) * ds1] = keep ? src[static_cast<int64_t>(i) * ss0 + static_cast<int64_t>(j) * ss1] : U(0);
}

template <bool UPPER>
int run_triangular(const tannic_tensor_t* src, tannic_tensor_t* dst, int k, hipStream_t stream) {
    size_t esize;
    switch (src->dtype) {
        case TANNIC_FLOAT16: case TANNIC_BFLOAT16: esize = 2; break;
        case TANNIC_INT32: case TANNIC_FLOAT32: esize = 4; break;
        case TANNIC_INT64: case TANNIC_FLOAT64: esize = 8; break;
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
    if (src->rank != 2) return TANNIC_UNSUPPORTED_DTYPE;   // src/cpu/triang.cpp:58
    if (dst->rank != 2 || dst->shape.sizes[0] != src->shape.sizes[0] || dst->shape.sizes[1] != src->shape.sizes[1]) {
        set_error_text("triu/tril: destination shape does not match");
        return TANNIC_ERROR;
    }
    const uint64_t rows = src->shape.sizes[0], cols = src->shape.sizes[1];
    if (rows * cols == 0) return TANNIC_SUCCESS;
    if (rows * cols >= (1ull << 31)) {
        set_error_text("triu/tril: 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    const dim3 grid(static_cast<uint32_t>((rows * cols + 255) / 256));
    const int64_t ss0 = src->strides.sizes[0], ss1 = src->strides.sizes[1], ds0 = dst->strides.sizes[0], ds1 = dst->strides.sizes[1];
    const FastDiv dc(static_cast<uint32_t>(cols));
    const uint32_t r = static_cast<uint32_t>(rows), c = static_cast<uint32_t>(cols);
    if (esize == 2) hipLaunchKernelGGL((triangular_kernel<uint16_t, UPPER>), grid, dim3(256), 0, stream, static_cast<const uint16_t*>(src->address), static_cast<uint16_t*>(dst->address), r, c, ss0, ss1, ds0, ds1, k, dc);
    else if (esize == 4) hipLaunchKernelGGL((triangular_kernel<uint32_t, UPPER>), grid, dim3(256), 0, stream, static_cast<const uint32_t*>(src->address), static_cast<uint32_t*>(dst->address), r, c, ss0, ss1, ds0, ds1, k, dc);
    else hipLaunchKernelGGL((triangular_kernel<uint64_t, UPPER>), grid, dim3(256), 0, stream, static_cast<const uint64_t*>(src->address), static_cast<uint64_t*>(dst->address), r, c, ss0, ss1, ds0, ds1, k, dc);
    return launch_status("triangular_kernel");
}

}  // namespace th

extern "C" {
int tannic_hip_repeat(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int axis, int reps) {
    if (!src || !dst) return TANNIC_ERROR;
    return th::run_repeat(src, dst, axis, reps, th::as_stream(stream));
}
int tannic_hip_triu(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int k) {
    if (!src || !dst) return TANNIC_ERROR;
    return th::run_triangular<true>(src, dst, k, th::as_stream(stream));
}
int tannic_hip_tril(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int k) {
    if (!src || !dst) return TANNIC_ERROR;
    return th::run_triangular<false>(src, dst, k, th::as_stream(stream));
}
}
