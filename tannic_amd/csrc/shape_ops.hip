// repeat (interleaved repetition along an axis), concat, outer, triu / tril.
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
    if (!destination_is(dst, src->dtype, "repeat: the destination's dtype is not the source's")) return TANNIC_ERROR;
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

// concat: dst[.., j, ..] = a[.., j, ..] for j < a.extent[axis], else b[.., j - a.extent[axis], ..]; both sources strided,
// destination contiguous.  The CPU path addresses the block behind the axis with one stride (src/cpu/concat.cpp:66,76),
// which is the same thing whenever at most one dimension follows the axis; further in, this kernel keeps indexing
// every dimension by its own stride.
struct ConcatPlan {
    int rank, axis;
    uint32_t total, first_extent;
    FastDiv div[8];
    int64_t stride_a[8], stride_b[8];
};

template <class U>
__global__ __launch_bounds__(256) void concat_kernel(const U* a, const U* b, U* dst, ConcatPlan q) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= q.total) return;
    // both sources' offsets are formed on the way through the dimensions (no coordinate array: one indexed by the axis
    // would live in scratch memory)
    uint32_t rest = idx;
    int64_t off_a = 0, off_b = 0;
    bool second = false;
    for (int d = q.rank - 1; d >= 0; --d) {
        uint32_t next, c;
        q.div[d].divmod(rest, next, c);
        rest = next;
        uint32_t cb = c;
        if (d == q.axis) {
            second = c >= q.first_extent;
            cb = c - q.first_extent;
        }
        off_a += static_cast<int64_t>(c) * q.stride_a[d];
        off_b += static_cast<int64_t>(cb) * q.stride_b[d];
    }
    dst[idx] = second ? b[off_b] : a[off_a];
}

// Both sources contiguous, and what each contributes to a row of the result (its extent along the axis times everything
// behind the axis) a whole number of 16-byte pieces: the result is, outer index by outer index, a run of `a` followed by a
// run of `b` (appending to a key / value cache).  A thread moves one piece.
__global__ __launch_bounds__(256) void concat_runs_kernel(const uint4* a, const uint4* b, uint4* dst, uint32_t run_a, uint32_t run_b, FastDiv row, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    uint32_t outer, at;
    row.divmod(idx, outer, at);
    dst[idx] = at < run_a ? a[static_cast<size_t>(outer) * run_a + at] : b[static_cast<size_t>(outer) * run_b + (at - run_a)];
}

int run_concat(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, int axis, hipStream_t stream) {
    size_t esize;
    switch (dst->dtype) {   // src/cpu/concat.cpp:104-118 dispatches on the destination
        case TANNIC_INT8: esize = 1; break;
        case TANNIC_INT16: case TANNIC_FLOAT16: case TANNIC_BFLOAT16: esize = 2; break;
        case TANNIC_INT32: case TANNIC_FLOAT32: esize = 4; break;
        case TANNIC_INT64: case TANNIC_FLOAT64: esize = 8; break;
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
    const int rank = dst->rank;
    if (rank < 1 || rank > 8 || a->rank != rank || b->rank != rank || axis < 0 || axis >= rank || a->dtype != dst->dtype || b->dtype != dst->dtype) {
        set_error_text("concat: ranks, dtypes or axis do not match");
        return TANNIC_ERROR;
    }
    uint64_t total = 1;
    ConcatPlan q{};
    for (int d = 0; d < rank; ++d) {
        const size_t want = d == axis ? a->shape.sizes[d] + b->shape.sizes[d] : a->shape.sizes[d];
        if (dst->shape.sizes[d] != want || (d != axis && b->shape.sizes[d] != a->shape.sizes[d])) {
            set_error_text("concat: shapes do not match");
            return TANNIC_ERROR;
        }
        total *= want;
        q.div[d] = FastDiv(static_cast<uint32_t>(want));
        q.stride_a[d] = a->strides.sizes[d];
        q.stride_b[d] = b->strides.sizes[d];
    }
    if (total == 0) return TANNIC_SUCCESS;
    if (total >= (1ull << 31)) {
        set_error_text("concat: destination of 2^31 elements or more is not supported");
        return TANNIC_ERROR;
    }
    q.rank = rank;
    q.axis = axis;
    q.total = static_cast<uint32_t>(total);
    q.first_extent = static_cast<uint32_t>(a->shape.sizes[axis]);
    {
        size_t behind = 1;
        for (int d = axis + 1; d < rank; ++d) behind *= a->shape.sizes[d];
        const size_t bytes_a = a->shape.sizes[axis] * behind * esize, bytes_b = b->shape.sizes[axis] * behind * esize;
        auto at16 = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
        if (a->layout == TANNIC_CONTIGUOUS && b->layout == TANNIC_CONTIGUOUS && bytes_a % 16 == 0 && bytes_b % 16 == 0 && at16(a->address) && at16(b->address) &&
            at16(dst->address)) {
            const uint32_t run_a = static_cast<uint32_t>(bytes_a / 16), run_b = static_cast<uint32_t>(bytes_b / 16);
            const uint32_t pieces = static_cast<uint32_t>(total * esize / 16);
            hipLaunchKernelGGL(concat_runs_kernel, dim3((pieces + 255) / 256), dim3(256), 0, stream, static_cast<const uint4*>(a->address),
                               static_cast<const uint4*>(b->address), static_cast<uint4*>(dst->address), run_a, run_b, FastDiv(run_a + run_b), pieces);
            return launch_status("concat_runs_kernel");
        }
    }
    const dim3 grid((q.total + 255) / 256);
    switch (esize) {
        case 1: hipLaunchKernelGGL((concat_kernel<uint8_t>), grid, dim3(256), 0, stream, static_cast<const uint8_t*>(a->address), static_cast<const uint8_t*>(b->address), static_cast<uint8_t*>(dst->address), q); break;
        case 2: hipLaunchKernelGGL((concat_kernel<uint16_t>), grid, dim3(256), 0, stream, static_cast<const uint16_t*>(a->address), static_cast<const uint16_t*>(b->address), static_cast<uint16_t*>(dst->address), q); break;
        case 4: hipLaunchKernelGGL((concat_kernel<uint32_t>), grid, dim3(256), 0, stream, static_cast<const uint32_t*>(a->address), static_cast<const uint32_t*>(b->address), static_cast<uint32_t*>(dst->address), q); break;
        default: hipLaunchKernelGGL((concat_kernel<uint64_t>), grid, dim3(256), 0, stream, static_cast<const uint64_t*>(a->address), static_cast<const uint64_t*>(b->address), static_cast<uint64_t*>(dst->address), q); break;
    }
    return launch_status("concat_kernel");
}

// outer: dst[i][j] = a[i] * b[j] in the type the CPU path's table gives the pair (src/cpu/outer.cpp:54-99).  It is the
// product of a column [n1,1] and a row [1,n2], so it runs as the broadcasting multiply — for the pairs whose table type
// is also what the front end sizes the destination with (the larger dtype code, include/tannic/transformations.hpp:208-212).
// For the others (int8 x int8 -> int32, fp16 x fp16 -> fp32, ...) the CPU kernel writes wider elements than the
// destination holds; those are not offered.
static int outer_table(int first, int second) {
    auto is_int = [](int t) { return t >= TANNIC_INT8 && t <= TANNIC_INT64; };
    if (is_int(first) && is_int(second)) {
        if (first == TANNIC_INT64 || second == TANNIC_INT64) return TANNIC_INT64;
        if (first == TANNIC_INT32 && second == TANNIC_INT32) return TANNIC_INT64;
        return TANNIC_INT32;
    }
    auto half = [](int t) { return t == TANNIC_FLOAT16 || t == TANNIC_BFLOAT16; };
    const int lo = first < second ? first : second, hi = first < second ? second : first;
    if (half(first) && half(second)) return first == second ? TANNIC_FLOAT32 : -1;
    if (lo == TANNIC_INT32 && (half(hi) || hi == TANNIC_FLOAT32)) return TANNIC_FLOAT32;
    if (lo == TANNIC_INT32 && hi == TANNIC_FLOAT64) return TANNIC_FLOAT64;
    if (half(lo) && hi == TANNIC_FLOAT32) return TANNIC_FLOAT32;
    if (half(lo) && hi == TANNIC_FLOAT64) return TANNIC_FLOAT64;
    if (lo == TANNIC_FLOAT32 && hi == TANNIC_FLOAT32) return TANNIC_FLOAT32;
    if ((lo == TANNIC_FLOAT32 || lo == TANNIC_FLOAT64) && hi == TANNIC_FLOAT64) return TANNIC_FLOAT64;
    return -1;
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

// Rows contiguous and 16-byte friendly in both tensors: a thread writes one 16-byte piece, and reads it only when some of it
// is kept (the zeroed half of the matrix is not read at all).
template <class U, bool UPPER>
__global__ __launch_bounds__(256) void triangular_pieces_kernel(const U* src, U* dst, uint32_t pieces_per_row, uint32_t total, int64_t ss0, int64_t ds0, int k, FastDiv div_pieces) {
    constexpr uint32_t E = 16 / sizeof(U);
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    uint32_t i, piece;
    div_pieces.divmod(idx, i, piece);
    const uint32_t j0 = piece * E;
    const uint64_t edge = static_cast<uint64_t>(i) + static_cast<uint64_t>(static_cast<int64_t>(k));   // as in the kernel above
    bool keep[E], any = false;
#pragma unroll
    for (uint32_t e = 0; e < E; ++e) {
        keep[e] = UPPER ? static_cast<uint64_t>(j0 + e) >= edge : static_cast<uint64_t>(j0 + e) <= edge;
        any = any || keep[e];
    }
    U v[E];
    if (any) {
        const uint4 bits = *reinterpret_cast<const uint4*>(src + static_cast<int64_t>(i) * ss0 + j0);
        __builtin_memcpy(v, &bits, 16);
    }
#pragma unroll
    for (uint32_t e = 0; e < E; ++e) v[e] = (any && keep[e]) ? v[e] : U(0);
    uint4 out;
    __builtin_memcpy(&out, v, 16);
    *reinterpret_cast<uint4*>(dst + static_cast<int64_t>(i) * ds0 + j0) = out;
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
    if (!destination_is(dst, src->dtype, "triu/tril: the destination's dtype is not the source's")) return TANNIC_ERROR;
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
    const uint64_t per = 16 / esize;
    if (ss1 == 1 && ds1 == 1 && cols % per == 0 && ss0 % static_cast<int64_t>(per) == 0 && ds0 % static_cast<int64_t>(per) == 0 &&
        reinterpret_cast<uintptr_t>(src->address) % 16 == 0 && reinterpret_cast<uintptr_t>(dst->address) % 16 == 0) {
        const uint32_t pieces = static_cast<uint32_t>(cols / per), total = r * pieces;
        const dim3 pgrid((total + 255) / 256);
        const FastDiv dp(pieces);
        if (esize == 2) hipLaunchKernelGGL((triangular_pieces_kernel<uint16_t, UPPER>), pgrid, dim3(256), 0, stream, static_cast<const uint16_t*>(src->address), static_cast<uint16_t*>(dst->address), pieces, total, ss0, ds0, k, dp);
        else if (esize == 4) hipLaunchKernelGGL((triangular_pieces_kernel<uint32_t, UPPER>), pgrid, dim3(256), 0, stream, static_cast<const uint32_t*>(src->address), static_cast<uint32_t*>(dst->address), pieces, total, ss0, ds0, k, dp);
        else hipLaunchKernelGGL((triangular_pieces_kernel<uint64_t, UPPER>), pgrid, dim3(256), 0, stream, static_cast<const uint64_t*>(src->address), static_cast<uint64_t*>(dst->address), pieces, total, ss0, ds0, k, dp);
        return launch_status("triangular_pieces_kernel");
    }
    if (esize == 2) hipLaunchKernelGGL((triangular_kernel<uint16_t, UPPER>), grid, dim3(256), 0, stream, static_cast<const uint16_t*>(src->address), static_cast<uint16_t*>(dst->address), r, c, ss0, ss1, ds0, ds1, k, dc);
    else if (esize == 4) hipLaunchKernelGGL((triangular_kernel<uint32_t, UPPER>), grid, dim3(256), 0, stream, static_cast<const uint32_t*>(src->address), static_cast<uint32_t*>(dst->address), r, c, ss0, ss1, ds0, ds1, k, dc);
    else hipLaunchKernelGGL((triangular_kernel<uint64_t, UPPER>), grid, dim3(256), 0, stream, static_cast<const uint64_t*>(src->address), static_cast<uint64_t*>(dst->address), r, c, ss0, ss1, ds0, ds1, k, dc);
    return launch_status("triangular_kernel");
}

}  // namespace th

extern "C" {
int tannic_hip_repeat(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int axis, int reps) {
    if (!src || !dst) return TANNIC_ERROR;
    if (!th::have_storage(src, dst)) return TANNIC_ERROR;
    return th::run_repeat(src, dst, axis, reps, th::as_stream(stream));
}
int tannic_hip_concat(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream, int axis) {
    if (!a || !b || !dst) return TANNIC_ERROR;
    if (!th::have_storage(a, b, dst)) return TANNIC_ERROR;
    return th::run_concat(a, b, dst, axis, th::as_stream(stream));
}
int tannic_hip_outer(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!a || !b || !dst) return TANNIC_ERROR;
    if (!th::have_storage(a, b, dst)) return TANNIC_ERROR;
    const int result = th::outer_table(a->dtype, b->dtype);
    const int sized_as = a->dtype > b->dtype ? a->dtype : b->dtype;
    if (result < 0 || result != sized_as || dst->dtype != result) return TANNIC_UNSUPPORTED_DTYPE;
    if (a->rank != 1 || b->rank != 1 || dst->rank != 2 || dst->shape.sizes[0] != a->shape.sizes[0] || dst->shape.sizes[1] != b->shape.sizes[0]) {
        th::set_error_text("outer: operands must be vectors and the destination their [n1, n2] product");
        return TANNIC_ERROR;
    }
    tannic_tensor_t column = *a, row = *b;
    column.rank = row.rank = 2;
    column.shape.sizes[1] = 1;
    column.strides.sizes[1] = 0;
    row.shape.sizes[1] = b->shape.sizes[0];
    row.strides.sizes[1] = b->strides.sizes[0];
    row.shape.sizes[0] = 1;
    row.strides.sizes[0] = 0;
    column.layout = row.layout = TANNIC_STRIDED;
    return tannic_hip_mul(&column, &row, dst, stream);
}
int tannic_hip_triu(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int k) {
    if (!src || !dst) return TANNIC_ERROR;
    if (!th::have_storage(src, dst)) return TANNIC_ERROR;
    return th::run_triangular<true>(src, dst, k, th::as_stream(stream));
}
int tannic_hip_tril(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int k) {
    if (!src || !dst) return TANNIC_ERROR;
    if (!th::have_storage(src, dst)) return TANNIC_ERROR;
    return th::run_triangular<false>(src, dst, k, th::as_stream(stream));
}
}
