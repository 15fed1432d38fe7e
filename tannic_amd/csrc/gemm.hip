// gemm entry point: problem description, dtype table, generic kernel.
//
// Destination type per operand pair as in src/cpu/matmul.cpp:189-252.  The
// 16-bit same-type pairs, int8 x int8 and fp32 go to the MFMA kernels (gemm_mfma.hip,
// gemm_dtl.hip) when their layout conditions hold; every other pair, and the leftovers, run the
// LDS-tiled scalar kernel below, which accepts any strides.
//
// Differences from the reference CPU path, all documented at the ABI:
//   - f16 x f16 and bf16 x bf16 accumulate in fp32 and round once (the CPU
//     path accumulates in the 16-bit type);
//   - fp32 sums are formed in a different order (tiles of K);
//   - batch counts above 255 are handled (the CPU path narrows the batch
//     counter to uint8_t, src/cpu/matmul.cpp:102);
//   - an operand is addressed by both of its matrix strides (the CPU path
//     takes the smaller one to be 1, src/cpu/matmul.cpp:87-94);
//   - the batch coordinate of an operand with fewer batch dims than the
//     destination is multiplied by the stride of the dim it was looked up in
//     (right-aligned).  The CPU path looks the coordinate up right-aligned and
//     multiplies it by the stride at the left-aligned position
//     (src/cpu/matmul.cpp:107-118), which steps a[3,M,K] in a[3,M,K] x
//     b[2,3,K,N] by its row stride;
//   - operand extents are checked against the destination's (the CPU path
//     takes M and N from the destination and K from the first operand on trust).
#include <utility>

#include "gemm_common.hpp"

namespace th {

int describe_gemm(const tannic_tensor_t* a, const tannic_tensor_t* b, const tannic_tensor_t* c, GemmProblem& p) {
    if (a->rank < 2 || b->rank < 2 || c->rank < 2 || c->rank > 8) {
        set_error_text("gemm: operands must have rank >= 2");
        return TANNIC_ERROR;
    }
    const size_t M = c->shape.sizes[c->rank - 2], N = c->shape.sizes[c->rank - 1], K = a->shape.sizes[a->rank - 1];
    if (M >= (1ull << 31) || N >= (1ull << 31) || K >= (1ull << 31)) {
        set_error_text("gemm: dimension of 2^31 or more");
        return TANNIC_ERROR;
    }
    // The kernels index both operands by the destination's M, N and batch coordinates and by the first operand's K:
    // anything that does not fit would be read outside its storage.
    if (a->shape.sizes[a->rank - 2] != M || b->shape.sizes[b->rank - 2] != K || b->shape.sizes[b->rank - 1] != N) {
        set_error_text("gemm: operand extents do not fit the destination ([.., M, K] x [.., K, N] -> [.., M, N])");
        return TANNIC_ERROR;
    }
    if (a->rank > c->rank || b->rank > c->rank) {
        set_error_text("gemm: an operand has more dims than the destination");
        return TANNIC_ERROR;
    }
    for (const tannic_tensor_t* s : {a, b})
        for (int sd = 0; sd < s->rank - 2; ++sd) {
            const size_t extent = s->shape.sizes[sd];
            if (extent != 1 && extent != c->shape.sizes[sd + (c->rank - s->rank)]) {
                set_error_text("gemm: a batch extent of an operand is neither 1 nor the destination's");
                return TANNIC_ERROR;
            }
        }
    p.M = static_cast<uint32_t>(M);
    p.N = static_cast<uint32_t>(N);
    p.K = static_cast<uint32_t>(K);
    // Both matrix strides of an operand are used as they are.  (The CPU path takes the larger one as the leading
    // dimension and the other one to be 1, src/cpu/matmul.cpp:87-94,135-137: the same thing for a slab or its
    // transpose, and the wrong elements for a view whose inner stride is not 1.)
    p.a_rs = a->strides.sizes[a->rank - 2];
    p.a_cs = a->strides.sizes[a->rank - 1];
    p.b_rs = b->strides.sizes[b->rank - 2];
    p.b_cs = b->strides.sizes[b->rank - 1];
    p.c_rs = c->strides.sizes[c->rank - 2];
    p.row_bias = nullptr;
    p.c_group = p.c_group_live = 0;
    p.c_group_stride = p.b_group_stride = 0;
    p.c_group_div = FastDiv(1);
    p.batch_rank = c->rank - 2;
    p.batches = 1;
    for (int d = 0; d < 6; ++d) {
        p.batch_extent[d] = 1;
        p.a_bs[d] = p.b_bs[d] = p.c_bs[d] = 0;
    }
    size_t batches = 1;
    for (int d = 0; d < p.batch_rank; ++d) {
        p.batch_extent[d] = static_cast<uint32_t>(c->shape.sizes[d]);
        batches *= c->shape.sizes[d];
        p.c_bs[d] = c->strides.sizes[d];
        // the coordinate of an operand is looked up right-aligned (size-1 and missing dims give 0,
        // src/cpu/matmul.cpp:107-112) and multiplied by the stride of that same dim
        auto stride_of = [&](const tannic_tensor_t* s) -> int64_t {
            const int sd = d + (s->rank - c->rank);
            if (sd < 0 || s->shape.sizes[sd] == 1) return 0;
            return s->strides.sizes[sd];
        };
        p.a_bs[d] = stride_of(a);
        p.b_bs[d] = stride_of(b);
    }
    if (batches >= (1ull << 31)) {
        set_error_text("gemm: too many batches");
        return TANNIC_ERROR;
    }
    p.batches = static_cast<uint32_t>(batches);
    return TANNIC_SUCCESS;
}

template <class A, class B> struct GemmResult {
    static auto pick() {
        constexpr bool ia = std::is_integral_v<A>, ib = std::is_integral_v<B>;
        constexpr bool ha = is_16bit<A>::value, hb = is_16bit<B>::value;
        constexpr bool ca = std::is_same_v<A, c64> || std::is_same_v<A, c128>, cb = std::is_same_v<B, c64> || std::is_same_v<B, c128>;
        if constexpr (ca || cb) return type_tag<void>{};
        else if constexpr (ia && ib) {
            if constexpr (sizeof(A) == 8 || sizeof(B) == 8 || (sizeof(A) == 4 && sizeof(B) == 4)) return type_tag<int64_t>{};
            else return type_tag<int32_t>{};
        } else if constexpr (ha && hb) {
            if constexpr (std::is_same_v<A, B>) return type_tag<A>{}; else return type_tag<void>{};
        } else if constexpr (ha || hb) {
            using O = std::conditional_t<ha, B, A>;
            if constexpr (std::is_same_v<O, double> || std::is_same_v<O, int64_t>) return type_tag<double>{};
            else return type_tag<float>{};
        } else if constexpr (ia || ib) {
            using I = std::conditional_t<ia, A, B>;
            using F = std::conditional_t<ia, B, A>;
            if constexpr (std::is_same_v<I, int32_t>) return type_tag<F>{}; else return type_tag<void>{};
        } else {
            if constexpr (std::is_same_v<A, double> || std::is_same_v<B, double>) return type_tag<double>{};
            else return type_tag<float>{};
        }
    }
    using type = typename decltype(pick())::type;
};

// 64x64 output tile per block of 256 threads, 4x4 outputs per thread, K in
// steps of 16 through LDS.  Products are formed in the accumulator type
// (static_cast<D>(a) * static_cast<D>(b), src/cpu/matmul.cpp:36) — fp32 for a
// 16-bit destination.
template <class A, class B, class D>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const A* a, const B* b, D* c, GemmProblem p) {
    using Acc = std::conditional_t<is_16bit<D>::value, float, D>;
    constexpr int T = 64, KT = 16;
    __shared__ Acc sa[KT][T + 1];
    __shared__ Acc sb[KT][T + 1];
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.z, oa, ob, oc);
    a += oa;
    b += ob;
    c += oc;
    const uint32_t m0 = blockIdx.y * T, n0 = blockIdx.x * T;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    Acc acc[4][4] = {};
    for (uint32_t k0 = 0; k0 < p.K; k0 += KT) {
        for (int i = threadIdx.x; i < T * KT; i += 256) {
            // A tile: consecutive threads along k when k is the contiguous index, else along m
            const int kk = p.a_cs == 1 ? i % KT : i / T, mm = p.a_cs == 1 ? i / KT : i % T;
            const uint32_t m = m0 + mm, k = k0 + kk;
            sa[kk][mm] = (m < p.M && k < p.K) ? static_cast<Acc>(widen(a[m * p.a_rs + k * p.a_cs])) : Acc(0);
            const int kb = p.b_rs == 1 ? i % KT : i / T, nn = p.b_rs == 1 ? i / KT : i % T;
            const uint32_t n = n0 + nn, k2 = k0 + kb;
            sb[kb][nn] = (n < p.N && k2 < p.K) ? static_cast<Acc>(widen(b[k2 * p.b_rs + n * p.b_cs])) : Acc(0);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KT; ++kk) {
            Acc x[4], y[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { x[i] = sa[kk][ty * 4 + i]; y[i] = sb[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += x[i] * y[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < p.M && n < p.N) c[m * p.c_rs + n] = narrow<D>(acc[i][j]);
        }
}

// A handful of rows over a long K, both operands contiguous along K (a linear layer on a few tokens, in float64, an integer
// type or a mixed pair): the kernel above would give each 64 x 64 tile to one block that walks all of K.  Here a
// wavefront owns four columns of the result and ROWS rows; its lanes stride over K (whole lines of B's rows, A's rows from
// the caches) and the 4 * ROWS sums meet in a butterfly at the end.  Integer sums are exact in any order; floating sums
// are a tree instead of the CPU path's sequence, within rounding of it.
template <class A, class B, class D, int ROWS>
__global__ __launch_bounds__(256) void gemm_generic_few_rows_kernel(const A* a, const B* b, D* c, GemmProblem p) {
    using Acc = std::conditional_t<is_16bit<D>::value, float, D>;
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.z, oa, ob, oc);
    a += oa;
    b += ob;
    c += oc;
    const uint32_t lane = threadIdx.x % 64, n0 = (blockIdx.x * 4 + threadIdx.x / 64) * 4, m0 = blockIdx.y * ROWS;
    if (n0 >= p.N) return;   // whole wavefronts; nothing below synchronises across them
    Acc acc[ROWS][4] = {};
    for (uint32_t k = lane; k < p.K; k += 64) {
        Acc y[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) y[j] = static_cast<Acc>(widen(b[static_cast<int64_t>(n0 + j < p.N ? n0 + j : n0) * p.b_cs + k]));
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
            const Acc x = static_cast<Acc>(widen(a[static_cast<int64_t>(m0 + i < p.M ? m0 + i : m0) * p.a_rs + k]));
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] += x * y[j];
        }
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            Acc v = acc[i][j];
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) v += __shfl_xor(v, step, 64);
            if (lane == 0 && m0 + i < p.M && n0 + j < p.N) c[static_cast<int64_t>(m0 + i) * p.c_rs + n0 + j] = narrow<D>(v);
        }
}

// Few results under a long K (a handful of dot products: 48 x 13 over K = 12000), any types and strides: a tile kernel has
// one or two blocks that walk all of K alone.  Here a workgroup owns 4 x 4 results and its 256 lanes stride over K
// together (consecutive lanes, consecutive k); the sums meet in a butterfly per wavefront and in LDS across the four.
// Integer sums are exact in any order; floating sums are a tree, within rounding of the CPU path's sequence.
template <class A, class B, class D>
__global__ __launch_bounds__(256) void gemm_generic_few_results_kernel(const A* a, const B* b, D* c, GemmProblem p, uint32_t tiles_n) {
    using Acc = std::conditional_t<is_16bit<D>::value, float, D>;
    __shared__ Acc part[4][16];
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.y, oa, ob, oc);
    const uint32_t m0 = (blockIdx.x / tiles_n) * 4, n0 = (blockIdx.x % tiles_n) * 4;
    const A* pa[4];
    const B* pb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        pa[i] = a + oa + static_cast<int64_t>(m0 + i < p.M ? m0 + i : m0) * p.a_rs + static_cast<int64_t>(threadIdx.x) * p.a_cs;
        pb[i] = b + ob + static_cast<int64_t>(n0 + i < p.N ? n0 + i : n0) * p.b_cs + static_cast<int64_t>(threadIdx.x) * p.b_rs;
    }
    const int64_t step_a = 256 * p.a_cs, step_b = 256 * p.b_rs;
    Acc acc[4][4] = {};
#pragma unroll 2
    for (uint32_t k = threadIdx.x; k < p.K; k += 256) {
        Acc x[4], y[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[i] = static_cast<Acc>(widen(*pa[i]));
            y[i] = static_cast<Acc>(widen(*pb[i]));
            pa[i] += step_a;
            pb[i] += step_b;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] += x[i] * y[j];
    }
    const uint32_t lane = threadIdx.x % 64, wave = threadIdx.x / 64;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            Acc v = acc[i][j];
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) v += __shfl_xor(v, step, 64);
            if (lane == 0) part[wave][i * 4 + j] = v;
        }
    __syncthreads();
    if (threadIdx.x < 16) {
        const uint32_t m = m0 + threadIdx.x / 4, n = n0 + threadIdx.x % 4;
        Acc v = part[0][threadIdx.x] + part[1][threadIdx.x] + part[2][threadIdx.x] + part[3][threadIdx.x];
        if (m >= p.M || n >= p.N) return;
        // (a convolution's product: a per-row start value, columns in groups that go image by image)
        if (p.row_bias) v += static_cast<Acc>(widen(static_cast<const D*>(p.row_bias)[m]));
        int64_t at = oc + n;
        if (p.c_group) {
            uint32_t g, j;
            p.c_group_div.divmod(n, g, j);
            if (j >= p.c_group_live) return;
            at = static_cast<int64_t>(g) * p.c_group_stride + j;
        }
        c[at + static_cast<int64_t>(m) * p.c_rs] = narrow<D>(v);
    }
}

// Whether the kernel above is the one to run: few results (what a few 64 x 64 tiles hold) under a K of 256 or more.
// (`most`: 8192 where tiles that share K exist for larger products, 32768 for the types that only have kernels whose blocks walk all of K)
inline bool few_results_under_a_long_k(const GemmProblem& p, uint64_t most) {
    return p.M != 0 && p.N != 0 && p.batches != 0 && p.batches <= 65535 && p.K >= 256 && static_cast<uint64_t>(p.M) * p.N * p.batches <= most;
}

template <class A, class B, class D>
int run_few_results(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    const uint32_t tiles_m = (p.M + 3) / 4, tiles_n = (p.N + 3) / 4;
    hipLaunchKernelGGL((gemm_generic_few_results_kernel<A, B, D>), dim3(tiles_m * tiles_n, p.batches), dim3(256), 0, stream, static_cast<const A*>(a), static_cast<const B*>(b),
                       static_cast<D*>(c), p, tiles_n);
    return launch_status("gemm_generic_few_results_kernel");
}

// The same for a caller inside the library (the unfolded batch of a convolution): both operands and the result of one type.
int gemm_few_results(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream) {
    if (!few_results_under_a_long_k(p, 8192)) return TANNIC_UNSUPPORTED_DTYPE;
    switch (dtype) {
        case TANNIC_FLOAT16: return run_few_results<f16, f16, f16>(p, a, b, c, stream);
        case TANNIC_BFLOAT16: return run_few_results<bf16, bf16, bf16>(p, a, b, c, stream);
        case TANNIC_FLOAT32: return run_few_results<float, float, float>(p, a, b, c, stream);
        case TANNIC_FLOAT64: return run_few_results<double, double, double>(p, a, b, c, stream);
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
}

// c[m * c_rs + n] = t[n * M + m]: the few rows of a transposed result back into the columns they belong to
template <class U>
__global__ __launch_bounds__(256) void gemm_columns_from_rows_kernel(const U* t, U* c, uint32_t M, uint32_t N, int64_t c_rs, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const uint32_t m = idx / N, n = idx % N;
    c[static_cast<int64_t>(m) * c_rs + n] = t[static_cast<size_t>(n) * M + m];
}

template <class A, class B, class D>
int run_generic(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    if (p.M == 0 || p.N == 0 || p.batches == 0) return TANNIC_SUCCESS;
    if (p.M <= 16 && p.a_cs == 1 && p.b_rs == 1 && p.K >= 256 && p.batches <= 65535) {
        const dim3 grid((p.N + 15) / 16, (p.M + 7) / 8, p.batches);
        if (p.M <= 4) {
            hipLaunchKernelGGL((gemm_generic_few_rows_kernel<A, B, D, 4>), dim3(grid.x, (p.M + 3) / 4, p.batches), dim3(256), 0, stream, static_cast<const A*>(a),
                               static_cast<const B*>(b), static_cast<D*>(c), p);
        } else {
            hipLaunchKernelGGL((gemm_generic_few_rows_kernel<A, B, D, 8>), grid, dim3(256), 0, stream, static_cast<const A*>(a), static_cast<const B*>(b),
                               static_cast<D*>(c), p);
        }
        return launch_status("gemm_generic_few_rows_kernel");
    }
    const uint32_t gx = (p.N + 63) / 64, gy = (p.M + 63) / 64;
    if (gy > 65535 || p.batches > 65535) {
        set_error_text("gemm: generic kernel grid limit exceeded");
        return TANNIC_ERROR;
    }
    hipLaunchKernelGGL((gemm_generic_kernel<A, B, D>), dim3(gx, gy, p.batches), dim3(256), 0, stream, static_cast<const A*>(a),
                       static_cast<const B*>(b), static_cast<D*>(c), p);
    return launch_status("gemm_generic_kernel");
}

}  // namespace th

using namespace th;

namespace {

// A dense copy of `t` in the element type `dtype`, laid out in the order of t's own strides (a transposed matrix stays
// transposed: the copy reads and writes along the same dimension).  `out` describes the copy with t's extents.
// TANNIC_UNSUPPORTED_DTYPE: t is not copied (broadcast or reversed dims, too large).
int dense_copy_as(const tannic_tensor_t* t, int dtype, tannic_tensor_t& out, void*& held, tannic_stream_t stream) {
    held = nullptr;
    const int rank = t->rank;
    uint64_t elements = 1;
    int order[TANNIC_DIMENSIONS];
    for (int d = 0; d < rank; ++d) {
        if (t->shape.sizes[d] != 1 && t->strides.sizes[d] <= 0) return TANNIC_UNSUPPORTED_DTYPE;
        elements *= t->shape.sizes[d];
        order[d] = d;
    }
    if (elements == 0 || elements >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    // dims by stride, largest first; extents of 1 (whose stride is never used) lead
    auto key = [&](int d) { return t->shape.sizes[d] == 1 ? INT64_MAX : t->strides.sizes[d]; };
    for (int i = 1; i < rank; ++i)
        for (int j = i; j > 0 && key(order[j]) > key(order[j - 1]); --j) std::swap(order[j], order[j - 1]);
    tannic_tensor_t source = *t, dense = *t;
    int64_t pitch = 1;
    for (int i = rank - 1; i >= 0; --i) {
        source.shape.sizes[i] = dense.shape.sizes[i] = t->shape.sizes[order[i]];
        source.strides.sizes[i] = t->strides.sizes[order[i]];
        dense.strides.sizes[i] = pitch;
        pitch *= static_cast<int64_t>(dense.shape.sizes[i]);
    }
    source.layout = TANNIC_STRIDED;
    if (scratch_acquire(&held, elements * dtype_size(dtype), as_stream(stream)) != TANNIC_SUCCESS) return TANNIC_ERROR;
    dense.address = held;
    dense.dtype = static_cast<tannic_type>(dtype);
    dense.layout = TANNIC_CONTIGUOUS;
    dense.size = elements;
    const int status = tannic_hip_cast(&source, &dense, stream);
    if (status != TANNIC_SUCCESS) {
        scratch_release(held, as_stream(stream));
        held = nullptr;
        return status;
    }
    out = *t;
    out.address = held;
    out.dtype = static_cast<tannic_type>(dtype);
    out.layout = TANNIC_STRIDED;
    for (int i = 0; i < rank; ++i) out.strides.sizes[order[i]] = dense.strides.sizes[i];
    return TANNIC_SUCCESS;
}

int gemm_entry(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream, const GemmWorkspace* workspace) {
    if (!a || !b || !dst) return TANNIC_ERROR;
    if (!have_storage(a, b, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    hipStream_t s = as_stream(stream);
    with_type(a->dtype, [&](auto ta) {
        with_type(b->dtype, [&](auto tb) {
            using A = typename decltype(ta)::type;
            using B = typename decltype(tb)::type;
            using D = typename GemmResult<A, B>::type;
            if constexpr (!std::is_void_v<D>) {
                if (!destination_is(dst, dtype_code<D>(), "gemm: the destination's dtype is not the pair's product type")) {
                    status = TANNIC_ERROR;
                    return;
                }
                GemmProblem p;
                status = describe_gemm(a, b, dst, p);
                if (status != TANNIC_SUCCESS) return;
                if constexpr (!std::is_same_v<A, B> && (std::is_same_v<D, float> || std::is_same_v<D, double>)) {
                    // A product of two different types whose result is fp32 or float64 multiplies static_cast<D>(a) by
                    // static_cast<D>(b) (src/cpu/matmul.cpp:36): the same numbers as the product of the operands converted
                    // to D first, which runs on the matrix pipe where this pair has the scalar kernel only.  Worth the
                    // copies from a few million multiply-adds on; never on the path that must not allocate.
                    // (with few rows the scalar kernels stream the large operand once as it is: converting it first would
                    // read and write it once more - fp32 x bf16, 16 rows over 4096 x 4096: 37 against 39 us, float64 x fp32 67 against 114)
                    const bool few_rows_stream = p.M <= 16 && p.a_cs == 1 && p.b_rs == 1 && p.K >= 256 && !std::is_same_v<B, D>;
                    if (workspace == nullptr && !few_rows_stream && static_cast<double>(p.M) * p.N * p.K * p.batches >= static_cast<double>(1 << 24)) {
                        tannic_tensor_t a2 = *a, b2 = *b;
                        void* held[2] = {nullptr, nullptr};
                        int copied = TANNIC_SUCCESS;
                        if (!std::is_same_v<A, D>) copied = dense_copy_as(a, dtype_code<D>(), a2, held[0], stream);
                        if (copied == TANNIC_SUCCESS && !std::is_same_v<B, D>) copied = dense_copy_as(b, dtype_code<D>(), b2, held[1], stream);
                        if (copied == TANNIC_SUCCESS) copied = gemm_entry(&a2, &b2, dst, stream, workspace);
                        for (void* h : held)
                            if (h) scratch_release(h, s);
                        if (copied != TANNIC_UNSUPPORTED_DTYPE) {
                            status = copied;
                            return;
                        }
                    }
                }
                const void *first = a->address, *second = b->address;
                if constexpr (std::is_same_v<A, B>) {
                    // A matrix times a column, y = A . v: the same numbers are v^T . A^T, one row times a matrix whose "rows of
                    // W" are A's rows - the shape the kernels for few rows stream (a column of results lies in memory like a row).
                    if (p.N == 1 && p.M > 1 && p.c_rs == 1) {
                        GemmProblem t = p;
                        t.M = 1;
                        t.N = p.M;
                        t.a_rs = p.b_cs;   // a single row: its pitch is never used
                        t.a_cs = p.b_rs;
                        t.b_rs = p.a_cs;
                        t.b_cs = p.a_rs;
                        t.c_rs = p.M;
                        for (int d = 0; d < 6; ++d) {
                            t.a_bs[d] = p.b_bs[d];
                            t.b_bs[d] = p.a_bs[d];
                        }
                        p = t;
                        first = b->address;
                        second = a->address;
                    }
                }
                constexpr bool tiled = std::is_same_v<A, B> && (is_16bit<A>::value || std::is_same_v<A, int8_t> || std::is_same_v<A, float>);
                if constexpr (std::is_same_v<A, B> && (is_16bit<A>::value || std::is_same_v<A, float>)) {
                    // Many rows times a few columns (a classifier's last layer over a batch): C^T = W . X^T has the few as its
                    // rows, which the streaming kernel takes - X goes by once - and the small result is turned back.  Only
                    // where that kernel will take it (whole windows of K, aligned K-contiguous rows) and scratch may be had.
                    constexpr uint32_t window = 128 / sizeof(A), unit = 16 / sizeof(A);
                    const bool streams = p.N >= 2 && p.N <= 32 && p.M >= 256 && p.batches == 1 && workspace == nullptr && p.a_cs == 1 && p.b_rs == 1 &&
                                         p.K % window == 0 && p.a_rs % unit == 0 && p.b_cs % unit == 0 && p.a_rs >= static_cast<int64_t>(p.K) &&
                                         p.b_cs >= static_cast<int64_t>(p.K) && p.a_rs < (1 << 22) && p.b_cs < (1 << 22) &&
                                         reinterpret_cast<uintptr_t>(first) % 16 == 0 && reinterpret_cast<uintptr_t>(second) % 16 == 0 &&
                                         static_cast<uint64_t>(p.M) * p.K >= (1u << 21) &&
                                         // (16-bit tiles already fill the chip from 16384 rows on, and a short K leaves the streaming
                                         // kernel's blocks too little each; fp32 tiles pay the matrix pipe for every padded column)
                                         (sizeof(A) == 2 ? (p.M <= 16384 && p.K >= 1024) : p.K >= 512);
                    if (streams) {
                        GemmProblem t = p;
                        t.M = p.N;
                        t.N = p.M;
                        t.a_rs = p.b_cs;
                        t.a_cs = p.b_rs;
                        t.b_rs = p.a_cs;
                        t.b_cs = p.a_rs;
                        t.c_rs = p.M;
                        void* turned = nullptr;
                        if (scratch_acquire(&turned, static_cast<size_t>(p.M) * p.N * sizeof(A), s) != TANNIC_SUCCESS) {
                            status = TANNIC_ERROR;
                            return;
                        }
                        if constexpr (is_16bit<A>::value) status = gemm_skinny_16bit(t, a->dtype, second, first, turned, s);
                        else status = gemm_skinny_f32(t, static_cast<const float*>(second), static_cast<const float*>(first), static_cast<float*>(turned), s);
                        if (status == TANNIC_SUCCESS) {
                            using U = typename std::conditional<sizeof(A) == 2, uint16_t, uint32_t>::type;
                            const uint32_t total = p.M * p.N;
                            hipLaunchKernelGGL((gemm_columns_from_rows_kernel<U>), dim3((total + 255) / 256), dim3(256), 0, s, static_cast<const U*>(turned),
                                               static_cast<U*>(dst->address), p.M, p.N, p.c_rs, total);
                            status = launch_status("gemm_columns_from_rows_kernel");
                        }
                        scratch_release(turned, s);
                        if (status != TANNIC_UNSUPPORTED_DTYPE) return;   // (refused after all: on with the product as it is)
                    }
                }
                constexpr bool shares_k = std::is_same_v<A, B> && (is_16bit<A>::value || std::is_same_v<A, float> || std::is_same_v<A, int8_t>);
                if (few_results_under_a_long_k(p, shares_k ? 8192 : 32768)) {
                    // (not where the tiles share K or W is streamed: aligned K-contiguous operands of the 16-bit types and
                    // fp32, of int8 up to 32 rows; nor the few rows that the row-major kernel below or the scalar kernel
                    // for few rows streams)
                    bool elsewhere = !shares_k && p.M <= 16 && p.a_cs == 1 && p.b_rs == 1;
                    if constexpr (shares_k) {
                        constexpr int64_t unit = 16 / sizeof(A);
                        const bool aligned_nt = p.a_cs == 1 && p.b_rs == 1 && p.K % (std::is_same_v<A, int8_t> ? 128 : unit) == 0 && p.a_rs % unit == 0 && p.b_cs % unit == 0 &&
                                                reinterpret_cast<uintptr_t>(first) % 16 == 0 && reinterpret_cast<uintptr_t>(second) % 16 == 0;
                        if (aligned_nt && (!std::is_same_v<A, int8_t> || p.M <= 32)) elsewhere = true;
                        if (!std::is_same_v<A, int8_t> && p.M <= 8 && p.b_cs == 1 && p.b_rs != 1 && p.N >= 256 && p.N % 4 == 0) elsewhere = true;   // gemm_rows_nn
                    }
                    if (!elsewhere) {
                        status = run_few_results<A, B, D>(p, first, second, dst->address, s);
                        return;
                    }
                }
                if constexpr (std::is_same_v<A, B> && (is_16bit<A>::value || std::is_same_v<A, float>)) {
                    // at most eight rows times a matrix that lies row by row (x . W as written): W is read once, along its rows
                    if (workspace == nullptr) {
                        status = gemm_rows_nn(p, a->dtype, first, second, dst->address, s);
                        if (status != TANNIC_UNSUPPORTED_DTYPE) return;
                    }
                }
                if constexpr (tiled) {
                    // operands that do not lie as the tiled kernels want them are copied first when that pays (never on the
                    // path that must not allocate)
                    GemmProblem q;
                    const void *pa = first, *pb = second;
                    void* held[2] = {nullptr, nullptr};
                    const int repacked = gemm_repack(p, sizeof(A), first, second, s, workspace == nullptr, q, pa, pb, held);
                    if (repacked == TANNIC_ERROR) {
                        status = TANNIC_ERROR;
                        return;
                    }
                    const GemmProblem& use = repacked == TANNIC_SUCCESS ? q : p;
                    if constexpr (is_16bit<A>::value) status = gemm_mfma_16bit(use, a->dtype, pa, pb, dst->address, s, workspace);
                    else if constexpr (std::is_same_v<A, int8_t>) status = gemm_mfma_int8(use, pa, pb, dst->address, s);
                    else status = gemm_mfma_f32(use, static_cast<const float*>(pa), static_cast<const float*>(pb), static_cast<float*>(dst->address), s, workspace);
                    for (void* h : held)
                        if (h) scratch_release(h, s);
                    if (status != TANNIC_UNSUPPORTED_DTYPE) return;
                }
                if constexpr (std::is_same_v<A, double> && std::is_same_v<B, double>) {
                    status = gemm_mfma_f64(p, static_cast<const double*>(first), static_cast<const double*>(second), static_cast<double*>(dst->address), s);
                    if (status != TANNIC_UNSUPPORTED_DTYPE) return;
                }
                status = run_generic<A, B, D>(p, first, second, dst->address, s);
            }
        });
    });
    return status;
}

// Partial sums of tannic_hip_gemm_noalloc: device memory that exists from the moment the library's code is loaded on a
// device until the process ends, one copy per device.
constexpr size_t kNoAllocScratchBytes = TANNIC_GEMM_NOALLOC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

// The array's address on the current device.  In host code the name `scratch` is only a handle for this lookup; the
// kernels are given the address it returns.  Looked up once per device, with that device current.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_address[kMaxDevices];

int scratch_address(void** out) {
    int device = 0;
    TH_TRY(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) {
        set_error_text("gemm_noalloc: device id beyond the table of scratch addresses");
        return TANNIC_ERROR;
    }
    void* ptr = g_scratch_address[device].load(std::memory_order_acquire);
    if (!ptr) {
        TH_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        g_scratch_address[device].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return TANNIC_SUCCESS;
}

}  // namespace

extern "C" int tannic_hip_gemm(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream) {
    return gemm_entry(a, b, dst, stream, nullptr);
}

extern "C" int tannic_hip_gemm_noalloc(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream) {
    void* base = nullptr;
    if (int rc = scratch_address(&base)) return rc;
    const GemmWorkspace workspace{base, kNoAllocScratchBytes};
    return gemm_entry(a, b, dst, stream, &workspace);
}
