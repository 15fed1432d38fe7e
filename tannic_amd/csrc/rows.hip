// Row-wise operators the reference does not have: RMS normalisation, softmax, rotary embedding.
// A Tannic program writes each as a chain of the reference's operators (mean of squares, rsqrt, products;
// max, difference, exp, sum, products; products and sums on stride-2 slices), which moves every intermediate
// through HBM once per operator.  Here a row is read once, kept in registers, and written once; the arithmetic
// is float (double for float64) with one rounding at the end.
//   rms_norm : y[r, i] = x[r, i] / sqrt(mean_i(x[r, i]^2) + eps) * gain[i]           over the last axis
//   softmax  : s = x[r, i] * scale + mask[r mod Q, i];  y = exp(s - max_i s) / sum_i exp(s - max_i s)
//              over the last axis; mask is optional, [Q, L] with Q = x's second-to-last extent.  A row whose
//              s are all -inf gives NaN, as the chain of operators does.
//   rope     : pairs (2i, 2i+1) of the last axis rotated by the angle of position n (second-to-last axis):
//              y[2i] = x[2i] * cos[n, i] - x[2i+1] * sin[n, i],  y[2i+1] = x[2i] * sin[n, i] + x[2i+1] * cos[n, i]
// HBM-bound: one wavefront per row for short rows (four rows per block), one block per row for long ones,
// 16-byte accesses per lane; rows that are misaligned, ragged or longer than the registers hold take a scalar
// kernel that re-reads the row from cache.
#include "elementwise.hpp"
#include "lanes.hpp"

namespace th {

constexpr int kRowBlock = 256;
constexpr int kRowMaxChunks = 8;   // 16-byte pieces of a row held per thread

template <class T> using RowAcc = std::conditional_t<std::is_same_v<T, double>, double, float>;

struct AddOp {
    template <class A> __device__ static inline A combine(A x, A y) { return x + y; }
};
struct MaxOp {
    __device__ static inline float combine(float x, float y) { return fmaxf(x, y); }
    __device__ static inline double combine(double x, double y) { return fmax(x, y); }
};

// One value per group of G threads (a wavefront, or the whole block through LDS), identical in every thread.
template <class Op, int G, class A>
__device__ inline A group_reduce(A v, A* lds) {
    v = wave_reduce<Op>(v);
    if constexpr (G > 64) {
        __syncthreads();   // the previous use of lds has been read
        if (threadIdx.x % 64 == 0) lds[threadIdx.x / 64] = v;
        __syncthreads();
        v = Op::combine(Op::combine(lds[0], lds[1]), Op::combine(lds[2], lds[3]));
    }
    return v;
}

template <class A> __device__ inline A fast_exp(A x, bool coarse) {
    if constexpr (std::is_same_v<A, double>) return exp(x);
    else return coarse ? __expf(x) : expf(x);
}

// ---- RMS normalisation ----------------------------------------------------------
template <class T, int G, int NCH>
__global__ __launch_bounds__(kRowBlock) void rms_norm_kernel(const T* x, const T* gain, T* y, uint32_t rows, uint32_t L, double eps) {
    constexpr int VEC = 16 / sizeof(T);
    using A = RowAcc<T>;
    __shared__ A lds[4];
    const uint32_t t = threadIdx.x % G;
    const uint32_t row = blockIdx.x * (kRowBlock / G) + threadIdx.x / G;
    const bool live = row < rows;
    const uint32_t chunks = L / VEC;
    const size_t base = static_cast<size_t>(live ? row : 0) * L;
    Pack<T, VEC> v[NCH];
    A ss = 0;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = t + i * G;
        if (live && c < chunks) {
            v[i] = load_pack<T, VEC>(x + base + static_cast<size_t>(c) * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const A a = static_cast<A>(widen(v[i].v[e]));
                ss += a * a;
            }
        }
    }
    ss = group_reduce<AddOp, G>(ss, lds);
    const A r = A(1) / sqrt(ss / static_cast<A>(L) + static_cast<A>(eps));
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = t + i * G;
        if (live && c < chunks) {
            const Pack<T, VEC> g = *reinterpret_cast<const Pack<T, VEC>*>(gain + static_cast<size_t>(c) * VEC);
            Pack<T, VEC> out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) out.v[e] = narrow<T>(static_cast<A>(widen(v[i].v[e])) * r * static_cast<A>(widen(g.v[e])));
            store_pack<T, VEC>(y + base + static_cast<size_t>(c) * VEC, out);
        }
    }
}

// any length, any alignment: one block per row, the row read twice
template <class T>
__global__ __launch_bounds__(kRowBlock) void rms_norm_any_kernel(const T* x, const T* gain, T* y, uint32_t L, double eps) {
    using A = RowAcc<T>;
    __shared__ A lds[4];
    const size_t base = static_cast<size_t>(blockIdx.x) * L;
    A ss = 0;
    for (uint32_t i = threadIdx.x; i < L; i += kRowBlock) {
        const A a = static_cast<A>(widen(x[base + i]));
        ss += a * a;
    }
    ss = group_reduce<AddOp, kRowBlock>(ss, lds);
    const A r = A(1) / sqrt(ss / static_cast<A>(L) + static_cast<A>(eps));
    for (uint32_t i = threadIdx.x; i < L; i += kRowBlock)
        y[base + i] = narrow<T>(static_cast<A>(widen(x[base + i])) * r * static_cast<A>(widen(gain[i])));
}

// ---- softmax ----------------------------------------------------------------------
template <class T, int G, int NCH, bool MASK>
__global__ __launch_bounds__(kRowBlock) void softmax_kernel(const T* x, const T* mask, T* y, uint32_t rows, uint32_t L, FastDiv q, float scale) {
    constexpr int VEC = 16 / sizeof(T);
    using A = RowAcc<T>;
    __shared__ A lds[4];
    const uint32_t t = threadIdx.x % G;
    const uint32_t row = blockIdx.x * (kRowBlock / G) + threadIdx.x / G;
    const bool live = row < rows;
    const uint32_t chunks = L / VEC;
    const size_t base = static_cast<size_t>(live ? row : 0) * L;
    uint32_t mrow = 0, quotient = 0;
    if (MASK) q.divmod(live ? row : 0, quotient, mrow);
    A s[NCH][VEC];
    A top = -INFINITY;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = t + i * G;
        if (live && c < chunks) {
            const Pack<T, VEC> v = load_pack<T, VEC>(x + base + static_cast<size_t>(c) * VEC);
            Pack<T, VEC> m;
            if (MASK) m = *reinterpret_cast<const Pack<T, VEC>*>(mask + static_cast<size_t>(mrow) * L + static_cast<size_t>(c) * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                A a = static_cast<A>(widen(v.v[e])) * static_cast<A>(scale);
                if (MASK) a += static_cast<A>(widen(m.v[e]));
                s[i][e] = a;
                top = MaxOp::combine(top, a);
            }
        }
    }
    top = group_reduce<MaxOp, G>(top, lds);
    A sum = 0;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = t + i * G;
        if (live && c < chunks) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                s[i][e] = fast_exp(s[i][e] - top, is_16bit<T>::value);
                sum += s[i][e];
            }
        }
    }
    sum = group_reduce<AddOp, G>(sum, lds);
    const A inv = A(1) / sum;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const uint32_t c = t + i * G;
        if (live && c < chunks) {
            Pack<T, VEC> out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) out.v[e] = narrow<T>(s[i][e] * inv);
            store_pack<T, VEC>(y + base + static_cast<size_t>(c) * VEC, out);
        }
    }
}

// Rows of up to 64 * NE elements whose length or start no 16-byte access fits (attention over 197 or 1025 positions): a
// wavefront per row, a lane holding elements lane, lane + 64, ...: one read of the row, single-element accesses that a
// wavefront still makes as whole lines.
template <class T, int NE, bool MASK>
__global__ __launch_bounds__(kRowBlock) void softmax_wave_kernel(const T* x, const T* mask, T* y, uint32_t rows, uint32_t L, FastDiv q, float scale) {
    using A = RowAcc<T>;
    const uint32_t lane = threadIdx.x % 64, row = blockIdx.x * (kRowBlock / 64) + threadIdx.x / 64;
    if (row >= rows) return;   // whole wavefronts; nothing below synchronises across them
    const size_t base = static_cast<size_t>(row) * L;
    uint32_t mrow = 0, quotient = 0;
    if (MASK) q.divmod(row, quotient, mrow);
    A s[NE];
    A top = -INFINITY;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        const uint32_t i = lane + 64 * e;
        s[e] = -INFINITY;
        if (i < L) {
            s[e] = static_cast<A>(widen(x[base + i])) * static_cast<A>(scale);
            if (MASK) s[e] += static_cast<A>(widen(mask[static_cast<size_t>(mrow) * L + i]));
        }
        top = MaxOp::combine(top, s[e]);
    }
    top = wave_reduce<MaxOp>(top);
    A sum = 0;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        s[e] = lane + 64 * e < L ? fast_exp(s[e] - top, is_16bit<T>::value) : A(0);
        sum += s[e];
    }
    sum = wave_reduce<AddOp>(sum);
    const A inv = A(1) / sum;
#pragma unroll
    for (int e = 0; e < NE; ++e)
        if (lane + 64 * e < L) y[base + lane + 64 * e] = narrow<T>(s[e] * inv);
}

// Many rows of at most 16 elements (of one: the softmax over a dim of extent 1): a lane per row, the row in its registers.
template <class T, bool MASK>
__global__ __launch_bounds__(kRowBlock) void softmax_lane_kernel(const T* x, const T* mask, T* y, uint32_t rows, uint32_t L, FastDiv q, float scale) {
    using A = RowAcc<T>;
    const uint32_t row = blockIdx.x * kRowBlock + threadIdx.x;
    if (row >= rows) return;
    const size_t base = static_cast<size_t>(row) * L;
    uint32_t mrow = 0, quotient = 0;
    if (MASK) q.divmod(row, quotient, mrow);
    A s[16];
    A top = -INFINITY;
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i) {
        s[i] = -INFINITY;
        if (i < L) {
            s[i] = static_cast<A>(widen(x[base + i])) * static_cast<A>(scale);
            if (MASK) s[i] += static_cast<A>(widen(mask[static_cast<size_t>(mrow) * L + i]));
        }
        top = MaxOp::combine(top, s[i]);
    }
    A sum = 0;
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i) {
        s[i] = i < L ? fast_exp(s[i] - top, is_16bit<T>::value) : A(0);
        sum += s[i];
    }
    const A inv = A(1) / sum;
#pragma unroll
    for (uint32_t i = 0; i < 16; ++i)
        if (i < L) y[base + i] = narrow<T>(s[i] * inv);
}

// any length, any alignment: one block per row, the row read three times (from cache after the first), four elements of a
// thread on their way at a time
template <class T, bool MASK>
__global__ __launch_bounds__(kRowBlock) void softmax_any_kernel(const T* x, const T* mask, T* y, uint32_t L, FastDiv q, float scale) {
    using A = RowAcc<T>;
    __shared__ A lds[4];
    const size_t base = static_cast<size_t>(blockIdx.x) * L;
    uint32_t mrow = 0, quotient = 0;
    if (MASK) q.divmod(blockIdx.x, quotient, mrow);
    const T* mk = MASK ? mask + static_cast<size_t>(mrow) * L : nullptr;
    auto value = [&](uint32_t i) {
        A a = static_cast<A>(widen(x[base + i])) * static_cast<A>(scale);
        if (MASK) a += static_cast<A>(widen(mk[i]));
        return a;
    };
    // four values at i, i + 256, ... (-inf past the end of the row)
    auto four = [&](uint32_t i, A (&v)[4]) {
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * kRowBlock < L ? value(i + u * kRowBlock) : static_cast<A>(-INFINITY);
    };
    A top = -INFINITY;
    for (uint32_t i = threadIdx.x; i < L; i += 4 * kRowBlock) {
        A v[4];
        four(i, v);
#pragma unroll
        for (int u = 0; u < 4; ++u) top = MaxOp::combine(top, v[u]);
    }
    top = group_reduce<MaxOp, kRowBlock>(top, lds);
    A sum = 0;
    for (uint32_t i = threadIdx.x; i < L; i += 4 * kRowBlock) {
        A v[4];
        four(i, v);
#pragma unroll
        for (int u = 0; u < 4; ++u) sum += i + u * kRowBlock < L ? fast_exp(v[u] - top, is_16bit<T>::value) : A(0);
    }
    sum = group_reduce<AddOp, kRowBlock>(sum, lds);
    const A inv = A(1) / sum;
    for (uint32_t i = threadIdx.x; i < L; i += 4 * kRowBlock) {
        A v[4];
        four(i, v);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (i + u * kRowBlock < L) y[base + i + u * kRowBlock] = narrow<T>(fast_exp(v[u] - top, is_16bit<T>::value) * inv);
    }
}

// A few very long rows (the probabilities of a vocabulary's logits, one row per sequence): one block per row leaves the
// chip idle and walks the row three times.  Here a row is shared by gridDim.x blocks.  The first kernel leaves, per block,
// the largest value of its range and the sum of exp(value - that); the second combines a row's pairs (every block for
// itself: they are few) into the row's maximum and sum and writes its range.
template <class T, bool MASK>
__global__ __launch_bounds__(kRowBlock) void softmax_shared_rows_first_kernel(const T* x, const T* mask, RowAcc<T>* partial, uint32_t L, FastDiv q, float scale,
                                                                              uint32_t per_block) {
    using A = RowAcc<T>;
    __shared__ A lds[4];
    const uint32_t row = blockIdx.y, first = blockIdx.x * per_block, end = first + per_block < L ? first + per_block : L;
    const size_t base = static_cast<size_t>(row) * L;
    uint32_t mrow = 0, quotient = 0;
    if (MASK) q.divmod(row, quotient, mrow);
    const T* mk = MASK ? mask + static_cast<size_t>(mrow) * L : nullptr;
    auto value = [&](uint32_t i) {
        A a = static_cast<A>(widen(x[base + i])) * static_cast<A>(scale);
        if (MASK) a += static_cast<A>(widen(mk[i]));
        return a;
    };
    A top = -INFINITY;
    for (uint32_t i = first + threadIdx.x; i < end; i += 4 * kRowBlock) {
        A v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * kRowBlock < end ? value(i + u * kRowBlock) : static_cast<A>(-INFINITY);
#pragma unroll
        for (int u = 0; u < 4; ++u) top = MaxOp::combine(top, v[u]);
    }
    top = group_reduce<MaxOp, kRowBlock>(top, lds);
    A sum = 0;
    for (uint32_t i = first + threadIdx.x; i < end; i += 4 * kRowBlock) {
        A v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = i + u * kRowBlock < end ? value(i + u * kRowBlock) : static_cast<A>(-INFINITY);
#pragma unroll
        for (int u = 0; u < 4; ++u) sum += i + u * kRowBlock < end ? fast_exp(v[u] - top, is_16bit<T>::value) : A(0);
    }
    sum = group_reduce<AddOp, kRowBlock>(sum, lds);
    if (threadIdx.x == 0) {
        A* out = partial + (static_cast<size_t>(row) * gridDim.x + blockIdx.x) * 2;
        out[0] = top;
        out[1] = top == static_cast<A>(-INFINITY) ? A(0) : sum;   // a range of -inf only: nothing to add (its own sum is NaN)
    }
}

template <class T, bool MASK>
__global__ __launch_bounds__(kRowBlock) void softmax_shared_rows_second_kernel(const T* x, const T* mask, T* y, const RowAcc<T>* partial, uint32_t L, FastDiv q,
                                                                               float scale, uint32_t per_block) {
    using A = RowAcc<T>;
    const uint32_t row = blockIdx.y, first = blockIdx.x * per_block, end = first + per_block < L ? first + per_block : L;
    const size_t base = static_cast<size_t>(row) * L;
    // the row's maximum and sum from its blocks' pairs (at most 64 of them: a lane each, every wavefront for itself)
    const uint32_t lane = threadIdx.x % 64;
    const A* pairs = partial + static_cast<size_t>(row) * gridDim.x * 2;
    const A my_top = lane < gridDim.x ? pairs[2 * lane] : static_cast<A>(-INFINITY);
    const A my_sum = lane < gridDim.x ? pairs[2 * lane + 1] : A(0);
    const A top = wave_reduce<MaxOp>(my_top);
    // a block whose range held nothing above -inf contributes nothing; a row of -inf only has the sum 0 and, from
    // exp(-inf - -inf) below, NaN everywhere, as the definition has it
    const A sum = wave_reduce<AddOp>(my_top == static_cast<A>(-INFINITY) ? A(0) : my_sum * fast_exp(my_top - top, false));
    const A inv = A(1) / sum;
    uint32_t mrow = 0, quotient = 0;
    if (MASK) q.divmod(row, quotient, mrow);
    const T* mk = MASK ? mask + static_cast<size_t>(mrow) * L : nullptr;
    for (uint32_t i = first + threadIdx.x; i < end; i += kRowBlock) {
        A a = static_cast<A>(widen(x[base + i])) * static_cast<A>(scale);
        if (MASK) a += static_cast<A>(widen(mk[i]));
        y[base + i] = narrow<T>(fast_exp(a - top, is_16bit<T>::value) * inv);
    }
}

// ---- rotary embedding -----------------------------------------------------------------
struct RopeMap {
    int outer;                              // dims in front of the last one
    uint32_t extent[TANNIC_DIMENSIONS];
    FastDiv div[TANNIC_DIMENSIONS];
    int64_t stride[TANNIC_DIMENSIONS];      // of x, in elements
    int64_t last_stride;
    uint32_t d, row_items;                  // last extent; threads per row
    FastDiv item_div;
    uint32_t total;
};

// PAIRS rotations per thread: PAIRS * 2 consecutive elements of the last axis
template <class T, int PAIRS>
__global__ __launch_bounds__(kRowBlock) void rope_kernel(const T* x, const T* cs, const T* sn, T* y, RopeMap m) {
    using A = RowAcc<T>;
    const uint32_t idx = blockIdx.x * kRowBlock + threadIdx.x;
    if (idx >= m.total) return;
    uint32_t row, item;
    m.item_div.divmod(idx, row, item);
    int64_t off = 0;
    uint32_t pos = 0, rest = row;
    for (int k = m.outer - 1; k >= 0; --k) {
        uint32_t qv, c;
        m.div[k].divmod(rest, qv, c);
        rest = qv;
        off += static_cast<int64_t>(c) * m.stride[k];
        if (k == m.outer - 1) pos = c;
    }
    const uint32_t col = item * (2 * PAIRS);
    const size_t table = static_cast<size_t>(pos) * (m.d / 2) + item * PAIRS;
    Pack<T, 2 * PAIRS> v;
    Pack<T, PAIRS> c, s;
    if constexpr (PAIRS > 1) {
        v = load_pack<T, 2 * PAIRS>(x + off + col);
        c = *reinterpret_cast<const Pack<T, PAIRS>*>(cs + table);
        s = *reinterpret_cast<const Pack<T, PAIRS>*>(sn + table);
    } else {
        v.v[0] = x[off + static_cast<int64_t>(col) * m.last_stride];
        v.v[1] = x[off + static_cast<int64_t>(col + 1) * m.last_stride];
        c.v[0] = cs[table];
        s.v[0] = sn[table];
    }
    Pack<T, 2 * PAIRS> out;
#pragma unroll
    for (int i = 0; i < PAIRS; ++i) {
        const A a = static_cast<A>(widen(v.v[2 * i])), b = static_cast<A>(widen(v.v[2 * i + 1]));
        const A co = static_cast<A>(widen(c.v[i])), si = static_cast<A>(widen(s.v[i]));
        out.v[2 * i] = narrow<T>(a * co - b * si);
        out.v[2 * i + 1] = narrow<T>(a * si + b * co);
    }
    T* dst = y + static_cast<size_t>(row) * m.d + col;
    if constexpr (PAIRS > 1) {
        store_pack<T, 2 * PAIRS>(dst, out);
    } else {
        dst[0] = out.v[0];
        dst[1] = out.v[1];
    }
}

// ---- host side ---------------------------------------------------------------------------
inline bool is_contiguous(const tannic_tensor_t* t) {
    int64_t run = 1;
    for (int d = t->rank - 1; d >= 0; --d) {
        if (t->shape.sizes[d] != 1 && t->strides.sizes[d] != run) return false;
        run *= static_cast<int64_t>(t->shape.sizes[d]);
    }
    return true;
}

inline bool same_shape(const tannic_tensor_t* a, const tannic_tensor_t* b) {
    if (a->rank != b->rank) return false;
    for (int d = 0; d < a->rank; ++d)
        if (a->shape.sizes[d] != b->shape.sizes[d]) return false;
    return true;
}

inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

// Group width and chunks per thread for rows of `chunks` 16-byte pieces; false when the registers cannot hold a row.
inline bool row_shape(uint32_t chunks, uint32_t rows, int& group, int& nch) {
    group = (chunks <= 64 * 4 && rows >= 1024) || chunks <= 64 ? 64 : kRowBlock;
    const uint32_t per = (chunks + group - 1) / group;
    if (per > kRowMaxChunks) return false;
    nch = per <= 1 ? 1 : per <= 2 ? 2 : per <= 4 ? 4 : 8;
    return true;
}

template <class T, int G, int NCH>
int launch_rms(const T* x, const T* g, T* y, uint32_t rows, uint32_t L, double eps, hipStream_t stream) {
    const uint32_t per_block = kRowBlock / G;
    hipLaunchKernelGGL((rms_norm_kernel<T, G, NCH>), dim3((rows + per_block - 1) / per_block), dim3(kRowBlock), 0, stream, x, g, y, rows, L, eps);
    return launch_status("rms_norm_kernel");
}

template <class T, int G>
int pick_rms(int nch, const T* x, const T* g, T* y, uint32_t rows, uint32_t L, double eps, hipStream_t stream) {
    switch (nch) {
        case 1: return launch_rms<T, G, 1>(x, g, y, rows, L, eps, stream);
        case 2: return launch_rms<T, G, 2>(x, g, y, rows, L, eps, stream);
        case 4: return launch_rms<T, G, 4>(x, g, y, rows, L, eps, stream);
        default: return launch_rms<T, G, 8>(x, g, y, rows, L, eps, stream);
    }
}

template <class T>
int run_rms(const tannic_tensor_t* x, const tannic_tensor_t* gain, tannic_tensor_t* dst, double eps, hipStream_t stream) {
    const uint32_t L = static_cast<uint32_t>(x->shape.sizes[x->rank - 1]);
    const size_t count = element_count(x);
    if (count == 0) return TANNIC_SUCCESS;
    const size_t rows64 = count / L;
    if (rows64 >= (1ull << 31)) {
        set_error_text("rms_norm: 2^31 rows or more are not supported");
        return TANNIC_ERROR;
    }
    const uint32_t rows = static_cast<uint32_t>(rows64);
    const T* px = static_cast<const T*>(x->address);
    const T* pg = static_cast<const T*>(gain->address);
    T* py = static_cast<T*>(dst->address);
    constexpr uint32_t VEC = 16 / sizeof(T);
    int group, nch;
    if (L % VEC == 0 && aligned16(px) && aligned16(pg) && aligned16(py) && row_shape(L / VEC, rows, group, nch)) {
        if (group == 64) return pick_rms<T, 64>(nch, px, pg, py, rows, L, eps, stream);
        return pick_rms<T, kRowBlock>(nch, px, pg, py, rows, L, eps, stream);
    }
    hipLaunchKernelGGL((rms_norm_any_kernel<T>), dim3(rows), dim3(kRowBlock), 0, stream, px, pg, py, L, eps);
    return launch_status("rms_norm_any_kernel");
}

template <class T, int G, int NCH>
int launch_softmax(const T* x, const T* mask, T* y, uint32_t rows, uint32_t L, uint32_t q, float scale, hipStream_t stream) {
    const uint32_t per_block = kRowBlock / G;
    const dim3 grid((rows + per_block - 1) / per_block);
    if (mask) hipLaunchKernelGGL((softmax_kernel<T, G, NCH, true>), grid, dim3(kRowBlock), 0, stream, x, mask, y, rows, L, FastDiv(q), scale);
    else hipLaunchKernelGGL((softmax_kernel<T, G, NCH, false>), grid, dim3(kRowBlock), 0, stream, x, mask, y, rows, L, FastDiv(1), scale);
    return launch_status("softmax_kernel");
}

template <class T, int G>
int pick_softmax(int nch, const T* x, const T* mask, T* y, uint32_t rows, uint32_t L, uint32_t q, float scale, hipStream_t stream) {
    switch (nch) {
        case 1: return launch_softmax<T, G, 1>(x, mask, y, rows, L, q, scale, stream);
        case 2: return launch_softmax<T, G, 2>(x, mask, y, rows, L, q, scale, stream);
        case 4: return launch_softmax<T, G, 4>(x, mask, y, rows, L, q, scale, stream);
        default: return launch_softmax<T, G, 8>(x, mask, y, rows, L, q, scale, stream);
    }
}

template <class T>
int run_softmax(const tannic_tensor_t* x, const tannic_tensor_t* mask, tannic_tensor_t* dst, float scale, hipStream_t stream) {
    const uint32_t L = static_cast<uint32_t>(x->shape.sizes[x->rank - 1]);
    const uint32_t Q = x->rank >= 2 ? static_cast<uint32_t>(x->shape.sizes[x->rank - 2]) : 1;
    const size_t count = element_count(x);
    if (count == 0) return TANNIC_SUCCESS;
    const size_t rows64 = count / L;
    if (rows64 >= (1ull << 31)) {
        set_error_text("softmax: 2^31 rows or more are not supported");
        return TANNIC_ERROR;
    }
    const uint32_t rows = static_cast<uint32_t>(rows64);
    const T* px = static_cast<const T*>(x->address);
    const T* pm = mask ? static_cast<const T*>(mask->address) : nullptr;
    T* py = static_cast<T*>(dst->address);
    constexpr uint32_t VEC = 16 / sizeof(T);
    int group, nch;
    if (L % VEC == 0 && aligned16(px) && aligned16(pm) && aligned16(py) && row_shape(L / VEC, rows, group, nch)) {
        if (group == 64) return pick_softmax<T, 64>(nch, px, pm, py, rows, L, Q, scale, stream);
        return pick_softmax<T, kRowBlock>(nch, px, pm, py, rows, L, Q, scale, stream);
    }
    if (rows <= 64 && L >= 16384) {
        // a handful of very long rows: up to 64 blocks per row, two kernels
        uint32_t splits = L / 4096;
        if (splits > 64) splits = 64;
        while (splits > 2 && splits * rows > 1024) splits /= 2;
        const uint32_t per_block = (L + splits - 1) / splits;
        RowAcc<T>* partial = nullptr;
        if (scratch_acquire(reinterpret_cast<void**>(&partial), sizeof(RowAcc<T>) * 2 * splits * rows, stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
        const dim3 grid(splits, rows);
        if (pm) hipLaunchKernelGGL((softmax_shared_rows_first_kernel<T, true>), grid, dim3(kRowBlock), 0, stream, px, pm, partial, L, FastDiv(Q), scale, per_block);
        else hipLaunchKernelGGL((softmax_shared_rows_first_kernel<T, false>), grid, dim3(kRowBlock), 0, stream, px, pm, partial, L, FastDiv(1), scale, per_block);
        int status = launch_status("softmax_shared_rows_first_kernel");
        if (status == TANNIC_SUCCESS) {
            if (pm) hipLaunchKernelGGL((softmax_shared_rows_second_kernel<T, true>), grid, dim3(kRowBlock), 0, stream, px, pm, py, partial, L, FastDiv(Q), scale, per_block);
            else hipLaunchKernelGGL((softmax_shared_rows_second_kernel<T, false>), grid, dim3(kRowBlock), 0, stream, px, pm, py, partial, L, FastDiv(1), scale, per_block);
            status = launch_status("softmax_shared_rows_second_kernel");
        }
        scratch_release(partial, stream);
        return status;
    }
    if (L <= 16 && rows >= 4096) {
        const dim3 grid((rows + kRowBlock - 1) / kRowBlock);
        if (pm) hipLaunchKernelGGL((softmax_lane_kernel<T, true>), grid, dim3(kRowBlock), 0, stream, px, pm, py, rows, L, FastDiv(Q), scale);
        else hipLaunchKernelGGL((softmax_lane_kernel<T, false>), grid, dim3(kRowBlock), 0, stream, px, pm, py, rows, L, FastDiv(1), scale);
        return launch_status("softmax_lane_kernel");
    }
    if (L <= 64 * 32 && rows >= 256) {
        // short rows that the vector kernel cannot take: a wavefront per row
        const dim3 grid((rows + kRowBlock / 64 - 1) / (kRowBlock / 64));
        auto launch = [&](auto with_mask, auto without) {
            if (pm) hipLaunchKernelGGL(with_mask, grid, dim3(kRowBlock), 0, stream, px, pm, py, rows, L, FastDiv(Q), scale);
            else hipLaunchKernelGGL(without, grid, dim3(kRowBlock), 0, stream, px, pm, py, rows, L, FastDiv(1), scale);
        };
        if (L <= 64 * 4) launch(softmax_wave_kernel<T, 4, true>, softmax_wave_kernel<T, 4, false>);
        else if (L <= 64 * 8) launch(softmax_wave_kernel<T, 8, true>, softmax_wave_kernel<T, 8, false>);
        else if (L <= 64 * 16) launch(softmax_wave_kernel<T, 16, true>, softmax_wave_kernel<T, 16, false>);
        else launch(softmax_wave_kernel<T, 32, true>, softmax_wave_kernel<T, 32, false>);
        return launch_status("softmax_wave_kernel");
    }
    if (pm) hipLaunchKernelGGL((softmax_any_kernel<T, true>), dim3(rows), dim3(kRowBlock), 0, stream, px, pm, py, L, FastDiv(Q), scale);
    else hipLaunchKernelGGL((softmax_any_kernel<T, false>), dim3(rows), dim3(kRowBlock), 0, stream, px, pm, py, L, FastDiv(1), scale);
    return launch_status("softmax_any_kernel");
}

template <class T>
int run_rope(const tannic_tensor_t* x, const tannic_tensor_t* cs, const tannic_tensor_t* sn, tannic_tensor_t* dst, hipStream_t stream) {
    const size_t count = element_count(x);
    if (count == 0) return TANNIC_SUCCESS;
    if (count >= (1ull << 31)) {
        set_error_text("rope: tensors of 2^31 elements or more are not supported");
        return TANNIC_ERROR;
    }
    RopeMap m{};
    m.outer = x->rank - 1;
    m.d = static_cast<uint32_t>(x->shape.sizes[x->rank - 1]);
    m.last_stride = x->shape.sizes[x->rank - 1] == 1 ? 0 : x->strides.sizes[x->rank - 1];
    constexpr int VEC = 16 / sizeof(T);
    bool wide = VEC >= 4 && m.d % VEC == 0 && m.last_stride == 1 && aligned16(x->address) && aligned16(dst->address) &&
                reinterpret_cast<uintptr_t>(cs->address) % (sizeof(T) * VEC / 2) == 0 && reinterpret_cast<uintptr_t>(sn->address) % (sizeof(T) * VEC / 2) == 0;
    for (int k = 0; k < m.outer; ++k) {
        m.extent[k] = static_cast<uint32_t>(x->shape.sizes[k]);
        m.div[k] = FastDiv(m.extent[k]);
        m.stride[k] = x->shape.sizes[k] == 1 ? 0 : x->strides.sizes[k];
        if (m.stride[k] % VEC) wide = false;
    }
    const T* px = static_cast<const T*>(x->address);
    const T* pc = static_cast<const T*>(cs->address);
    const T* ps = static_cast<const T*>(sn->address);
    T* py = static_cast<T*>(dst->address);
    const uint32_t rows = static_cast<uint32_t>(count / m.d);
    if constexpr (VEC >= 4) {
        if (wide) {
            m.row_items = m.d / VEC;
            m.item_div = FastDiv(m.row_items);
            m.total = rows * m.row_items;
            hipLaunchKernelGGL((rope_kernel<T, VEC / 2>), dim3((m.total + kRowBlock - 1) / kRowBlock), dim3(kRowBlock), 0, stream, px, pc, ps, py, m);
            return launch_status("rope_kernel");
        }
    }
    m.row_items = m.d / 2;
    m.item_div = FastDiv(m.row_items);
    m.total = rows * m.row_items;
    hipLaunchKernelGGL((rope_kernel<T, 1>), dim3((m.total + kRowBlock - 1) / kRowBlock), dim3(kRowBlock), 0, stream, px, pc, ps, py, m);
    return launch_status("rope_kernel");
}

template <class F> inline int with_float_type(int dtype, F&& f) {
    switch (dtype) {
        case TANNIC_FLOAT16: return f(type_tag<f16>{});
        case TANNIC_BFLOAT16: return f(type_tag<bf16>{});
        case TANNIC_FLOAT32: return f(type_tag<float>{});
        case TANNIC_FLOAT64: return f(type_tag<double>{});
        default: return TANNIC_UNSUPPORTED_DTYPE;
    }
}

}  // namespace th

using namespace th;

extern "C" {

int tannic_hip_rms_norm(const tannic_tensor_t* x, const tannic_tensor_t* gain, tannic_tensor_t* dst, tannic_stream_t stream, float eps) {
    if (!x || !gain || !dst) return TANNIC_ERROR;
    if (!have_storage(x, gain, dst)) return TANNIC_ERROR;
    if (x->dtype != gain->dtype || x->dtype != dst->dtype) return TANNIC_UNSUPPORTED_DTYPE;
    if (x->rank < 1 || !same_shape(x, dst) || !is_contiguous(x) || !is_contiguous(dst) || !is_contiguous(gain) ||
        element_count(gain) != x->shape.sizes[x->rank - 1]) {
        set_error_text("rms_norm: x and dst must be contiguous with one shape, gain must hold one value per element of the last axis");
        return TANNIC_ERROR;
    }
    return with_float_type(x->dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        return run_rms<T>(x, gain, dst, static_cast<double>(eps), as_stream(stream));
    });
}

int tannic_hip_softmax(const tannic_tensor_t* x, const tannic_tensor_t* mask, tannic_tensor_t* dst, tannic_stream_t stream, float scale) {
    if (!x || !dst) return TANNIC_ERROR;
    if (!have_storage(x, mask, dst)) return TANNIC_ERROR;
    if (x->dtype != dst->dtype || (mask && mask->dtype != x->dtype)) return TANNIC_UNSUPPORTED_DTYPE;
    if (x->rank < 1 || !same_shape(x, dst) || !is_contiguous(x) || !is_contiguous(dst)) {
        set_error_text("softmax: x and dst must be contiguous with one shape");
        return TANNIC_ERROR;
    }
    if (mask) {
        const size_t L = x->shape.sizes[x->rank - 1], Q = x->rank >= 2 ? x->shape.sizes[x->rank - 2] : 1;
        const bool shaped = (mask->rank == 2 && mask->shape.sizes[0] == Q && mask->shape.sizes[1] == L) || (mask->rank == 1 && Q == 1 && mask->shape.sizes[0] == L);
        if (!shaped || !is_contiguous(mask)) {
            set_error_text("softmax: mask must be contiguous with the last two extents of x");
            return TANNIC_ERROR;
        }
    }
    return with_float_type(x->dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        return run_softmax<T>(x, mask, dst, scale, as_stream(stream));
    });
}

int tannic_hip_rope(const tannic_tensor_t* x, const tannic_tensor_t* cos, const tannic_tensor_t* sin, tannic_tensor_t* dst, tannic_stream_t stream) {
    if (!x || !cos || !sin || !dst) return TANNIC_ERROR;
    if (!have_storage(x, cos, sin, dst)) return TANNIC_ERROR;
    if (x->dtype != dst->dtype || cos->dtype != x->dtype || sin->dtype != x->dtype) return TANNIC_UNSUPPORTED_DTYPE;
    bool ok = x->rank >= 2 && same_shape(x, dst) && is_contiguous(dst) && is_contiguous(cos) && is_contiguous(sin) && same_shape(cos, sin) && cos->rank == 2;
    if (ok) {
        const size_t n = x->shape.sizes[x->rank - 2], d = x->shape.sizes[x->rank - 1];
        ok = d % 2 == 0 && cos->shape.sizes[0] == n && cos->shape.sizes[1] == d / 2;
    }
    if (!ok) {
        set_error_text("rope: x [.., n, d] with even d, cos and sin contiguous [n, d/2], dst contiguous with x's shape");
        return TANNIC_ERROR;
    }
    return with_float_type(x->dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        return run_rope<T>(x, cos, sin, dst, as_stream(stream));
    });
}

}  // extern "C"
