// The streaming engine behind every elementwise entry point.
//
// HBM-bound work: the goal is 16-byte accesses per lane, every byte of every
// operand touched once, and index arithmetic cheap enough to hide behind the
// memory stream.  No matrix cores are involved.
//
// Host side: the destination's index space and the operands' element strides
// (size-1 dims already rewritten to stride 0, operands right-aligned on the
// destination) are collapsed: dims of extent 1 vanish and neighbours that are
// jointly contiguous for every operand merge.  A full-size contiguous operand
// pair thus becomes ONE dim, X[64,4096,1024] (+) Z[1,4096,1] becomes three.
//
// Device side: the last collapsed dim is the "row".  A thread owns VEC
// consecutive row elements (VEC*sizeof = 16 bytes); an operand whose row
// stride is 0 is loaded once and splat.  The row number is decoded into outer
// coordinates with multiply-shift division by launch-time constants.  When
// alignment or strides rule out vectors the same kernel is instantiated with
// VEC = 1 and arbitrary row strides.
#pragma once

#include "common.hpp"

namespace th {

constexpr int kMaxOperands = 3;  // two sources + destination

struct Plan {
    int rank;                              // collapsed rank, >= 1
    uint32_t extent[TANNIC_DIMENSIONS];    // collapsed extents
    FastDiv div[TANNIC_DIMENSIONS];        // division by extent[d]
    int64_t stride[kMaxOperands][TANNIC_DIMENSIONS];  // element strides per operand
    uint32_t row_vectors;                  // vectors per row (set at launch)
    FastDiv row_div;                       // division by row_vectors
    uint32_t total_vectors;                // rows * row_vectors
};

// Collapses `rank` dims.  strides[o][d] are element strides of operand o.
// Returns false when the index space cannot be addressed (see below); the launch checks the vector count.
inline bool build_plan(Plan& p, int rank, const size_t* extent, const int64_t (*strides)[TANNIC_DIMENSIONS], int operands) {
    size_t ext[TANNIC_DIMENSIONS];
    int64_t st[kMaxOperands][TANNIC_DIMENSIONS];
    int r = 0;
    for (int d = 0; d < rank; ++d) {
        if (extent[d] == 1) continue;
        bool merged = false;
        if (r > 0) {
            merged = true;
            for (int o = 0; o < operands; ++o)
                if (st[o][r - 1] != strides[o][d] * static_cast<int64_t>(extent[d])) merged = false;
            if (merged) {
                ext[r - 1] *= extent[d];
                for (int o = 0; o < operands; ++o) st[o][r - 1] = strides[o][d];
            }
        }
        if (!merged) {
            ext[r] = extent[d];
            for (int o = 0; o < operands; ++o) st[o][r] = strides[o][d];
            ++r;
        }
    }
    if (r == 0) {
        ext[0] = 1;
        for (int o = 0; o < operands; ++o) st[o][0] = 1;
        r = 1;
    }
    // A thread's index counts 16-byte vectors and stays below 2^31 (what the multiply-shift division takes); the element
    // count may go beyond that.  A dim of 2^31 elements or more (a large contiguous tensor collapses to one) is cut in
    // two at a power of two, so that every extent fits; what cannot be cut that way is refused.
    for (int d = 0; d < r; ++d) {
        if (ext[d] < (1ull << 31)) continue;
        if (r == TANNIC_DIMENSIONS) return false;
        size_t inner = size_t(1) << 20;
        while (inner > 1 && ext[d] % inner != 0) inner >>= 1;
        if (ext[d] / inner >= (1ull << 31)) return false;
        for (int e = r; e > d + 1; --e) {
            ext[e] = ext[e - 1];
            for (int o = 0; o < operands; ++o) st[o][e] = st[o][e - 1];
        }
        ext[d + 1] = inner;
        ext[d] /= inner;
        for (int o = 0; o < operands; ++o) {
            st[o][d + 1] = st[o][d];
            st[o][d] = st[o][d] * static_cast<int64_t>(inner);
        }
        ++r;
        ++d;
    }
    size_t total = 1;
    for (int d = 0; d < r; ++d) {
        total *= ext[d];
        if (total >= (1ull << 36)) return false;
    }
    p.rank = r;
    for (int d = 0; d < TANNIC_DIMENSIONS; ++d) {
        p.extent[d] = d < r ? static_cast<uint32_t>(ext[d]) : 1;
        p.div[d] = FastDiv(p.extent[d]);
        for (int o = 0; o < kMaxOperands; ++o) p.stride[o][d] = (d < r && o < operands) ? st[o][d] : 0;
    }
    return true;
}

template <class T, int N>
struct alignas(sizeof(T) * N >= 16 ? 16 : sizeof(T) * N) Pack {
    T v[N];
};

// Register image of BYTES bytes that the memory instructions understand.
template <int BYTES> struct RawBits;
template <> struct RawBits<16> { using type = unsigned int __attribute__((ext_vector_type(4))); };
template <> struct RawBits<8> { using type = unsigned int __attribute__((ext_vector_type(2))); };
template <> struct RawBits<4> { using type = unsigned int; };
template <> struct RawBits<2> { using type = unsigned short; };
template <> struct RawBits<1> { using type = unsigned char; };

#ifndef TH_NONTEMPORAL
#define TH_NONTEMPORAL 1
#endif

// Loads N consecutive elements with one access of sizeof(T)*N bytes.  Operand
// streams are read once and results written once, so both bypass temporal
// caching.
template <class T, int N>
__device__ inline Pack<T, N> load_pack(const T* p) {
    static_assert(sizeof(T) * N <= 16, "a pack is at most 16 bytes");
    using Raw = typename RawBits<sizeof(T) * N>::type;
#if TH_NONTEMPORAL
    const Raw raw = __builtin_nontemporal_load(reinterpret_cast<const Raw*>(p));
#else
    const Raw raw = *reinterpret_cast<const Raw*>(p);
#endif
    Pack<T, N> r;
    __builtin_memcpy(&r, &raw, sizeof r);
    return r;
}

template <class T, int N>
__device__ inline void store_pack(T* p, const Pack<T, N>& v) {
    using Raw = typename RawBits<sizeof(T) * N>::type;
    Raw raw;
    __builtin_memcpy(&raw, &v, sizeof raw);
#if TH_NONTEMPORAL
    __builtin_nontemporal_store(raw, reinterpret_cast<Raw*>(p));
#else
    *reinterpret_cast<Raw*>(p) = raw;
#endif
}

template <class T, int N>
__device__ inline Pack<T, N> load_or_splat(const T* p, bool splat) {
    if (!splat) return load_pack<T, N>(p);
    Pack<T, N> r;
    const T s = *p;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = s;
    return r;
}

constexpr int kBlock = 256;

// Element offsets of vector `v` in the three operands.
struct Offsets {
    int64_t o0, o1, od;
};

template <int VEC>
__device__ inline Offsets decode(const Plan& p, uint32_t v) {
    const int last = p.rank - 1;
    uint32_t row, col;
    p.row_div.divmod(v, row, col);
    col *= VEC;
    Offsets o;
    o.o0 = static_cast<int64_t>(col) * p.stride[0][last];
    o.o1 = static_cast<int64_t>(col) * p.stride[1][last];
    o.od = static_cast<int64_t>(col) * p.stride[2][last];
    for (int d = last - 1; d >= 0; --d) {
        uint32_t q, c;
        p.div[d].divmod(row, q, c);
        row = q;
        o.o0 += static_cast<int64_t>(c) * p.stride[0][d];
        o.o1 += static_cast<int64_t>(c) * p.stride[1][d];
        o.od += static_cast<int64_t>(c) * p.stride[2][d];
    }
    return o;
}

// F: { using S0, S1, D; static constexpr int sources; const S0* a; const S1* b; D* out;
//      __device__ D operator()(S0, S1) const; }   (S1/b unused when sources == 1)
// UNROLL vectors per thread, kBlock apart.  One is best for plain contiguous operands; with a broadcast operand a
// thread lives longer (row decoding, the dependent load of the repeated value) and two keep enough bytes in flight.
template <class F, int VEC, int UNROLL>
__global__ __launch_bounds__(kBlock) void elementwise_kernel(F f, Plan p) {
    constexpr int kUnroll = UNROLL;
    using S0 = typename F::S0;
    using S1 = typename F::S1;
    using D = typename F::D;
    const int last = p.rank - 1;
    const bool splat0 = p.stride[0][last] == 0;
    const bool splat1 = p.stride[1][last] == 0;
    const uint32_t base = blockIdx.x * (kBlock * kUnroll) + threadIdx.x;
    if constexpr (VEC == 1) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t v = base + u * kBlock;
            if (v < p.total_vectors) {
                const Offsets o = decode<1>(p, v);
                if constexpr (F::sources == 2) f.out[o.od] = f(f.a[o.o0], f.b[o.o1]);
                else f.out[o.od] = f(f.a[o.o0], S1{});
            }
        }
    } else {
        // all loads of the unrolled group are issued before any store
        Pack<S0, VEC> a[kUnroll];
        Pack<S1, VEC> b[kUnroll];
        Offsets o[kUnroll];
        bool live[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t v = base + u * kBlock;
            live[u] = v < p.total_vectors;
            if (live[u]) {
                o[u] = decode<VEC>(p, v);
                a[u] = load_or_splat<S0, VEC>(f.a + o[u].o0, splat0);
                if constexpr (F::sources == 2) b[u] = load_or_splat<S1, VEC>(f.b + o[u].o1, splat1);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (live[u]) {
                Pack<D, VEC> r;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    if constexpr (F::sources == 2) r.v[i] = f(a[u].v[i], b[u].v[i]);
                    else r.v[i] = f(a[u].v[i], S1{});
                }
                store_pack<D, VEC>(f.out + o[u].od, r);
            }
        }
    }
}

// Rows whose length is not a multiple of the vector (softmax over 197 columns: x - max, x / sum) when every operand is
// either contiguous over the whole index space or constant along the row: the kernel above would go element by element,
// but the contiguous operands do not care where a row ends.  A thread owns VEC consecutive elements of the flat index
// space (the last thread of all a shorter tail); the row-constant operand is looked up for the row of the thread's first
// element and, when the vector runs over the row's end, for the next row (rows are at least VEC long: two rows at most).
struct FlatPlan {
    Plan p;                 // the collapsed plan; p.row_div divides by the row length
    uint64_t elements;      // all of them
    uint32_t rows;          // product of the outer extents
    bool full[2];           // source o is contiguous over everything (else constant along the row)
};

template <class T>
__device__ inline int64_t outer_offset(const Plan& p, int o, uint32_t row) {
    int64_t off = 0;
    for (int d = p.rank - 2; d >= 0; --d) {
        uint32_t q, c;
        p.div[d].divmod(row, q, c);
        row = q;
        off += static_cast<int64_t>(c) * p.stride[o][d];
    }
    return off;
}

template <class T, int VEC>
__device__ inline Pack<T, VEC> flat_source(const FlatPlan& fp, int o, const T* base, uint64_t first, uint32_t row, uint32_t col, uint32_t live) {
    Pack<T, VEC> r;
    if (fp.full[o]) {
        if (live == VEC) return load_pack<T, VEC>(base + first);
#pragma unroll
        for (int i = 0; i < VEC; ++i) r.v[i] = static_cast<uint32_t>(i) < live ? base[first + i] : T{};
        return r;
    }
    const uint32_t length = fp.p.extent[fp.p.rank - 1];
    const T here = base[outer_offset<T>(fp.p, o, row)];
    const bool runs_over = col + VEC > length && row + 1 < fp.rows;
    const T next = runs_over ? base[outer_offset<T>(fp.p, o, row + 1)] : here;
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.v[i] = col + i < length ? here : next;
    return r;
}

template <class F, int VEC>
__global__ __launch_bounds__(kBlock) void elementwise_flat_kernel(F f, FlatPlan fp, uint32_t vectors) {
    using S0 = typename F::S0;
    using S1 = typename F::S1;
    using D = typename F::D;
    const uint32_t v = blockIdx.x * kBlock + threadIdx.x;
    if (v >= vectors) return;
    const uint64_t first = static_cast<uint64_t>(v) * VEC;
    const uint32_t live = fp.elements - first < VEC ? static_cast<uint32_t>(fp.elements - first) : VEC;
    uint32_t row = 0, col = 0;
    if (fp.p.rank > 1) fp.p.row_div.divmod(static_cast<uint32_t>(first), row, col);   // fewer than 2^31 elements (the launch checks)
    const Pack<S0, VEC> a = flat_source<S0, VEC>(fp, 0, f.a, first, row, col, live);
    Pack<S1, VEC> b;
    if constexpr (F::sources == 2) b = flat_source<S1, VEC>(fp, 1, f.b, first, row, col, live);
    Pack<D, VEC> r;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        if constexpr (F::sources == 2) r.v[i] = f(a.v[i], b.v[i]);
        else r.v[i] = f(a.v[i], S1{});
    }
    if (live == VEC) {
        store_pack<D, VEC>(f.out + first, r);
    } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
            if (static_cast<uint32_t>(i) < live) f.out[first + i] = r.v[i];
    }
}

template <class A, class B>
constexpr size_t max_size() { return sizeof(A) > sizeof(B) ? sizeof(A) : sizeof(B); }

// Whether operand `o` allows VEC-wide access: row stride 0 or 1, every outer
// stride and the base address multiples of the vector.
template <class T>
inline bool vector_ok(const Plan& p, int o, const T* ptr, int vec, bool is_dst) {
    const int last = p.rank - 1;
    const int64_t rs = p.stride[o][last];
    if (is_dst ? rs != 1 : (rs != 0 && rs != 1)) return false;
    if (rs == 0) return true;  // splat operand: scalar loads, no alignment needed
    if (reinterpret_cast<uintptr_t>(ptr) % (sizeof(T) * vec)) return false;
    for (int d = 0; d < last; ++d)
        if (p.stride[o][d] % vec) return false;
    return true;
}

// Enqueues F over the plan.  Destination operand index is 2.
template <class F>
int launch_elementwise(F f, Plan p, hipStream_t stream) {
    using S0 = typename F::S0;
    using S1 = typename F::S1;
    using D = typename F::D;
    constexpr size_t widest = F::sources == 2 ? (max_size<S0, S1>() > sizeof(D) ? max_size<S0, S1>() : sizeof(D))
                                              : max_size<S0, D>();
    constexpr int VEC = widest >= 16 ? 1 : static_cast<int>(16 / widest);
    const int last = p.rank - 1;
    uint64_t rows = 1;
    for (int d = 0; d < last; ++d) rows *= p.extent[d];
    bool vec = VEC > 1 && p.extent[last] % VEC == 0 && vector_ok(p, 0, f.a, VEC, false) &&
               vector_ok(p, 2, f.out, VEC, true);
    if (F::sources == 2) vec = vec && vector_ok(p, 1, f.b, VEC, false);
    if constexpr (VEC > 1) {
        if (!vec) {
            // contiguous operands next to row-constant ones, a row length the vector does not divide: vectors over the flat index
            FlatPlan fp;
            fp.elements = rows * p.extent[last];
            auto contiguous = [&](int o) {
                int64_t expect = 1;
                for (int d = last; d >= 0; --d) {
                    if (p.stride[o][d] != expect) return false;
                    expect *= p.extent[d];
                }
                return true;
            };
            auto aligned_to = [](const void* ptr, size_t bytes) { return reinterpret_cast<uintptr_t>(ptr) % bytes == 0; };
            bool flat = fp.elements > 0 && fp.elements < (1ull << 31) && contiguous(2) && aligned_to(f.out, sizeof(D) * VEC);
            bool any_constant = false;
            fp.full[0] = fp.full[1] = true;
            if (flat) {
                fp.full[0] = contiguous(0);
                flat = fp.full[0] ? aligned_to(f.a, sizeof(S0) * VEC) : p.stride[0][last] == 0;
                any_constant = !fp.full[0];
            }
            if (flat && F::sources == 2) {
                fp.full[1] = contiguous(1);
                flat = fp.full[1] ? aligned_to(f.b, sizeof(S1) * VEC) : p.stride[1][last] == 0;
                any_constant = any_constant || !fp.full[1];
            }
            if (flat && any_constant && (p.rank < 2 || p.extent[last] < static_cast<uint32_t>(VEC))) flat = false;
            if (flat) {
                fp.rows = static_cast<uint32_t>(rows);
                p.row_div = FastDiv(p.extent[last]);
                fp.p = p;
                const uint32_t vectors = static_cast<uint32_t>((fp.elements + VEC - 1) / VEC);
                hipLaunchKernelGGL((elementwise_flat_kernel<F, VEC>), dim3((vectors + kBlock - 1) / kBlock), dim3(kBlock), 0, stream, f, fp, vectors);
                return launch_status("elementwise_flat_kernel");
            }
        }
    }
    p.row_vectors = vec ? p.extent[last] / VEC : p.extent[last];
    p.row_div = FastDiv(p.row_vectors);
    if (rows * p.row_vectors >= (1ull << 31)) {
        set_error_text("elementwise: more than 2^31 vectors (16 bytes each where the operands allow, single elements otherwise)");
        return TANNIC_ERROR;
    }
    p.total_vectors = static_cast<uint32_t>(rows * p.row_vectors);
    if (p.total_vectors == 0) return TANNIC_SUCCESS;
    const bool repeats = p.rank > 1 || p.stride[0][last] == 0 || (F::sources == 2 && p.stride[1][last] == 0);
    // Two vectors per thread pay only when the blocks are many generations deep (1 GiB with a broadcast operand: 6 %
    // faster); at the sizes of a layer's activations (16 MB: one or two generations) one vector per thread and twice
    // the blocks let stores of early blocks overlap loads of late ones (15 of a decoder layer's 600 us).
    const bool two = repeats && p.total_vectors >= (1u << 23);
    const uint32_t per_block = kBlock * (two ? 2 : 1);
    const uint32_t grid = (p.total_vectors + per_block - 1) / per_block;
    if constexpr (VEC > 1) {
        if (vec) {
            if (two) hipLaunchKernelGGL((elementwise_kernel<F, VEC, 2>), dim3(grid), dim3(kBlock), 0, stream, f, p);
            else hipLaunchKernelGGL((elementwise_kernel<F, VEC, 1>), dim3(grid), dim3(kBlock), 0, stream, f, p);
            return launch_status("elementwise_kernel");
        }
    }
    if (two) hipLaunchKernelGGL((elementwise_kernel<F, 1, 2>), dim3(grid), dim3(kBlock), 0, stream, f, p);
    else hipLaunchKernelGGL((elementwise_kernel<F, 1, 1>), dim3(grid), dim3(kBlock), 0, stream, f, p);
    return launch_status("elementwise_kernel");
}

// ---- copies that transpose -------------------------------------------------------------------------------------------
// A copy whose source is contiguous along another dimension than the destination's last one (a transposed matrix made
// contiguous, [B, S, H, D] read as [B, D, S, H] ...): element by element, either the loads or the stores of a wavefront
// are a line apart each.  Here a block moves a 64 x 64 tile of those two dimensions through LDS: it reads rows along the
// source's contiguous dimension and writes rows along the destination's, both as whole lines.  The other dimensions are
// decoded from the block number.
struct TransposePlan {
    int outer;                         // dimensions besides the two of the tile
    FastDiv div[TANNIC_DIMENSIONS];    // their extents, innermost last
    int64_t src_stride[TANNIC_DIMENSIONS], dst_stride[TANNIC_DIMENSIONS];
    uint32_t extent_c, extent_l;       // the source's contiguous dimension, the destination's last one
    int64_t src_stride_l, dst_stride_c;
    uint32_t tiles_c, tiles_l;
};

template <class U>
__global__ __launch_bounds__(256) void transposed_copy_kernel(const U* src, U* dst, TransposePlan q) {
    constexpr int TILE = 64;
    __shared__ U tile[TILE][TILE + 1];
    uint32_t rest = blockIdx.x;
    const uint32_t tc = rest % q.tiles_c;
    rest /= q.tiles_c;
    const uint32_t tl = rest % q.tiles_l;
    rest /= q.tiles_l;
    int64_t from = 0, to = 0;
    for (int d = q.outer - 1; d >= 0; --d) {
        uint32_t next, c;
        q.div[d].divmod(rest, next, c);
        rest = next;
        from += static_cast<int64_t>(c) * q.src_stride[d];
        to += static_cast<int64_t>(c) * q.dst_stride[d];
    }
    const uint32_t c0 = tc * TILE, l0 = tl * TILE, tx = threadIdx.x % TILE, ty = threadIdx.x / TILE;
#pragma unroll 4
    for (int i = 0; i < TILE; i += 4) {
        const uint32_t c = c0 + tx, l = l0 + ty + i;
        if (c < q.extent_c && l < q.extent_l) tile[ty + i][tx] = src[from + c + static_cast<int64_t>(l) * q.src_stride_l];
    }
    __syncthreads();
#pragma unroll 4
    for (int i = 0; i < TILE; i += 4) {
        const uint32_t l = l0 + tx, c = c0 + ty + i;
        if (c < q.extent_c && l < q.extent_l) dst[to + l + static_cast<int64_t>(c) * q.dst_stride_c] = tile[tx][ty + i];
    }
}

// Runs the copy described by `p` (operand 0 the source, operand 2 the destination) through the tiles above when it is one
// of those; TANNIC_UNSUPPORTED_DTYPE otherwise.  U: an unsigned type (or 16-byte struct) of the element's size.
template <class U>
inline int transposed_copy(const Plan& p, const void* src, void* dst, hipStream_t stream) {
    const int last = p.rank - 1;
    if (p.rank < 2 || p.stride[2][last] != 1 || p.stride[0][last] == 1 || p.stride[0][last] == 0) return TANNIC_UNSUPPORTED_DTYPE;
    int c = -1;
    for (int d = last - 1; d >= 0; --d)
        if (p.stride[0][d] == 1) { c = d; break; }
    if (c < 0 || p.extent[c] < 16 || p.extent[last] < 16) return TANNIC_UNSUPPORTED_DTYPE;
    TransposePlan q{};
    uint64_t blocks = 1;
    for (int d = 0; d < last; ++d) {
        if (d == c) continue;
        q.div[q.outer] = p.div[d];
        q.src_stride[q.outer] = p.stride[0][d];
        q.dst_stride[q.outer] = p.stride[2][d];
        ++q.outer;
        blocks *= p.extent[d];
    }
    q.extent_c = p.extent[c];
    q.extent_l = p.extent[last];
    q.src_stride_l = p.stride[0][last];
    q.dst_stride_c = p.stride[2][c];
    q.tiles_c = (q.extent_c + 63) / 64;
    q.tiles_l = (q.extent_l + 63) / 64;
    blocks *= static_cast<uint64_t>(q.tiles_c) * q.tiles_l;
    if (blocks == 0) return TANNIC_SUCCESS;
    if (blocks >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    hipLaunchKernelGGL((transposed_copy_kernel<U>), dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream, static_cast<const U*>(src), static_cast<U*>(dst), q);
    return launch_status("transposed_copy_kernel");
}

template <int BYTES> struct BitsOf;
template <> struct BitsOf<1> { using type = uint8_t; };
template <> struct BitsOf<2> { using type = uint16_t; };
template <> struct BitsOf<4> { using type = uint32_t; };
template <> struct BitsOf<8> { using type = uint64_t; };
struct alignas(16) SixteenBytes { uint64_t lo, hi; };
template <> struct BitsOf<16> { using type = SixteenBytes; };

// Strides of `t` right-aligned on a destination of `rank` dims with `extent`;
// size-1 dims (and missing leading dims) get stride 0
// (src/cpu/ops-binary.cpp:89-95).
inline void aligned_strides(const tannic_tensor_t* t, int rank, int64_t* out) {
    const int off = rank - t->rank;
    for (int d = 0; d < rank; ++d) {
        if (d < off) { out[d] = 0; continue; }
        out[d] = t->shape.sizes[d - off] == 1 ? 0 : t->strides.sizes[d - off];
    }
}

// Whether `t`, right-aligned on `dst`, matches it in every dim or has extent 1 there: the kernels index `t` by
// dst's coordinates, so anything else would read outside `t`.
inline bool broadcasts_to(const tannic_tensor_t* t, const tannic_tensor_t* dst) {
    if (t->rank > dst->rank) return false;
    const int off = dst->rank - t->rank;
    for (int d = 0; d < t->rank; ++d)
        if (t->shape.sizes[d] != 1 && t->shape.sizes[d] != dst->shape.sizes[d + off]) return false;
    return true;
}

// Same rank and extents: what the kernels that walk one tensor by another's coordinates rely on.
inline bool same_extents(const tannic_tensor_t* a, const tannic_tensor_t* b) {
    if (a->rank != b->rank) return false;
    for (int d = 0; d < a->rank; ++d)
        if (a->shape.sizes[d] != b->shape.sizes[d]) return false;
    return true;
}

inline int shape_mismatch(const char* what) {
    set_error_text(what);
    return TANNIC_ERROR;
}

inline void contiguous_strides(int rank, const size_t* extent, int64_t* out) {
    int64_t run = 1;
    for (int d = rank - 1; d >= 0; --d) {
        out[d] = run;
        run *= static_cast<int64_t>(extent[d]);
    }
}

}  // namespace th
