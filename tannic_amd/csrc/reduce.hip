// Axis reductions: argsum, argmean, argmax, argmin (+ value max / min).
//
// HBM-bound: every source byte is read once with 16-byte accesses.  A
// contiguous source is seen as [outer, R, inner] (src/cpu/argred.cpp:186-212):
//   inner == 1  -> "rows":    a wavefront (or a whole block) owns a row, lanes
//                             stride over it, partials meet in a DPP tree and,
//                             for block-wide rows, in LDS;
//   inner  > 1  -> "columns": a lane owns VEC adjacent columns so that a
//                             wavefront reads contiguous bytes, the waves of
//                             a block (and, when the output is small, several
//                             blocks) take interleaved slices of R; partials
//                             meet in LDS, then in a second small pass.
// Strided sources take a one-thread-per-output walk.
//
// Arithmetic follows src/cpu/argred.cpp:151-181 with two documented
// differences: partial sums are combined as a tree (fp32 results differ from
// the sequential CPU sum within rounding), and 16-bit sums accumulate in fp32
// and round once.  Integer sums wrap exactly as the sequential sum does.
// argmax/argmin: strict comparison from a -inf/+inf (lowest/max) start, lowest
// index wins ties, NaN never wins (src/cpu/argred.cpp:95-101, :317-347).
#include "common.hpp"
#include "lanes.hpp"

namespace th {

constexpr int kWave = 64;
constexpr int kThreads = 256;

// ---- reduction policies -------------------------------------------------------
template <class T> struct SumAcc { using type = T; };
template <> struct SumAcc<f16> { using type = float; };
template <> struct SumAcc<bf16> { using type = float; };
template <> struct SumAcc<int8_t> { using type = uint32_t; };   // wraps; narrowed at the end
template <> struct SumAcc<int16_t> { using type = uint32_t; };
template <> struct SumAcc<int32_t> { using type = uint32_t; };
template <> struct SumAcc<int64_t> { using type = uint64_t; };

template <class T, bool MEAN>
struct SumOp {
    using S = T;
    using A = typename SumAcc<T>::type;
    using Out = T;
    static constexpr bool needs_source = false;
    __device__ static inline A init() { return A(0); }
    __device__ static inline A step(A acc, T v, uint32_t) {
        if constexpr (std::is_integral_v<T>) return acc + static_cast<A>(v);
        else return acc + static_cast<A>(widen(v));
    }
    __device__ static inline A combine(A x, A y) { return x + y; }
    __device__ static inline Out finish(A acc, uint32_t count) {
        if constexpr (MEAN) return narrow<T>(acc / static_cast<A>(count));
        else if constexpr (std::is_integral_v<T>) return static_cast<T>(acc);
        else return narrow<T>(acc);
    }
};

template <class T>
struct Best {
    T value;
    uint32_t index;
};
template <> struct Best<f16> { f16 value; uint16_t pad; uint32_t index; };
template <> struct Best<bf16> { bf16 value; uint16_t pad; uint32_t index; };
template <> struct Best<int8_t> { int8_t value; int8_t pad[3]; uint32_t index; };
template <> struct Best<int16_t> { int16_t value; int16_t pad; uint32_t index; };
template <> struct Best<double> { double value; uint32_t index; uint32_t pad; };
template <> struct Best<int64_t> { int64_t value; uint32_t index; uint32_t pad; };

template <class T> __device__ inline bool gt(T a, T b) {
    if constexpr (std::is_same_v<T, bf16>) return to_float(a) > to_float(b); else return a > b;
}
template <class T> __device__ inline bool same(T a, T b) {
    if constexpr (std::is_same_v<T, bf16>) return to_float(a) == to_float(b); else return a == b;
}

template <class T, bool MAX> __device__ inline T arg_start() {
    if constexpr (std::is_same_v<T, int8_t>) return MAX ? INT8_MIN : INT8_MAX;
    else if constexpr (std::is_same_v<T, int16_t>) return MAX ? INT16_MIN : INT16_MAX;
    else if constexpr (std::is_same_v<T, int32_t>) return MAX ? INT32_MIN : INT32_MAX;
    else if constexpr (std::is_same_v<T, int64_t>) return MAX ? INT64_MIN : INT64_MAX;
    else if constexpr (std::is_same_v<T, bf16>) return bf16{static_cast<uint16_t>(MAX ? 0xFF80u : 0x7F80u)};
    else return static_cast<T>(MAX ? -__builtin_inff() : __builtin_inff());
}

// VALUE = false: int64 index out.  VALUE = true: the source element at that index.
template <class T, bool MAX, bool VALUE>
struct ArgOp {
    using S = T;
    using A = Best<T>;
    using Out = std::conditional_t<VALUE, T, int64_t>;
    static constexpr bool needs_source = VALUE;
    __device__ static inline A init() {
        A a{};
        a.value = arg_start<T, MAX>();
        a.index = 0;
        return a;
    }
    __device__ static inline bool better(T v, uint32_t i, const A& than) {
        const bool strictly = MAX ? gt(v, than.value) : gt(than.value, v);
        return strictly || (same(v, than.value) && i < than.index);
    }
    // a lane meets its elements in increasing index order, so inside a lane "strictly better" is the whole
    // rule; the lower-index tie-break only matters when partial results meet (combine)
    __device__ static inline A step(A acc, T v, uint32_t r) {
        const bool strictly = MAX ? gt(v, acc.value) : gt(acc.value, v);
        A out;   // the padding of a 16-bit value is left unset: carrying it along costs three instructions per element
        out.value = strictly ? v : acc.value;
        out.index = strictly ? r : acc.index;
        return out;
    }
    __device__ static inline A combine(A x, A y) { return better(y.value, y.index, x) ? y : x; }
    __device__ static inline int64_t finish(A acc, uint32_t) { return static_cast<int64_t>(acc.index); }
};

// The larger (smaller) of two values the way the hardware's maximum instructions order them: numbers by value,
// +0 above -0, a NaN loses against a number.  The order of the operands does not matter, so partial results may meet
// in any order and still give the same bits.
template <class T, bool MAX> __device__ inline T extreme(T a, T b) {
    if constexpr (std::is_same_v<T, float>) return MAX ? __builtin_fmaxf(a, b) : __builtin_fminf(a, b);
    else if constexpr (std::is_same_v<T, double>) return MAX ? __builtin_fmax(a, b) : __builtin_fmin(a, b);
    else if constexpr (std::is_same_v<T, f16>) {
        const float r = MAX ? __builtin_fmaxf(static_cast<float>(a), static_cast<float>(b)) : __builtin_fminf(static_cast<float>(a), static_cast<float>(b));
        return static_cast<f16>(r);   // one of the operands: exact
    } else if constexpr (std::is_same_v<T, bf16>) {
        const float r = MAX ? __builtin_fmaxf(to_float(a), to_float(b)) : __builtin_fminf(to_float(a), to_float(b));
        return bf16{static_cast<uint16_t>(__builtin_bit_cast(uint32_t, r) >> 16)};   // one of the operands: exact
    } else return (MAX ? a > b : b > a) ? a : b;
}

// Value max / min: the largest (smallest) number of the slice, +0 counting as larger than -0 and NaNs as absent.
// The fold starts from -inf / +inf (the lowest / highest integer); when nothing beats the start (a slice of NaN,
// of -inf, of the integer minimum) the answer is the slice's first element, which is also what argmax points at.
template <class T, bool MAX>
struct ValueOp {
    using S = T;
    using A = T;
    using Out = T;
    static constexpr bool needs_source = true;
    static constexpr bool value_only = true;
    __device__ static inline A init() { return arg_start<T, MAX>(); }
    __device__ static inline A step(A acc, T v, uint32_t) { return extreme<T, MAX>(acc, v); }
    __device__ static inline A combine(A x, A y) { return extreme<T, MAX>(x, y); }
};

// an index search over 16-bit elements: eight compare-and-select pairs per 16-byte load
template <class Op> struct folds_slowly { static constexpr bool value = false; };
template <class T, bool MAX, bool VALUE> struct folds_slowly<ArgOp<T, MAX, VALUE>> { static constexpr bool value = sizeof(T) == 2; };

template <class Op, class = void> struct is_value_only { static constexpr bool value = false; };
template <class Op> struct is_value_only<Op, std::enable_if_t<Op::value_only>> { static constexpr bool value = true; };

template <class T, int N>
struct alignas(sizeof(T) * N >= 16 ? 16 : sizeof(T) * N) Vec {
    T v[N];
};

template <class T, int N>
__device__ inline Vec<T, N> load_vec(const T* p) {
    if constexpr (N == 1) {
        Vec<T, 1> r;
        r.v[0] = *p;
        return r;
    } else {
        using Raw = unsigned int __attribute__((ext_vector_type(sizeof(T) * N / 4)));
        const Raw raw = __builtin_nontemporal_load(reinterpret_cast<const Raw*>(p));
        Vec<T, N> r;
        __builtin_memcpy(&r, &raw, sizeof r);
        return r;
    }
}

// Writes the result for output slot `slot`.  `first` / `step` locate the slice
// in the source for value reductions.
template <class Op>
__device__ inline void emit(typename Op::A acc, uint32_t count, typename Op::Out* dst, size_t slot,
                            const typename Op::S* src, size_t first, size_t step) {
    if constexpr (is_value_only<Op>::value) dst[slot] = (count != 0 && same(acc, Op::init())) ? src[first] : acc;   // an empty slice yields the start value
    else if constexpr (Op::needs_source) dst[slot] = src[first + static_cast<size_t>(acc.index) * step];
    else dst[slot] = Op::finish(acc, count);
}

// ---- rows: inner == 1 ----------------------------------------------------------
// WAVES waves cooperate on one row; a block of 256 threads holds 4 / WAVES rows.
// RAGGED: rows that do not start at multiples of 16 bytes or whose length no vector divides (a softmax over 197 columns).
// The aligned middle of a row is read as vectors all the same; the up to VEC - 1 elements before it and after it are
// taken one per lane by the row's first wavefront, before and after its share of the middle, so that a lane still meets
// its elements in increasing index order.
template <class Op, int VEC, int WAVES, bool RAGGED = false>
__global__ __launch_bounds__(kThreads) void reduce_rows_kernel(const typename Op::S* src, typename Op::Out* dst, uint32_t rows, uint32_t R) {
    using A = typename Op::A;
    using T = typename Op::S;
    constexpr int ROWS_PER_BLOCK = (kThreads / kWave) / WAVES;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const uint32_t row = blockIdx.x * ROWS_PER_BLOCK + wave / WAVES;
    const int part = wave % WAVES;  // which slice of the row this wave takes
    __shared__ A shared[kThreads / kWave];
    A acc = Op::init();
    if (row < rows) {
        const T* p = src + static_cast<size_t>(row) * R;
        constexpr uint32_t STRIDE = kWave * WAVES * VEC;
        uint32_t head = 0, end = R;   // [head, end): whole aligned vectors
        if constexpr (RAGGED) {
            head = static_cast<uint32_t>((VEC - (reinterpret_cast<uintptr_t>(p) / sizeof(T)) % VEC) % VEC);
            if (head > R) head = R;
            end = head + (R - head) / VEC * VEC;
            if (part == 0 && static_cast<uint32_t>(lane) < head) acc = Op::step(acc, p[lane], lane);
        }
        uint32_t r = head + (part * kWave + lane) * VEC;
        // two independent accumulators keep two 16-byte loads in flight per lane
        A acc2 = Op::init();
        for (; r + STRIDE + VEC <= end; r += 2 * STRIDE) {
            const Vec<T, VEC> x = load_vec<T, VEC>(p + r);
            const Vec<T, VEC> y = load_vec<T, VEC>(p + r + STRIDE);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc = Op::step(acc, x.v[i], r + i);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc2 = Op::step(acc2, y.v[i], r + STRIDE + i);
        }
        for (; r + VEC <= end; r += STRIDE) {
            const Vec<T, VEC> x = load_vec<T, VEC>(p + r);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc = Op::step(acc, x.v[i], r + i);
        }
        if constexpr (RAGGED) {
            if (part == 0 && end + lane < R) acc = Op::step(acc, p[end + lane], end + lane);
        }
        acc = Op::combine(acc, acc2);
    }
    acc = wave_reduce<Op>(acc);
    if constexpr (WAVES == 1) {
        if (lane == 0 && row < rows) emit<Op>(acc, R, dst, row, src, static_cast<size_t>(row) * R, 1);
    } else {
        if (lane == 0) shared[wave] = acc;
        __syncthreads();
        if (threadIdx.x == 0 && row < rows) {
            A total = shared[0];
            for (int w = 1; w < WAVES; ++w) total = Op::combine(total, shared[w]);
            emit<Op>(total, R, dst, row, src, static_cast<size_t>(row) * R, 1);
        }
    }
}

// ---- rows, argmax / argmin of 16-bit floats ------------------------------------------------------
// The generic row kernel carries (value, index) pairs through every step, which makes these the one
// reduction bound by the vector ALU rather than by HBM.  Here a wavefront holds its row in registers (up
// to four 16-byte pieces per lane), finds the extreme VALUE first (one max/min per element, NaN ignored,
// the -inf / +inf start kept when nothing beats it), then the lowest index holding it.  Same answers as
// the strict comparison from the start value: ties go to the lowest index, NaN never wins, and a row in
// which nothing beats the start gives 0 (src/cpu/argred.cpp:95-101, :317-347).
template <bool MAX> struct ExtremeOp {
    __device__ static inline float combine(float x, float y) { return MAX ? fmaxf(x, y) : fminf(x, y); }
};

// A wavefront takes kArgRows rows at once: all their loads are issued before any arithmetic, which keeps enough
// bytes in flight per compute unit for the longer life of these wavefronts.
constexpr int kArgRows = 2;

template <class T, bool MAX, int NCH>
__global__ __launch_bounds__(kThreads) void arg_rows16_kernel(const T* src, int64_t* dst, uint32_t rows, uint32_t R) {
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const uint32_t row0 = (blockIdx.x * (kThreads / kWave) + wave) * kArgRows;
    if (row0 >= rows) return;   // whole wavefronts; nothing below synchronises across them
    const uint32_t chunks = R / 8;
    const float start = MAX ? -__builtin_inff() : __builtin_inff();
    Vec<T, 8> raw[kArgRows][NCH];
#pragma unroll
    for (int r = 0; r < kArgRows; ++r) {
        const uint32_t row = row0 + r < rows ? row0 + r : rows - 1;   // the odd last row is done twice
        const T* p = src + static_cast<size_t>(row) * R;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const uint32_t c = lane + i * kWave;
            raw[r][i] = load_vec<T, 8>(p + static_cast<size_t>(c < chunks ? c : 0) * 8);
        }
    }
#pragma unroll
    for (int r = 0; r < kArgRows; ++r) {
        float f[NCH][8], piece_best[NCH];
        float best = start;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            float m = start;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                f[i][e] = widen(raw[r][i].v[e]);
                m = ExtremeOp<MAX>::combine(m, f[i][e]);
            }
            piece_best[i] = lane + i * kWave < chunks ? m : __builtin_nanf("");   // an absent piece equals nothing
            best = ExtremeOp<MAX>::combine(best, piece_best[i]);
        }
        best = wave_reduce<ExtremeOp<MAX>>(best);
        // Nothing beat the start (all NaN, or only the start value itself): the strict comparison never moved off 0.
        // Otherwise the lowest index holding the extreme is in the first piece (pieces are 64 lanes apart) that any
        // lane found it in, in the lowest such lane: a ballot names both, and only that piece is searched.
        uint32_t index = 0;
        if (best != start) {
            bool found = false;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const uint64_t holders = __ballot(piece_best[i] == best);
                if (!found && holders != 0) {
                    found = true;
                    const int holder = __builtin_ctzll(holders);
                    int pos = 7;
#pragma unroll
                    for (int e = 6; e >= 0; --e) pos = f[i][e] == best ? e : pos;
                    index = (static_cast<uint32_t>(i) * kWave + holder) * 8 + __builtin_amdgcn_readlane(pos, holder);
                }
            }
        }
        if (lane == 0 && row0 + r < rows) dst[row0 + r] = static_cast<int64_t>(index);
    }
}

template <class T, bool MAX>
int launch_arg_rows16(const T* src, int64_t* dst, uint32_t rows, uint32_t R, hipStream_t stream) {
    const uint32_t per_lane = (R / 8 + kWave - 1) / kWave;
    const uint32_t per_block = (kThreads / kWave) * kArgRows;
    const dim3 grid((rows + per_block - 1) / per_block);
    if (per_lane <= 1) hipLaunchKernelGGL((arg_rows16_kernel<T, MAX, 1>), grid, dim3(kThreads), 0, stream, src, dst, rows, R);
    else if (per_lane <= 2) hipLaunchKernelGGL((arg_rows16_kernel<T, MAX, 2>), grid, dim3(kThreads), 0, stream, src, dst, rows, R);
    else hipLaunchKernelGGL((arg_rows16_kernel<T, MAX, 4>), grid, dim3(kThreads), 0, stream, src, dst, rows, R);
    return launch_status("arg_rows16_kernel");
}

template <class Op> struct ArgRows16 { static constexpr bool value = false; };
template <class T, bool MAX> struct ArgRows16<ArgOp<T, MAX, false>> {
    static constexpr bool value = is_16bit<T>::value;
    static int run(const T* src, int64_t* dst, uint32_t rows, uint32_t R, hipStream_t stream) { return launch_arg_rows16<T, MAX>(src, dst, rows, R, stream); }
};

// ---- columns: inner > 1 ----------------------------------------------------------
// Thread (tx, ty): VEC columns starting at (blockIdx.x*TX + tx)*VEC, rows
// ty + k*TY*gridDim.z offset by blockIdx.z*TY.  LOG_TX picks the block shape.
template <class Op, int VEC, int TX>
__global__ __launch_bounds__(kThreads) void reduce_columns_kernel(const typename Op::S* src, typename Op::Out* dst, typename Op::A* partial,
                                                                   uint32_t R, uint32_t inner, uint32_t slots) {
    using A = typename Op::A;
    using T = typename Op::S;
    constexpr int TY = kThreads / TX;
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const uint32_t col = (blockIdx.x * TX + tx) * VEC;
    const uint32_t outer = blockIdx.y;
    const bool live = col < inner;
    __shared__ A shared[kThreads][VEC > 4 ? 4 : VEC];  // see the loop over `pass` below
    A acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = Op::init();
    if (live) {
        const T* p = src + static_cast<size_t>(outer) * R * inner + col;
        const uint32_t stride = TY * gridDim.z;
        uint32_t r = blockIdx.z * TY + ty;
        if constexpr (folds_slowly<Op>::value) {
            // Groups of rows, two groups in turn: the loads of the next group are on their way while the current
            // one is folded, so a lane keeps requests outstanding through the arithmetic (an index search over 16-bit
            // elements spends some hundred instructions per group, and only two waves share a SIMD at two blocks per
            // compute unit).  Folds of a few instructions per load stream better without it.
            constexpr int G = 4;   // rows per group; two-row groups (as many loads outstanding as the plain loop) stream a tenth slower
            const size_t hop = static_cast<size_t>(stride) * inner;
            const T* q = p + static_cast<size_t>(r) * inner;
            auto fetch = [&](Vec<T, VEC> (&x)[G]) {
#pragma unroll
                for (int k = 0; k < G; ++k) x[k] = load_vec<T, VEC>(q + k * hop);
                q += G * hop;
            };
            auto fold = [&](const Vec<T, VEC> (&x)[G]) {
#pragma unroll
                for (int k = 0; k < G; ++k)
#pragma unroll
                    for (int i = 0; i < VEC; ++i) acc[i] = Op::step(acc[i], x[k].v[i], r + k * stride);
                r += G * stride;
            };
            if (r + (G - 1) * stride < R) {
                Vec<T, VEC> even[G], odd[G];
                fetch(even);
                for (;;) {
                    if (!(r + (2 * G - 1) * stride < R)) { fold(even); break; }
                    fetch(odd);
                    fold(even);
                    if (!(r + (2 * G - 1) * stride < R)) { fold(odd); break; }
                    fetch(even);
                    fold(odd);
                }
            }
        } else {
            for (; r + 3 * stride < R; r += 4 * stride) {
                Vec<T, VEC> x[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) x[k] = load_vec<T, VEC>(p + static_cast<size_t>(r + k * stride) * inner);
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int i = 0; i < VEC; ++i) acc[i] = Op::step(acc[i], x[k].v[i], r + k * stride);
            }
        }
        for (; r < R; r += stride) {
            const Vec<T, VEC> x = load_vec<T, VEC>(p + static_cast<size_t>(r) * inner);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] = Op::step(acc[i], x.v[i], r);
        }
    }
    // fold the TY slices through LDS, at most four columns of the vector at a time
    constexpr int CH = VEC > 4 ? 4 : VEC;
#pragma unroll
    for (int pass = 0; pass < VEC / CH; ++pass) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < CH; ++i) shared[threadIdx.x][i] = acc[pass * CH + i];
        __syncthreads();
        if (ty == 0 && live) {
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                A total = shared[tx][i];
                for (int y = 1; y < TY; ++y) total = Op::combine(total, shared[y * TX + tx][i]);
                const size_t slot = static_cast<size_t>(outer) * inner + col + pass * CH + i;
                if (gridDim.z == 1) emit<Op>(total, R, dst, slot, src, static_cast<size_t>(outer) * R * inner + col + pass * CH + i, inner);
                else partial[static_cast<size_t>(blockIdx.z) * slots + slot] = total;
            }
        }
    }
}

// A few very long rows (the index of the largest of 128 256 logits, one row per sequence): a row is shared by `gridDim.x`
// blocks, each folding a range of its aligned vectors (the first block also the elements before and after them), and
// reduce_finish_kernel folds the blocks' results.
template <class Op, int VEC>
__global__ __launch_bounds__(kThreads) void reduce_rows_split_kernel(const typename Op::S* src, typename Op::A* partial, uint32_t rows, uint32_t R,
                                                                      uint32_t vectors_per_split) {
    using A = typename Op::A;
    using T = typename Op::S;
    const uint32_t row = blockIdx.y, split = blockIdx.x, tid = threadIdx.x;
    const T* p = src + static_cast<size_t>(row) * R;
    uint32_t head = static_cast<uint32_t>((VEC - (reinterpret_cast<uintptr_t>(p) / sizeof(T)) % VEC) % VEC);
    if (head > R) head = R;
    const uint32_t vectors = (R - head) / VEC, end = head + vectors * VEC;
    const uint32_t v0 = split * vectors_per_split, v1 = v0 + vectors_per_split < vectors ? v0 + vectors_per_split : vectors;
    __shared__ A shared[kThreads / kWave];
    A acc = Op::init();
    if (split == 0 && tid < head) acc = Op::step(acc, p[tid], tid);
    for (uint32_t v = v0 + tid; v < v1; v += kThreads) {
        const Vec<T, VEC> x = load_vec<T, VEC>(p + head + static_cast<size_t>(v) * VEC);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc = Op::step(acc, x.v[i], head + v * VEC + i);
    }
    if (split == 0 && end + tid < R) acc = Op::step(acc, p[end + tid], end + tid);
    acc = wave_reduce<Op>(acc);
    if (tid % kWave == 0) shared[tid / kWave] = acc;
    __syncthreads();
    if (tid == 0) {
        A total = shared[0];
        for (int w = 1; w < kThreads / kWave; ++w) total = Op::combine(total, shared[w]);
        partial[static_cast<size_t>(split) * rows + row] = total;
    }
}

// Second pass of the split-R column reduction: folds `splits` partials per slot.
template <class Op>
__global__ __launch_bounds__(kThreads) void reduce_finish_kernel(const typename Op::A* partial, typename Op::Out* dst, const typename Op::S* src,
                                                                  uint32_t splits, uint32_t slots, uint32_t R, uint32_t inner) {
    const uint32_t slot = blockIdx.x * kThreads + threadIdx.x;
    if (slot >= slots) return;
    typename Op::A total = partial[slot];
    // sixteen partial results are fetched before they are folded (in split order): one after the other, each waiting for
    // its own load, 64 of them took 16 us
    uint32_t s = 1;
    for (; s + 16 <= splits; s += 16) {
        typename Op::A part[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) part[k] = partial[static_cast<size_t>(s + k) * slots + slot];
#pragma unroll
        for (int k = 0; k < 16; ++k) total = Op::combine(total, part[k]);
    }
    if (s < splits) {
        typename Op::A part[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) part[k] = partial[static_cast<size_t>(s + k < splits ? s + k : s) * slots + slot];
#pragma unroll
        for (int k = 0; k < 16; ++k)
            if (s + k < splits) total = Op::combine(total, part[k]);
    }
    const uint32_t outer = slot / inner, col = slot % inner;
    emit<Op>(total, R, dst, slot, src, static_cast<size_t>(outer) * R * inner + col, inner);
}

// ---- strided sources: one thread per output slot (src/cpu/argred.cpp:44-76) -----
struct StridedWalk {
    int rank, axis;
    uint32_t extent[TANNIC_DIMENSIONS];
    int64_t stride[TANNIC_DIMENSIONS];
};

template <class Op>
__global__ __launch_bounds__(kThreads) void reduce_strided_kernel(const typename Op::S* src, typename Op::Out* dst, StridedWalk w, uint32_t slots) {
    const uint32_t slot = blockIdx.x * kThreads + threadIdx.x;
    if (slot >= slots) return;
    uint32_t rem = slot;
    int64_t base = 0;
    for (int d = w.rank - 1; d >= 0; --d) {
        if (d == w.axis) continue;
        base += static_cast<int64_t>(rem % w.extent[d]) * w.stride[d];
        rem /= w.extent[d];
    }
    const uint32_t R = w.extent[w.axis];
    const int64_t step = w.stride[w.axis];
    typename Op::A acc = Op::init();
    for (uint32_t r = 0; r < R; ++r) acc = Op::step(acc, src[base + static_cast<int64_t>(r) * step], r);
    if constexpr (is_value_only<Op>::value) dst[slot] = (R != 0 && same(acc, Op::init())) ? src[base] : acc;
    else if constexpr (Op::needs_source) dst[slot] = src[base + static_cast<int64_t>(acc.index) * step];
    else dst[slot] = Op::finish(acc, R);
}

// Few results over a long reduced dim (a lane per result would walk it alone): a wavefront per result, its lanes
// striding over R in increasing order, combined like the lanes of a row.
template <class Op>
__global__ __launch_bounds__(kThreads) void reduce_strided_wave_kernel(const typename Op::S* src, typename Op::Out* dst, StridedWalk w, uint32_t slots) {
    const uint32_t slot = blockIdx.x * (kThreads / kWave) + threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (slot >= slots) return;   // whole wavefronts; nothing below synchronises across them
    uint32_t rem = slot;
    int64_t base = 0;
    for (int d = w.rank - 1; d >= 0; --d) {
        if (d == w.axis) continue;
        base += static_cast<int64_t>(rem % w.extent[d]) * w.stride[d];
        rem /= w.extent[d];
    }
    const uint32_t R = w.extent[w.axis];
    const int64_t step = w.stride[w.axis];
    typename Op::A acc = Op::init();
    for (uint32_t r = lane; r < R; r += kWave) acc = Op::step(acc, src[base + static_cast<int64_t>(r) * step], r);
    acc = wave_reduce<Op>(acc);
    if (lane != 0) return;
    if constexpr (is_value_only<Op>::value) dst[slot] = (R != 0 && same(acc, Op::init())) ? src[base] : acc;
    else if constexpr (Op::needs_source) dst[slot] = src[base + static_cast<int64_t>(acc.index) * step];
    else dst[slot] = Op::finish(acc, R);
}

// ---- host side -------------------------------------------------------------------
template <class Op>
int run_reduce(const tannic_tensor_t* src, tannic_tensor_t* dst, hipStream_t stream, uint8_t axis) {
    using T = typename Op::S;
    using Out = typename Op::Out;
    using A = typename Op::A;
    if (axis >= src->rank) {
        set_error_text("reduce: axis out of range");
        return TANNIC_ERROR;
    }
    const T* ps = static_cast<const T*>(src->address);
    Out* pd = static_cast<Out*>(dst->address);
    const size_t R = src->shape.sizes[axis];
    if (R >= (1ull << 32)) {
        set_error_text("reduce: reduced axis of 2^32 elements or more is not supported");
        return TANNIC_ERROR;
    }
    // A view that is a dense tensor with its dims in another order (a transposed matrix) is still [outer, R, inner] in
    // memory when the dims that stay keep their order among themselves: the results then come out in the order the
    // destination holds them.  (Summing a transposed [3589, 2141] along its rows is the column sum of the matrix as it lies.)
    size_t outer = 1, inner = 1;
    bool as_slab = src->layout == TANNIC_CONTIGUOUS;
    if (as_slab) {
        for (int d = 0; d < src->rank; ++d) {
            if (d < axis) outer *= src->shape.sizes[d];
            else if (d > axis) inner *= src->shape.sizes[d];
        }
    } else {
        int order[TANNIC_DIMENSIONS];
        int count = 0;
        for (int d = 0; d < src->rank; ++d)
            if (src->shape.sizes[d] != 1 || d == axis) order[count++] = d;
        for (int i = 1; i < count; ++i)
            for (int j = i; j > 0 && src->strides.sizes[order[j]] > src->strides.sizes[order[j - 1]]; --j) {
                const int t = order[j];
                order[j] = order[j - 1];
                order[j - 1] = t;
            }
        bool dense = true, in_order = true;
        int64_t expect = 1;
        int last_kept = -1;
        for (int i = count - 1; i >= 0; --i) {
            if (src->shape.sizes[order[i]] != 1 && src->strides.sizes[order[i]] != expect) dense = false;
            expect *= static_cast<int64_t>(src->shape.sizes[order[i]]);
        }
        for (int i = 0; i < count; ++i) {
            if (order[i] == axis) continue;
            if (order[i] < last_kept) in_order = false;
            last_kept = order[i];
        }
        if (dense && in_order && R > 0) {
            bool before = true;
            for (int i = 0; i < count; ++i) {
                if (order[i] == axis) before = false;
                else if (before) outer *= src->shape.sizes[order[i]];
                else inner *= src->shape.sizes[order[i]];
            }
            as_slab = true;
        }
    }
    if (!as_slab) {
        StridedWalk w{};
        w.rank = src->rank;
        w.axis = axis;
        size_t slots = 1;
        for (int d = 0; d < src->rank; ++d) {
            w.extent[d] = static_cast<uint32_t>(src->shape.sizes[d]);
            w.stride[d] = src->strides.sizes[d];
            if (d != axis) slots *= src->shape.sizes[d];
        }
        if (slots == 0) return TANNIC_SUCCESS;
        if (slots >= (1ull << 31)) { set_error_text("reduce: too many outputs"); return TANNIC_ERROR; }
        if (element_count(dst) != slots) { set_error_text("reduce: the destination does not hold one element per reduced slice"); return TANNIC_ERROR; }
        if (R >= 256 && slots <= 65536) {
            constexpr uint32_t per_block = kThreads / kWave;
            hipLaunchKernelGGL((reduce_strided_wave_kernel<Op>), dim3((static_cast<uint32_t>(slots) + per_block - 1) / per_block), dim3(kThreads), 0, stream, ps, pd, w,
                               static_cast<uint32_t>(slots));
            return launch_status("reduce_strided_wave_kernel");
        }
        // Neighbouring lanes are neighbouring results: the last dim that stays.  Where its stride is not 1 (a view with its
        // outer dims swapped, reduced over the innermost) every lane reads a line of its own; a large view is then copied
        // into a contiguous tensor first - one transposing pass - and reduced as a slab.
        int last_kept = -1;
        for (int d = src->rank - 1; d >= 0 && last_kept < 0; --d)
            if (d != axis && src->shape.sizes[d] != 1) last_kept = d;
        const size_t elements = slots * R;
        if (last_kept >= 0 && src->strides.sizes[last_kept] != 1 && elements >= (1u << 18) && elements < (1ull << 31)) {
            tannic_tensor_t dense = *src;
            int64_t pitch = 1;
            for (int d = src->rank - 1; d >= 0; --d) {
                dense.strides.sizes[d] = pitch;
                pitch *= static_cast<int64_t>(src->shape.sizes[d]);
            }
            dense.layout = TANNIC_CONTIGUOUS;
            dense.size = elements;
            void* copy = nullptr;
            if (scratch_acquire(&copy, elements * sizeof(T), stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
            dense.address = copy;
            tannic_stream_t on{reinterpret_cast<uintptr_t>(stream)};
            int status = tannic_hip_repack(src, &dense, on);
            if (status == TANNIC_SUCCESS) status = run_reduce<Op>(&dense, dst, stream, axis);
            scratch_release(copy, stream);
            return status;
        }
        hipLaunchKernelGGL((reduce_strided_kernel<Op>), dim3((slots + kThreads - 1) / kThreads), dim3(kThreads), 0, stream, ps, pd, w,
                           static_cast<uint32_t>(slots));
        return launch_status("reduce_strided_kernel");
    }
    const size_t slots = outer * inner;
    if (slots == 0) return TANNIC_SUCCESS;
    if (slots >= (1ull << 31) || outer >= (1ull << 31)) { set_error_text("reduce: too many outputs"); return TANNIC_ERROR; }
    if (element_count(dst) != slots) { set_error_text("reduce: the destination does not hold one element per reduced slice"); return TANNIC_ERROR; }
    constexpr int VEC = sizeof(T) >= 16 ? 1 : static_cast<int>(16 / sizeof(T));
    const bool aligned = reinterpret_cast<uintptr_t>(ps) % 16 == 0;

    if (inner == 1 && R <= 16) {
        // rows of a few elements (of one, when the reduced dim has extent 1): a lane per row instead of a wavefront
        StridedWalk w{};
        w.rank = 2; w.axis = 1;
        w.extent[0] = static_cast<uint32_t>(outer); w.extent[1] = static_cast<uint32_t>(R);
        w.stride[0] = static_cast<int64_t>(R); w.stride[1] = 1;
        hipLaunchKernelGGL((reduce_strided_kernel<Op>), dim3((slots + kThreads - 1) / kThreads), dim3(kThreads), 0, stream, ps, pd, w, static_cast<uint32_t>(slots));
        return launch_status("reduce_strided_kernel");
    }
    if (inner == 1) {
        const uint32_t rows = static_cast<uint32_t>(outer);
        const bool vec = VEC > 1 && aligned && R % VEC == 0;
        if constexpr (ArgRows16<Op>::value) {
            // rows that fit the registers of one wavefront (four 16-byte pieces per lane)
            if (vec && R <= 8 * kWave * 4 && rows >= 1024) return ArgRows16<Op>::run(ps, pd, rows, static_cast<uint32_t>(R), stream);
        }
        // a handful of very long rows: several blocks per row and a second pass over their results
        if (VEC > 1 && rows <= 64 && R >= 16384 && reinterpret_cast<uintptr_t>(ps) % sizeof(T) == 0) {
            uint32_t splits = static_cast<uint32_t>(R / 4096);
            if (splits > 64) splits = 64;
            while (splits > 2 && static_cast<size_t>(splits) * rows > 512) splits /= 2;
            const uint32_t vectors_per_split = (static_cast<uint32_t>(R / VEC) + splits - 1) / splits;
            A* partial = nullptr;
            if (scratch_acquire(reinterpret_cast<void**>(&partial), sizeof(A) * splits * rows, stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
            hipLaunchKernelGGL((reduce_rows_split_kernel<Op, VEC>), dim3(splits, rows), dim3(kThreads), 0, stream, ps, partial, rows, static_cast<uint32_t>(R),
                               vectors_per_split);
            int status = launch_status("reduce_rows_split_kernel");
            if (status == TANNIC_SUCCESS) {
                hipLaunchKernelGGL((reduce_finish_kernel<Op>), dim3((rows + kThreads - 1) / kThreads), dim3(kThreads), 0, stream, partial, pd, ps, splits, rows,
                                   static_cast<uint32_t>(R), 1u);
                status = launch_status("reduce_finish_kernel");
            }
            scratch_release(partial, stream);
            return status;
        }
        // few long rows: a whole block per row
        const bool wide = rows < 2048 && R >= 8192;
        const uint32_t grid = wide ? rows : (rows + 3) / 4;
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), 0, stream, ps, pd, rows, static_cast<uint32_t>(R));
        };
        // Rows of any start and length still read their aligned middle as vectors when they are long (fp16 sums, us against
        // element by element: rows of 4097 7.1 / 11.3, of 1025 14.4 / 17.4; of 511 36 / 37, of 197 18.5 / 13.3 - a short row
        // has too few vectors for a wavefront's lanes, and its two ends wait one after the other).
        const bool ragged = VEC > 1 && !vec && R >= 1024 && reinterpret_cast<uintptr_t>(ps) % sizeof(T) == 0;
        if (vec && wide) launch(reduce_rows_kernel<Op, VEC, 4>);
        else if (vec) launch(reduce_rows_kernel<Op, VEC, 1>);
        else if (ragged && wide) launch(reduce_rows_kernel<Op, VEC, 4, true>);
        else if (ragged) launch(reduce_rows_kernel<Op, VEC, 1, true>);
        else if (wide) launch(reduce_rows_kernel<Op, 1, 4>);
        else launch(reduce_rows_kernel<Op, 1, 1>);
        return launch_status("reduce_rows_kernel");
    }

    if (outer > 65535) {
        // grid.y carries `outer`; fold the excess into a strided walk instead
        StridedWalk w{};
        w.rank = 3; w.axis = 1;
        w.extent[0] = static_cast<uint32_t>(outer); w.extent[1] = static_cast<uint32_t>(R); w.extent[2] = static_cast<uint32_t>(inner);
        w.stride[0] = static_cast<int64_t>(R * inner); w.stride[1] = static_cast<int64_t>(inner); w.stride[2] = 1;
        hipLaunchKernelGGL((reduce_strided_kernel<Op>), dim3((slots + kThreads - 1) / kThreads), dim3(kThreads), 0, stream, ps, pd, w,
                           static_cast<uint32_t>(slots));
        return launch_status("reduce_strided_kernel");
    }

    const bool vec = VEC > 1 && aligned && inner % VEC == 0;
    const uint32_t column_groups = static_cast<uint32_t>(vec ? inner / VEC : inner);
    // block shape: TX lanes across columns, the rest of the 256 threads across R.  About two blocks per compute unit
    // (512) stream best on this chip: fewer leave units idle, more only add partial results and a longer second pass.
    int TX = column_groups >= 64 ? 64 : column_groups >= 16 ? 16 : 4;
    if (TX == 64) {
        // narrow blocks reach that count without sharing R between blocks: no partial results, no second kernel
        const size_t narrow = static_cast<size_t>((column_groups + 15) / 16) * outer;
        const size_t wide_blocks = static_cast<size_t>((column_groups + 63) / 64) * outer;
        if (wide_blocks < 512 && narrow >= 512 && narrow < 1024 && R >= 512) TX = 16;
    }
    const int TY = kThreads / TX;
    const uint32_t gx = (column_groups + TX - 1) / TX;
    uint32_t splits = 1;
    const size_t base_blocks = static_cast<size_t>(gx) * outer;
    // (down to eight rows per thread: the partial results are then still a sixteenth of the source at most, and a matrix
    // summed over its rows - one slice, a few thousand columns - gets its two blocks per compute unit: [4097, 4096] fp16
    // 27 us with 256 blocks)
    while (base_blocks * splits < 512 && R / (static_cast<size_t>(TY) * splits * 2) >= 4 && splits < 64) splits *= 2;
    A* partial = nullptr;
    if (splits > 1) {
        if (scratch_acquire(reinterpret_cast<void**>(&partial), sizeof(A) * splits * slots, stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
    }
    const dim3 grid(gx, static_cast<uint32_t>(outer), splits);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(kThreads), 0, stream, ps, pd, partial, static_cast<uint32_t>(R), static_cast<uint32_t>(inner),
                           static_cast<uint32_t>(slots));
    };
    if (vec) {
        if (TX == 64) launch(reduce_columns_kernel<Op, VEC, 64>);
        else if (TX == 16) launch(reduce_columns_kernel<Op, VEC, 16>);
        else launch(reduce_columns_kernel<Op, VEC, 4>);
    } else {
        if (TX == 64) launch(reduce_columns_kernel<Op, 1, 64>);
        else if (TX == 16) launch(reduce_columns_kernel<Op, 1, 16>);
        else launch(reduce_columns_kernel<Op, 1, 4>);
    }
    int status = launch_status("reduce_columns_kernel");
    if (splits > 1) {
        if (status == TANNIC_SUCCESS) {
            hipLaunchKernelGGL((reduce_finish_kernel<Op>), dim3((slots + kThreads - 1) / kThreads), dim3(kThreads), 0, stream, partial, pd, ps,
                               splits, static_cast<uint32_t>(slots), static_cast<uint32_t>(R), static_cast<uint32_t>(inner));
            status = launch_status("reduce_finish_kernel");
        }
        scratch_release(partial, stream);
    }
    return status;
}

enum ReduceKind { R_SUM, R_MEAN, R_ARGMAX, R_ARGMIN, R_MAX, R_MIN };

template <int K>
int reduce_entry(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, uint8_t axis) {
    if (!src || !dst) return TANNIC_ERROR;
    if (!have_storage(src, dst)) return TANNIC_ERROR;
    int status = TANNIC_UNSUPPORTED_DTYPE;
    with_type(src->dtype, [&](auto t) {
        using T = typename decltype(t)::type;
        constexpr bool cplx = std::is_same_v<T, c64> || std::is_same_v<T, c128>;
        if constexpr (!cplx) {
            hipStream_t s = as_stream(stream);
            // indices leave as int64, everything else in the source's type
            const int out = (K == R_ARGMAX || K == R_ARGMIN) ? static_cast<int>(TANNIC_INT64) : dtype_code<T>();
            if (!destination_is(dst, out, "reduction: the destination's dtype does not fit the result")) {
                status = TANNIC_ERROR;
                return;
            }
            // coverage: src/cpu/argred.cpp:289-347 (mean: floating types only)
            if constexpr (K == R_SUM) status = run_reduce<SumOp<T, false>>(src, dst, s, axis);
            else if constexpr (K == R_MEAN) { if constexpr (!std::is_integral_v<T>) status = run_reduce<SumOp<T, true>>(src, dst, s, axis); }
            else if constexpr (K == R_ARGMAX) status = run_reduce<ArgOp<T, true, false>>(src, dst, s, axis);
            else if constexpr (K == R_ARGMIN) status = run_reduce<ArgOp<T, false, false>>(src, dst, s, axis);
            else if constexpr (K == R_MAX) status = run_reduce<ValueOp<T, true>>(src, dst, s, axis);
            else status = run_reduce<ValueOp<T, false>>(src, dst, s, axis);
        }
    });
    return status;
}

}  // namespace th

using namespace th;

extern "C" {
int tannic_hip_argsum(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st, uint8_t ax) { return reduce_entry<R_SUM>(s, d, st, ax); }
int tannic_hip_argmean(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st, uint8_t ax) { return reduce_entry<R_MEAN>(s, d, st, ax); }
int tannic_hip_argmax(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st, uint8_t ax) { return reduce_entry<R_ARGMAX>(s, d, st, ax); }
int tannic_hip_argmin(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st, uint8_t ax) { return reduce_entry<R_ARGMIN>(s, d, st, ax); }
int tannic_hip_max(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st, uint8_t ax) { return reduce_entry<R_MAX>(s, d, st, ax); }
int tannic_hip_min(const tannic_tensor_t* s, tannic_tensor_t* d, tannic_stream_t st, uint8_t ax) { return reduce_entry<R_MIN>(s, d, st, ax); }
}
