// MFMA matrix-multiply kernels for gfx950.
//
// 16-bit operands (fp16, bf16), fp32 accumulation:
//   v_mfma_f32_32x32x16_{f16,bf16}; a block of 256 threads (4 wavefronts, 2x2)
//   owns a BM x BN tile of C and walks K in steps of 64.  Both operand tiles
//   live in LDS as [row][64 k] with the eight 16-byte chunks of a row XOR-
//   swizzled by the row number, so that the 16-byte fragment reads of a
//   wavefront (32 rows x 2 chunks) and the tile writes are bank-conflict free.
//   Tiles are double buffered: the global loads of step i+1 are issued before
//   the MFMAs of step i and written to the other buffer after them; one barrier
//   per step.  An operand that is contiguous along K is copied chunk by chunk;
//   an operand that is contiguous along its row index (a transposed view of A,
//   a plain row-major B) is read as 8x8 micro-blocks and transposed in
//   registers on its way to LDS.
//
// fp32 operands: v_mfma_f32_32x32x2f32 (true fp32), same tiling with K steps
//   of 16; fragments are single LDS words.
//
// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2, so
// the id is first folded (id % 8 selects the XCD's contiguous share of tiles)
// and then walked in groups of four tile rows: the tiles that run together on
// one XCD share A and B panels.
#include "gemm_common.hpp"

namespace th {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bfloat8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

template <class T> struct Mfma16;
template <> struct Mfma16<f16> {
    __device__ static inline float16v run(uint4v a, uint4v b, float16v c) {
        half8 x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, c, 0, 0, 0);
    }
};
template <> struct Mfma16<bf16> {
    __device__ static inline float16v run(uint4v a, uint4v b, float16v c) {
        bfloat8 x, y;
        __builtin_memcpy(&x, &a, 16);
        __builtin_memcpy(&y, &b, 16);
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, c, 0, 0, 0);
    }
};

constexpr int kBK = 64;          // K elements per step (16-bit kernels)
constexpr int kChunk = 8;        // 16-bit elements per 16-byte chunk
constexpr int kThreads = 256;

// Maps the hardware workgroup id to a tile: XCD folding, then grouped rows.
__device__ inline void tile_of(uint32_t wg, uint32_t tiles_m, uint32_t tiles_n, uint32_t& tm, uint32_t& tn) {
    const uint32_t total = tiles_m * tiles_n;
    uint32_t id = wg;
    if (total % 8 == 0) id = (wg % 8) * (total / 8) + wg / 8;
    constexpr uint32_t GROUP = 4;
    const uint32_t width = GROUP * tiles_n;
    const uint32_t group = id / width;
    const uint32_t first = group * GROUP;
    const uint32_t rows = tiles_m - first < GROUP ? tiles_m - first : GROUP;
    tm = first + (id % width) % rows;
    tn = (id % width) / rows;
}

// One operand of the product seen as rows x K: element (r, k) at
// base[r * row_stride + k * k_stride]; exactly one of the strides is 1.
struct Operand {
    const void* base;
    int64_t row_stride, k_stride;
    uint32_t rows;  // M for A, N for B
};

// Swizzled element offset of (row, chunk) inside a [ROWS][64] tile.
__device__ inline uint32_t tile_offset(uint32_t row, uint32_t chunk) { return row * kBK + ((chunk ^ (row & 7u)) * kChunk); }

// ---- global -> registers -> LDS, operand contiguous along K -------------------
template <class T, int ROWS>
struct KMajorLoader {
    static constexpr int PASSES = ROWS / 32;
    uint4v regs[PASSES];
    __device__ inline void fetch(const Operand& op, uint32_t row0, uint32_t k0, uint32_t K) {
        const uint32_t chunk = threadIdx.x % 8, r = threadIdx.x / 8;
        const uint32_t k = k0 + chunk * kChunk;
        const T* base = static_cast<const T*>(op.base);
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            const uint32_t row = row0 + r + 32 * i;
            if (row < op.rows && k < K) regs[i] = *reinterpret_cast<const uint4v*>(base + static_cast<int64_t>(row) * op.row_stride + k);
            else regs[i] = uint4v{0, 0, 0, 0};
        }
    }
    __device__ inline void commit(T* tile) const {
        const uint32_t chunk = threadIdx.x % 8, r = threadIdx.x / 8;
#pragma unroll
        for (int i = 0; i < PASSES; ++i) *reinterpret_cast<uint4v*>(tile + tile_offset(r + 32 * i, chunk)) = regs[i];
    }
};

// ---- operand contiguous along its row index: 8x8 micro-blocks, transposed --------
template <class T, int ROWS>
struct RowMajorLoader {
    // ROWS/8 row-blocks x 8 k-blocks micro-blocks, 256 threads
    static constexpr int PASSES = (ROWS + 255) / 256;
    uint4v regs[PASSES][8];
    __device__ inline void fetch(const Operand& op, uint32_t row0, uint32_t k0, uint32_t K) {
        const T* base = static_cast<const T*>(op.base);
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            const uint32_t mb = threadIdx.x + kThreads * i;
            const uint32_t kb = mb % 8, rb = mb / 8;
            const uint32_t row = row0 + rb * 8;
            const bool live = rb < ROWS / 8 && row < op.rows;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                const uint32_t k = k0 + kb * 8 + kk;
                if (live && k < K) regs[i][kk] = *reinterpret_cast<const uint4v*>(base + static_cast<int64_t>(k) * op.k_stride + row);
                else regs[i][kk] = uint4v{0, 0, 0, 0};
            }
        }
    }
    __device__ inline void commit(T* tile) const {
#pragma unroll
        for (int i = 0; i < PASSES; ++i) {
            const uint32_t mb = threadIdx.x + kThreads * i;
            const uint32_t kb = mb % 8, rb = mb / 8;
            if (rb >= ROWS / 8) continue;
            uint16_t in[8][8], out[8][8];
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) __builtin_memcpy(in[kk], &regs[i][kk], 16);
#pragma unroll
            for (int rr = 0; rr < 8; ++rr)
#pragma unroll
                for (int kk = 0; kk < 8; ++kk) out[rr][kk] = in[kk][rr];
#pragma unroll
            for (int rr = 0; rr < 8; ++rr) {
                uint4v v;
                __builtin_memcpy(&v, out[rr], 16);
                *reinterpret_cast<uint4v*>(tile + tile_offset(rb * 8 + rr, kb)) = v;
            }
        }
    }
};

template <class T, int ROWS, bool K_MAJOR>
using Loader = std::conditional_t<K_MAJOR, KMajorLoader<T, ROWS>, RowMajorLoader<T, ROWS>>;

template <class T, int BM, int BN, bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(kThreads) void gemm16_kernel(const T* A, const T* B, T* C, GemmProblem p, uint32_t tiles_m, uint32_t tiles_n) {
    constexpr int WM = BM / 2, WN = BN / 2;   // 2 x 2 wavefronts
    constexpr int TM = WM / 32, TN = WN / 32;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);
    T* sA[2] = {lds, lds + BM * kBK};
    T* sB[2] = {lds + 2 * BM * kBK, lds + 2 * BM * kBK + BN * kBK};

    uint32_t tm, tn;
    tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.y, oa, ob, oc);
    const Operand opA{A + oa, p.a_rs, p.a_cs, p.M};
    const Operand opB{B + ob, p.b_cs, p.b_rs, p.N};   // rows of B's operand are the columns n
    const uint32_t m0 = tm * BM, n0 = tn * BN;

    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int wm = (wave / 2) * WM, wn = (wave % 2) * WN;
    const uint32_t frag_row = lane % 32, frag_chunk = lane / 32;

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    Loader<T, BM, A_KMAJOR> la;
    Loader<T, BN, B_KMAJOR> lb;
    la.fetch(opA, m0, 0, p.K);
    lb.fetch(opB, n0, 0, p.K);
    la.commit(sA[0]);
    lb.commit(sB[0]);
    __syncthreads();

    const uint32_t steps = (p.K + kBK - 1) / kBK;
    for (uint32_t s = 0; s < steps; ++s) {
        const int cur = s & 1;
        if (s + 1 < steps) {
            la.fetch(opA, m0, (s + 1) * kBK, p.K);
            lb.fetch(opB, n0, (s + 1) * kBK, p.K);
        }
        const T* a_tile = sA[cur];
        const T* b_tile = sB[cur];
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
            uint4v fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const uint4v*>(a_tile + tile_offset(wm + i * 32 + frag_row, ks * 2 + frag_chunk));
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const uint4v*>(b_tile + tile_offset(wn + j * 32 + frag_row, ks * 2 + frag_chunk));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = Mfma16<T>::run(fa[i], fb[j], acc[i][j]);
        }
        if (s + 1 < steps) {
            la.commit(sA[cur ^ 1]);
            lb.commit(sB[cur ^ 1]);
        }
        __syncthreads();
    }

    // accumulator layout of a 32x32 tile: lane -> column lane % 32; value v ->
    // row 8 * (v / 4) + 4 * (lane / 32) + v % 4
    T* c = C + oc;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t col = n0 + wn + j * 32 + lane % 32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t row = m0 + wm + i * 32 + 8 * (v / 4) + 4 * (lane / 32) + v % 4;
                if (row < p.M && col < p.N) c[static_cast<int64_t>(row) * p.c_rs + col] = narrow<T>(acc[i][j][v]);
            }
        }
}

template <class T, int BM, int BN, bool AK, bool BK_>
int launch16(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    const uint32_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    constexpr size_t lds_bytes = sizeof(T) * 2 * (BM + BN) * kBK;
    auto kernel = gemm16_kernel<T, BM, BN, AK, BK_>;
    static bool configured = false;
    if (!configured) {
        TH_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
        configured = true;
    }
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, p.batches), dim3(kThreads), lds_bytes, stream, static_cast<const T*>(a),
                       static_cast<const T*>(b), static_cast<T*>(c), p, tiles_m, tiles_n);
    return launch_status("gemm16_kernel");
}

template <class T, int BM, int BN>
int pick_layout16(const GemmProblem& p, bool ak, bool bk, const void* a, const void* b, void* c, hipStream_t s) {
    if (ak && bk) return launch16<T, BM, BN, true, true>(p, a, b, c, s);
    if (ak) return launch16<T, BM, BN, true, false>(p, a, b, c, s);
    if (bk) return launch16<T, BM, BN, false, true>(p, a, b, c, s);
    return launch16<T, BM, BN, false, false>(p, a, b, c, s);
}

template <class T>
int run16(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    if (p.M == 0 || p.N == 0 || p.batches == 0) return TANNIC_SUCCESS;
    // layout of each operand: along which index is it contiguous?
    const bool ak = p.a_cs == 1, bk = p.b_rs == 1;
    if (!ak && p.a_rs != 1) return TANNIC_UNSUPPORTED_DTYPE;
    if (!bk && p.b_cs != 1) return TANNIC_UNSUPPORTED_DTYPE;
    // 16-byte accesses: addresses, leading dimensions, batch strides and the
    // contiguous extent must be multiples of 8 elements
    auto mult8 = [](int64_t v) { return v % 8 == 0; };
    if (reinterpret_cast<uintptr_t>(a) % 16 || reinterpret_cast<uintptr_t>(b) % 16) return TANNIC_UNSUPPORTED_DTYPE;
    if (!mult8(ak ? p.a_rs : p.a_cs) || !mult8(bk ? p.b_cs : p.b_rs)) return TANNIC_UNSUPPORTED_DTYPE;
    if (!mult8(ak ? p.K : p.M) || !mult8(bk ? p.K : p.N)) return TANNIC_UNSUPPORTED_DTYPE;
    for (int d = 0; d < p.batch_rank; ++d)
        if (!mult8(p.a_bs[d]) || !mult8(p.b_bs[d])) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.batches > 65535) return TANNIC_UNSUPPORTED_DTYPE;
    // large tiles when they still give every CU work, smaller ones otherwise
    const uint64_t big = static_cast<uint64_t>((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batches;
    if (big >= 200) return pick_layout16<T, 256, 256>(p, ak, bk, a, b, c, stream);
    const uint64_t mid = static_cast<uint64_t>((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batches;
    if (mid >= 128 || p.M > 64) return pick_layout16<T, 128, 128>(p, ak, bk, a, b, c, stream);
    return pick_layout16<T, 64, 128>(p, ak, bk, a, b, c, stream);
}

int gemm_mfma_16bit(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream) {
    if (dtype == TANNIC_FLOAT16) return run16<f16>(p, a, b, c, stream);
    if (dtype == TANNIC_BFLOAT16) return run16<bf16>(p, a, b, c, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

int gemm_mfma_f32(const GemmProblem&, const float*, const float*, float*, hipStream_t) { return TANNIC_UNSUPPORTED_DTYPE; }

}  // namespace th
