// MFMA matrix-multiply kernels for gfx950.
//
// 16-bit operands (fp16, bf16), fp32 accumulation:
//   v_mfma_f32_32x32x16_{f16,bf16}; a block of 256 threads (4 wavefronts, 2x2)
//   owns a BM x BN tile of C and walks K in steps of 64.  Both operand tiles
//   live in LDS as [row][64 k] with the eight 16-byte chunks of a row XOR-
//   swizzled by the row number, so that the 16-byte fragment reads of a
//   wavefront (32 rows x 2 chunks) and the tile writes are bank-conflict free.
//   Tiles are double buffered in LDS and a third tile is in flight in registers:
//   during step s every register of tile s+1 is written to the other LDS buffer
//   and refilled from global memory with tile s+2, one memory operation between
//   two MFMAs; one barrier per step, placed where the fragments of the next 16
//   MFMAs are in registers already.  An operand that is contiguous along K is copied chunk by chunk;
//   an operand that is contiguous along its row index (a transposed view of A,
//   a plain row-major B) goes to LDS as it lies in memory, [k][row], and is
//   transposed on the way out by ds_read_b64_tr_b16, two per fragment.
//
// fp32 operands: v_mfma_f32_32x32x2f32 (true fp32), the same kernel with K steps
//   of 32 (rows of a tile stay 128 bytes): a 16-byte fragment feeds four MFMAs,
//   one per element; which k an element stands for is the same permutation for
//   both operands.  The result is written from the accumulators as 16 bytes per lane.
//
// Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2, so
// the id is first folded (id % 8 selects the XCD's contiguous share of tiles)
// and then walked in groups of four tile rows: the tiles that run together on
// one XCD share A and B panels.
#include "gemm_common.hpp"

#include "gemm_tiles.hpp"

namespace th {

// One operand of the product seen as rows x K: element (r, k) at
// base[r * row_stride + k * k_stride]; exactly one of the strides is 1.
struct Operand {
    const void* base;
    int64_t row_stride, k_stride;
    uint32_t rows;  // M for A, N for B
    // Rows in groups that lie apart (only the loaders for rows that are contiguous in memory, in their mode for any
    // alignment, look at this): row r is element r % group of group r / group, which exists when it is below group_live,
    // and a group starts group_stride elements after the one before.  Plain rows: one group that holds them all.
    FastDiv group;
    uint32_t group_live;
    int64_t group_stride;
};


typedef unsigned int uint4_any __attribute__((ext_vector_type(4), aligned(2)));
// The piece of 16 bytes that starts at element `first` of a run of `extent` elements at `run`, which may lie at any
// address: one load when the whole piece lies inside the run, else element by element, with zero for what lies past the end.
template <class T>
__device__ inline uint4v piece_of_run(const T* run, uint32_t first, uint32_t extent) {
    constexpr uint32_t E = 16 / sizeof(T);
    using U = std::conditional_t<sizeof(T) == 2, uint16_t, uint32_t>;
    const U* from = reinterpret_cast<const U*>(run) + first;
    if (first + E <= extent) return *reinterpret_cast<const uint4_any*>(from);
    U piece[E];
#pragma unroll
    for (uint32_t e = 0; e < E; ++e) piece[e] = first + e < extent ? from[e] : U(0);
    uint4v out;
    __builtin_memcpy(&out, piece, 16);
    return out;
}


// ---- global -> registers -> LDS, operand contiguous along K -------------------
// Rows past the operand's end read a clamped (valid) address: they only feed
// rows/columns of C that are never stored.  K past the end must contribute
// zero; that is decided when the registers are written to LDS, so that nothing
// touches the loaded values (and waits for them) early.
// Both loaders expose their work as single memory operations (fetch_one /
// commit_one) so that the main loop can spread them between MFMAs.
// ALIGNED = false: the operand's address, leading dimension or K is not a multiple of 16 bytes.  A chunk that lies inside
// K is still one 16-byte load, at an address that is a multiple of the element size only; the chunk that straddles K's
// end is gathered element by element (each checked against K; what lies past it reads as zero).
template <class T, int ROWS, int THREADS, bool ALIGNED = true>
struct KMajorLoader {
    static constexpr int ROWS_PER_PASS = THREADS / 8;
    static constexpr int LOADS = ROWS / ROWS_PER_PASS, STORES = ROWS / ROWS_PER_PASS;
    uint4v regs[LOADS];
    const T* base;      // operand base + this thread's k offset for the tile being fetched
    bool k_live;
    uint32_t k_left;    // ALIGNED = false: how many of the chunk's elements lie inside K
    __device__ inline void begin_fetch(const Operand& op, uint32_t k0, uint32_t K) {
        const uint32_t k = k0 + (threadIdx.x % 8) * kChunkOf<T>;
        k_live = k < K;
        k_left = k_live ? K - k : 0;
        base = static_cast<const T*>(op.base) + (k_live ? k : 0);
    }
    __device__ inline void fetch_one(int i, const Operand& op, uint32_t row0) {
        const uint32_t row = row0 + threadIdx.x / 8 + ROWS_PER_PASS * i;
        const uint32_t srow = row < op.rows ? row : op.rows - 1;
        if constexpr (ALIGNED) {
            regs[i] = *reinterpret_cast<const uint4v*>(base + static_cast<int64_t>(srow) * op.row_stride);
        } else {
            using U = std::conditional_t<sizeof(T) == 2, uint16_t, uint32_t>;
            const U* from = reinterpret_cast<const U*>(base + static_cast<int64_t>(srow) * op.row_stride);
            if (k_left >= static_cast<uint32_t>(kChunkOf<T>)) {
                // the whole chunk lies inside K: one 16-byte load at whatever address that is (the hardware splits what it must)
                regs[i] = *reinterpret_cast<const uint4_any*>(from);
            } else {
                U piece[kChunkOf<T>];
#pragma unroll
                for (int e = 0; e < kChunkOf<T>; ++e) piece[e] = static_cast<uint32_t>(e) < k_left ? from[e] : U(0);
                __builtin_memcpy(&regs[i], piece, 16);
            }
        }
    }
    template <bool MASK>
    __device__ inline void commit_one(int i, T* tile) const {
        *reinterpret_cast<uint4v*>(tile + tile_offset<T>(threadIdx.x / 8 + ROWS_PER_PASS * i, threadIdx.x % 8)) =
            (!MASK || k_live) ? regs[i] : uint4v{0, 0, 0, 0};
    }
    // Order of the step's memory operations: register i is written to LDS and refilled right away, so
    // that every load has a whole step to arrive.
    static constexpr int OPS = STORES + LOADS;
    static constexpr bool is_commit(int o) { return o % 2 == 0; }
    static constexpr int index_of(int o) { return o / 2; }
};

// ---- fp32 operand contiguous along its row index: E x E micro-blocks (E elements per 16 bytes), transposed ----
// ALIGNED = false: as for the loader above, with the operand's rows in the place of K.
template <class T, int ROWS, int THREADS, bool ALIGNED = true>
struct RowMajorLoader {
    static constexpr int E = kChunkOf<T>;
    using U = std::conditional_t<sizeof(T) == 2, uint16_t, uint32_t>;
    // ROWS/E row-blocks x 8 k-blocks micro-blocks over THREADS threads
    static constexpr int BLOCKS = ROWS / E * 8;
    static constexpr int PASSES = (BLOCKS + THREADS - 1) / THREADS;
    static constexpr int LOADS = E * PASSES, STORES = E * PASSES;
    uint4v regs[PASSES][E];
    uint32_t kfirst, k_count;  // first k of this thread's micro-block; how many of its E k values are inside K
    uint32_t K_;
    __device__ inline void begin_fetch(const Operand&, uint32_t k0, uint32_t K) {
        kfirst = k0 + (threadIdx.x % 8) * E;
        k_count = kfirst >= K ? 0 : (K - kfirst < E ? K - kfirst : E);
        K_ = K;
    }
    __device__ inline void fetch_one(int idx, const Operand& op, uint32_t row0) {
        const int i = idx / E, kk = idx % E;
        const uint32_t rb = (threadIdx.x + THREADS * i) / 8;
        const uint32_t row = row0 + rb * E;
        const uint32_t srow = (rb < ROWS / E && row < op.rows) ? row : 0;
        const uint32_t k = kfirst + kk;
        const T* run = static_cast<const T*>(op.base) + static_cast<int64_t>(k < K_ ? k : 0) * op.k_stride;
        if constexpr (ALIGNED) {
            regs[i][kk] = *reinterpret_cast<const uint4v*>(run + srow);
        } else {
            uint32_t g, j;
            op.group.divmod(srow, g, j);
            regs[i][kk] = piece_of_run<T>(run + static_cast<int64_t>(g) * op.group_stride, j, op.group_live);
        }
    }
    template <bool MASK>
    __device__ inline void commit_one(int idx, T* tile) const {
        const int i = idx / E, rr = idx % E;
        const uint32_t mb = threadIdx.x + THREADS * i;
        const uint32_t kb = mb % 8, rb = mb / 8;
        if (rb >= ROWS / E) return;
        // row rr of the transposed micro-block: element rr of each of the E loaded vectors
        U out[E];
#pragma unroll
        for (int kk = 0; kk < E; ++kk) {
            U in[E];
            __builtin_memcpy(in, &regs[i][kk], 16);
            out[kk] = (!MASK || static_cast<uint32_t>(kk) < k_count) ? in[rr] : U(0);
        }
        uint4v v;
        __builtin_memcpy(&v, out, 16);
        *reinterpret_cast<uint4v*>(tile + tile_offset<T>(rb * E + rr, kb)) = v;
    }
    // A micro-block is transposed out of all of its registers: the E writes of a pass, then its E refills.
    static constexpr int OPS = STORES + LOADS;
    static constexpr bool is_commit(int o) { return o % (2 * E) < E; }
    static constexpr int index_of(int o) { return (o / (2 * E)) * E + o % E; }
};

// ---- 16-bit operand contiguous along its row index: the tile goes to LDS as it lies in memory -----------------
// [k][row] with a pitch of ROWS + 32 elements.  The transposition happens on the way out: gfx950's
// ds_read_b64_tr_b16 hands lane i of a group of 16 lanes, whose lanes 4e+q point at four elements each, element i % 4
// of the four pointers with q = i / 4 - that is, pointed at k-row e and rows 4q..4q+3, it returns to lane i four
// consecutive k of row i.  Two such reads make the 8 k of a lane's MFMA fragment.  The 64 bytes added to the pitch put
// the four k-rows that 32 lanes read together on different banks.
// ALIGNED = false: as for the loaders above.
template <class T, int ROWS, int THREADS, bool ALIGNED = true>
struct AsIsLoader {
    static constexpr int PITCH = ROWS + 32;
    static constexpr int CHUNKS = ROWS / 8;                    // 16-byte chunks per k-row
    static constexpr int LOADS = kBKof<T> * CHUNKS / THREADS, STORES = LOADS;
    static_assert(kBKof<T> * CHUNKS % THREADS == 0, "whole passes");
    uint4v regs[LOADS];
    uint32_t k0_, K_;
    __device__ inline void begin_fetch(const Operand&, uint32_t k0, uint32_t K) { k0_ = k0; K_ = K; }
    __device__ inline void fetch_one(int i, const Operand& op, uint32_t row0) {
        const uint32_t id = threadIdx.x + THREADS * i, k = k0_ + id / CHUNKS, row = row0 + (id % CHUNKS) * 8;
        const T* run = static_cast<const T*>(op.base) + static_cast<int64_t>(k < K_ ? k : 0) * op.k_stride;
        if constexpr (ALIGNED) {
            regs[i] = *reinterpret_cast<const uint4v*>(run + (row < op.rows ? row : 0));
        } else {
            uint32_t g, j;
            op.group.divmod(row < op.rows ? row : 0, g, j);
            regs[i] = piece_of_run<T>(run + static_cast<int64_t>(g) * op.group_stride, j, op.group_live);
        }
    }
    template <bool MASK>
    __device__ inline void commit_one(int i, T* tile) const {
        const uint32_t id = threadIdx.x + THREADS * i, k = id / CHUNKS;
        *reinterpret_cast<uint4v*>(tile + k * PITCH + (id % CHUNKS) * 8) = (!MASK || k0_ + k < K_) ? regs[i] : uint4v{0, 0, 0, 0};
    }
    static constexpr int OPS = STORES + LOADS;
    static constexpr bool is_commit(int o) { return o % 2 == 0; }
    static constexpr int index_of(int o) { return o / 2; }
};

typedef short short4v __attribute__((ext_vector_type(4)));
// the lane's fragment of k-slice ks for the 32 rows starting at row0; lane_offset: see the kernel
template <class T, int PITCH> __device__ inline uint4v read_transposed(const T* tile, uint32_t row0, int ks, uint32_t lane_offset) {
    using Lds = __attribute__((address_space(3))) short4v;
    const T* at = tile + lane_offset + static_cast<uint32_t>(ks) * 16 * PITCH + row0;
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((Lds*)at);
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((Lds*)(at + 4 * PITCH));
    uint4v out;
    __builtin_memcpy(&out, &lo, 8);
    __builtin_memcpy(reinterpret_cast<char*>(&out) + 8, &hi, 8);
    return out;
}

template <class T, bool K_MAJOR> constexpr bool kAsIs = !K_MAJOR && sizeof(T) == 2;
// elements of LDS that one buffer of an operand's tile takes
template <class T, int ROWS, bool K_MAJOR> constexpr uint32_t kTileElements = kAsIs<T, K_MAJOR> ? kBKof<T> * (ROWS + 32) : ROWS * kBKof<T>;

template <class T, int ROWS, int THREADS, bool K_MAJOR, bool ALIGNED = true>
using Loader = std::conditional_t<K_MAJOR, KMajorLoader<T, ROWS, THREADS, ALIGNED>,
                                  std::conditional_t<sizeof(T) == 2, AsIsLoader<T, ROWS, THREADS, ALIGNED>, RowMajorLoader<T, ROWS, THREADS, ALIGNED>>>;

// WAVES_N: wavefronts along N (2 -> 256 threads, one wavefront per SIMD; 4 -> 512 threads, two per SIMD, so that
// one wavefront's waits are covered by the other's MFMAs); always two wavefronts along M.

// SPLIT: several blocks share an output tile, each taking a range of K and storing its fp32 accumulators; a second
// kernel adds the shares in split order, rounds once and writes C.
template <class T, int BM, int BN, int WAVES_N, bool A_KMAJOR, bool B_KMAJOR, bool SPLIT = false, bool ALIGNED = true>
__global__ __launch_bounds__(128 * WAVES_N) void gemm16_kernel(const T* A, const T* B, T* C, GemmProblem p, uint32_t tiles_m, uint32_t tiles_n, SplitK sk) {
    constexpr int THREADS = 128 * WAVES_N;
    constexpr int WM = BM / 2, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    // layout: A buffer 0, A buffer 1, B buffer 0, B buffer 1 (offsets in elements)
    T* lds = reinterpret_cast<T*>(lds_raw);
    constexpr int kBK = kBKof<T>;   // K elements per step
    constexpr uint32_t A_TILE = kTileElements<T, BM, A_KMAJOR>, B_TILE = kTileElements<T, BN, B_KMAJOR>, B_BASE = 2 * A_TILE;

    uint32_t tm, tn;
    const uint32_t tile_id = SPLIT ? blockIdx.x / sk.splits : blockIdx.x, split = SPLIT ? blockIdx.x % sk.splits : 0;
    tile_of(tile_id, tiles_m, tiles_n, tm, tn);
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.y, oa, ob, oc);
    // this block's range of K: all of it, or its share
    const uint32_t k_first = SPLIT ? split * sk.k_chunk : 0;
    const uint32_t K = SPLIT ? (p.K - k_first < sk.k_chunk ? p.K - k_first : sk.k_chunk) : p.K;
    const FastDiv one_group = FastDiv::beyond_all();
    const Operand opA{A + oa + static_cast<int64_t>(k_first) * p.a_cs, p.a_rs, p.a_cs, p.M, one_group, p.M, 0};
    // rows of B's operand are the columns n
    const Operand opB{B + ob + static_cast<int64_t>(k_first) * p.b_rs, p.b_cs, p.b_rs, p.N, p.b_group_stride ? p.c_group_div : one_group,
                      p.b_group_stride ? p.c_group_live : p.N, p.b_group_stride};
    const uint32_t m0 = tm * BM, n0 = tn * BN;

    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
    const uint32_t frag_row = lane % 32, frag_chunk = lane / 32;
    // transposing reads: lane 16b + 4e + q points at k-row 8 * (b / 2) + e, rows 16 * (b % 2) + 4q .. + 3 of the fragment
    const uint32_t tr_k = 8 * (lane / 32) + (lane % 16) / 4, tr_row = 16 * ((lane / 16) % 2) + 4 * (lane % 4);

    // an accumulator holds C transposed: the lane's row of C is lane % 32, so a per-row bias is one value per lane
    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const uint32_t row = tm * BM + (wave / WAVES_N) * WM + i * 32 + lane % 32;
        // (blocks that share K leave the start value to the pass that adds up their partial sums)
        const float start = (!SPLIT && p.row_bias && row < p.M) ? static_cast<float>(widen(static_cast<const T*>(p.row_bias)[row])) : 0.0f;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = start;
    }

    using LA = Loader<T, BM, THREADS, A_KMAJOR, ALIGNED>;
    using LB = Loader<T, BN, THREADS, B_KMAJOR, ALIGNED>;
    LA la;
    LB lb;
    const uint32_t steps = (K + kBK - 1) / kBK;

    // prologue: tile 0 into LDS buffer 0, tile 1 into registers
    la.begin_fetch(opA, 0, K);
    lb.begin_fetch(opB, 0, K);
#pragma unroll
    for (int i = 0; i < LA::LOADS; ++i) la.fetch_one(i, opA, m0);
#pragma unroll
    for (int i = 0; i < LB::LOADS; ++i) lb.fetch_one(i, opB, n0);
#pragma unroll
    for (int i = 0; i < LA::STORES; ++i) la.template commit_one<true>(i, lds);
#pragma unroll
    for (int i = 0; i < LB::STORES; ++i) lb.template commit_one<true>(i, lds + B_BASE);
    if (steps > 1) {
        la.begin_fetch(opA, kBK, K);
        lb.begin_fetch(opB, kBK, K);
#pragma unroll
        for (int i = 0; i < LA::LOADS; ++i) la.fetch_one(i, opA, m0);
#pragma unroll
        for (int i = 0; i < LB::LOADS; ++i) lb.fetch_one(i, opB, n0);
    }
    __syncthreads();

    // One K step, rotated by one k-slice: the step for tile s issues the MFMAs of the LAST 16-wide k-slice of
    // tile s-1 (its fragments are in registers already) and those of the first three slices of tile s.  The
    // barrier thus sits where every wavefront still has 16 MFMAs to issue whose operands need no LDS, so the
    // LDS latency of the first fragment reads of the new tile is covered.  The barrier at the end of step s-1
    // tells that (a) all of tile s is in LDS and (b) nobody reads tile s-1 any more, so its buffer takes tile s+1.
    // The registers hold tile s+1 on entry.  Between the MFMAs, one memory operation at a time: register i
    // goes to LDS (tile s+1) and is refilled from global memory (tile s+2).  sched_barrier pins that
    // interleaving so that neither the load unit nor the LDS ever sees a burst while the matrix pipe idles.
    constexpr int KS = 4, PER_KS = TM * TN;   // a k-slice is two chunks: one per half of the wavefront
    uint4v fa[2][TM], fb[2][TN];
    auto read_fragments = [&](const T* a_tile, const T* b_tile, int ks, int into) {
#pragma unroll
        for (int x = 0; x < TM; ++x) {
            if constexpr (kAsIs<T, A_KMAJOR>) fa[into][x] = read_transposed<T, BM + 32>(a_tile, wm + x * 32, ks, tr_k * (BM + 32) + tr_row);
            else fa[into][x] = *reinterpret_cast<const uint4v*>(a_tile + tile_offset<T>(wm + x * 32 + frag_row, ks * 2 + frag_chunk));
        }
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            if constexpr (kAsIs<T, B_KMAJOR>) fb[into][y] = read_transposed<T, BN + 32>(b_tile, wn + y * 32, ks, tr_k * (BN + 32) + tr_row);
            else fb[into][y] = *reinterpret_cast<const uint4v*>(b_tile + tile_offset<T>(wn + y * 32 + frag_row, ks * 2 + frag_chunk));
        }
    };
    // (for tile 0 the "previous tile's" fragments are zeros: 16 MFMAs that add nothing keep the loop free of a
    // peeled first iteration, whose extra copy of the code costs more than it saves)
#pragma unroll
    for (int x = 0; x < TM; ++x) fa[(KS - 1) & 1][x] = uint4v{0, 0, 0, 0};
#pragma unroll
    for (int y = 0; y < TN; ++y) fb[(KS - 1) & 1][y] = uint4v{0, 0, 0, 0};
    auto step = [&](uint32_t s, auto commit_tag, auto fetch_tag, auto mask_tag) {
        constexpr bool COMMIT = decltype(commit_tag)::value, FETCH = decltype(fetch_tag)::value, MASK = decltype(mask_tag)::value;
        constexpr int MFMAS = KS * PER_KS;
        constexpr int OPS = LA::OPS + LB::OPS;
        const uint32_t cur = s & 1;
        const T* a_tile = lds + cur * A_TILE;
        const T* b_tile = lds + B_BASE + cur * B_TILE;
        T* a_next = lds + (cur ^ 1) * A_TILE;
        T* b_next = lds + B_BASE + (cur ^ 1) * B_TILE;
        if constexpr (FETCH) {
            la.begin_fetch(opA, (s + 2) * kBK, K);
            lb.begin_fetch(opB, (s + 2) * kBK, K);
        }
        read_fragments(a_tile, b_tile, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        static_for<MFMAS>([&](auto m_tag) {
            constexpr int m = decltype(m_tag)::value;
            constexpr int slot = m;
            constexpr int group = slot / PER_KS;           // 0: slice 3 of the previous tile; g > 0: slice g-1 of this tile
            constexpr int i = (slot % PER_KS) / TN, j = slot % TN;
            constexpr int now = group == 0 ? (KS - 1) & 1 : (group - 1) & 1;
            if constexpr (slot % PER_KS == 0 && group > 0) {
                // fragments of slice `group` are requested before the MFMAs of slice group-1
                read_fragments(a_tile, b_tile, group, group & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            acc[i][j] = Mfma16<T>::run(fb[now][j], fa[now][i], acc[i][j]);
            // memory operations [first, last) of the step go right after this MFMA
            constexpr int first = m * OPS / MFMAS, last = (m + 1) * OPS / MFMAS;
            static_for<last - first>([&](auto o_tag) {
                constexpr int o = first + decltype(o_tag)::value;
                if constexpr (o < LA::OPS) {
                    if constexpr (LA::is_commit(o)) { if constexpr (COMMIT) la.template commit_one<MASK>(LA::index_of(o), a_next); }
                    else { if constexpr (FETCH) la.fetch_one(LA::index_of(o), opA, m0); }
                } else {
                    constexpr int ob = o - LA::OPS;
                    if constexpr (LB::is_commit(ob)) { if constexpr (COMMIT) lb.template commit_one<MASK>(LB::index_of(ob), b_next); }
                    else { if constexpr (FETCH) lb.fetch_one(LB::index_of(ob), opB, n0); }
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
    };
    static_assert(KS == 4, "the rotation below assumes four k-slices per tile");
    using Yes = std::true_type;
    using No = std::false_type;
    // only the last tile can reach past K: the tiles the main loop writes to LDS need no mask
    uint32_t s = 0;
    for (; s + 2 < steps; ++s) step(s, Yes{}, Yes{}, No{});
    if (s + 1 < steps) { step(s, Yes{}, No{}, Yes{}); ++s; }
    step(s, No{}, No{}, No{});
    // the last slice of the last tile
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma16<T>::run(fb[(KS - 1) & 1][j], fa[(KS - 1) & 1][i], acc[i][j]);

    // The B fragment is the MFMA's first operand, so a 32x32 accumulator holds C transposed: lane -> row
    // lane % 32 of C; value v -> column 8 * (v / 4) + 4 * (lane / 32) + v % 4, i.e. runs of four consecutive
    // columns.  Each wavefront rounds its WM x WN block into its own LDS area (nobody reads operand tiles any
    // more after the last barrier) and writes it out as whole rows: 16 bytes per lane, WN / 8 lanes per row, so
    // that the memory system sees full lines instead of fragments.
    if constexpr (SPLIT) {
        // lane: row lane % 32 of each 32x32 block, runs of four consecutive columns
        float* mine = sk.partials + (static_cast<size_t>(split) * p.batches + blockIdx.y) * p.M * p.N;
        const bool quads = p.N % 4 == 0;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const uint32_t row = m0 + wm + i * 32 + lane % 32;
            if (row >= p.M) continue;
            float* rp = mine + static_cast<size_t>(row) * p.N;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t col = n0 + wn + j * 32 + g * 8 + 4 * (lane / 32);
                    if (quads) {
                        if (col < p.N) *reinterpret_cast<float4*>(rp + col) = float4{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
                    } else if (col < p.N) {
                        // rows that start anywhere, or end inside a piece: 16 bytes at whatever address, the last piece element by element
                        const float4 four{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
                        store_piece_anywhere(rp + col, &four, p.N - col < 4 ? p.N - col : 4u);
                    }
                }
        }
        return;
    }
    T* c = C + oc;
    if constexpr (sizeof(T) == 4) {
        // four consecutive columns per lane are 16 bytes already
        const bool quads = p.c_rs % 4 == 0 && p.N % 4 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0;
        if (p.c_group) {
            // columns in groups (an image each): every piece of four finds its own place
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const uint32_t row = m0 + wm + i * 32 + lane % 32;
                if (row >= p.M) continue;
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const uint32_t col = n0 + wn + j * 32 + g * 8 + 4 * (lane / 32);
                        if (col >= p.N) continue;
                        uint32_t live;
                        T* dst = grouped_piece(c, p, row, col, 4, live);
                        const float4 four{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
                        if (live) store_piece_anywhere(dst, &four, live);
                    }
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const uint32_t row = m0 + wm + i * 32 + lane % 32;
            if (row >= p.M) continue;
            T* rp = c + static_cast<int64_t>(row) * p.c_rs;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const uint32_t col = n0 + wn + j * 32 + g * 8 + 4 * (lane / 32);
                    if (quads) {
                        if (col < p.N) *reinterpret_cast<float4*>(rp + col) = float4{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
                    } else if (col < p.N) {
                        const float4 four{acc[i][j][g * 4], acc[i][j][g * 4 + 1], acc[i][j][g * 4 + 2], acc[i][j][g * 4 + 3]};
                        store_piece_anywhere(rp + col, &four, p.N - col < 4 ? p.N - col : 4u);
                    }
                }
        }
        return;
    }
    // Rounded into LDS (each wavefront its own block) and written as pieces of 16 bytes: aligned stores when every row of C
    // starts at a multiple of 16 bytes and is whole pieces long, otherwise stores at whatever address a piece has (the last
    // piece of a row element by element): a result whose rows are 4098 long no longer costs 80 % more than one of 4096.
    const bool aligned_rows = p.c_rs % 8 == 0 && p.N % 8 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0;
    {
        constexpr int PITCH = WN + 8;                       // elements: rows stay 16-byte aligned and shift by four banks
        T* stage = lds + wave * (WM * PITCH);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    T out[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) out[e] = narrow_result<T>(acc[i][j][g * 4 + e]);
                    uint2 bits;
                    __builtin_memcpy(&bits, out, 8);
                    *reinterpret_cast<uint2*>(stage + (i * 32 + lane % 32) * PITCH + j * 32 + g * 8 + 4 * (lane / 32)) = bits;
                }
        // same wavefront reads what it wrote: LDS operations of a wavefront complete in order
        constexpr int LANES_PER_ROW = WN / 8, ROWS_PER_PASS = 64 / LANES_PER_ROW;
        const uint32_t col = n0 + wn + (lane % LANES_PER_ROW) * 8;
        if (p.c_group) {
            // columns in groups (an image each): the lane's piece belongs to one group, at one place in it, for every row
            uint32_t live = 0;
            T* first = col < p.N ? grouped_piece(c, p, 0, col, 8, live) : c;
#pragma unroll
            for (int r0 = 0; r0 < WM; r0 += ROWS_PER_PASS) {
                const uint32_t r = r0 + lane / LANES_PER_ROW, row = m0 + wm + r;
                const uint4v bits = *reinterpret_cast<const uint4v*>(stage + r * PITCH + (lane % LANES_PER_ROW) * 8);
                if (live && row < p.M) store_piece_anywhere(first + static_cast<int64_t>(row) * p.c_rs, &bits, live);
            }
            return;
        }
        if (!aligned_rows) {
            const uint32_t live = col >= p.N ? 0u : p.N - col < 8 ? p.N - col : 8u;
#pragma unroll
            for (int r0 = 0; r0 < WM; r0 += ROWS_PER_PASS) {
                const uint32_t r = r0 + lane / LANES_PER_ROW, row = m0 + wm + r;
                const uint4v bits = *reinterpret_cast<const uint4v*>(stage + r * PITCH + (lane % LANES_PER_ROW) * 8);
                if (live && row < p.M) store_piece_anywhere(c + static_cast<int64_t>(row) * p.c_rs + col, &bits, live);
            }
            return;
        }
#pragma unroll
        for (int r0 = 0; r0 < WM; r0 += ROWS_PER_PASS) {
            const uint32_t r = r0 + lane / LANES_PER_ROW, row = m0 + wm + r;
            const uint4v bits = *reinterpret_cast<const uint4v*>(stage + r * PITCH + (lane % LANES_PER_ROW) * 8);
            if (row < p.M && col < p.N) *reinterpret_cast<uint4v*>(c + static_cast<int64_t>(row) * p.c_rs + col) = bits;
        }
    }
}

template <class T, int BM, int BN, int WAVES_N, bool AK, bool BK_, bool SPLIT = false, bool ALIGNED = true>
int launch16(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream, SplitK sk = SplitK{1, 0, nullptr}) {
    const uint32_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    // operand tiles (two buffers each); the same memory later stages the output, BM*BN elements in padded rows
    constexpr size_t tile_bytes = sizeof(T) * 2 * (kTileElements<T, BM, AK> + kTileElements<T, BN, BK_>);
    constexpr size_t stage_bytes = sizeof(T) * 2 * WAVES_N * (BM / 2) * (BN / WAVES_N + 8);
    constexpr size_t lds_bytes = (sizeof(T) == 2 && stage_bytes > tile_bytes) ? stage_bytes : tile_bytes;   // fp32 results are not staged
    auto kernel = gemm16_kernel<T, BM, BN, WAVES_N, AK, BK_, SPLIT, ALIGNED>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n * sk.splits, p.batches), dim3(128 * WAVES_N), lds_bytes, stream, static_cast<const T*>(a),
                       static_cast<const T*>(b), static_cast<T*>(c), p, tiles_m, tiles_n, sk);
    return launch_status("gemm16_kernel");
}

template <class T, int BM, int BN, int WAVES_N>
int pick_layout16(const GemmProblem& p, bool ak, bool bk, const void* a, const void* b, void* c, hipStream_t s) {
    if (ak && bk) return launch16<T, BM, BN, WAVES_N, true, true>(p, a, b, c, s);
    if (ak) return launch16<T, BM, BN, WAVES_N, true, false>(p, a, b, c, s);
    if (bk) return launch16<T, BM, BN, WAVES_N, false, true>(p, a, b, c, s);
    return launch16<T, BM, BN, WAVES_N, false, false>(p, a, b, c, s);
}

// C[batch][m][n] = sum over splits of partials[split][batch][m][n], four columns per thread
template <class T>
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(const float* partials, T* C, GemmProblem p, uint32_t splits, uint32_t quads_per_row, uint32_t total) {
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const uint32_t r = idx / quads_per_row, col = (idx % quads_per_row) * 4;
    const uint32_t batch = r / p.M, m = r % p.M;
    const size_t share = static_cast<size_t>(p.batches) * p.M * p.N;
    const float* src = partials + static_cast<size_t>(r) * p.N + col;
    // the row's start value (the bias of a convolution) first, then the shares of K in their order
    const float start = p.row_bias ? static_cast<float>(widen(static_cast<const T*>(p.row_bias)[m])) : 0.0f;
    float sum[4] = {start, start, start, start};
    const uint32_t live = p.N - col < 4 ? p.N - col : 4;
    if (p.N % 4 == 0) {   // rows of the partial sums start at multiples of 16 bytes
        for (uint32_t sp = 0; sp < splits; ++sp) {
            const float4 v = *reinterpret_cast<const float4*>(src + sp * share);
            sum[0] += v.x; sum[1] += v.y; sum[2] += v.z; sum[3] += v.w;
        }
    } else {
        for (uint32_t sp = 0; sp < splits; ++sp)
            for (uint32_t e = 0; e < live; ++e) sum[e] += src[sp * share + e];
    }
    int64_t oa, ob, oc;
    batch_offsets(p, batch, oa, ob, oc);
    T* dst = C + oc + static_cast<int64_t>(m) * p.c_rs + col;
    if (p.c_group) {
        uint32_t there;
        dst = grouped_piece(C, p, m, col, 4, there);
        for (uint32_t e = 0; e < there; ++e) dst[e] = narrow_result<T>(sum[e]);
        return;
    }
    if (live == 4 && reinterpret_cast<uintptr_t>(dst) % (4 * sizeof(T)) == 0) {
        T out[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = narrow_result<T>(sum[e]);
        using Quad = std::conditional_t<sizeof(T) == 2, uint2, uint4>;
        Quad bits;
        __builtin_memcpy(&bits, out, sizeof(Quad));
        *reinterpret_cast<Quad*>(dst) = bits;
    } else {
        for (uint32_t e = 0; e < live; ++e) dst[e] = narrow_result<T>(sum[e]);
    }
}

// Few tiles and a long K: each tile is shared by `splits` blocks.
template <class T, int BM>
int run16_split(const GemmProblem& p, bool ak, bool bk, uint32_t splits, const void* a, const void* b, void* c, hipStream_t stream, const GemmWorkspace* workspace) {
    constexpr int BN = 128;
    const uint32_t steps = (p.K + kBK - 1) / kBK;
    SplitK sk{};
    sk.k_chunk = (steps + splits - 1) / splits * kBK;
    sk.splits = (p.K + sk.k_chunk - 1) / sk.k_chunk;   // no block without a step
    count(kCounterKShares, sk.splits, true);
    const uint64_t rows = static_cast<uint64_t>(p.batches) * p.M, quads_per_row = (p.N + 3) / 4;
    if (rows * quads_per_row >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    const size_t bytes = static_cast<size_t>(sk.splits) * rows * p.N * sizeof(float);
    if (workspace) {
        if (bytes > workspace->bytes) {
            char text[160];
            snprintf(text, sizeof text, "gemm: this product shares K between blocks and needs %zu bytes for partial sums; the workspace holds %zu", bytes, workspace->bytes);
            set_error_text(text);
            return TANNIC_ERROR;
        }
        sk.partials = static_cast<float*>(workspace->base);
    } else if (scratch_acquire(reinterpret_cast<void**>(&sk.partials), bytes, stream) != TANNIC_SUCCESS) {
        return TANNIC_ERROR;
    }
    int status = TANNIC_UNSUPPORTED_DTYPE;
    if constexpr (sizeof(T) == 2 && (BM == 128 || BM == 64)) status = gemm16_dtl_split<T>(p, BM, sk.splits, sk.k_chunk, sk.partials, a, b, stream);
    if (status != TANNIC_UNSUPPORTED_DTYPE) {}
    else if (ak && bk) status = launch16<T, BM, BN, 2, true, true, true>(p, a, b, c, stream, sk);
    else if (ak) status = launch16<T, BM, BN, 2, true, false, true>(p, a, b, c, stream, sk);
    else if (bk) status = launch16<T, BM, BN, 2, false, true, true>(p, a, b, c, stream, sk);
    else status = launch16<T, BM, BN, 2, false, false, true>(p, a, b, c, stream, sk);
    if (status == TANNIC_SUCCESS) {
        const uint32_t total = static_cast<uint32_t>(rows * quads_per_row);
        hipLaunchKernelGGL((gemm_split_reduce_kernel<T>), dim3((total + 255) / 256), dim3(256), 0, stream, sk.partials, static_cast<T*>(c), p, sk.splits,
                           static_cast<uint32_t>(quads_per_row), total);
        status = launch_status("gemm_split_reduce_kernel");
    }
    if (!workspace) scratch_release(sk.partials, stream);
    return status;
}

// What a 256-row tile narrower than 256 columns loses per column it is narrower (operand bytes per multiply-add), as a
// fraction of its time.
constexpr double kNarrowTilePenalty = 0.001;

template <class T>
int run16(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream, const GemmWorkspace* workspace) {
    if (p.M == 0 || p.N == 0 || p.batches == 0) return TANNIC_SUCCESS;
    // No products to add: the operands hold no elements (their addresses may be null) and the tile loaders would still
    // fetch a first tile.  The scalar kernel, whose K loop then does not run, writes the zeros.
    if (p.K == 0) return TANNIC_UNSUPPORTED_DTYPE;
    // layout of each operand: along which index is it contiguous?
    const bool ak = p.a_cs == 1, bk = p.b_rs == 1;
    if (!ak && p.a_rs != 1) return TANNIC_UNSUPPORTED_DTYPE;
    if (!bk && p.b_cs != 1) return TANNIC_UNSUPPORTED_DTYPE;
    // 16-byte accesses: addresses, leading dimensions, batch strides and the
    // contiguous extent must be multiples of a chunk (8 elements of 16 bits, 4 of 32)
    auto mult8 = [](int64_t v) { return v % kChunkOf<T> == 0; };
    bool aligned = !(reinterpret_cast<uintptr_t>(a) % 16 || reinterpret_cast<uintptr_t>(b) % 16);
    aligned = aligned && mult8(ak ? p.a_rs : p.a_cs) && mult8(bk ? p.b_cs : p.b_rs) && mult8(ak ? p.K : p.M) && mult8(bk ? p.K : p.N);
    for (int d = 0; d < p.batch_rank; ++d) aligned = aligned && mult8(p.a_bs[d]) && mult8(p.b_bs[d]);
    if (p.batches > 65535) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.b_group_stride) {
        // B's columns in groups: the loaders for any alignment know about them; A is a parameter matrix, K-contiguous
        if (!p.c_group || bk || !ak || p.batches != 1) return TANNIC_UNSUPPORTED_DTYPE;
        const uint64_t tiles128 = static_cast<uint64_t>((p.M + 127) / 128) * ((p.N + 127) / 128);
        if (p.M > 64 && tiles128 >= 200) return launch16<T, 128, 128, 2, true, false, false, false>(p, a, b, c, stream);
        return launch16<T, 64, 128, 2, true, false, false, false>(p, a, b, c, stream);
    }
    if (!aligned) {
        // An extent, a row pitch or an address that is odd: the loaders fetch their 16-byte pieces at whatever address they
        // lie (only the piece that straddles the end of a row is gathered element by element) and the product stays on the
        // matrix cores.
        if (ak && bk) {
            if (p.M > 64) return launch16<T, 128, 128, 2, true, true, false, false>(p, a, b, c, stream);
            return launch16<T, 64, 128, 2, true, true, false, false>(p, a, b, c, stream);
        }
        if (ak) return launch16<T, 128, 128, 2, true, false, false, false>(p, a, b, c, stream);
        if (bk) return launch16<T, 128, 128, 2, false, true, false, false>(p, a, b, c, stream);
        return launch16<T, 128, 128, 2, false, false, false, false>(p, a, b, c, stream);
    }
    // Tile height by M (a tile taller than M multiplies padding).  Large tiles when they give (nearly) every compute unit one.  Tile width: 256 unless a narrower one needs less time
    // for its rounds over the 256 compute units (2048 x 14336: 448 tiles 256 wide are two rounds, the second three
    // quarters full; 512 tiles 224 wide are two full rounds of tiles that take 7/8 of the time; 2048 x 6144 is 192 tiles
    // 256 wide, and exactly 256 tiles 192 wide).  A narrower tile reads more operand bytes per multiply-add: it has to win
    // by more than that.
    const uint64_t tiles_m = (p.M + 255) / 256;
    int width = 0;
    double least = 1e30;
    for (int w : {256, 224, 192}) {
        if (w != 256 && (sizeof(T) != 2 || !(ak && bk))) continue;   // fp32 tiles and k-row tiles are powers of two wide
        const uint64_t tiles = tiles_m * ((p.N + w - 1) / w) * p.batches;
        if (tiles < 200) continue;
        const double cost = static_cast<double>((tiles + 255) / 256) * w * (1.0 + (256 - w) * kNarrowTilePenalty);
        if (cost < least) { least = cost; width = w; }
    }
    // Not when the last (or only) column of large tiles would be mostly empty (attention's P . V has 64 or 128 columns: fp16
    // [200, 200] . [200, 64] x 384 takes 31 us on 256 x 256 tiles and 17-19 us on the smaller ones, fp32 140 against 60), and
    // for fp32 only under a long K: its matrix pipe, not the operand traffic, sets the pace, so what counts is how little
    // of a tile is padding and how many blocks overlap their starts and ends ([2048, 128] . [128, 2048] x 32: 437 us on
    // 256 x 256 tiles, 383 on 128 x 128; 4096^3: 1094 against 1105).
    const bool large_ok = static_cast<double>(p.N) >= 0.75 * (((p.N + 255) / 256) * 256.0) && (sizeof(T) == 2 || p.K >= 1024);
    if constexpr (sizeof(T) == 2) {
        if (large_ok && p.M > 192 && width && width != 256) {
            const int rc = gemm16_dtl<T>(p, 256, width, a, b, c, stream);
            if (rc != TANNIC_UNSUPPORTED_DTYPE) return rc;
        }
    }
    if (large_ok && p.M > 192 && tiles_m * ((p.N + 255) / 256) * p.batches >= 200) {
        if constexpr (sizeof(T) == 2) {
            const int rc = gemm16_dtl<T>(p, 256, 256, a, b, c, stream);
            if (rc != TANNIC_UNSUPPORTED_DTYPE) return rc;
        }
        return pick_layout16<T, 256, 256, 2>(p, ak, bk, a, b, c, stream);
    }
    // Fewer large tiles than compute units: choose between the smaller tiles (256 x 128, 128 x 128, 64 x 128) and between
    // whole K per block and a share of it, by a model of the time (microseconds): blocks on the busiest compute unit x
    // steps per block x the measured time of one 64-wide step of that tile, a fixed start-up and write-out, and for
    // shared K the second pass over the fp32 partial sums.
    const bool tall = p.M > 64;
    const double steps_all = (p.K + 63) / 64;
    double best_cost = 1e30;
    int best_bm = tall ? 128 : 64;
    uint32_t best_splits = 1;
    // (fp32: equal costs go to the 128-row tile, which is tried first)
    const int heights[3] = {sizeof(T) == 4 ? 128 : 256, sizeof(T) == 4 ? 256 : 128, 64};
    // Under a short K a block's start and end count: about 2 us for the 128- and 256-row tiles and 0.7 us for the 64-row
    // one, per round of blocks (fp16, K = 64, [192, 64] . [64, 192] x 384: 23 us on 128 x 128 tiles, 15 us on 64 x 128).
    const bool short_k = steps_all <= 4 && sizeof(T) == 2;
    for (int bm : heights) {
        if ((bm == 128 && !tall) || (bm == 256 && p.M <= 192)) continue;
        const double block_fixed = short_k ? (bm == 64 ? 0.7 : 2.0) : 0.0;
        const uint64_t tiles = static_cast<uint64_t>((p.M + bm - 1) / bm) * ((p.N + 127) / 128) * p.batches;
        for (uint32_t splits : {1u, 2u, 4u, 8u, 16u}) {
            if (splits > 1 && (bm == 256 || splits > p.K / (sizeof(T) == 4 ? 64 : 256))) break;
            const double blocks = static_cast<double>(tiles) * splits;
            const double rounds = static_cast<double>((static_cast<uint64_t>(blocks) + 255) / 256);
            // a step costs more the more compute units pull operands through the L2s at the same time
            const double busy = blocks < 256.0 ? blocks / 256.0 : 1.0;
            // (A 64-row tile that walks all of K is register-staged with two stages: between other kernels, with its operands
            // in no cache, its steps take a fifth longer than in a loop over the same product — 40 against 29 us for
            // 512 x 4096 x 4096 inside a decoder layer — which those of the direct-to-LDS tiles do not: 33 us with K shared.)
            double step_us = bm == 256 ? 1.0 : bm == 128 ? 0.375 + 0.175 * busy : splits == 1 ? 0.36 + 0.09 * busy : 0.30 + 0.075 * busy;
            // fp32: the matrix pipe, sixteen times slower than for the 16-bit types, sets the pace of a step
            // (2 * bm * 128 * 64 flops at 157.3 TFLOP/s over 256 compute units)
            if constexpr (sizeof(T) == 4) step_us = std::max(step_us, 2.0 * bm * 128 * 64 / (157.3e6 / 256));
            double cost = rounds * ((steps_all / splits) * step_us + block_fixed) + 5.0;
            if (splits > 1) cost += 4.0 + (splits + 0.5) * static_cast<double>(p.M) * p.N * p.batches * 4.0 / 5.0e6;
            if (cost < best_cost) { best_cost = cost; best_bm = bm; best_splits = splits; }
        }
    }
    if (best_splits > 1) {
        if (best_bm == 128) return run16_split<T, 128>(p, ak, bk, best_splits, a, b, c, stream, workspace);
        return run16_split<T, 64>(p, ak, bk, best_splits, a, b, c, stream, workspace);
    }
    if constexpr (sizeof(T) == 2) {
        if (best_bm >= 128) {
            const int rc = gemm16_dtl<T>(p, best_bm, 128, a, b, c, stream);
            if (rc != TANNIC_UNSUPPORTED_DTYPE) return rc;
        }
    }
    if (best_bm == 256) return pick_layout16<T, 256, 128, 2>(p, ak, bk, a, b, c, stream);
    if (best_bm == 128) return pick_layout16<T, 128, 128, 2>(p, ak, bk, a, b, c, stream);
    return pick_layout16<T, 64, 128, 2>(p, ak, bk, a, b, c, stream);
}

int gemm_mfma_16bit(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream, const GemmWorkspace* workspace) {
    // a handful of rows: stream the other operand once, no tiles
    const int skinny = gemm_skinny_16bit(p, dtype, a, b, c, stream);
    if (skinny != TANNIC_UNSUPPORTED_DTYPE) return skinny;
    if (dtype == TANNIC_FLOAT16) return run16<f16>(p, a, b, c, stream, workspace);
    if (dtype == TANNIC_BFLOAT16) return run16<bf16>(p, a, b, c, stream, workspace);
    return TANNIC_UNSUPPORTED_DTYPE;
}

int gemm_mfma_f32(const GemmProblem& p, const float* a, const float* b, float* c, hipStream_t stream, const GemmWorkspace* workspace) {
    // a handful of rows: stream the other operand once
    const int skinny = gemm_skinny_f32(p, a, b, c, stream);
    if (skinny != TANNIC_UNSUPPORTED_DTYPE) return skinny;
    const int small = gemm_small_f32(p, a, b, c, stream);
    if (small != TANNIC_UNSUPPORTED_DTYPE) return small;
    return run16<float>(p, a, b, c, stream, workspace);
}

}  // namespace th
