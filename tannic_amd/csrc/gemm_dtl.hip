// 16-bit matrix product with both operands contiguous along K (X . W^T, a linear layer): 256 x 256 tiles whose operand
// tiles are filled by direct global -> LDS loads and multiplied with v_mfma_f32_16x16x32.
//
// Tile, wavefront layout (2 x 2 wavefronts of 128 x 128) and the swizzled LDS rows of 128 bytes are those of gemm16_kernel
// in gemm_mfma.hip.  Two things differ.
//
// How a tile gets into LDS: `buffer_load_dwordx4 ... lds` moves 16 bytes per lane from global memory straight into LDS:
// no register holds operand data on its way and no ds_write is issued.  Such a load writes the 64 lanes' 16 bytes to
// consecutive LDS addresses, 1 KB = eight 128-byte tile rows; the swizzle permutes the eight 16-byte chunks inside a row,
// so it is applied on the global side: the lane that fills slot c of row r fetches chunk c ^ ((r >> 1) & 7) of that row
// (still whole 128-byte lines).  LDS holds STAGES tiles (2 for 256 x 256, 3 for 256 x 128, 4 for 128 x 128): the loads of
// tile s+STAGES-1 are issued between the first MFMAs of step s into the buffer tile s-1 has left, and a step ends with
// a wait for the loads of tile s+1 only (loads complete in order, so "at most (STAGES-2) tiles' worth outstanding")
// and one barrier.  Operands are addressed through buffer resources, whose range check returns zeros for rows past the
// operand's end.
//
// The MFMA: per multiply-add the 16 x 16 x 32 instruction reads and writes half the accumulator registers of the
// 32 x 32 x 16 one (and twice the operand registers, which are a quarter of the size).  Under the chip's power limit it
// sustains a higher clock: the MFMA-only probes of probes.hip give about 16 % more on N(0,1) x N(0,0.02) operands.  A
// wavefront's 128 x 128 block is 8 x 8 accumulators of four registers; a K step of 64 is two k-slices of 32, each 8 + 8
// fragment reads (lane l: row l % 16, k chunk l / 16 of the slice) and 64 MFMAs.  The B fragment is the first operand,
// so an accumulator holds C transposed: lane l has row l % 16 of the 16 x 16 block and its four values are columns
// 4 * (l / 16) .. + 3.  Sums are formed in the same order of k as in gemm16_kernel: results are bit-identical.
//
// int8 x int8 -> int32 runs the same kernel on v_mfma_i32_16x16x64_i8: a 128-byte tile row is 128 elements, a k-slice 64.
//
// An operand that is contiguous along its other index (A stored as [K][M], B as [K][N]: the X . W, X^T . W and X^T . W^T
// products) keeps that order in LDS: a tile is 64 k-rows of BM (BN) elements, filled by the same loads, and a fragment
// is two ds_read_b64_tr_b16, the transposing LDS read of gfx950: in every group of 16 lanes, lane j supplies the
// address of four consecutive elements and receives element j % 4 of the lanes j / 4, j / 4 + 4, j / 4 + 8, j / 4 + 12.
// With lane 16 g + m pointing at row 8 g + m / 4 (+ 4 for the second read), elements 4 * (m % 4) .. + 3 of the
// fragment's 16 columns, lane 16 g + j ends up with column j, k = 8 g .. 8 g + 7: the MFMA's operand layout.  The
// 32-byte units of a k-row are XOR-swizzled by (k % 4) + 4 * ((k / 8) % 2), on the global side as above, so that the 32
// lanes of a read pass (rows 0..3 and 8..11, or 16..19 and 24..27, 32 bytes each) cover all banks.
#include "gemm_tiles.hpp"

namespace th {

typedef __attribute__((address_space(3))) void* lds_void;

typedef float float4v __attribute__((ext_vector_type(4)));
typedef int int4v __attribute__((ext_vector_type(4)));

// int8 operands: v_mfma_i32_16x16x64_i8, the same 16-byte fragments (lane l: row l % 16, the 16 k of chunk l / 16 of a
// 64-byte slice), int32 accumulators that wrap like the CPU path's; results are written from the registers.
template <class T> struct DtlTypes { using Acc = float4v; using Out = T; };
template <> struct DtlTypes<int8_t> { using Acc = int4v; using Out = int32_t; };

template <class T> __device__ inline void mfma16x16_in_place(typename DtlTypes<T>::Acc& acc, const uint4v& first, const uint4v& second) {
    if constexpr (std::is_same_v<T, int8_t>) {
        int4v x, y;
        __builtin_memcpy(&x, &first, 16);
        __builtin_memcpy(&y, &second, 16);
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(x, y, acc, 0, 0, 0);
    } else if constexpr (std::is_same_v<T, f16>) {
        half8 x, y;
        __builtin_memcpy(&x, &first, 16);
        __builtin_memcpy(&y, &second, 16);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, acc, 0, 0, 0);
    } else {
        bfloat8 x, y;
        __builtin_memcpy(&x, &first, 16);
        __builtin_memcpy(&y, &second, 16);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, acc, 0, 0, 0);
    }
}

// BM x BN: 256 x 256, 256 x 224, 256 x 192, 256 x 128 or 128 x 128 (2 x 2 wavefronts each; BN any multiple of 32 for
// operands contiguous along K, a power of two for k-rows).  The smaller tiles are for products with too few
// large tiles to fill the chip; two workgroups of the smallest share a compute unit.
// SPLIT: `sk.splits` workgroups share a tile, each taking sk.k_chunk of K and storing its fp32 accumulators.
// A_T, B_T: the operand is contiguous along M (N) and its tile is kept as k-rows.
template <class T, int BM, int BN, int STAGES, int BLOCKS_PER_CU, bool SPLIT = false, bool A_T = false, bool B_T = false>
__global__ __launch_bounds__(256, BLOCKS_PER_CU) void gemm16_dtl_kernel(const T* A, const T* B, typename DtlTypes<T>::Out* C, GemmProblem p, uint32_t tiles_m, uint32_t tiles_n, SplitK sk) {
#if defined(__HIP_DEVICE_COMPILE__)   // the host pass needs the launch stub only (and loses it over the body's device-only builtins)
    constexpr int ES = sizeof(T), BK = 128 / ES, WAVES_N = 2;   // a tile row is 128 bytes: 64 elements of 16 bits, 128 of 8
    constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 16, TN = WN / 16;
    constexpr uint32_t A_TILE = BM * BK, B_TILE = BN * BK, STAGE = A_TILE + B_TILE;   // elements
    constexpr int LOADS_A = BM / 32, LOADS_B = BN / 32, LOADS = LOADS_A + LOADS_B;     // 1 KB loads per wavefront and tile
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);           // stage s: A tile at s * STAGE, B tile right behind it

    uint32_t tm, tn;
    const uint32_t split = SPLIT ? blockIdx.x % sk.splits : 0;
    tile_of(SPLIT ? blockIdx.x / sk.splits : blockIdx.x, tiles_m, tiles_n, tm, tn);
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.y, oa, ob, oc);
    const uint32_t m0 = tm * BM, n0 = tn * BN;
    // this workgroup's range of K: all of it, or its share (whole steps)
    const uint32_t k_first = SPLIT ? split * sk.k_chunk : 0;
    const uint32_t steps = (SPLIT ? (p.K - k_first < sk.k_chunk ? p.K - k_first : sk.k_chunk) : p.K) / BK;

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
    const uint32_t frag_row = lane % 16, frag_chunk = lane / 16;

    // Buffer resources starting at the tile's first row: offsets stay below 2^31 and rows past the end are out of range.
    // (A k-row operand starts at the tile's first column.  Its last tile may reach past the operand's extent: those
    // lanes then read the head of the next k-row, rows or columns of the product that are never stored, and past the
    // last k-row the range check returns zeros.)
    const T* a_base = A + oa + static_cast<int64_t>(m0) * p.a_rs;
    const T* b_base = B + ob + static_cast<int64_t>(n0) * p.b_cs;
    auto records = [](uint64_t rows_left, int64_t stride, uint32_t K) -> uint32_t {
        const uint64_t bytes = ((rows_left - 1) * static_cast<uint64_t>(stride) + K) * ES;
        return bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(bytes);
    };
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(a_base), 0, A_T ? records(p.K, p.a_cs, p.M - m0 < BM ? p.M - m0 : BM) : records(p.M - m0, p.a_rs, p.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(b_base), 0, B_T ? records(p.K, p.b_rs, p.N - n0 < BN ? p.N - n0 : BN) : records(p.N - n0, p.b_cs, p.K), 0x00020000);
    // Load j of a wavefront fills 1 KB of a tile (j < LOADS_A: bytes 1024 * (LOADS_A * wave + j) .. of A's, then B's
    // likewise): eight rows of 128 bytes, or 1024 / (2 BM) k-rows; the lane's byte offset from the tile's first element:
    uint32_t voff[LOADS];
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
        const bool of_a = j < LOADS_A;
        const uint32_t slot = (of_a ? wave * LOADS_A + j : wave * LOADS_B + (j - LOADS_A)) * 64 + lane;   // 16-byte slot of the tile
        if ((of_a && A_T) || (!of_a && B_T)) {
            const uint32_t per_row = (of_a ? BM : BN) / 8, k = slot / per_row, in_row = slot % per_row;
            const uint32_t unit = (in_row / 2) ^ ((k % 4) + 4 * ((k / 8) % 2));
            voff[j] = k * static_cast<uint32_t>(of_a ? p.a_cs : p.b_rs) * ES + (unit * 2 + in_row % 2) * 16;
        } else {
            const uint32_t row = slot / 8;
            const uint32_t chunk = (lane % 8) ^ ((row >> 1) & 7u);
            voff[j] = row * static_cast<uint32_t>(of_a ? p.a_rs : p.b_cs) * ES + chunk * 16;
        }
    }
    // the tile that starts at element k of K
    const uint32_t a_kstep = A_T ? static_cast<uint32_t>(p.a_cs) * ES : ES, b_kstep = B_T ? static_cast<uint32_t>(p.b_rs) * ES : ES;
    auto issue_load = [&](int j, uint32_t stage, uint32_t k) {
        const uint32_t at = stage * (STAGE * ES) + (j < LOADS_A ? (wave * LOADS_A + j) * 1024 : A_TILE * ES + (wave * LOADS_B + (j - LOADS_A)) * 1024);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(j < LOADS_A ? rsrc_a : rsrc_b, (lds_void)(lds_raw + at), 16, voff[j], k * (j < LOADS_A ? a_kstep : b_kstep), 0, 0);
    };

    using Acc = typename DtlTypes<T>::Acc;
    // a lane's four values of an accumulator are four columns of ONE row of C: a per-row start value (the bias of a 1x1
    // convolution, src/cpu/conv2d.cpp:90) seeds them, as in the register-staged kernel
    Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        Acc start = Acc{0, 0, 0, 0};
        if constexpr (!SPLIT && ES == 2) {
            const uint32_t row = m0 + wm + i * 16 + lane % 16;
            if (p.row_bias && row < p.M) {
                const float b = static_cast<float>(widen(static_cast<const T*>(p.row_bias)[row]));
                start = Acc{b, b, b, b};
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = start;
    }

    // Tile loads complete in the order they were issued: waiting until at most AHEAD of them are outstanding leaves the
    // tiles that are not needed yet in flight.
    constexpr int AHEAD = (STAGES - 2) * LOADS;
    auto wait_loads = [](bool all) {
        if (all) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AHEAD) : "memory");
    };
    // own LDS traffic done, then everybody's: no fence beyond that (a fence would also wait for the loads in flight)
    auto meet = [] {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // prologue: tiles 0 .. STAGES-2 into their stages
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t) {
        if (static_cast<uint32_t>(t) < steps) {
#pragma unroll
            for (int j = 0; j < LOADS; ++j) issue_load(j, t, k_first + t * BK);
        }
    }
    wait_loads(steps < static_cast<uint32_t>(STAGES - 1));
    meet();

    constexpr int PER_KS = TM * TN;   // MFMAs per k-slice
    constexpr int LOAD_EVERY = PER_KS / LOADS > 0 ? PER_KS / LOADS : 1;   // the loads of a step go out during its first half
    // The fragment reads of a half are spread evenly over it.  A 16-byte read of a wavefront keeps the LDS busy for 8 clocks
    // and the four wavefronts of a workgroup run in step: sixteen reads each behind sixteen consecutive MFMAs ask for
    // 512 clocks of LDS time during 256 clocks of matrix work, and the wavefront that cannot hand its read over does not
    // issue its next MFMA either (measured: 1240 clocks for a half of 64 MFMAs, 1024 of them matrix work).
    constexpr int READ_EVERY = PER_KS / (TM + TN) > 0 ? PER_KS / (TM + TN) : 1;
    uint4v fa[2][TM], fb[2][TN];
    // fragment of the 16 rows (columns) from `first` on, k-slice ks of a tile
    const uint32_t tr_unit = (frag_row / 4) + 4 * (frag_chunk % 2), tr_row = 8 * frag_chunk + frag_row / 4, tr_quad = (frag_row % 4) * 4;
    // The transposing reads are written as assembly: as a builtin, every such read that follows a global -> LDS load in
    // program order is made to wait for that load (the two might touch the same LDS bytes, for all the compiler knows),
    // which puts the memory latency into every step.  The price: the compiler does not count them in lgkmcnt, so the
    // MFMAs of a half are preceded by an explicit wait for the reads issued during the half before.
    const uint32_t lds_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void)(lds_raw)));   // of the dynamic area
    auto fragment = [&](const T* tile, auto transposed_tag, auto width_tag, uint32_t first, auto ks_tag) -> uint4v {
        constexpr int ks = decltype(ks_tag)::value;
        if constexpr (decltype(transposed_tag)::value) {
            constexpr uint32_t WIDTH = decltype(width_tag)::value;
            typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
            const uint32_t at = lds_address + static_cast<uint32_t>(tile - lds) * ES + (tr_row * WIDTH + ((first / 16) ^ tr_unit) * 16 + tr_quad) * ES;
            uint2v low, high;
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(low) : "v"(at), "n"(ks * 32 * WIDTH * ES));
            asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(high) : "v"(at), "n"((ks * 32 + 4) * WIDTH * ES));
            return uint4v{low[0], low[1], high[0], high[1]};
        } else {
            return *reinterpret_cast<const uint4v*>(tile + tile_offset<T>(first + frag_row, ks * 4 + frag_chunk));
        }
    };
    auto wait_fragments = [] {
        if constexpr (A_T || B_T) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    using ATag = std::integral_constant<bool, A_T>;
    using BTag = std::integral_constant<bool, B_T>;
    using AWidth = std::integral_constant<uint32_t, BM>;
    using BWidth = std::integral_constant<uint32_t, BN>;
    auto read_fragments = [&](const T* a_tile, const T* b_tile, auto ks_tag, int into) {
#pragma unroll
        for (int x = 0; x < TM; ++x) fa[into][x] = fragment(a_tile, ATag{}, AWidth{}, wm + x * 16, ks_tag);
#pragma unroll
        for (int y = 0; y < TN; ++y) fb[into][y] = fragment(b_tile, BTag{}, BWidth{}, wn + y * 16, ks_tag);
    };
    // fragment read r of a k-slice: the first A fragment and the B fragments first, in the order the MFMAs want them
    auto read_one = [&](const T* a_tile, const T* b_tile, auto ks_tag, int into, int r) {
        if (r == 0) fa[into][0] = fragment(a_tile, ATag{}, AWidth{}, wm, ks_tag);
        else if (r <= TN) fb[into][r - 1] = fragment(b_tile, BTag{}, BWidth{}, wn + (r - 1) * 16, ks_tag);
        else fa[into][r - TN] = fragment(a_tile, ATag{}, AWidth{}, wm + (r - TN) * 16, ks_tag);
    };
    // A step issues the MFMAs of the second k-slice of the previous tile (its fragments are in registers since before
    // the barrier) and those of the first slice of this tile.  Spread over the MFMAs of each half go the fragment
    // reads of the slice the NEXT half multiplies (their registers were last read by the half before this one), and,
    // spread over the first half, the loads of the next tile.
    auto step = [&](uint32_t s, uint32_t cur, uint32_t fill, auto first_tag, auto fetch_tag) {   // cur: stage of tile s; fill: stage tile s-1 has left
        constexpr bool FIRST = decltype(first_tag)::value, FETCH = decltype(fetch_tag)::value;
        const T* a_tile = lds + cur * STAGE;
        const T* b_tile = a_tile + A_TILE;
        // the first step has no MFMAs in its first half: its fragment reads go out at once
        if constexpr (FIRST) read_fragments(a_tile, b_tile, std::integral_constant<int, 0>{}, 0);
        __builtin_amdgcn_sched_barrier(0);
        static_for<2 * PER_KS>([&](auto m_tag) {
            constexpr int m = decltype(m_tag)::value;
            constexpr int group = m / PER_KS;           // 0: slice 1 of the previous tile (set 1); 1: slice 0 of this tile (set 0)
            constexpr int q = m % PER_KS, i = q / TN, j = q % TN;
            constexpr int now = group == 0 ? 1 : 0;
            if constexpr (q == 0) wait_fragments();
            if constexpr (!(FIRST && group == 0)) mfma16x16_in_place<T>(acc[i][j], fb[now][j], fa[now][i]);
            if constexpr (q % READ_EVERY == 0 && q / READ_EVERY < TM + TN && !(FIRST && group == 0)) read_one(a_tile, b_tile, std::integral_constant<int, group == 0 ? 0 : 1>{}, group == 0 ? 0 : 1, q / READ_EVERY);
            constexpr int slot = FIRST ? m - PER_KS : m;
            if constexpr (FETCH && slot >= 0 && slot % LOAD_EVERY == LOAD_EVERY / 2 && slot / LOAD_EVERY < LOADS) issue_load(slot / LOAD_EVERY, fill, k_first + (s + STAGES - 1) * BK);
            __builtin_amdgcn_sched_barrier(0);
        });
        wait_loads(!FETCH);    // tile s+1 is in LDS (steps that issue no loads wait for all that are left)
        meet();
    };
    using Yes = std::true_type;
    using No = std::false_type;
    auto next = [](uint32_t stage) { return stage + 1 == STAGES ? 0u : stage + 1; };
    uint32_t s = 0, cur = 0, fill = STAGES - 1;
    if (steps > STAGES - 1) step(0, cur, fill, Yes{}, Yes{});
    else step(0, cur, fill, Yes{}, No{});
    for (s = 1, cur = next(cur), fill = next(fill); s + STAGES - 1 < steps; ++s, cur = next(cur), fill = next(fill)) step(s, cur, fill, No{}, Yes{});
    for (; s < steps; ++s, cur = next(cur), fill = next(fill)) step(s, cur, fill, No{}, No{});
    // the second slice of the last tile
    wait_fragments();
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma16x16_in_place<T>(acc[i][j], fb[1][j], fa[1][i]);

    // Each wavefront rounds its block into its own LDS area (no operand tile is read after the last barrier) and
    // writes it out as whole rows, 16 bytes per lane.
    if constexpr (SPLIT) {
        // fp32 partial sums, [split][batch][M][N]: a lane's four consecutive columns are 16 bytes
        float* mine = sk.partials + (static_cast<size_t>(split) * p.batches + blockIdx.y) * p.M * p.N;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const uint32_t row = m0 + wm + i * 16 + lane % 16;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const uint32_t col = n0 + wn + j * 16 + 4 * (lane / 16);
                if (row < p.M && col < p.N) *reinterpret_cast<Acc*>(mine + static_cast<size_t>(row) * p.N + col) = acc[i][j];
            }
        }
        return;
    } else if constexpr (ES == 1) {
        // int32 results: a lane's four consecutive columns are 16 bytes already (rows that start anywhere, or end inside
        // them, go through the store for any alignment)
        int32_t* c32 = C + oc;
        const bool quads = (p.c_rs | p.N) % 4 == 0 && reinterpret_cast<uintptr_t>(c32) % 16 == 0;
        if (quads) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const uint32_t row = m0 + wm + i * 16 + lane % 16;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const uint32_t col = n0 + wn + j * 16 + 4 * (lane / 16);
                    if (row < p.M && col < p.N) *reinterpret_cast<int4v*>(c32 + static_cast<int64_t>(row) * p.c_rs + col) = acc[i][j];
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const uint32_t row = m0 + wm + i * 16 + lane % 16;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const uint32_t col = n0 + wn + j * 16 + 4 * (lane / 16);
                    if (row < p.M && col < p.N) store_piece_anywhere<int32_t>(c32 + static_cast<int64_t>(row) * p.c_rs + col, &acc[i][j], p.N - col < 4 ? p.N - col : 4);
                }
            }
        }
        return;
    } else {
    T* c = C + oc;
    constexpr int PITCH = WN + 8;
    T* stage = lds + wave * (WM * PITCH);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            T out[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) out[e] = narrow_result<T>(acc[i][j][e]);
            uint2 bits;
            __builtin_memcpy(&bits, out, 8);
            *reinterpret_cast<uint2*>(stage + (i * 16 + lane % 16) * PITCH + j * 16 + 4 * (lane / 16)) = bits;
        }
    // a row of the wavefront's block is WN / 8 stores of 16 bytes: that many lanes per row, or the next power of two with the
    // lanes beyond the row idle (tile widths that are not a power of two)
    constexpr int PIECES = WN / 8, LANES_PER_ROW = PIECES <= 4 ? 4 : PIECES <= 8 ? 8 : 16, ROWS_PER_PASS = 64 / LANES_PER_ROW;
    static_assert(PIECES <= 16, "a wavefront's block is at most 128 columns wide");
    const uint32_t piece = lane % LANES_PER_ROW, col = n0 + wn + piece * 8;
    const bool aligned_rows = (p.c_rs | p.N) % 8 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0;
    if (p.c_group || !aligned_rows) {
        // Columns in groups (an image each): the lane's piece belongs to one group, at one place in it, for every row.
        // Plain rows that do not start at multiples of 16 bytes, or end inside a piece, are stored the same way.
        uint32_t live = 0;
        T* first = c;
        if (piece < PIECES && col < p.N) {
            if (p.c_group) {
                first = grouped_piece(c, p, 0, col, 8, live);
            } else {
                first = c + col;
                live = p.N - col < 8 ? p.N - col : 8;
            }
        }
#pragma unroll
        for (int r0 = 0; r0 < WM; r0 += ROWS_PER_PASS) {
            const uint32_t r = r0 + lane / LANES_PER_ROW, row = m0 + wm + r;
            if (live && row < p.M) {
                const uint4v bits = *reinterpret_cast<const uint4v*>(stage + r * PITCH + piece * 8);
                store_piece_anywhere(first + static_cast<int64_t>(row) * p.c_rs, &bits, live);
            }
        }
        return;
    }
#pragma unroll
    for (int r0 = 0; r0 < WM; r0 += ROWS_PER_PASS) {
        const uint32_t r = r0 + lane / LANES_PER_ROW, row = m0 + wm + r;
        if (piece < PIECES && row < p.M && col < p.N)
            *reinterpret_cast<uint4v*>(c + static_cast<int64_t>(row) * p.c_rs + col) = *reinterpret_cast<const uint4v*>(stage + r * PITCH + piece * 8);
    }
    }
#endif
}

template <class T, int BM, int BN, int STAGES, bool SPLIT = false, bool A_T = false, bool B_T = false>
static int launch_dtl(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream, SplitK sk = SplitK{1, 0, nullptr}) {
    const uint32_t tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    constexpr size_t tile_bytes = STAGES * (BM + BN) * 128, stage_bytes = sizeof(T) == 2 ? 2 * 4 * (BM / 2) * (BN / 2 + 8) : 0;   // the operand stages; the output staging (16-bit results)
    constexpr size_t lds_bytes = tile_bytes > stage_bytes ? tile_bytes : stage_bytes;
    auto kernel = gemm16_dtl_kernel<T, BM, BN, STAGES, (lds_bytes <= 80 * 1024 ? 2 : 1), SPLIT, A_T, B_T>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n * sk.splits, p.batches), dim3(256), lds_bytes, stream, static_cast<const T*>(a), static_cast<const T*>(b),
                       static_cast<typename DtlTypes<T>::Out*>(c), p, tiles_m, tiles_n, sk);
    return launch_status("gemm16_dtl_kernel");
}

// This file is compiled in parts (TH_DTL_PART): 0 holds the entry points and the kernels for operands contiguous along
// K, 1 and 2 the kernels with k-row operands for float16 and bfloat16.
#ifndef TH_DTL_PART
#define TH_DTL_PART 0
#endif

// the kernels with k-row operands: a_t / b_t say which operand is one; splits == 0: whole K per workgroup
template <class T>
int gemm16_dtl_krows(const GemmProblem& p, int bm, int bn, bool a_t, bool b_t, SplitK sk, const void* a, const void* b, void* c, hipStream_t stream);

#if TH_DTL_PART != 0
template <class T, int BM, int BN, int STAGES, bool SPLIT>
static int launch_dtl_krows(const GemmProblem& p, bool a_t, bool b_t, SplitK sk, const void* a, const void* b, void* c, hipStream_t stream) {
    if (a_t && b_t) return launch_dtl<T, BM, BN, STAGES, SPLIT, true, true>(p, a, b, c, stream, sk);
    if (a_t) return launch_dtl<T, BM, BN, STAGES, SPLIT, true, false>(p, a, b, c, stream, sk);
    return launch_dtl<T, BM, BN, STAGES, SPLIT, false, true>(p, a, b, c, stream, sk);
}

template <class T>
int gemm16_dtl_krows(const GemmProblem& p, int bm, int bn, bool a_t, bool b_t, SplitK sk, const void* a, const void* b, void* c, hipStream_t stream) {
    if (sk.splits) return bm == 128 && bn == 128 ? launch_dtl_krows<T, 128, 128, 4, true>(p, a_t, b_t, sk, a, b, c, stream) : TANNIC_UNSUPPORTED_DTYPE;
    sk.splits = 1;
    if (bm == 256 && bn == 256) return launch_dtl_krows<T, 256, 256, 2, false>(p, a_t, b_t, sk, a, b, c, stream);
    if (bm == 256 && bn == 128) return launch_dtl_krows<T, 256, 128, 3, false>(p, a_t, b_t, sk, a, b, c, stream);
    if (bm == 128 && bn == 128) return launch_dtl_krows<T, 128, 128, 4, false>(p, a_t, b_t, sk, a, b, c, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}
#if TH_DTL_PART == 1
template int gemm16_dtl_krows<f16>(const GemmProblem&, int, int, bool, bool, SplitK, const void*, const void*, void*, hipStream_t);
#else
template int gemm16_dtl_krows<bf16>(const GemmProblem&, int, int, bool, bool, SplitK, const void*, const void*, void*, hipStream_t);
#endif

#else   // TH_DTL_PART == 0

// Whether the operands are this kernel's (tile bm x bn): each contiguous along K, or (16-bit types) along its other
// index; whole K steps; rows that do not overlap; offsets that fit 32 bits.
template <class T>
static bool operands_fit(const GemmProblem& p, int bm, int bn, bool& a_t, bool& b_t) {
    a_t = p.a_cs != 1;
    b_t = p.b_rs != 1;
    if ((a_t || b_t) && sizeof(T) != 2) return false;
    if ((a_t && p.a_rs != 1) || (b_t && p.b_cs != 1)) return false;
    constexpr int step = 128 / sizeof(T);
    if (p.K == 0 || p.K % step != 0) return false;       // whole K steps only
    // a row's offset inside a tile is a 32-bit byte count; rows must not overlap (the range check relies on it)
    if (!a_t && (p.a_rs < static_cast<int64_t>(p.K) || p.a_rs >= (1 << 22))) return false;
    if (!b_t && (p.b_cs < static_cast<int64_t>(p.K) || p.b_cs >= (1 << 22))) return false;
    // k-row operands: 16-byte pieces along the contiguous index, 32-bit byte offsets along K
    // (a last tile that reaches past the extent is fine, see the kernel; with a short K the register-staged tiles, which
    // start multiplying sooner, are as fast or faster: 12.1 against 11.0 us for [128,512] . [512,784] x 32)
    if (((a_t && p.M % bm != 0) || (b_t && p.N % bn != 0)) && p.K < 2048) return false;
    if (a_t && (p.M % 8 != 0 || p.a_cs < static_cast<int64_t>(p.M) || static_cast<uint64_t>(p.K) * p.a_cs * sizeof(T) >= (1ull << 32))) return false;
    if (b_t && (p.N % 8 != 0 || p.b_rs < static_cast<int64_t>(p.N) || static_cast<uint64_t>(p.K) * p.b_rs * sizeof(T) >= (1ull << 32))) return false;
    return true;
}

template <class T>
int gemm16_dtl_split(const GemmProblem& p, int bm, uint32_t splits, uint32_t k_chunk, float* partials, const void* a, const void* b, hipStream_t stream) {
    bool a_t, b_t;
    if (!operands_fit<T>(p, bm, 128, a_t, b_t) || p.N % 4 != 0 || k_chunk % 64 != 0) return TANNIC_UNSUPPORTED_DTYPE;   // (a row start value is added with the partial sums)
    const SplitK sk{splits, k_chunk, partials};
    if (bm == 64) {
        // 64 x 128 tiles, six stages: a workgroup's share of K is short and its operands are in no cache, so what counts
        // is how much of that share is on its way at once (operands contiguous along K only: a k-row tile is at least
        // 128 wide)
        if (a_t || b_t) return TANNIC_UNSUPPORTED_DTYPE;
        return launch_dtl<T, 64, 128, 6, true>(p, a, b, nullptr, stream, sk);
    }
    if (bm != 128) return TANNIC_UNSUPPORTED_DTYPE;
    if constexpr (sizeof(T) == 2) {
        if (a_t || b_t) return gemm16_dtl_krows<T>(p, 128, 128, a_t, b_t, sk, a, b, nullptr, stream);
    }
    return launch_dtl<T, 128, 128, 4, true>(p, a, b, nullptr, stream, sk);
}
template int gemm16_dtl_split<f16>(const GemmProblem&, int, uint32_t, uint32_t, float*, const void*, const void*, hipStream_t);
template int gemm16_dtl_split<bf16>(const GemmProblem&, int, uint32_t, uint32_t, float*, const void*, const void*, hipStream_t);

// Returns TANNIC_UNSUPPORTED_DTYPE when the problem is not this kernel's: the caller then takes the register-staged one.
template <class T>
int gemm16_dtl(const GemmProblem& p, int bm, int bn, const void* a, const void* b, void* c, hipStream_t stream) {
    bool a_t, b_t;
    if (!operands_fit<T>(p, bm, bn, a_t, b_t)) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.c_group && (sizeof(T) != 2 || p.N % 8 != 0)) return TANNIC_UNSUPPORTED_DTYPE;   // column groups: 16-bit results, whole pieces of eight
    // (results may lie anywhere: the kernel looks at the alignment of its own rows)
    if (reinterpret_cast<uintptr_t>(c) % sizeof(typename DtlTypes<T>::Out) != 0) return TANNIC_UNSUPPORTED_DTYPE;
    if constexpr (sizeof(T) == 2) {
        if (a_t || b_t) return gemm16_dtl_krows<T>(p, bm, bn, a_t, b_t, SplitK{0, 0, nullptr}, a, b, c, stream);
    }
    // as many stages as LDS holds (160 KB): the smaller the tile, the shorter its step and the more steps a load needs to arrive
    if (bm == 256 && bn == 256) return launch_dtl<T, 256, 256, 2>(p, a, b, c, stream);
    if constexpr (sizeof(T) == 2) {
        // widths between the powers of two, for extents that leave the last round of 256-wide tiles mostly empty
        if (bm == 256 && bn == 224) return launch_dtl<T, 256, 224, 2>(p, a, b, c, stream);
        if (bm == 256 && bn == 192) return launch_dtl<T, 256, 192, 2>(p, a, b, c, stream);
    }
    if (bm == 256 && bn == 128) return launch_dtl<T, 256, 128, 3>(p, a, b, c, stream);
    if (bm == 128 && bn == 128) return launch_dtl<T, 128, 128, 4>(p, a, b, c, stream);
    return TANNIC_UNSUPPORTED_DTYPE;
}

template int gemm16_dtl<f16>(const GemmProblem&, int, int, const void*, const void*, void*, hipStream_t);
template int gemm16_dtl<bf16>(const GemmProblem&, int, int, const void*, const void*, void*, hipStream_t);
template int gemm16_dtl<int8_t>(const GemmProblem&, int, int, const void*, const void*, void*, hipStream_t);

// int8 x int8 -> int32 (src/cpu/matmul.cpp:191-209): exact, so the tiled kernel's results are the scalar kernel's bit for
// bit.  Both operands K-contiguous and 16-byte friendly; the tile follows the number of tiles it leaves.
int gemm_mfma_int8(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    if (p.M == 0 || p.N == 0 || p.batches == 0) return TANNIC_SUCCESS;
    if (p.a_cs != 1 || p.b_rs != 1 || p.K % 128 != 0 || p.batches > 65535) return TANNIC_UNSUPPORTED_DTYPE;
    if (reinterpret_cast<uintptr_t>(a) % 16 || reinterpret_cast<uintptr_t>(b) % 16 || p.a_rs % 16 || p.b_cs % 16) return TANNIC_UNSUPPORTED_DTYPE;
    for (int d = 0; d < p.batch_rank; ++d)
        if (p.a_bs[d] % 16 || p.b_bs[d] % 16) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.M <= 32) {
        const int status = gemm_skinny_int8(p, a, b, c, stream);
        if (status != TANNIC_UNSUPPORTED_DTYPE) return status;
    }
    auto tiles = [&](uint64_t bm, uint64_t bn) { return ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.batches; };
    if (p.M > 192 && tiles(256, 256) >= 200) return gemm16_dtl<int8_t>(p, 256, 256, a, b, c, stream);
    if (p.M > 192 && tiles(256, 128) >= 128) return gemm16_dtl<int8_t>(p, 256, 128, a, b, c, stream);
    // (also a handful of rows: a mostly empty 128-row tile still walks W at the tiles' pace, 17 us for 4096 x 4096 where the
    // scalar kernel takes 570)
    return gemm16_dtl<int8_t>(p, 128, 128, a, b, c, stream);
}

#endif   // TH_DTL_PART == 0

}  // namespace th
