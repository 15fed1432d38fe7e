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
// (still whole 128-byte lines).  The loads of tile s+1 are issued between the first MFMAs of step s into the buffer tile
// s-1 has left; the step ends with vmcnt(0) and one barrier.  Operands are addressed through buffer resources, whose
// range check returns zeros for rows past the operand's end.
//
// The MFMA: per multiply-add the 16 x 16 x 32 instruction reads and writes half the accumulator registers of the
// 32 x 32 x 16 one (and twice the operand registers, which are a quarter of the size).  Under the chip's power limit it
// sustains a higher clock: the MFMA-only probes of probes.hip give about 16 % more on N(0,1) x N(0,0.02) operands.  A
// wavefront's 128 x 128 block is 8 x 8 accumulators of four registers; a K step of 64 is two k-slices of 32, each 8 + 8
// fragment reads (lane l: row l % 16, k chunk l / 16 of the slice) and 64 MFMAs.  The B fragment is the first operand,
// so an accumulator holds C transposed: lane l has row l % 16 of the 16 x 16 block and its four values are columns
// 4 * (l / 16) .. + 3.  Sums are formed in the same order of k as in gemm16_kernel: results are bit-identical.
#include "gemm_tiles.hpp"

namespace th {

typedef __attribute__((address_space(3))) void* lds_void;

typedef float float4v __attribute__((ext_vector_type(4)));

template <class T> __device__ inline void mfma16x16_in_place(float4v& acc, const uint4v& first, const uint4v& second) {
    if constexpr (std::is_same_v<T, f16>) {
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

template <class T, int LOAD_EVERY>
__global__ __launch_bounds__(256) void gemm16_dtl16_kernel(const T* A, const T* B, T* C, GemmProblem p, uint32_t tiles_m, uint32_t tiles_n) {
    constexpr int BM = 256, BN = 256, BK = 64;
    constexpr int WM = 128, WN = 128, TM = 8, TN = 8, WAVES_N = 2;
    constexpr uint32_t TILE = 256 * BK;
    constexpr uint32_t TILE_BYTES = TILE * 2, STAGE_BYTES = 2 * TILE_BYTES;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);

    uint32_t tm, tn;
    tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
    int64_t oa, ob, oc;
    batch_offsets(p, blockIdx.y, oa, ob, oc);
    const uint32_t m0 = tm * BM, n0 = tn * BN;
    const uint32_t steps = p.K / BK;

    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
    const uint32_t frag_row = lane % 16, frag_chunk = lane / 16;

    const T* a_base = A + oa + static_cast<int64_t>(m0) * p.a_rs;
    const T* b_base = B + ob + static_cast<int64_t>(n0) * p.b_cs;
    auto records = [](uint64_t rows_left, int64_t stride, uint32_t K) -> uint32_t {
        const uint64_t bytes = ((rows_left - 1) * static_cast<uint64_t>(stride) + K) * 2;
        return bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(bytes);
    };
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(a_base), 0, records(p.M - m0, p.a_rs, p.K), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(b_base), 0, records(p.N - n0, p.b_cs, p.K), 0x00020000);
    uint32_t voff[16];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t row = (wave * 8 + j) * 8 + lane / 8;
        const uint32_t chunk = (lane % 8) ^ ((row >> 1) & 7u);
        voff[j] = row * static_cast<uint32_t>(p.a_rs) * 2 + chunk * 16;
        voff[8 + j] = row * static_cast<uint32_t>(p.b_cs) * 2 + chunk * 16;
    }
    auto issue_load = [&](int j, uint32_t stage, uint32_t k_bytes) {
        const uint32_t at = stage * STAGE_BYTES + (j < 8 ? 0 : TILE_BYTES) + (wave * 8 + (j & 7)) * 1024;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(j < 8 ? rsrc_a : rsrc_b, (lds_void)(lds_raw + at), 16, voff[j], k_bytes, 0, 0);
    };

    float4v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = float4v{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
    for (int j = 0; j < 16; ++j) issue_load(j, 0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    constexpr int PER_KS = TM * TN;   // 64 MFMAs per k-slice
    uint4v fa[2][TM], fb[2][TN];
    auto read_fragments = [&](const T* a_tile, const T* b_tile, int ks, int into) {
#pragma unroll
        for (int x = 0; x < TM; ++x) fa[into][x] = *reinterpret_cast<const uint4v*>(a_tile + tile_offset<T>(wm + x * 16 + frag_row, ks * 4 + frag_chunk));
#pragma unroll
        for (int y = 0; y < TN; ++y) fb[into][y] = *reinterpret_cast<const uint4v*>(b_tile + tile_offset<T>(wn + y * 16 + frag_row, ks * 4 + frag_chunk));
    };

    // A step issues the MFMAs of the second k-slice of the previous tile (fragments in registers since before the
    // barrier) and those of the first slice of this tile; the loads of the next tile go between the first of them.
    // fragment read r of a k-slice: the B fragments and the first A fragment first, in the order the MFMAs want them
    auto read_one = [&](const T* a_tile, const T* b_tile, int ks, int into, int r) {
        if (r == 0) fa[into][0] = *reinterpret_cast<const uint4v*>(a_tile + tile_offset<T>(wm + frag_row, ks * 4 + frag_chunk));
        else if (r <= TN) fb[into][r - 1] = *reinterpret_cast<const uint4v*>(b_tile + tile_offset<T>(wn + (r - 1) * 16 + frag_row, ks * 4 + frag_chunk));
        else fa[into][r - TN] = *reinterpret_cast<const uint4v*>(a_tile + tile_offset<T>(wm + (r - TN) * 16 + frag_row, ks * 4 + frag_chunk));
    };
    auto step = [&](uint32_t s, auto first_tag, auto fetch_tag) {
        constexpr bool FIRST = decltype(first_tag)::value, FETCH = decltype(fetch_tag)::value;
        const uint32_t cur = s & 1;
        const T* a_tile = lds + cur * 2 * TILE;
        const T* b_tile = a_tile + TILE;
        // the first step has no MFMAs in its first half: its fragment reads go out at once
        if constexpr (FIRST) read_fragments(a_tile, b_tile, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        static_for<2 * PER_KS>([&](auto m_tag) {
            constexpr int m = decltype(m_tag)::value;
            constexpr int group = m / PER_KS;           // 0: slice 1 of the previous tile (set 1); 1: slice 0 of this tile (set 0)
            constexpr int q = m % PER_KS, i = q / TN, j = q % TN;
            constexpr int now = group == 0 ? 1 : 0;
            if constexpr (!(FIRST && group == 0)) mfma16x16_in_place<T>(acc[i][j], fb[now][j], fa[now][i]);
            // behind the first 16 MFMAs of a half: the fragment reads of the slice the NEXT half multiplies (its registers were
            // last read by the half before this one)
            if constexpr (q < TM + TN && !(FIRST && group == 0)) read_one(a_tile, b_tile, group == 0 ? 0 : 1, group == 0 ? 0 : 1, q);
            constexpr int slot = FIRST ? m - PER_KS : m;
            if constexpr (FETCH && slot >= 0 && slot % LOAD_EVERY == LOAD_EVERY / 2 && slot / LOAD_EVERY < 16) issue_load(slot / LOAD_EVERY, cur ^ 1, (s + 1) * (BK * 2));
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (FETCH) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };
    using Yes = std::true_type;
    using No = std::false_type;
    if (steps == 1) {
        step(0, Yes{}, No{});
    } else {
        step(0, Yes{}, Yes{});
        uint32_t s = 1;
        for (; s + 1 < steps; ++s) step(s, No{}, Yes{});
        step(s, No{}, No{});
    }
    // the second slice of the last tile
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mfma16x16_in_place<T>(acc[i][j], fb[1][j], fa[1][i]);

    // Each wavefront rounds its 128 x 128 block into its own LDS area (no operand tile is read after the last barrier)
    // and writes it out as whole rows, 16 bytes per lane.
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
    constexpr int LANES_PER_ROW = WN / 8, ROWS_PER_PASS = 64 / LANES_PER_ROW;
    const uint32_t col = n0 + wn + (lane % LANES_PER_ROW) * 8;
#pragma unroll
    for (int r0 = 0; r0 < WM; r0 += ROWS_PER_PASS) {
        const uint32_t r = r0 + lane / LANES_PER_ROW, row = m0 + wm + r;
        const uint4v bits = *reinterpret_cast<const uint4v*>(stage + r * PITCH + (lane % LANES_PER_ROW) * 8);
        if (row < p.M && col < p.N) *reinterpret_cast<uint4v*>(c + static_cast<int64_t>(row) * p.c_rs + col) = bits;
    }
}

template <class T, int LOAD_EVERY>
static int launch_dtl16(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    const uint32_t tiles_m = (p.M + 255) / 256, tiles_n = (p.N + 255) / 256;
    constexpr size_t lds_bytes = 2 * 4 * 128 * (128 + 8);
    auto kernel = gemm16_dtl16_kernel<T, LOAD_EVERY>;
    static std::atomic<uint64_t> configured{0};
    if (int rc = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds_bytes, configured)) return rc;
    hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, p.batches), dim3(256), lds_bytes, stream, static_cast<const T*>(a), static_cast<const T*>(b),
                       static_cast<T*>(c), p, tiles_m, tiles_n);
    return launch_status("gemm16_dtl16_kernel");
}

// Returns TANNIC_UNSUPPORTED_DTYPE when the problem is not this kernel's: the caller then takes the register-staged one.
template <class T>
int gemm16_dtl(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream) {
    if (p.a_cs != 1 || p.b_rs != 1) return TANNIC_UNSUPPORTED_DTYPE;                     // both operands K-contiguous
    if (p.K == 0 || p.K % 64 != 0 || p.row_bias) return TANNIC_UNSUPPORTED_DTYPE;         // whole K steps only, no start values
    if (p.N % 8 != 0 || p.c_rs % 8 != 0 || reinterpret_cast<uintptr_t>(c) % 16 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    for (int d = 0; d < p.batch_rank; ++d)
        if (p.c_bs[d] % 8 != 0) return TANNIC_UNSUPPORTED_DTYPE;
    // a row's offset inside a tile is a 32-bit byte count; rows must not overlap (the range check relies on it)
    if (p.a_rs < static_cast<int64_t>(p.K) || p.b_cs < static_cast<int64_t>(p.K)) return TANNIC_UNSUPPORTED_DTYPE;
    if (p.a_rs >= (1 << 22) || p.b_cs >= (1 << 22)) return TANNIC_UNSUPPORTED_DTYPE;
    return launch_dtl16<T, 4>(p, a, b, c, stream);
}

template int gemm16_dtl<f16>(const GemmProblem&, const void*, const void*, void*, hipStream_t);
template int gemm16_dtl<bf16>(const GemmProblem&, const void*, const void*, void*, hipStream_t);

}  // namespace th
