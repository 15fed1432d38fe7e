// Operands the tiled kernels cannot take as they lie — rows that start at odd addresses, a K no 16-byte piece divides,
// int8 operands that are not contiguous along K — are copied once into dense K-contiguous rows, K padded with zeros to
// whole steps, and the product then runs on the aligned kernels with everything they have (large tiles, K shared
// between blocks, the streaming kernel for few rows).  The copy costs one read and one write of the operand, which a
// large product repays many times: the kernels for misaligned operands run 128 x 128 tiles that walk all of K, and an
// int8 product that is not K-contiguous otherwise runs the scalar kernel.
// (The product itself: src/cpu/matmul.cpp:60-124; zeros added to both operands along K change no sum.)
#include "gemm_common.hpp"

namespace th {

// 16 bytes at any multiple of the element size
template <int BYTES> struct PieceAt;
template <> struct PieceAt<1> { typedef unsigned int type __attribute__((ext_vector_type(4), aligned(1))); };
template <> struct PieceAt<2> { typedef unsigned int type __attribute__((ext_vector_type(4), aligned(2))); };
template <> struct PieceAt<4> { typedef unsigned int type __attribute__((ext_vector_type(4), aligned(4))); };

// dst[r][k] = k < K ? src[r * row_stride + k * k_stride] : 0 for r < rows, k < Kp; dst rows are Kp elements long.
// k_stride == 1: a thread moves one 16-byte piece of a destination row.
template <class U>
__global__ __launch_bounds__(256) void repack_rows_kernel(const U* src, U* dst, uint32_t rows, uint32_t K, uint32_t Kp, int64_t row_stride, uint32_t pieces_per_row,
                                                          uint32_t total, int64_t src_batch_stride) {
    constexpr uint32_t E = 16 / sizeof(U);
    using uint4_elem = typename PieceAt<sizeof(U)>::type;
    const uint32_t idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    src += static_cast<int64_t>(blockIdx.y) * src_batch_stride;   // one product of a batch per blockIdx.y, its copy rows * Kp further on
    dst += static_cast<size_t>(blockIdx.y) * rows * Kp;
    const uint32_t r = idx / pieces_per_row, k0 = (idx % pieces_per_row) * E;
    const U* from = src + static_cast<int64_t>(r) * row_stride + k0;
    uint4 bits;
    if (k0 + E <= K) {
        const uint4_elem v = *reinterpret_cast<const uint4_elem*>(from);
        __builtin_memcpy(&bits, &v, 16);
    } else {
        U v[E];
#pragma unroll
        for (uint32_t e = 0; e < E; ++e) v[e] = k0 + e < K ? from[e] : U(0);
        __builtin_memcpy(&bits, v, 16);
    }
    *reinterpret_cast<uint4*>(dst + static_cast<size_t>(r) * Kp + k0) = bits;
}

// row_stride == 1 (the operand is contiguous along its rows): 64 x 64 tiles through LDS, read along the rows, written along K.
template <class U>
__global__ __launch_bounds__(256) void repack_transposed_kernel(const U* src, U* dst, uint32_t rows, uint32_t K, uint32_t Kp, int64_t k_stride, uint32_t tiles_r,
                                                                int64_t src_batch_stride) {
    constexpr int TILE = 64;
    __shared__ U tile[TILE][TILE + 1];
    src += static_cast<int64_t>(blockIdx.y) * src_batch_stride;
    dst += static_cast<size_t>(blockIdx.y) * rows * Kp;
    const uint32_t tr = blockIdx.x % tiles_r, tk = blockIdx.x / tiles_r;
    const uint32_t r0 = tr * TILE, k0 = tk * TILE, tx = threadIdx.x % TILE, ty = threadIdx.x / TILE;
#pragma unroll 4
    for (int i = 0; i < TILE; i += 4) {
        const uint32_t r = r0 + tx, k = k0 + ty + i;
        tile[ty + i][tx] = (r < rows && k < K) ? src[r + static_cast<int64_t>(k) * k_stride] : U(0);
    }
    __syncthreads();
#pragma unroll 4
    for (int i = 0; i < TILE; i += 4) {
        const uint32_t k = k0 + tx, r = r0 + ty + i;
        if (r < rows && k < Kp) dst[static_cast<size_t>(r) * Kp + k] = tile[tx][ty + i];
    }
}

template <class U>
static int repack_operand(const void* src, void* dst, uint32_t rows, uint32_t K, uint32_t Kp, int64_t row_stride, int64_t k_stride, uint32_t copies, int64_t batch_stride,
                          hipStream_t stream) {
    if (k_stride == 1) {
        const uint32_t pieces = Kp / (16 / sizeof(U));
        const uint64_t total = static_cast<uint64_t>(rows) * pieces;
        if (total >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
        hipLaunchKernelGGL((repack_rows_kernel<U>), dim3(static_cast<uint32_t>((total + 255) / 256), copies), dim3(256), 0, stream, static_cast<const U*>(src),
                           static_cast<U*>(dst), rows, K, Kp, row_stride, pieces, static_cast<uint32_t>(total), batch_stride);
        return launch_status("repack_rows_kernel");
    }
    const uint32_t tiles_r = (rows + 63) / 64, tiles_k = (Kp + 63) / 64;
    if (static_cast<uint64_t>(tiles_r) * tiles_k >= (1ull << 31)) return TANNIC_UNSUPPORTED_DTYPE;
    hipLaunchKernelGGL((repack_transposed_kernel<U>), dim3(tiles_r * tiles_k, copies), dim3(256), 0, stream, static_cast<const U*>(src), static_cast<U*>(dst), rows, K, Kp,
                       k_stride, tiles_r, batch_stride);
    return launch_status("repack_transposed_kernel");
}

// Whether one operand, seen as rows x K with the given strides, can go to the aligned kernels as it lies.
// unit: elements per 16 bytes.  k_only: the kernels take this element type K-contiguous only (int8).
static bool lies_well(const void* base, uint32_t rows, uint32_t K, int64_t row_stride, int64_t k_stride, uint32_t unit, bool k_only) {
    if (reinterpret_cast<uintptr_t>(base) % 16 != 0) return false;
    if (k_stride == 1) return row_stride % unit == 0 && K % unit == 0;
    if (k_only) return false;
    if (row_stride == 1) return k_stride % unit == 0 && rows % unit == 0;
    return false;
}

// Decides, copies, and describes the product over the copies (a single product, or an int8 batch along one dim).  Returns TANNIC_UNSUPPORTED_DTYPE when nothing was done
// (the caller goes on with the operands as they are); otherwise `q`, `a2`, `b2` are what to multiply and `held[0..1]` what
// to release after the product has been queued.
int gemm_repack(const GemmProblem& p, size_t esize, const void* a, const void* b, hipStream_t stream, bool may_copy, GemmProblem& q, const void*& a2, const void*& b2,
                void* held[2]) {
    held[0] = held[1] = nullptr;
    if (p.c_group || p.b_group_stride || p.M == 0 || p.N == 0 || p.K == 0 || p.batches == 0 || p.batches > 65535) return TANNIC_UNSUPPORTED_DTYPE;
    // a batch along one dim: an operand is copied product by product, or once when every product reads the same one
    if (p.batches != 1 && p.batch_rank != 1) return TANNIC_UNSUPPORTED_DTYPE;
    const bool batched = p.batches != 1;
    if (batched && (p.a_bs[0] < 0 || p.b_bs[0] < 0)) return TANNIC_UNSUPPORTED_DTYPE;
    const bool int8 = esize == 1;
    const uint32_t unit = static_cast<uint32_t>(16 / esize);
    q = p;
    // a single row (column) has no pitch: whatever the descriptor says, it lies K-contiguously when its elements do
    if (q.M == 1 && q.a_cs == 1) q.a_rs = q.K;
    if (q.N == 1 && q.b_rs == 1) q.b_cs = q.K;
    const uint32_t k_step = int8 ? 128 : unit;
    const bool k_fits = q.K % k_step == 0;
    bool a_ok = k_fits && lies_well(a, q.M, q.K, q.a_rs, q.a_cs, unit, int8);
    bool b_ok = k_fits && lies_well(b, q.N, q.K, q.b_cs, q.b_rs, unit, int8);
    if (batched) {   // every product's operand has to start at a multiple of 16 bytes as well
        a_ok = a_ok && q.a_bs[0] % unit == 0;
        b_ok = b_ok && q.b_bs[0] % unit == 0;
    }
    a2 = a;
    b2 = b;
    if (a_ok && b_ok) {
        // only the single-row normalisation may have changed something
        return (q.a_rs != p.a_rs || q.b_cs != p.b_cs) ? TANNIC_SUCCESS : TANNIC_UNSUPPORTED_DTYPE;
    }
    const bool normalised = q.a_rs != p.a_rs || q.b_cs != p.b_cs;
    const int untouched = normalised ? TANNIC_SUCCESS : TANNIC_UNSUPPORTED_DTYPE;   // (with q = p but for the single row's pitch)
    if (!may_copy) return untouched;
    // the copy kernels read along K or along the rows
    if ((!a_ok && q.a_cs != 1 && q.a_rs != 1) || (!b_ok && q.b_rs != 1 && q.b_cs != 1)) return untouched;
    // Worth two more launches: the int8 alternative is the scalar kernel; for the others the kernels for misaligned
    // operands are within a few microseconds of this on small products.
    const double work = static_cast<double>(q.M) * q.N * q.K * q.batches, moved = (static_cast<double>(q.M) + q.N) * q.K * esize * q.batches;
    if (int8 ? work < 1.0e5 : (work < 1.0e7 || moved < 2.0e6)) return untouched;
    // (batches of 16-bit and fp32 products keep their loaders for any alignment, which read a misaligned operand as it
    // lies at nearly the tiles' pace; an int8 batch has the scalar kernel only)
    if (batched && !int8) return untouched;
    const uint32_t Kp = k_fits ? q.K : (q.K + (int8 ? 127 : 63)) / (int8 ? 128 : 64) * (int8 ? 128 : 64);   // zeros are added to both or to neither
    const uint32_t copies_a = batched && q.a_bs[0] != 0 ? q.batches : 1, copies_b = batched && q.b_bs[0] != 0 ? q.batches : 1;
    const size_t bytes_a = a_ok ? 0 : static_cast<size_t>(q.M) * Kp * esize * copies_a, bytes_b = b_ok ? 0 : static_cast<size_t>(q.N) * Kp * esize * copies_b;
    if (bytes_a + bytes_b > (2ull << 30)) return untouched;
    auto copy = [&](const void* src, void* dst, uint32_t rows, int64_t row_stride, int64_t k_stride, uint32_t copies, int64_t batch_stride) {
        switch (esize) {
            case 1: return repack_operand<uint8_t>(src, dst, rows, q.K, Kp, row_stride, k_stride, copies, batch_stride, stream);
            case 2: return repack_operand<uint16_t>(src, dst, rows, q.K, Kp, row_stride, k_stride, copies, batch_stride, stream);
            default: return repack_operand<uint32_t>(src, dst, rows, q.K, Kp, row_stride, k_stride, copies, batch_stride, stream);
        }
    };
    int status = TANNIC_SUCCESS;
    if (!a_ok) {
        if (scratch_acquire(&held[0], bytes_a, stream) != TANNIC_SUCCESS) return TANNIC_ERROR;
        status = copy(a, held[0], q.M, q.a_rs, q.a_cs, copies_a, q.a_bs[0]);
        a2 = held[0];
        q.a_rs = Kp;
        q.a_cs = 1;
        if (batched) q.a_bs[0] = copies_a == 1 ? 0 : static_cast<int64_t>(q.M) * Kp;
    }
    if (status == TANNIC_SUCCESS && !b_ok) {
        if (scratch_acquire(&held[1], bytes_b, stream) != TANNIC_SUCCESS) status = TANNIC_ERROR;
        else {
            status = copy(b, held[1], q.N, q.b_cs, q.b_rs, copies_b, q.b_bs[0]);
            b2 = held[1];
            q.b_cs = Kp;
            q.b_rs = 1;
            if (batched) q.b_bs[0] = copies_b == 1 ? 0 : static_cast<int64_t>(q.N) * Kp;
        }
    }
    q.K = Kp;
    if (status != TANNIC_SUCCESS) {
        for (int i = 0; i < 2; ++i)
            if (held[i]) scratch_release(held[i], stream);
        held[0] = held[1] = nullptr;
        if (status != TANNIC_UNSUPPORTED_DTYPE) return TANNIC_ERROR;
        q = p;
        a2 = a;
        b2 = b;
        return TANNIC_UNSUPPORTED_DTYPE;
    }
    return TANNIC_SUCCESS;
}

}  // namespace th
