// Problem description shared by the matrix-multiply kernels.
#pragma once

#include "common.hpp"

namespace th {

// One batched product C[b] = A[b] * B[b].  Operands are addressed as
// base + batch_offset + row * rs + col * cs (element strides), which covers the
// four plain/transposed combinations the reference derives from strides
// (src/cpu/matmul.cpp:87-94, :132-137).
struct GemmProblem {
    uint32_t M, N, K;
    int64_t a_rs, a_cs;  // A[m,k]
    int64_t b_rs, b_cs;  // B[k,n]
    int64_t c_rs;        // C[m,n], column stride 1
    // batch dims of the destination, outermost first
    int batch_rank;
    uint32_t batches;
    uint32_t batch_extent[6];
    int64_t a_bs[6], b_bs[6], c_bs[6];
    // optional (MFMA 16-bit kernels only): one value of C's type per row of C, added before rounding
    const void* row_bias;
    // optional (MFMA f16 / bf16 / fp32 kernels, no batches): the columns of C come in groups of c_group (a multiple of 16
    // bytes of elements; 0: off).  Column j of group g goes to C + g * c_group_stride + row * c_rs + j when j < c_group_live
    // and nowhere otherwise; nothing about these addresses needs to be aligned.  (A convolution over a whole batch as one
    // product: a group is an image, its live columns the image's pixels.)
    uint32_t c_group, c_group_live;
    int64_t c_group_stride;
    FastDiv c_group_div;
    // optional, with c_group and B contiguous along n (b_cs == 1): B's columns lie in the same groups, element (k, j) of
    // group g at B + g * b_group_stride + k * b_rs + j for j < c_group_live, at any alignment; the other columns of a group
    // read as zero (0: off).  (The same convolution reading its images where they lie.)
    int64_t b_group_stride;
};

// Where the piece of E elements that starts at column `col` (a multiple of E) of row `row` goes, and how many of its elements exist.
template <class T>
__device__ inline T* grouped_piece(T* c, const GemmProblem& p, uint32_t row, uint32_t col, int E, uint32_t& live) {
    uint32_t g, j;
    p.c_group_div.divmod(col, g, j);
    live = j >= p.c_group_live ? 0u : p.c_group_live - j < static_cast<uint32_t>(E) ? p.c_group_live - j : static_cast<uint32_t>(E);
    return c + static_cast<int64_t>(g) * p.c_group_stride + static_cast<int64_t>(row) * p.c_rs + j;
}

// `live` of the E elements at `bits` (16 bytes) to dst, which may have any alignment
template <class T>
__device__ inline void store_piece_anywhere(T* dst, const void* bits, uint32_t live) {
    constexpr uint32_t E = 16 / sizeof(T);
    typedef unsigned int uint4_any __attribute__((ext_vector_type(4), aligned(2)));
    if (live == E) {
        uint4_any v;
        __builtin_memcpy(&v, bits, 16);
        *reinterpret_cast<uint4_any*>(dst) = v;
    } else {
        T e[E];
        __builtin_memcpy(e, bits, 16);
        for (uint32_t i = 0; i < live; ++i) dst[i] = e[i];
    }
}

__host__ __device__ inline void batch_offsets(const GemmProblem& p, uint32_t batch, int64_t& oa, int64_t& ob, int64_t& oc) {
    oa = ob = oc = 0;
    for (int d = p.batch_rank - 1; d >= 0; --d) {
        const uint32_t idx = batch % p.batch_extent[d];
        batch /= p.batch_extent[d];
        oa += static_cast<int64_t>(idx) * p.a_bs[d];
        ob += static_cast<int64_t>(idx) * p.b_bs[d];
        oc += static_cast<int64_t>(idx) * p.c_bs[d];
    }
}

// Fills `p` from the descriptors the way launchGemmKernel does
// (src/cpu/matmul.cpp:126-176).  Returns a status.
int describe_gemm(const tannic_tensor_t* a, const tannic_tensor_t* b, const tannic_tensor_t* c, GemmProblem& p);

// Where the kernels that share K between blocks leave their fp32 partial sums.  nullptr: a block from the library's
// scratch cache (allocated on first need); otherwise caller-supplied memory, and a need beyond `bytes` is an error.
struct GemmWorkspace {
    void* base;
    size_t bytes;
};

// MFMA paths; each returns TANNIC_UNSUPPORTED_DTYPE when the problem does not
// meet its layout/alignment conditions so that the caller can fall back.
int gemm_skinny_16bit(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream);
int gemm_skinny_f32(const GemmProblem& p, const float* a, const float* b, float* c, hipStream_t stream);
int gemm_skinny_int8(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream);
int gemm_rows_nn(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream);
int gemm_few_results(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream);
int gemm_mfma_f64(const GemmProblem& p, const double* a, const double* b, double* c, hipStream_t stream);
int gemm_mfma_16bit(const GemmProblem& p, int dtype, const void* a, const void* b, void* c, hipStream_t stream, const GemmWorkspace* workspace = nullptr);
int gemm_mfma_f32(const GemmProblem& p, const float* a, const float* b, float* c, hipStream_t stream, const GemmWorkspace* workspace = nullptr);
// Operands that do not lie as the tiled kernels want them, copied into dense K-contiguous rows (gemm_repack.hip).  SUCCESS:
// multiply q, a2, b2 instead and release held[0..1] (each may be null) afterwards; UNSUPPORTED: nothing was done.
int gemm_repack(const GemmProblem& p, size_t esize, const void* a, const void* b, hipStream_t stream, bool may_copy, GemmProblem& q, const void*& a2, const void*& b2,
                void* held[2]);
// fp32 products of a few hundred rows and columns (32 x 32 tiles whose wavefronts split K; gemm_small.hip)
int gemm_small_f32(const GemmProblem& p, const float* a, const float* b, float* c, hipStream_t stream);
// bm x bn tiles (256 x 256, 256 x 128, 128 x 128) filled by direct global -> LDS loads (gemm_dtl.hip); T is f16 or bf16
template <class T> int gemm16_dtl(const GemmProblem& p, int bm, int bn, const void* a, const void* b, void* c, hipStream_t stream);
// the 128 x 128 (bm = 128) or 64 x 128 (bm = 64) tiles with K shared between `splits` workgroups per tile (k_chunk elements each, a multiple of 64): fp32
// partial sums go to partials[split][batch][M][N], which the caller adds up
template <class T> int gemm16_dtl_split(const GemmProblem& p, int bm, uint32_t splits, uint32_t k_chunk, float* partials, const void* a, const void* b, hipStream_t stream);
// int8 x int8 -> int32 on the same tiles (v_mfma_i32_16x16x64_i8)
int gemm_mfma_int8(const GemmProblem& p, const void* a, const void* b, void* c, hipStream_t stream);

}  // namespace th
