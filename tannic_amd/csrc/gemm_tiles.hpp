// Pieces shared by the MFMA matrix-multiply kernels: fragment types, the MFMA wrappers, the tile-to-workgroup
// mapping and the swizzled LDS tile layout.
#pragma once

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

// A tile row is 128 bytes = eight 16-byte chunks for every element type.
template <class T> constexpr int kBKof = 128 / sizeof(T);      // K elements per step: 64 (16-bit), 32 (fp32)
template <class T> constexpr int kChunkOf = 16 / sizeof(T);    // elements per 16-byte chunk
template <> struct Mfma16<float> {
    // element e of both fragments is one k: four 32x32x2 MFMAs (lanes 0-31 hold one k of the pair, lanes 32-63 the other)
    __device__ static inline float16v run(uint4v a, uint4v b, float16v c) {
        float x[4], y[4];
        __builtin_memcpy(x, &a, 16);
        __builtin_memcpy(y, &b, 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(x[e], y[e], c, 0, 0, 0);
        return c;
    }
};

constexpr int kBK = 64;          // K granule the host splits by (a multiple of every type's step)

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
// Calls f(std::integral_constant<int, 0>{}) ... f(std::integral_constant<int, N-1>{}).
template <int N, class F, int I = 0>
__device__ inline void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, F, I + 1>(static_cast<F&&>(f));
    }
}

// Swizzled element offset of (row, chunk) inside a [ROWS][128 bytes] tile.
// LDS serves 16 lanes of a 16-byte read per clock out of a 256-byte bank window,
// i.e. two 128-byte rows: consecutive row PAIRS get different chunk rotations so
// that 16 consecutive rows of one logical chunk land in 16 different slots.
template <class T> __device__ inline uint32_t tile_offset(uint32_t row, uint32_t chunk) { return row * kBKof<T> + ((chunk ^ ((row >> 1) & 7u)) * kChunkOf<T>); }


// Where a block of a split product leaves its share: fp32, [split][batch][M][N].
struct SplitK {
    uint32_t splits, k_chunk;    // blocks per tile; K elements per block, a multiple of kBK
    float* partials;
};

}  // namespace th
