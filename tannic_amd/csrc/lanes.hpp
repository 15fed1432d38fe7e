// Moving values between the 64 lanes of a wavefront, and the all-lanes fold built on it.
#pragma once

#include "common.hpp"

namespace th {

// ---- moving values between lanes -------------------------------------------
template <int CTRL>
__device__ inline uint32_t dpp32(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, false));
}

template <int CTRL, class T>
__device__ inline T dpp(T v) {
    // DPP moves 32-bit registers: narrower values ride in one
    constexpr size_t WORDS = (sizeof(T) + 3) / 4;
    uint32_t w[WORDS] = {};
    __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
    for (size_t i = 0; i < WORDS; ++i) w[i] = dpp32<CTRL>(w[i]);
    T r;
    __builtin_memcpy(&r, w, sizeof(T));
    return r;
}

template <class T>
__device__ inline T read_lane(T v, int lane) {
    constexpr size_t WORDS = (sizeof(T) + 3) / 4;
    uint32_t w[WORDS] = {};
    __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
    for (size_t i = 0; i < WORDS; ++i) w[i] = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(w[i]), lane));
    T r;
    __builtin_memcpy(&r, w, sizeof(T));
    return r;
}

// All 64 lanes -> one value, identical in every lane.  Four DPP steps fold
// each row of 16 lanes (quad swaps, half-row mirror, row mirror), the four row
// results are read out as scalars.
template <class Op, class A>
__device__ inline A wave_reduce(A v) {
    v = Op::combine(v, dpp<0xB1>(v));   // quad_perm [1,0,3,2]
    v = Op::combine(v, dpp<0x4E>(v));   // quad_perm [2,3,0,1]
    v = Op::combine(v, dpp<0x141>(v));  // row_half_mirror
    v = Op::combine(v, dpp<0x140>(v));  // row_mirror
    const A r0 = read_lane(v, 0), r1 = read_lane(v, 16), r2 = read_lane(v, 32), r3 = read_lane(v, 48);
    return Op::combine(Op::combine(r0, r1), Op::combine(r2, r3));
}

}  // namespace th
