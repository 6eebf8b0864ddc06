// Moves and sums among the 16 lanes of a row of a wave (data-parallel moves between neighbouring
// lanes: no trip through LDS, which is what a shuffle costs).
#pragma once
#include "common.h"

// v of the lane `N` places further round its row of 16 lanes
template <int N>
__device__ __forceinline__ float row_rotated(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xf, 0xf, false));
}
// the sum over the 16 lanes of a row, in every lane
__device__ __forceinline__ float row_sum16(float v) {
    v += row_rotated<8>(v);
    v += row_rotated<4>(v);
    v += row_rotated<2>(v);
    v += row_rotated<1>(v);
    return v;
}
