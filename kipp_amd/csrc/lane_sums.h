// Sums over a few lanes that stand side by side in a wave, without a trip through LDS.
#pragma once
#include "common.h"

// v + the v of the lane whose number differs in one bit, for bits 0 to 3 by the data-parallel moves inside a row of 16
// lanes (no trip through LDS): neighbours in a quad, the other pair of a quad, the other quad of a half row (a mirror
// inside 8 lanes, where every lane of a quad already holds the quad's sum), the other half row (a mirror inside 16).
template <int STEP>
__device__ __forceinline__ float lane_pair_sum(float v) {
    constexpr int ctrl = STEP == 1 ? 0xB1 : (STEP == 2 ? 0x4E : (STEP == 4 ? 0x141 : 0x140));
    if constexpr (STEP <= 8) return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), ctrl, 0xF, 0xF, true));
    else return v + __shfl_xor(v, STEP, KIPP_WAVE);
}

// The sum over the PARTS lanes of a column, in every one of them: pairs, pairs of pairs, ...
template <int PARTS>
__device__ __forceinline__ float column_sum(float v) {
    if constexpr (PARTS >= 2) v = lane_pair_sum<1>(v);
    if constexpr (PARTS >= 4) v = lane_pair_sum<2>(v);
    if constexpr (PARTS >= 8) v = lane_pair_sum<4>(v);
    if constexpr (PARTS >= 16) v = lane_pair_sum<8>(v);
    if constexpr (PARTS >= 32) v = lane_pair_sum<16>(v);
    if constexpr (PARTS >= 64) v = lane_pair_sum<32>(v);
    return v;
}
