// gsx_wave.h - cross-lane helpers for 64-wide wavefronts (gfx950): DPP row permutes, the permlane swaps and the
// 16-component wave sum the backward rasterizers use.
#pragma once
#include "gsx_common.h"

namespace gsx {

// ---- cross-lane helpers -----------------------------------------------------------------------
// One halving step of a wave reduction: lanes of the lower half want lo_mine + lo_partner, lanes of the upper half
// want hi_mine + hi_partner.  v_permlane32_swap / v_permlane16_swap exchange the upper (odd-row) lanes of their first
// operand with the lower (even-row) lanes of the second, so swap(lo, hi) followed by one add is the whole step.
__device__ __forceinline__ float halve_swap32(float lo, float hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(f2u(lo), f2u(hi), false, false);
    return u2f(r[0]) + u2f(r[1]);
}
__device__ __forceinline__ float halve_swap16(float lo, float hi) {
    const auto r = __builtin_amdgcn_permlane16_swap(f2u(lo), f2u(hi), false, false);
    return u2f(r[0]) + u2f(r[1]);
}
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), CTRL, 0xf, 0xf, true));
}
static constexpr int kDppRowMirror = 0x140;     // lane i <-> 15 - i inside a row of 16
static constexpr int kDppHalfMirror = 0x141;    // lane i <-> 7 - i inside a half row of 8
static constexpr int kDppQuadXor1 = 0xB1;       // quad_perm [1,0,3,2]
static constexpr int kDppQuadXor2 = 0x4E;       // quad_perm [2,3,0,1]

// Sum of 16 values over the 64 lanes of a wave with a halving butterfly: 8 + 4 swap steps across the rows, then
// 2 + 1 mirror steps inside a row, then the quad.  On return lane L holds the wave total of component
// ((L>>5)&1)*8 + ((L>>4)&1)*4 + ((L>>3)&1)*2 + ((L>>2)&1).
__device__ __forceinline__ float wave_reduce16(float (&v)[16], uint32_t lane) {
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i)
        v[i] = halve_swap32(v[i], v[i + 8]);
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i)
        v[i] = halve_swap16(v[i], v[i + 4]);
    {
        const bool upper = (lane & 8u) != 0;
        const float a0 = v[0] + dpp<kDppRowMirror>(v[0]), b0 = v[2] + dpp<kDppRowMirror>(v[2]);
        const float a1 = v[1] + dpp<kDppRowMirror>(v[1]), b1 = v[3] + dpp<kDppRowMirror>(v[3]);
        v[0] = upper ? b0 : a0;
        v[1] = upper ? b1 : a1;
    }
    {
        const bool upper = (lane & 4u) != 0;
        const float a0 = v[0] + dpp<kDppHalfMirror>(v[0]), b0 = v[1] + dpp<kDppHalfMirror>(v[1]);
        v[0] = upper ? b0 : a0;
    }
    v[0] += dpp<kDppQuadXor2>(v[0]);
    v[0] += dpp<kDppQuadXor1>(v[0]);
    return v[0];
}


} // namespace gsx
