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


// ---- the same butterfly for 13 and for 9 values ------------------------------------------------------------------
// With fewer than 16 values some components of the butterfly do not exist.  A step whose partner component is missing
// still needs its swap (the lower lanes want the upper lanes' share), but its second operand can be any value the
// caller no longer needs - here the register the previous swap has just handed back - instead of a fresh zero; the
// lanes that would own the missing component then hold a meaningless sum, and wave_reduce*_index tells them so.
// A pair of components that are both missing costs nothing.
struct Halved {
    float sum, spare;
};
__device__ __forceinline__ Halved halve32(float lo, float hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(f2u(lo), f2u(hi), false, false);
    return {u2f(r[0]) + u2f(r[1]), u2f(r[1])};
}
__device__ __forceinline__ Halved halve16(float lo, float hi) {
    const auto r = __builtin_amdgcn_permlane16_swap(f2u(lo), f2u(hi), false, false);
    return {u2f(r[0]) + u2f(r[1]), u2f(r[1])};
}
__device__ __forceinline__ float reduce_rows(float v0, float v1, uint32_t lane) { // last pair of components + the quad
    const float a = v0 + dpp<kDppHalfMirror>(v0), b = v1 + dpp<kDppHalfMirror>(v1);
    float v = (lane & 4u) != 0 ? b : a;
    v += dpp<kDppQuadXor2>(v);
    v += dpp<kDppQuadXor1>(v);
    return v;
}
// Which of the N values lane L holds the wave total of (lanes with L & 3 == 0 are the ones that use it), or 15: none.
// Components as in wave_reduce16; 13 values sit in components 0-6 and 8-13, 9 values in 0, 1, 2, 4, 5, 8, 9, 10, 12.
__device__ __forceinline__ uint32_t wave_component(uint32_t lane) {
    return ((lane >> 5) & 1u) * 8u + ((lane >> 4) & 1u) * 4u + ((lane >> 3) & 1u) * 2u + ((lane >> 2) & 1u);
}
__device__ __forceinline__ uint32_t wave_reduce13_index(uint32_t lane) {
    return (uint32_t)(0xFFCBA987F6543210ull >> (4u * wave_component(lane))) & 15u;
}
__device__ __forceinline__ uint32_t wave_reduce9_index(uint32_t lane) {
    return (uint32_t)(0xFFF7F654FF83F210ull >> (4u * wave_component(lane))) & 15u;
}
// 7 + 4 swap steps, then as wave_reduce16: 34 instructions instead of 39 (no zeros to make, one pair fewer).
__device__ __forceinline__ float wave_reduce13(const float (&a)[13], uint32_t lane) {
    const Halved s0 = halve32(a[0], a[7]), s1 = halve32(a[1], a[8]), s2 = halve32(a[2], a[9]);
    const Halved s3 = halve32(a[3], a[10]), s4 = halve32(a[4], a[11]), s5 = halve32(a[5], a[12]);
    const Halved s6 = halve32(a[6], s5.spare);
    const Halved t0 = halve16(s0.sum, s4.sum), t1 = halve16(s1.sum, s5.sum), t2 = halve16(s2.sum, s6.sum);
    const Halved t3 = halve16(s3.sum, t2.spare);
    const bool upper = (lane & 8u) != 0;
    const float a0 = t0.sum + dpp<kDppRowMirror>(t0.sum), b0 = t2.sum + dpp<kDppRowMirror>(t2.sum);
    const float a1 = t1.sum + dpp<kDppRowMirror>(t1.sum), b1 = t3.sum + dpp<kDppRowMirror>(t3.sum);
    return reduce_rows(upper ? b0 : a0, upper ? b1 : a1, lane);
}
// 5 + 3 swap steps and three mirror steps: 26 instructions.
__device__ __forceinline__ float wave_reduce9(const float (&a)[9], uint32_t lane) {
    const Halved s0 = halve32(a[0], a[4]), s1 = halve32(a[1], a[5]), s2 = halve32(a[2], a[6]);
    const Halved s4 = halve32(a[3], a[7]);
    const Halved s5 = halve32(a[8], s4.spare);
    const Halved t0 = halve16(s0.sum, s4.sum), t1 = halve16(s1.sum, s5.sum);
    const Halved t2 = halve16(s2.sum, t1.spare);
    const float a0 = t0.sum + dpp<kDppRowMirror>(t0.sum), b0 = t2.sum + dpp<kDppRowMirror>(t2.sum);
    const float a1 = t1.sum + dpp<kDppRowMirror>(t1.sum);
    return reduce_rows((lane & 8u) != 0 ? b0 : a0, a1, lane);
}

} // namespace gsx
