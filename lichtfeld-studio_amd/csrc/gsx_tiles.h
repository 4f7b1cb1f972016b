// gsx_tiles.h - the tile rectangle of a projected Gaussian and its packed form (device side; shared by intersect.hip
// and tile_lists.hip).
#pragma once
#include "gsx_common.h"

namespace gsx {

struct TileRect {
    uint32_t x0, y0, x1, y1;
};

// IntersectTile.cu:56-76.  The float -> uint32 conversions saturate (negative -> 0): that is what the
// reference's hardware conversion does, and plain C++ casts of negative floats are undefined.
__device__ __forceinline__ bool tile_rect_of(float2 m, int2 rad, float tile_size, uint32_t tile_width,
                                             uint32_t tile_height, TileRect* r) {
    const float radius_x = (float)rad.x, radius_y = (float)rad.y;
    if (radius_x <= 0 || radius_y <= 0)
        return false;
    const float tile_radius_x = radius_x / tile_size, tile_radius_y = radius_y / tile_size;
    const float tile_x = m.x / tile_size, tile_y = m.y / tile_size;
    r->x0 = min(sat_u32(gsx::floor(tile_x - tile_radius_x)), tile_width);
    r->y0 = min(sat_u32(gsx::floor(tile_y - tile_radius_y)), tile_height);
    r->x1 = min(sat_u32(gsx::ceil(tile_x + tile_radius_x)), tile_width);
    r->y1 = min(sat_u32(gsx::ceil(tile_y + tile_radius_y)), tile_height);
    return true;
}
__device__ __forceinline__ bool tile_rect(const float* __restrict__ means2d, const int32_t* __restrict__ radii,
                                          uint32_t idx, float tile_size, uint32_t tile_width, uint32_t tile_height,
                                          TileRect* r) {
    const int2 rad = reinterpret_cast<const int2*>(radii)[idx];
    if (rad.x <= 0 || rad.y <= 0)
        return false;
    return tile_rect_of(reinterpret_cast<const float2*>(means2d)[idx], rad, tile_size, tile_width, tile_height, r);
}

// Depth-ordered variant, one camera: the tile count rides in the high word of a sort key whose low word is the
// depth's bit pattern (what the low word of an intersection key holds; all ones for a Gaussian that touches no
// tile).  Sorting these N keys on their low 32 bits gives the visiting order AND the counts in that order.
// RECT (tile grids up to 255 x 255): the high word holds the tile rectangle x0 | y0 << 8 | x1 << 16 | y1 << 24
// instead (0 = no tile), from which both the count and the emission follow without going back to the Gaussian.
__device__ __forceinline__ uint32_t packed_rect_count(uint32_t hi) {
    return (((hi >> 24) & 255u) - ((hi >> 8) & 255u)) * (((hi >> 16) & 255u) - (hi & 255u));
}

// ---- visiting order of the tiles for the rasterizers: longest lists first -----------------------------------------
// The rasterizers' workgroups are handed out in launch order as slots free up; with the long lists first the short
// ones fill the end of the launch instead of a few long ones running on alone.  Counting sort on a logarithmic
// length class (16 classes per octave), descending; the order inside a class is whatever the atomics give (no
// result depends on the order tiles are visited in).
static constexpr uint32_t kLenClasses = 512;
__device__ __forceinline__ uint32_t tile_len_class(uint32_t len) {
    if (len == 0)
        return 0;
    const uint32_t e = 31u - (uint32_t)__clz((int)len);
    const uint32_t m = e >= 4 ? (len >> (e - 4)) & 15u : (len << (4 - e)) & 15u; // four bits below the leading one
    return min(e * 16u + m + 1u, kLenClasses - 1u);
}

// The whole sort by one workgroup of THREADS lanes (a multiple of 64, at most 1024); every lane of the workgroup
// calls it.  A tile's cost is tile_cost[tile], or with tile_cost == nullptr the length of its list in tile_offsets.
// cursor: LDS [kLenClasses], wave_total: LDS [16].
template <uint32_t THREADS>
__device__ __forceinline__ void tile_order_block(uint32_t n_tiles, uint32_t n_isects,
                                                 const int32_t* __restrict__ tile_offsets,
                                                 const uint32_t* __restrict__ tile_cost,
                                                 uint32_t* __restrict__ tile_order, uint32_t* cursor,
                                                 uint32_t* wave_total) {
    static_assert(THREADS % 64 == 0 && THREADS <= 1024 && kLenClasses % 64 == 0, "whole waves");
    const uint32_t t = threadIdx.x, lane = t & 63u, w = t >> 6;
    for (uint32_t c = t; c < kLenClasses; c += THREADS)
        cursor[c] = 0;
    __syncthreads();
    auto length = [&](uint32_t tile) {
        if (tile_cost != nullptr)
            return tile_cost[tile];
        const uint32_t end =
            (tile + 1 < n_tiles || n_isects == kCountInOffsets) ? (uint32_t)tile_offsets[tile + 1] : n_isects;
        return end - (uint32_t)tile_offsets[tile];
    };
    for (uint32_t tile = t; tile < n_tiles; tile += THREADS)
        atomicAdd(&cursor[tile_len_class(length(tile))], 1u);
    __syncthreads();
    // first position of every class, dearest class first: an exclusive scan over the classes in descending order,
    // THREADS classes at a time (virtual index v owns class kLenClasses - 1 - v)
    uint32_t carry = 0;
    for (uint32_t base = 0; base < kLenClasses; base += THREADS) {
        const uint32_t v = base + t;
        const uint32_t c = kLenClasses - 1u - v;
        const uint32_t n = v < kLenClasses ? cursor[c] : 0u;
        uint32_t incl = n;
#pragma unroll
        for (uint32_t off = 1; off < 64; off <<= 1) {
            const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
            if (lane >= off)
                incl += up;
        }
        if (lane == 63)
            wave_total[w] = incl;
        __syncthreads();
        uint32_t before = carry;
        for (uint32_t k = 0; k < w; ++k)
            before += wave_total[k];
        if (v < kLenClasses)
            cursor[c] = before + incl - n;
        for (uint32_t k = 0; k < THREADS / 64; ++k)
            carry += wave_total[k];
        __syncthreads();
    }
    for (uint32_t tile = t; tile < n_tiles; tile += THREADS)
        tile_order[atomicAdd(&cursor[tile_len_class(length(tile))], 1u)] = tile;
}

} // namespace gsx
