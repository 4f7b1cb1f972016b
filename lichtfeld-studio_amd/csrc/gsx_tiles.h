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

} // namespace gsx
