// gsx_record.h - the per-Gaussian record the tile rasterizers stage (host + device, no HIP dependency).
//
// For one global-shutter pinhole camera everything a (pixel, Gaussian) pair needs from the Gaussian is
//   M   = diag(1/scale) R(quat)^T            (RasterizeToPixelsFromWorld3DGSFwd.cu:214-226)
//   gro = M (ray_o - mean)                   (ray_o = camera centre, one per camera)
//   opacity, colour
// so it is built once per Gaussian (not once per tile the Gaussian touches) and kept as 96 bytes:
//   f4[0] = gro.xyz, opacity   f4[1] = M00 M01 M02 M10   f4[2] = M11 M12 M20 M21   f4[3] = M22, c0, c1, c2
//   f4[4] = jmin | jmax << 16, imin | imax << 16 (inclusive pixel-index bounds), power cut-off, A00
//   f4[5] = A01, A11, centre x, centre y     (pixel-space ellipse (p - c)^T A (p - c) <= 1)
// The last eight words describe where the pair can reach alpha >= 1/255 at all; the rasterizers use them to skip
// work whose result the reference discards anyway (alpha < 1/255 => `continue`), so they change no output.
//
// The region.  A pixel contributes iff alpha = min(0.999, o exp(-d^2 / 2)) >= 1/255, d = distance from the
// whitened-space origin to the pixel's ray, i.e. iff d^2 <= k = 2 ln(255 o) (power >= -k/2: the cut-off).  All
// rays start at gro, so {d^2 <= k} is the exact perspective silhouette of an ellipsoid: a conic in the image
// plane.  With B = M R_cw, (x0, y0, 1) the camera-space direction of the mean (depth z) and delta the offset from
// it, the whitened ray is -gro/z + B (delta, 0), which removes the large common component analytically:
//   |g^ x v|^2 <= (k/|g|^2) |v - gro/z|^2,   v = b1 dx + b2 dy,   g^ = gro/|gro|
// a 2x2 quadratic form: an ellipse with closed-form centre, extent and axis-aligned bounding box.  k is inflated
// for the rounding of the in-kernel evaluation of d^2 (whose absolute error grows with |gro|), the ellipse by
// 0.4 %, the bounding box by one pixel and the tested rectangles by a quarter, so the region is a superset of the
// contributing pixels; anything that is not a proper, well-conditioned ellipse (camera inside the k-ellipsoid,
// hyperbolic or nearly parabolic silhouette, non-finite numbers) falls back to "everywhere".
#pragma once

#include "gsx_math.h"

namespace gsx {

static constexpr uint32_t kRecordFloats = 24; // 96 bytes
static constexpr uint32_t kRecordF4 = 6;
static constexpr float kLogAlphaInv = 5.5412635f; // ln 255
static constexpr float kBlockMargin = 0.25f;        // pixels added around a block's pixel centres in the region test
static constexpr float kPowerFloor = -80.0f;      // no cut-off is below this: exp_nonpos stays in its domain

struct RecordRegion {
    int32_t jmin, imin, jmax, imax; // inclusive pixel-index bounds; empty when jmin > jmax
    float cut;                      // pairs with power < cut have alpha < 1/255
    float a00, a01, a11, pcx, pcy;  // (p - pc)^T A (p - pc) <= 1 in pixel coordinates; A = 0: everywhere
};

// viewmat: row-major [4,4] world->camera.  gro / M as stored in the record.
// pinhole = false (a distorted camera: straight lines of rays are not straight lines of pixels): only the power
// cut-off is claimed, the pixel region is "everywhere".
GSX_HD RecordRegion record_region(vec3 gro, const mat3& M, float opacity, vec3 mean, const float* viewmat, float fx,
                                  float fy, float cx, float cy, uint32_t W, uint32_t H, bool pinhole = true) {
    RecordRegion full = {0, 0, (int32_t)W - 1, (int32_t)H - 1, kPowerFloor, 0.f, 0.f, 0.f, 0.f, 0.f};
    RecordRegion empty = {1, 1, 0, 0, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (!(opacity > 0.f))
        return (opacity == opacity) ? empty : full; // NaN: no claim
    // k = 2 ln(255 o)
    float k = 2.0f * (kLogAlphaInv + gsx::log(opacity));
    if (!(k == k) || !(k < 150.f))
        return full;
    if (k < -1e-3f)
        return empty; // o clearly below 1/255: alpha never reaches the threshold
    k = gsx::fmax(k, 0.f);
    // the cut-off is compared with the power the kernel itself computes, so it only needs room for the rounding of
    // exp and log: o exp(cut) < 1/255 by 0.4 %
    full.cut = gsx::fmax(fma(-0.5f, k, -0.004f), kPowerFloor);
    if (!pinhole)
        return full;
    // the geometric region is derived in exact arithmetic: inflate k for the rounding of the kernel's d^2
    const float g2 = dot(gro, gro);
    k = fma(k, 1.002f, 0.004f) + 4e-6f * gsx::sqrt(g2 * k);
    if (!(k == k) || !(g2 == g2))
        return full;
    // camera-space mean
    const vec3 r0 = mk3(viewmat[0], viewmat[1], viewmat[2]);
    const vec3 r1 = mk3(viewmat[4], viewmat[5], viewmat[6]);
    const vec3 r2 = mk3(viewmat[8], viewmat[9], viewmat[10]);
    const float z = dot(r2, mean) + viewmat[11];
    if (!(z > 1e-6f) || !(g2 > k * 1.05f))
        return full;
    const float x0 = (dot(r0, mean) + viewmat[3]) / z;
    const float y0 = (dot(r1, mean) + viewmat[7]) / z;
    // b1, b2: images of the camera x / y axes (world rows 0 / 1 of the view rotation) under M
    const vec3 b1 = mul(M, r0), b2 = mul(M, r1);
    const float inv_g = 1.0f / gsx::sqrt(g2);
    const vec3 gh = scale(gro, inv_g);
    const vec3 w1 = cross(gh, b1), w2 = cross(gh, b2);
    const float kap = k / g2;
    const float a00 = dot(w1, w1) - kap * dot(b1, b1);
    const float a01 = dot(w1, w2) - kap * dot(b1, b2);
    const float a11 = dot(w2, w2) - kap * dot(b2, b2);
    const float be0 = kap * dot(b1, gro) / z, be1 = kap * dot(b2, gro) / z;
    const float det = a00 * a11 - a01 * a01;
    if (!(det > 0.f) || !(a00 > 0.f) || !(a11 > 0.f))
        return full;
    // A thin ellipse lying diagonally, or a silhouette that is nearly a parabola (a needle reaching towards the
    // camera plane), leaves det as the small difference of two products, and the quadratic form of the block test as
    // a small sum of large terms: both carry the rounding of a00, a01, a11 multiplied by a00 a11 / det.  Drawn needles
    // show the form at contributing pixels growing by ~ratio x 2^-22: it uses up the 0.8 % margin at a ratio of 2^15.
    // Past 2^11 (an axis ratio of 90 at 45 degrees) no region is claimed.
    if (!(det * 2048.0f > a00 * a11))
        return full;
    const float inv_det = 1.0f / det;
    const float dcx = -(a11 * be0 - a01 * be1) * inv_det;
    const float dcy = -(a00 * be1 - a01 * be0) * inv_det;
    const float r2v = (a11 * be0 * be0 - 2.0f * a01 * be0 * be1 + a00 * be1 * be1) * inv_det + k / (z * z);
    if (!(r2v > 0.f))
        return full;
    const float hx = gsx::sqrt(r2v * a11 * inv_det), hy = gsx::sqrt(r2v * a00 * inv_det);
    const float px_c = fma(fx, x0 + dcx, cx), py_c = fma(fy, y0 + dcy, cy);
    const float rx = fma(fx * hx, 1.004f, 1.0f), ry = fma(fy * hy, 1.004f, 1.0f);
    // pixel centres j + 0.5 inside [c - r, c + r]
    const float jlo = gsx::ceil(px_c - rx - 0.5f), jhi = gsx::floor(px_c + rx - 0.5f);
    const float ilo = gsx::ceil(py_c - ry - 0.5f), ihi = gsx::floor(py_c + ry - 0.5f);
    if (!(jlo == jlo) || !(jhi == jhi) || !(ilo == ilo) || !(ihi == ihi) || !(rx < 1e9f) || !(ry < 1e9f))
        return full;
    if (jhi < 0.f || ihi < 0.f || jlo > (float)W - 1.f || ilo > (float)H - 1.f)
        return empty;
    RecordRegion b = full;
    b.jmin = (int32_t)gsx::fmax(jlo, 0.f);
    b.imin = (int32_t)gsx::fmax(ilo, 0.f);
    b.jmax = (int32_t)gsx::fmin(jhi, (float)W - 1.f);
    b.imax = (int32_t)gsx::fmin(ihi, (float)H - 1.f);
    // the ellipse in pixel units, grown by 0.4 %: (p - pc)^T A (p - pc) <= 1
    const float sc = 1.0f / (r2v * 1.008016f);
    const float e00 = a00 * sc / (fx * fx), e01 = a01 * sc / (fx * fy), e11 = a11 * sc / (fy * fy);
    if (e00 == e00 && e01 == e01 && e11 == e11 && e00 < 1e30f && e11 < 1e30f && e00 > 0.f && e11 > 0.f) {
        b.a00 = e00, b.a01 = e01, b.a11 = e11;
        b.pcx = px_c, b.pcy = py_c;
    }
    return b;
}

// Can a pixel of the 8x8 block whose first pixel is (wi0, wj0) contribute?  Bounding box first, then the
// minimum of the ellipse's quadratic form over the block's rectangle of pixel centres grown by a quarter pixel
// (the brute-force comparison with every pixel finds no miss with no growth at all).
GSX_HD bool record_region_hits_block(int32_t jmin, int32_t imin, int32_t jmax, int32_t imax, float a00, float a01,
                                     float a11, float pcx, float pcy, int32_t wi0, int32_t wj0) {
    if (!(jmin <= wj0 + 7 && jmax >= wj0 && imin <= wi0 + 7 && imax >= wi0))
        return false;
    // rectangle relative to the ellipse centre
    const float x0 = ((float)wj0 + 0.5f - kBlockMargin) - pcx, x1 = ((float)wj0 + 7.5f + kBlockMargin) - pcx;
    const float y0 = ((float)wi0 + 0.5f - kBlockMargin) - pcy, y1 = ((float)wi0 + 7.5f + kBlockMargin) - pcy;
    if (x0 <= 0.f && x1 >= 0.f && y0 <= 0.f && y1 >= 0.f)
        return true; // centre inside
    // minimum of q over the four edges (q is convex, its unconstrained minimum lies outside the rectangle).  Where
    // along an edge the minimum lies needs no more than an approximate quotient: q is stationary there, so an error
    // of one unit in the last place in the position changes q by its square, far inside the ellipse's 0.4 % margin
    const float r11 = gsx::rcp_approx(a11), r00 = gsx::rcp_approx(a00);
    float qmin = 3.0e38f;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const float x = e ? x1 : x0;
        float y = -(a01 * x) * r11; // minimiser along the vertical edge
        y = gsx::fmin(gsx::fmax(y, y0), y1);
        qmin = gsx::fmin(qmin, fma(a11 * y, y, fma(2.0f * a01 * x, y, a00 * x * x)));
        const float yy = e ? y1 : y0;
        float xx = -(a01 * yy) * r00; // along the horizontal edge
        xx = gsx::fmin(gsx::fmax(xx, x0), x1);
        qmin = gsx::fmin(qmin, fma(a00 * xx, xx, fma(2.0f * a01 * xx, yy, a11 * yy * yy)));
    }
    return !(qmin > 1.0f); // NaN (A = 0: 0/0) counts as a hit
}

// M = diag(1/s) R(q)^T with the reference's operation order (reciprocal, then product)
GSX_HD mat3 record_whitening(quat q, vec3 s) {
    const mat3 R = quat_to_rotmat(q);
    const float is0 = 1.0f / s.x, is1 = 1.0f / s.y, is2 = 1.0f / s.z;
    mat3 M;
    M.m[0][0] = is0 * R.m[0][0], M.m[0][1] = is0 * R.m[1][0], M.m[0][2] = is0 * R.m[2][0];
    M.m[1][0] = is1 * R.m[0][1], M.m[1][1] = is1 * R.m[1][1], M.m[1][2] = is1 * R.m[2][1];
    M.m[2][0] = is2 * R.m[0][2], M.m[2][1] = is2 * R.m[1][2], M.m[2][2] = is2 * R.m[2][2];
    return M;
}

} // namespace gsx
