// gsx_record.h - the per-Gaussian record the tile rasterizers stage (host + device, no HIP dependency).
//
// For one global-shutter pinhole camera everything a (pixel, Gaussian) pair needs from the Gaussian is
//   M   = diag(1/scale) R(quat)^T            (RasterizeToPixelsFromWorld3DGSFwd.cu:214-226)
//   gro = M (ray_o - mean)                   (ray_o = camera centre, one per camera)
//   opacity, colour
// so it is built once per Gaussian (not once per tile the Gaussian touches) and kept as 80 bytes:
//   f4[0] = gro.xyz, opacity   f4[1] = M00 M01 M02 M10   f4[2] = M11 M12 M20 M21   f4[3] = M22, c0, c1, c2
//   f4[4] = inclusive pixel-index bounds (jmin, imin, jmax, imax as int32 bit patterns) outside which the pair
//           cannot reach alpha >= 1/255.
//
// The bounds.  A pixel contributes iff alpha = min(0.999, o exp(-d^2 / 2)) >= 1/255, d = distance from the
// whitened-space origin to the pixel's ray, i.e. iff d^2 <= k = 2 ln(255 o).  All rays start at gro, so the set
// {d^2 <= k} is the exact perspective silhouette of an ellipsoid: a conic in the image plane.  With B = M R_cw,
// (x0, y0, 1) the camera-space direction of the mean (depth z) and delta the offset from it, the whitened ray is
// -gro/z + B (delta, 0), which removes the large common component analytically:
//   |g^ x v|^2 <= (k/|g|^2) |v - gro/z|^2,   v = b1 dx + b2 dy,   g^ = gro/|gro|
// a 2x2 quadratic form whose axis-aligned bounding box is closed-form.  k is inflated for the rounding of the
// in-kernel evaluation of d^2 (whose absolute error grows with |gro|) and the box by a pixel margin, so the box is
// a superset of the contributing pixels; anything that is not a proper ellipse (camera inside the k-ellipsoid,
// hyperbolic silhouette, non-finite numbers) falls back to the whole image.
#pragma once

#include "gsx_math.h"

namespace gsx {

static constexpr uint32_t kRecordFloats = 20; // 80 bytes
static constexpr float kLogAlphaInv = 5.5412635f; // ln 255

struct RecordBounds {
    int32_t jmin, imin, jmax, imax;
};

// viewmat: row-major [4,4] world->camera.  gro / M as stored in the record.  Returns inclusive pixel-index
// bounds clamped to the image; an empty box has jmin > jmax.
GSX_HD RecordBounds record_bounds(vec3 gro, const mat3& M, float opacity, vec3 mean, const float* viewmat, float fx,
                                  float fy, float cx, float cy, uint32_t W, uint32_t H) {
    RecordBounds full = {0, 0, (int32_t)W - 1, (int32_t)H - 1};
    RecordBounds empty = {1, 1, 0, 0};
    if (!(opacity > 0.f))
        return (opacity == opacity) ? empty : full; // NaN: no claim
    // k = 2 ln(255 o), at most 2 * 5.55 (the kernels' own exp-free cut-off), inflated for rounding
    float k = 2.0f * (kLogAlphaInv + gsx::log(opacity));
    if (!(k == k))
        return full;
    if (k < -1e-3f)
        return empty; // o clearly below 1/255: alpha never reaches the threshold
    k = gsx::fmin(gsx::fmax(k, 0.f), 11.1f);
    const float g2 = dot(gro, gro);
    k = fma(k, 1.002f, 0.004f) + 4e-6f * gsx::sqrt(g2 * k);
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
    RecordBounds b;
    b.jmin = (int32_t)gsx::fmax(jlo, 0.f);
    b.imin = (int32_t)gsx::fmax(ilo, 0.f);
    b.jmax = (int32_t)gsx::fmin(jhi, (float)W - 1.f);
    b.imax = (int32_t)gsx::fmin(ihi, (float)H - 1.f);
    return b;
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
