// gsx_camera.h - the OpenCV fisheye and the equirectangular camera models of gsplat/Cameras.cuh:757-1037
// (host + device, no HIP dependency).  One source for the kernels and for the CPU checker: what pins it are the
// independent float64 models in tests/test_oracle_geometry.py (closed forms of the equidistant and the latitude /
// longitude mappings, numpy's polynomial roots for the field-of-view limit, round trips), not the kernel <-> checker
// comparison, which for these two models only shows that host and device builds agree bit for bit.
//
// The reference evaluates atan2 / sin / cos / cbrt with CUDA's fast-math library (and the equirectangular
// unprojection in double, through PI being used with double literals, Cameras.cuh:1027-1036); here everything is
// fp32 on the fixed primitives of gsx_math.h plus the three below.
#pragma once

#include "gsx_math.h"

namespace gsx {

// atan on [0, inf) (Cephes atanf: two range reductions, degree-4 odd polynomial in x^2)
GSX_HD float atan_pos(float x) {
    float y0 = 0.0f;
    if (x > 2.414213562373095f) { // tan(3 pi / 8)
        y0 = 1.57079632679489661923f;
        x = -1.0f / x;
    } else if (x > 0.4142135623730950f) { // tan(pi / 8)
        y0 = 0.78539816339744830962f;
        x = (x - 1.0f) / (x + 1.0f);
    }
    const float z = x * x;
    float p = 8.05374449538e-2f;
    p = fma(p, z, -1.38776856032e-1f);
    p = fma(p, z, 1.99777106478e-1f);
    p = fma(p, z, -3.33329491539e-1f);
    return y0 + fma(p * z, x, x);
}

// atan2 on the whole plane; atan2(0, 0) = 0
GSX_HD float atan2(float y, float x) {
    const float ax = gsx::fabs(x), ay = gsx::fabs(y);
    if (ax == 0.0f && ay == 0.0f)
        return 0.0f;
    float a = ay > ax ? 1.57079632679489661923f - atan_pos(ax / ay) : atan_pos(ay / ax);
    if (x < 0.0f)
        a = 3.14159265358979323846f - a;
    return y < 0.0f ? -a : a;
}

GSX_HD float asin(float x) { return 1.57079632679489661923f - gsx::acos(x); }

// cube root: exp(log|x| / 3) polished by two Newton steps
GSX_HD float cbrt(float x) {
    if (x == 0.0f)
        return 0.0f;
    const float a = gsx::fabs(x);
    float r = gsx::exp(gsx::log(a) * 0.33333333333333333f);
    r = r - (r * r * r - a) / (3.0f * r * r);
    r = r - (r * r * r - a) / (3.0f * r * r);
    return x < 0.0f ? -r : r;
}

static constexpr float kFloatMax = 3.402823466e+38f;

// ---- polynomials (Cameras.cuh:91-141, 169-211) ----
template <int N>
GSX_HD float poly_horner(const float (&c)[N], float x) {
    float y = 0.0f;
#pragma unroll
    for (int i = N - 1; i >= 0; --i)
        y = x * y + c[i];
    return y;
}
template <int N>
GSX_HD float poly_odd(const float (&c)[N], float x) { return x * poly_horner(c, x * x); }
template <int N>
GSX_HD float poly_even(const float (&c)[N], float x) { return poly_horner(c, x * x); }

// solve 1 + a x + b x^2 + c x^3 = 0 for its smallest positive root (Cameras.cuh:757-815); FLT_MAX if there is none
GSX_HD float fisheye_max_angle_sq(float a, float b, float c) {
    const float INF = kFloatMax;
    if (c == 0.0f) {
        if (b == 0.0f) {
            if (a >= 0.0f)
                return INF;
            return -1.0f / a;
        }
        float delta = a * a - 4.0f * b;
        if (delta >= 0.0f) {
            delta = gsx::sqrt(delta) - a;
            if (delta > 0.0f)
                return 2.0f / delta;
        }
    } else {
        const float boc = b / c;
        const float boc2 = boc * boc;
        const float t1 = (9.0f * a * boc - 2.0f * b * boc2 - 27.0f) / c;
        const float t2 = 3.0f * a / c - boc2;
        const float delta = t1 * t1 + 4.0f * t2 * t2 * t2;
        if (delta >= 0.0f) {
            const float d2 = gsx::sqrt(delta);
            const float cube_root = gsx::cbrt((d2 + t1) / 2.0f);
            if (cube_root != 0.0f) {
                const float soln = (cube_root - (t2 / cube_root) - boc) / 3.0f;
                if (soln > 0.0f)
                    return soln;
            }
        } else {
            // three real roots
            const float theta = gsx::atan2(gsx::sqrt(-delta), t1) / 3.0f;
            const float two_third_pi = 2.0f * 3.14159265358979323846f / 3.0f;
            const float t3 = 2.0f * gsx::sqrt(-t2);
            float soln = INF;
#pragma unroll
            for (int i = -1; i <= 1; ++i) {
                // the angles stay inside [-pi, pi]: theta in [0, pi/3]
                const float angle = theta + (float)i * two_third_pi;
                const float s = (t3 * gsx::cos(angle) - boc) / 3.0f;
                if (s > 0.0f)
                    soln = gsx::fmin(soln, s);
            }
            return soln;
        }
    }
    return INF;
}

// OpenCVFisheyeCameraModel (Cameras.cuh:817-1001)
struct Fisheye {
    float fx, fy, cx, cy, W, H;
    float fwd[5];    // theta + k1 theta^3 + ... as an odd polynomial
    float dfwd[5];   // its derivative as an even polynomial
    float approx[2]; // crude linear inverse: the Newton start
    float max_angle;
};

GSX_HD Fisheye fisheye_setup(const float* k /*4 radial coefficients, may be null*/, float fx, float fy, float cx,
                             float cy, uint32_t W, uint32_t H) {
    Fisheye f;
    f.fx = fx, f.fy = fy, f.cx = cx, f.cy = cy, f.W = (float)W, f.H = (float)H;
    const float k1 = k ? k[0] : 0.f, k2 = k ? k[1] : 0.f, k3 = k ? k[2] : 0.f, k4 = k ? k[3] : 0.f;
    f.fwd[0] = 1.f, f.fwd[1] = k1, f.fwd[2] = k2, f.fwd[3] = k3, f.fwd[4] = k4;
    f.dfwd[0] = 1.f, f.dfwd[1] = 3 * k1, f.dfwd[2] = 5 * k2, f.dfwd[3] = 7 * k3, f.dfwd[4] = 9 * k4;
    const float max_diag_x = gsx::fmax(f.W - cx, cx), max_diag_y = gsx::fmax(f.H - cy, cy);
    const float max_radius_pixels = gsx::sqrt(max_diag_x * max_diag_x + max_diag_y * max_diag_y);
    if (k4 == 0.f) {
        f.max_angle = gsx::sqrt(fisheye_max_angle_sq(3.f * k1, 5.f * k2, 7.f * k3));
    } else {
        // first positive zero of the derivative: Newton from 1.57 (Cameras.cuh:859-873)
        const float dd[4] = {6 * k1, 20 * k2, 42 * k3, 72 * k4};
        float x = 1.57f;
        bool converged = false;
        for (int j = 0; j < 20; ++j) {
            const float dfdx = poly_odd(dd, x);
            const float residual = poly_even(f.dfwd, x) - 0.f;
            const float dx = residual / dfdx;
            x -= dx;
            if (gsx::fabs(dx) < 1e-6f) {
                converged = true;
                break;
            }
        }
        f.max_angle = (!converged || x <= 0.f) ? kFloatMax : x;
    }
    f.max_angle = gsx::fmin(f.max_angle, gsx::fmax(max_radius_pixels / fx, max_radius_pixels / fy));
    const float max_normalized_dist = gsx::fmax(f.W / 2.f / fx, f.H / 2.f / fy);
    f.approx[0] = 0.f, f.approx[1] = f.max_angle / max_normalized_dist;
    return f;
}

GSX_HD bool in_image_margin(float x, float y, float W, float H, float margin_factor) { // Cameras.cuh:228-240
    const float mx = W * margin_factor, my = H * margin_factor;
    bool valid = true;
    valid &= (-mx) <= x && x < (W + mx);
    valid &= (-my) <= y && y < (H + my);
    return valid;
}

// camera_ray_to_image_point (Cameras.cuh:894-959)
GSX_HD bool fisheye_project(const Fisheye& f, vec3 cam, float margin_factor, vec2* out) {
    out->x = 0.f, out->y = 0.f;
    if (cam.z <= 0.f)
        return false;
    // numerically_stable_norm2 (:77-89)
    const float abs_x = gsx::fabs(cam.x), abs_y = gsx::fabs(cam.y);
    const float mn = gsx::fmin(abs_x, abs_y), mx = gsx::fmax(abs_x, abs_y);
    float norm = 0.f;
    if (mx > 0.f) {
        const float ratio = mn / mx;
        norm = mx * gsx::sqrt(1.f + ratio * ratio);
    }
    if (norm <= 0.f)
        norm = 1.1920928955078125e-7f; // FLT_EPSILON
    const float theta_full = gsx::atan2(norm, cam.z);
    const float theta = theta_full < f.max_angle ? theta_full : f.max_angle;
    const float delta = poly_odd(f.fwd, theta) / norm;
    if (delta <= 0.f)
        return false;
    out->x = f.fx * delta * cam.x + f.cx;
    out->y = f.fy * delta * cam.y + f.cy;
    bool valid = in_image_margin(out->x, out->y, f.W, f.H, margin_factor);
    // Cameras.cuh:953-955 tests "theta <= max_angle", which the clamp above makes always true: points beyond the
    // field of view are clamped onto its rim and stay valid, as in the reference
    valid &= theta <= f.max_angle;
    return valid;
}

// image_point_to_camera_ray (Cameras.cuh:961-1000); false = invalid ray
GSX_HD bool fisheye_unproject(const Fisheye& f, float px, float py, vec3* ray) {
    const float u = (px - f.cx) / f.fx, v = (py - f.cy) / f.fy;
    const float delta = gsx::sqrt(u * u + v * v);
    float x = poly_horner(f.approx, delta);
    bool converged = false;
    for (int j = 0; j < 20; ++j) {
        const float dfdx = poly_even(f.dfwd, x);
        const float residual = poly_odd(f.fwd, x) - delta;
        const float dx = residual / dfdx;
        x -= dx;
        if (gsx::fabs(dx) < 1e-6f) {
            converged = true;
            break;
        }
    }
    const float theta = x;
    ray->x = 0.f, ray->y = 0.f, ray->z = 1.f;
    if (theta < 0.f || theta >= f.max_angle || !converged)
        return false;
    if (delta >= 1e-6f) {
        // gsx::sin / cos cover [-pi, pi]; a field-of-view limit beyond pi (possible only with coefficients no lens
        // has) is folded back by one period
        const float th = theta > 3.14159265358979323846f ? theta - 2.0f * 3.14159265358979323846f : theta;
        const float scale_factor = gsx::sin(th) / delta;
        ray->x = scale_factor * u, ray->y = scale_factor * v, ray->z = gsx::cos(th);
    }
    return true;
}

// EquirectangularCameraModel (Cameras.cuh:1003-1037): always valid
GSX_HD void equirect_project(float W, float H, vec3 cam, vec2* out) {
    const float azimuth = gsx::atan2(cam.x, cam.z);
    const float len = gsx::sqrt(cam.x * cam.x + cam.y * cam.y + cam.z * cam.z);
    const float elevation = gsx::asin(cam.y / len);
    out->x = (azimuth / (2.0f * 3.14159265358979323846f) + 0.5f) * W;
    out->y = (elevation / 3.14159265358979323846f + 0.5f) * H;
}

GSX_HD void equirect_unproject(float W, float H, float px, float py, vec3* ray) {
    const float azimuth = 2.0f * 3.14159265358979323846f * (px / W - 0.5f);
    const float elevation = 3.14159265358979323846f * (py / H - 0.5f);
    const float ce = gsx::cos(elevation);
    const float dx = ce * gsx::sin(azimuth), dy = gsx::sin(elevation), dz = gsx::cos(azimuth) * ce;
    const float len = gsx::sqrt(dx * dx + dy * dy + dz * dz);
    ray->x = dx / len, ray->y = dy / len, ray->z = dz / len;
}

// ---- unscented transform through a perfect pinhole under one rigid pose (the training camera) ----
// The reference rotates each of the seven world-space sigma points by the pose's quaternion and divides twice per
// point (Cameras.cuh:1070-1119, 362-369, 431-455).  The same points, formed where they are used: the mean goes
// through the pose once, each of the three scaled axes through its rotation matrix once, and the points are
// mean_c +- axis_c; the perspective division is one reciprocal per point.  Mathematically the same map (rotation is
// linear), ~40 % of the instructions; pinned by the float64 unscented-transform model of
// tests/test_oracle_geometry.py, shared by the kernels and the CPU checker.
//   Rc, t : rotation matrix and translation of the pose;  Rg : rotation matrix of the Gaussian (mat3_cast);
//   sq    : sqrt(3 + lambda);  out[0] = mean, out[1..3] = mean + axis, out[4..6] = mean - axis (camera coordinates)
GSX_HD void ut_sigma_points_camera(const mat3& Rc, vec3 t, vec3 mean, const mat3& Rg, vec3 scl, float sq,
                                   vec3 (&out)[7]) {
    out[0] = add(mul(Rc, mean), t);
    const float sc[3] = {scl.x, scl.y, scl.z};
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
#endif
    for (int a = 0; a < 3; ++a) {
        const float s = sq * sc[a];
        const vec3 axis_c = mul(Rc, mk3(s * Rg.m[0][a], s * Rg.m[1][a], s * Rg.m[2][a]));
        out[a + 1] = add(out[0], axis_c);
        out[a + 4] = sub(out[0], axis_c);
    }
}

// camera_ray_to_image_point of the perfect pinhole (Cameras.cuh:431-455) with one reciprocal: invalid behind the
// camera, valid inside the image grown by margin_factor on every side
GSX_HD bool pinhole_project_point(vec3 pc, float fx, float fy, float cx, float cy, float W, float H,
                                  float margin_factor, vec2* out) {
    out->x = 0.f;
    out->y = 0.f;
    if (pc.z <= 0.f)
        return false;
    const float iz = 1.0f / pc.z;
    out->x = fma(pc.x * iz, fx, cx);
    out->y = fma(pc.y * iz, fy, cy);
    return in_image_margin(out->x, out->y, W, H, margin_factor);
}

} // namespace gsx
