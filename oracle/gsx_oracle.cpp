// gsx_oracle.cpp - CPU restatement of the reference's 3DGUT training-step kernels.
//
// TEST INFRASTRUCTURE ONLY.  This file is the checker the GPU kernels are compared against; the
// shipped library never links, loads or calls it.  Only tests/, __graft_entry__.smoke() and the
// cpu_baseline leg of bench.py may use it.
//
// Each function follows one kernel of the reference (file:line given at the function), one
// "thread" at a time, in the reference's operation order and with its thresholds.  The reference
// is compiled with --use_fast_math and links glm, neither of which can be reproduced here, so
// the fast-math intrinsics (__expf, __logf, rsqrtf, __frcp_rn, powf) and the glm routines are
// replaced by the fixed fp32 primitives of gsx_math.h (pinned against libm / closed forms in
// tests/test_oracle_math.py).  Sums that the reference forms with atomics in unspecified order
// (backward gradients) are accumulated here in double so that the checker is the well-defined
// value the toleranced comparison is made against.
//
// Pinning status (tests/test_oracle_*.py): every function below is pinned by closed forms,
// brute force, an independent float64 numpy model or a library routine, except where its header
// comment says "parity unpinned".
//
// Build: g++ -O2 -march=x86-64-v3 -ffp-contract=off -fopenmp -shared -fPIC (oracle/build.py).

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <numeric>
#include <vector>

#include "gsx_math.h"
#include "gsx_camera.h"

#if defined(_OPENMP)
#include <omp.h>
#endif

using gsx::mat3;
using gsx::quat;
using gsx::vec2;
using gsx::vec3;

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

constexpr float kAlphaThreshold = 1.f / 255.f; // gsplat/Common.h:54

// ---------------------------------------------------------------------------------------------
// camera pose helpers (gsplat/Cameras.cuh:33-71, 253-280)
// ---------------------------------------------------------------------------------------------

struct ShutterPose {
    vec3 t;
    quat q;
};

struct RollingShutter {
    vec3 t_start, t_end;
    quat q_start, q_end;
};

// Rolling-shutter state of the one camera (set by orc_set_rolling_shutter; GLOBAL = 4 and no end pose by default):
// the operators' `rs_type` / `viewmats1` arguments (Ops.h:69-98), kept out of every signature.
int g_rs_type = 4;
bool g_has_end_pose = false;
float g_end_pose[16];
uint32_t g_W = 0, g_H = 0; // image size for the unprojections and the shutter time (set with the camera model)

// Cameras.cuh:39-70 : rotation part of the row-major [4,4] world->camera matrix as a quaternion.
RollingShutter make_rolling_shutter(const float* se3_start, const float* se3_end) {
    RollingShutter rs;
    mat3 R;
    for (int r = 0; r < 3; ++r)
        for (int c = 0; c < 3; ++c)
            R.m[r][c] = se3_start[r * 4 + c];
    rs.q_start = gsx::quat_cast(R);
    rs.t_start = gsx::mk3(se3_start[3], se3_start[7], se3_start[11]);
    if (se3_end == nullptr && g_has_end_pose)
        se3_end = g_end_pose;
    if (se3_end == nullptr) {
        rs.q_end = rs.q_start;
        rs.t_end = rs.t_start;
    } else {
        for (int r = 0; r < 3; ++r)
            for (int c = 0; c < 3; ++c)
                R.m[r][c] = se3_end[r * 4 + c];
        rs.q_end = gsx::quat_cast(R);
        rs.t_end = gsx::mk3(se3_end[3], se3_end[7], se3_end[11]);
    }
    return rs;
}

// Cameras.cuh:268-280
ShutterPose interpolate_shutter_pose(float rel, const RollingShutter& rs) {
    ShutterPose p;
    p.t.x = (1.f - rel) * rs.t_start.x + rel * rs.t_end.x;
    p.t.y = (1.f - rel) * rs.t_start.y + rel * rs.t_end.y;
    p.t.z = (1.f - rel) * rs.t_start.z + rel * rs.t_end.z;
    p.q = gsx::slerp(rs.q_start, rs.q_end, rel);
    return p;
}

// Cameras.cuh:293-320 : when a pixel is exposed, as a fraction of the frame time (0 for a global shutter)
float shutter_relative_frame_time(float x, float y, uint32_t W, uint32_t H) {
    switch (g_rs_type) {
    case 0: return gsx::floor(y) / (float)(H - 1);
    case 1: return gsx::floor(x) / (float)(W - 1);
    case 2: return ((float)H - gsx::ceil(y)) / (float)(H - 1);
    case 3: return ((float)W - gsx::ceil(x)) / (float)(W - 1);
    default: return 0.f;
    }
}

// Cameras.cuh:416-455 : perfect pinhole projection with the 10 % margin validity test (:228-240)
bool pinhole_project(vec3 cam, float fx, float fy, float cx, float cy, uint32_t W, uint32_t H,
                     float margin_factor, vec2* out) {
    out->x = 0.f;
    out->y = 0.f;
    if (cam.z <= 0.f)
        return false;
    out->x = (cam.x / cam.z) * fx + cx;
    out->y = (cam.y / cam.z) * fy + cy;
    const float mx = (float)W * margin_factor;
    const float my = (float)H * margin_factor;
    bool valid = true;
    valid &= (-mx) <= out->x && out->x < ((float)W + mx);
    valid &= (-my) <= out->y && out->y < ((float)H + my);
    return valid;
}

// OpenCV pinhole model with radial (6), tangential (2) and thin-prism (4) distortion (Cameras.cuh:473-815).  The
// coefficients are process-wide checker state set by orc_set_distortion (off = the perfect pinhole model): every
// function below that projects a point or casts a pixel ray consults it, like the reference's dispatch on
// "any coefficient pointer given" (ProjectionUT3DGSFused.cu:86-113, RasterizeToPixelsFromWorld3DGSFwd.cu:90-116).
struct Distortion {
    bool on = false;
    float k[6] = {0, 0, 0, 0, 0, 0}, p[2] = {0, 0}, s[4] = {0, 0, 0, 0};
};
Distortion g_dist;
// camera model (gsx_camera_model values): 0 pinhole (g_dist), 2 OpenCV fisheye (g_dist.k[0..3] = radial), 3
// equirectangular - the two latter through the model code shared with the kernels (gsx_camera.h)
int g_model = 0;
bool g_fisheye_has_coeffs = false;

// Cameras.cuh:504-533
void compute_distortion(const Distortion& d, float u, float v, float* icD, float* delta_x, float* delta_y) {
    const float uu = u * u, vv = v * v;
    const float r2 = uu + vv;
    const float a1 = 2.f * u * v;
    const float a2 = r2 + 2.f * uu;
    const float a3 = r2 + 2.f * vv;
    const float num = 1.f + r2 * (d.k[0] + r2 * (d.k[1] + r2 * d.k[2]));
    const float den = 1.f + r2 * (d.k[3] + r2 * (d.k[4] + r2 * d.k[5]));
    *icD = num / den;
    *delta_x = d.p[0] * a1 + d.p[1] * a2 + r2 * (d.s[0] + r2 * d.s[1]);
    *delta_y = d.p[0] * a3 + d.p[1] * a1 + r2 * (d.s[2] + r2 * d.s[3]);
}

// Cameras.cuh:535-597 : camera_ray_to_image_point of the distorted model
bool opencv_project(const Distortion& d, vec3 cam, float fx, float fy, float cx, float cy, uint32_t W, uint32_t H,
                    float margin_factor, vec2* out) {
    out->x = 0.f;
    out->y = 0.f;
    if (cam.z <= 0.f)
        return false;
    const float u = cam.x / cam.z, v = cam.y / cam.z;
    float icD, dx, dy;
    compute_distortion(d, u, v, &icD, &dx, &dy);
    const bool valid_radial = icD > 0.8f;
    out->x = (icD * u + dx) * fx + cx;
    out->y = (icD * v + dy) * fy + cy;
    const float mx = (float)W * margin_factor;
    const float my = (float)H * margin_factor;
    bool valid = valid_radial;
    valid &= (-mx) <= out->x && out->x < ((float)W + mx);
    valid &= (-my) <= out->y && out->y < ((float)H + my);
    return valid;
}

bool project_point(vec3 cam, float fx, float fy, float cx, float cy, uint32_t W, uint32_t H, float margin_factor,
                   vec2* out) {
    if (g_model == 2) {
        const gsx::Fisheye fe = gsx::fisheye_setup(g_fisheye_has_coeffs ? g_dist.k : nullptr, fx, fy, cx, cy, W, H);
        return gsx::fisheye_project(fe, cam, margin_factor, out);
    }
    if (g_model == 3) {
        gsx::equirect_project((float)W, (float)H, cam, out);
        return true;
    }
    return g_dist.on ? opencv_project(g_dist, cam, fx, fy, cx, cy, W, H, margin_factor, out)
                     : pinhole_project(cam, fx, fy, cx, cy, W, H, margin_factor, out);
}

// Cameras.cuh:346-414 world_point_to_image_point_shutter_pose: a global shutter projects under the start pose; a
// rolling shutter starts from the start-pose projection (the end-pose one if only that is valid; neither valid =
// invalid) and iterates 10 times "exposure time of the current image point -> pose -> projection", returning the
// last image point as valid.
bool project_world_point_shutter(vec3 world, const RollingShutter& rs, float fx, float fy, float cx, float cy,
                                 uint32_t W, uint32_t H, float margin_factor, vec2* out) {
    vec2 p_start;
    const bool valid_start = project_point(gsx::add(gsx::quat_rotate(rs.q_start, world), rs.t_start), fx, fy, cx,
                                           cy, W, H, margin_factor, &p_start);
    if (g_rs_type == 4) {
        *out = p_start;
        return valid_start;
    }
    vec2 p_end;
    const bool valid_end =
        project_point(gsx::add(gsx::quat_rotate(rs.q_end, world), rs.t_end), fx, fy, cx, cy, W, H, margin_factor, &p_end);
    vec2 prev;
    if (valid_start) {
        prev = p_start;
    } else if (valid_end) {
        prev = p_end;
    } else {
        *out = p_end;
        return false;
    }
    for (int j = 0; j < 10; ++j) {
        const ShutterPose pose = interpolate_shutter_pose(shutter_relative_frame_time(prev.x, prev.y, W, H), rs);
        vec2 p;
        project_point(gsx::add(gsx::quat_rotate(pose.q, world), pose.t), fx, fy, cx, cy, W, H, margin_factor, &p);
        prev = p;
    }
    *out = prev;
    return true;
}

// Cameras.cuh:635-740 : Newton undistortion (at most 5 steps, stop at |step| < 1e-6).  The reference's double
// literals make parts of the Jacobian double arithmetic; the expressions are kept as written there.
bool opencv_undistort_newton(const Distortion& d, float xd, float yd, float* xo, float* yo) {
    const float k1 = d.k[0], k2 = d.k[1], k3 = d.k[2], k4 = d.k[3], k5 = d.k[4], k6 = d.k[5];
    const float p1 = d.p[0], p2 = d.p[1], s1 = d.s[0], s2 = d.s[1], s3 = d.s[2], s4 = d.s[3];
    float x = xd, y = yd;
    const float eps = 1e-6f;
    bool converged = false;
    for (int iter = 0; iter < 5; ++iter) {
        const float r = x * x + y * y;
        const float r2 = r * r;
        const float alpha = 1.0f + r * (k1 + r * (k2 + r * k3));
        const float beta = 1.0f + r * (k4 + r * (k5 + r * k6));
        const float dd = alpha / beta;
        if (dd <= 0.f)
            break;
        const float fx = dd * x + 2 * p1 * x * y + p2 * (r + 2 * x * x) + s1 * r + s2 * r2 - xd;
        const float fy = dd * y + 2 * p2 * x * y + p1 * (r + 2 * y * y) + s3 * r + s4 * r2 - yd;
        const float alpha_r = k1 + r * (2.0 * k2 + r * (3.0 * k3));
        const float beta_r = k4 + r * (2.0 * k5 + r * (3.0 * k6));
        const float d_r = (alpha_r * beta - alpha * beta_r) / (beta * beta);
        const float d_x = 2.0 * x * d_r;
        const float d_y = 2.0 * y * d_r;
        float fx_x = dd + d_x * x + 2.0 * p1 * y + 6.0 * p2 * x;
        fx_x += 2.0 * x * (s1 + 2.0 * s2 * r);
        float fx_y = d_y * x + 2.0 * p1 * x + 2.0 * p2 * y;
        fx_y += 2.0 * y * (s1 + 2.0 * s2 * r);
        float fy_x = d_x * y + 2.0 * p2 * y + 2.0 * p1 * x;
        fy_x += 2.0 * x * (s3 + 2.0 * s4 * r);
        float fy_y = dd + d_y * y + 2.0 * p2 * x + 6.0 * p1 * y;
        fy_y += 2.0 * y * (s3 + 2.0 * s4 * r);
        const float det = fx_y * fy_x - fx_x * fy_y;
        if (gsx::fabs(det) < eps)
            break;
        const float dx = (fx * fy_y - fy * fx_y) / det;
        const float dy = (fy * fx_x - fx * fy_x) / det;
        x += dx;
        y += dy;
        if (gsx::fabs(dx) < eps && gsx::fabs(dy) < eps) {
            converged = true;
            break;
        }
    }
    *xo = x;
    *yo = y;
    return converged;
}

// Cameras.cuh:457-470 / 742-755 + 253-266 + 322-339 : pixel centre -> world ray under the pose of the pixel's
// exposure time (the start pose for a global shutter: shutter_relative_frame_time has no GLOBAL case).  Returns the ray's valid flag (false
// only when the undistortion did not converge; then the ray is zero, :330-333).
bool pixel_world_ray(float px, float py, float fx, float fy, float cx, float cy,
                     const RollingShutter& rs, vec3* ray_o, vec3* ray_d) {
    vec3 d_cam;
    bool ok = true;
    if (g_model == 2) {
        const gsx::Fisheye fe = gsx::fisheye_setup(g_fisheye_has_coeffs ? g_dist.k : nullptr, fx, fy, cx, cy, g_W, g_H);
        ok = gsx::fisheye_unproject(fe, px, py, &d_cam);
    } else if (g_model == 3) {
        gsx::equirect_unproject((float)g_W, (float)g_H, px, py, &d_cam);
    } else {
        float u = (px - cx) / fx;
        float v = (py - cy) / fy;
        if (g_dist.on)
            ok = opencv_undistort_newton(g_dist, u, v, &u, &v);
        const vec3 cr = gsx::mk3(u, v, 1.f);
        const float len = gsx::sqrt(gsx::dot(cr, cr));
        d_cam = gsx::mk3(cr.x / len, cr.y / len, cr.z / len);
    }
    if (!ok) {
        *ray_o = gsx::mk3(0.f, 0.f, 0.f);
        *ray_d = gsx::mk3(0.f, 0.f, 0.f);
        return false;
    }
    const ShutterPose pose = interpolate_shutter_pose(shutter_relative_frame_time(px, py, g_W, g_H), rs);
    const mat3 R_inv = gsx::mat3_cast(gsx::quat_inverse(pose.q));
    *ray_o = gsx::neg(gsx::mul(R_inv, pose.t));
    *ray_d = gsx::mul(R_inv, d_cam);
    return true;
}

// M = diag(1/scale) * R(quat)^T  (RasterizeToPixelsFromWorld3DGSFwd.cu:214-226)
mat3 iscl_rot(quat q, vec3 s) {
    const mat3 R = gsx::quat_to_rotmat(q);
    const float is[3] = {1.0f / s.x, 1.0f / s.y, 1.0f / s.z};
    mat3 M;
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j)
            M.m[i][j] = is[i] * R.m[j][i];
    return M;
}

inline vec3 ld3(const float* p, int64_t i) { return gsx::mk3(p[3 * i], p[3 * i + 1], p[3 * i + 2]); }
inline quat ld4(const float* p, int64_t i) {
    quat q;
    q.w = p[4 * i];
    q.x = p[4 * i + 1];
    q.y = p[4 * i + 2];
    q.z = p[4 * i + 3];
    return q;
}

} // namespace

// =============================================================================================
// k1  projection_ut_3dgs_fused   gsplat/ProjectionUT3DGSFused.cu:17-210, Cameras.cuh:1064-1186
// Perfect pinhole + global shutter only (the path LichtFeld's trainer takes).
// Entries of means2d/depths/conics for culled Gaussians are left untouched, as in the reference.
// =============================================================================================
ORC_API int orc_projection_ut_3dgs_fused(
    uint32_t C, uint32_t N, const float* means, const float* quats, const float* scales,
    const float* opacities /*nullable*/, const float* viewmats0, const float* Ks, uint32_t image_width,
    uint32_t image_height, float eps2d, float near_plane, float far_plane, float radius_clip,
    float ut_alpha, float ut_beta, float ut_kappa, float ut_margin, int ut_require_all, int32_t* radii,
    float* means2d, float* depths, float* conics, float* compensations /*nullable*/) {
#pragma omp parallel for schedule(static)
    for (int64_t idx = 0; idx < (int64_t)C * N; ++idx) {
        const uint32_t cid = idx / N, gid = idx % N;
        const vec3 mean = ld3(means, gid);
        const vec3 scale = ld3(scales, gid);
        quat q = gsx::quat_normalize(ld4(quats, gid));
        const float fx = Ks[cid * 9 + 0], fy = Ks[cid * 9 + 4];
        const float cx = Ks[cid * 9 + 2], cy = Ks[cid * 9 + 5];
        const RollingShutter rs = make_rolling_shutter(viewmats0 + cid * 16, nullptr);

        // :76-82 centre-of-shutter pose, near/far cull.  The trainer's camera (see `plain` below) has one pose for
        // the whole frame: its mean in camera coordinates is the first sigma point, taken through the pose's matrix.
        const bool plain = g_model == 0 && !g_dist.on && g_rs_type == 4 && !g_has_end_pose;
        const ShutterPose pose = interpolate_shutter_pose(0.5f, rs);
        const vec3 mean_c = plain ? gsx::add(gsx::mul(gsx::mat3_cast(rs.q_start), mean), rs.t_start)
                                  : gsx::add(gsx::quat_rotate(pose.q, mean), pose.t);
        if ((mean_c.z < near_plane && g_model != 3) || mean_c.z > far_plane) { // :78
            radii[idx * 2] = 0;
            radii[idx * 2 + 1] = 0;
            continue;
        }

        // Cameras.cuh:1070-1119 sigma points and weights
        const float D = 3.0f;
        const float lambda = ut_alpha * ut_alpha * (D + ut_kappa) - D;
        const mat3 Rg = gsx::mat3_cast(q);
        vec3 pts[7];
        float wm[7], wc[7];
        pts[0] = mean;
        const float sq = gsx::sqrt(D + lambda);
        const float sc[3] = {scale.x, scale.y, scale.z};
        for (int i = 0; i < 3; ++i) {
            const float s = sq * sc[i];
            const vec3 delta = gsx::mk3(s * Rg.m[0][i], s * Rg.m[1][i], s * Rg.m[2][i]);
            pts[i + 1] = gsx::add(mean, delta);
            pts[i + 4] = gsx::sub(mean, delta);
        }
        wm[0] = lambda / (D + lambda);
        wc[0] = lambda / (D + lambda) + (1.f - ut_alpha * ut_alpha + ut_beta);
        for (int i = 0; i < 6; ++i) {
            wm[i + 1] = 1.f / (2.f * (D + lambda));
            wc[i + 1] = 1.f / (2.f * (D + lambda));
        }

        // Cameras.cuh:1127-1185 push the sigma points through the camera (start pose, :362-369)
        bool valid = ut_require_all != 0;
        bool culled = false;
        vec2 ip[7];
        vec2 m2 = {0.f, 0.f};
        // The perfect pinhole under a global shutter (the trainer's camera) takes the sigma points through the start
        // pose as a 3x3 matrix - R (mean +- s r_a) = R mean +- R (s r_a), so one product per axis serves two points -
        // and projects with one reciprocal of z per point: the same real-valued function as the general route
        // below, rounded differently (each image point within a few ulp).  The kernels take the same two helpers
        // under the same condition.
        vec3 pts_c[7];
        if (plain)
            gsx::ut_sigma_points_camera(gsx::mat3_cast(rs.q_start), rs.t_start, mean, Rg, scale, sq, pts_c);
        for (int i = 0; i < 7; ++i) {
            vec2 p;
            const bool pv = plain ? gsx::pinhole_project_point(pts_c[i], fx, fy, cx, cy, (float)image_width,
                                                               (float)image_height, ut_margin, &p)
                                  : project_world_point_shutter(pts[i], rs, fx, fy, cx, cy, image_width,
                                                                image_height, ut_margin, &p);
            if (ut_require_all) {
                valid &= pv;
                if (!pv) {
                    culled = true;
                    break;
                }
            } else {
                valid |= pv;
            }
            ip[i] = p;
            m2.x += wm[i] * p.x;
            m2.y += wm[i] * p.y;
        }
        if (culled || !valid) {
            radii[idx * 2] = 0;
            radii[idx * 2 + 1] = 0;
            continue;
        }
        float c00 = 0.f, c01 = 0.f, c11 = 0.f;
        for (int i = 0; i < 7; ++i) {
            const float dx = ip[i].x - m2.x, dy = ip[i].y - m2.y;
            c00 += wc[i] * (dx * dx);
            c01 += wc[i] * (dx * dy);
            c11 += wc[i] * (dy * dy);
        }

        // Utils.cuh:171-179 add_blur
        const float det_orig = c00 * c11 - c01 * c01;
        c00 += eps2d;
        c11 += eps2d;
        const float det = c00 * c11 - c01 * c01;
        const float compensation = gsx::sqrt(gsx::fmax(0.f, det_orig / det));
        if (det <= 0.f) {
            radii[idx * 2] = 0;
            radii[idx * 2 + 1] = 0;
            continue;
        }
        // :159 glm::inverse(mat2)
        const float ood = 1.0f / det;
        const float i00 = c11 * ood, i01 = -c01 * ood, i11 = c00 * ood;

        float extend = 3.33f;
        if (opacities != nullptr) {
            float opacity = opacities[gid];
            opacity *= compensation;
            if (opacity < kAlphaThreshold) {
                radii[idx * 2] = 0;
                radii[idx * 2 + 1] = 0;
                continue;
            }
            extend = gsx::fmin(extend, gsx::sqrt(2.0f * gsx::log(opacity / kAlphaThreshold)));
        }
        const float b = 0.5f * (c00 + c11);
        const float tmp = gsx::sqrt(gsx::fmax(0.01f, b * b - det));
        const float v1 = b + tmp;
        const float r1 = extend * gsx::sqrt(v1);
        const float radius_x = gsx::ceil(gsx::fmin(extend * gsx::sqrt(c00), r1));
        const float radius_y = gsx::ceil(gsx::fmin(extend * gsx::sqrt(c11), r1));
        if (radius_x <= radius_clip && radius_y <= radius_clip) {
            radii[idx * 2] = 0;
            radii[idx * 2 + 1] = 0;
            continue;
        }
        if (m2.x + radius_x <= 0 || m2.x - radius_x >= (float)image_width || m2.y + radius_y <= 0 ||
            m2.y - radius_y >= (float)image_height) {
            radii[idx * 2] = 0;
            radii[idx * 2 + 1] = 0;
            continue;
        }
        radii[idx * 2] = (int32_t)radius_x;
        radii[idx * 2 + 1] = (int32_t)radius_y;
        means2d[idx * 2] = m2.x;
        means2d[idx * 2 + 1] = m2.y;
        depths[idx] = mean_c.z;
        conics[idx * 3] = i00;
        conics[idx * 3 + 1] = i01;
        conics[idx * 3 + 2] = i11;
        if (compensations != nullptr)
            compensations[idx] = compensation;
    }
    return 0;
}

// =============================================================================================
// k2/k3  spherical harmonics   gsplat/SphericalHarmonicsCUDA.cu:20-110 (fwd), :112-371 (vjp)
// One (element, channel) per reference thread.  degree <= 4, K >= (degree+1)^2.
// Masked-out elements are left untouched (fwd) / left at the caller's zero fill (bwd).
// =============================================================================================
namespace {

// the basis values pSH_k(dir) exactly as formed in sh_coeffs_to_color_fast (:29-104)
int sh_basis(uint32_t degree, vec3 dir, float* B /*[25]*/) {
    B[0] = 0.2820947917738781f;
    if (degree < 1)
        return 1;
    const float inorm = gsx::rsqrt(dir.x * dir.x + dir.y * dir.y + dir.z * dir.z);
    const float x = dir.x * inorm, y = dir.y * inorm, z = dir.z * inorm;
    B[1] = -0.48860251190292f * y;
    B[2] = 0.48860251190292f * z;
    B[3] = -0.48860251190292f * x;
    if (degree < 2)
        return 4;
    const float z2 = z * z;
    const float fTmp0B = -1.092548430592079f * z;
    const float fC1 = x * x - y * y;
    const float fS1 = 2.f * x * y;
    B[6] = (0.9461746957575601f * z2 - 0.3153915652525201f);
    B[7] = fTmp0B * x;
    B[5] = fTmp0B * y;
    B[8] = 0.5462742152960395f * fC1;
    B[4] = 0.5462742152960395f * fS1;
    if (degree < 3)
        return 9;
    const float fTmp0C = -2.285228997322329f * z2 + 0.4570457994644658f;
    const float fTmp1B = 1.445305721320277f * z;
    const float fC2 = x * fC1 - y * fS1;
    const float fS2 = x * fS1 + y * fC1;
    B[12] = z * (1.865881662950577f * z2 - 1.119528997770346f);
    B[13] = fTmp0C * x;
    B[11] = fTmp0C * y;
    B[14] = fTmp1B * fC1;
    B[10] = fTmp1B * fS1;
    B[15] = -0.5900435899266435f * fC2;
    B[9] = -0.5900435899266435f * fS2;
    if (degree < 4)
        return 16;
    const float fTmp0D = z * (-4.683325804901025f * z2 + 2.007139630671868f);
    const float fTmp1C = 3.31161143515146f * z2 - 0.47308734787878f;
    const float fTmp2B = -1.770130769779931f * z;
    const float fC3 = x * fC2 - y * fS2;
    const float fS3 = x * fS2 + y * fC2;
    B[20] = (1.984313483298443f * z * B[12] - 1.006230589874905f * B[6]);
    B[21] = fTmp0D * x;
    B[19] = fTmp0D * y;
    B[22] = fTmp1C * fC1;
    B[18] = fTmp1C * fS1;
    B[23] = fTmp2B * fC2;
    B[17] = fTmp2B * fS2;
    B[24] = 0.6258357354491763f * fC3;
    B[16] = 0.6258357354491763f * fS3;
    return 25;
}

// colour of one channel: the reference's summation order (:29, :38-40, :54-56, :72-76, :95-103)
float sh_color(uint32_t degree, vec3 dir, const float* coeffs /*[K,3]*/, uint32_t c) {
    float result = 0.2820947917738781f * coeffs[c];
    if (degree >= 1) {
        const float inorm = gsx::rsqrt(dir.x * dir.x + dir.y * dir.y + dir.z * dir.z);
        const float x = dir.x * inorm, y = dir.y * inorm, z = dir.z * inorm;
        result += 0.48860251190292f * (-y * coeffs[1 * 3 + c] + z * coeffs[2 * 3 + c] - x * coeffs[3 * 3 + c]);
        if (degree >= 2) {
            float B[25];
            sh_basis(degree, dir, B);
            result += B[4] * coeffs[4 * 3 + c] + B[5] * coeffs[5 * 3 + c] + B[6] * coeffs[6 * 3 + c] +
                      B[7] * coeffs[7 * 3 + c] + B[8] * coeffs[8 * 3 + c];
            if (degree >= 3) {
                result += B[9] * coeffs[9 * 3 + c] + B[10] * coeffs[10 * 3 + c] + B[11] * coeffs[11 * 3 + c] +
                          B[12] * coeffs[12 * 3 + c] + B[13] * coeffs[13 * 3 + c] + B[14] * coeffs[14 * 3 + c] +
                          B[15] * coeffs[15 * 3 + c];
                if (degree >= 4) {
                    result += B[16] * coeffs[16 * 3 + c] + B[17] * coeffs[17 * 3 + c] +
                              B[18] * coeffs[18 * 3 + c] + B[19] * coeffs[19 * 3 + c] +
                              B[20] * coeffs[20 * 3 + c] + B[21] * coeffs[21 * 3 + c] +
                              B[22] * coeffs[22 * 3 + c] + B[23] * coeffs[23 * 3 + c] +
                              B[24] * coeffs[24 * 3 + c];
                }
            }
        }
    }
    return result;
}

} // namespace

ORC_API int orc_spherical_harmonics_fwd(uint32_t N, uint32_t K, uint32_t degree, const float* dirs,
                                        const float* coeffs, const uint8_t* masks /*nullable*/,
                                        float* colors) {
#pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < (int64_t)N; ++e) {
        if (masks != nullptr && !masks[e])
            continue;
        const vec3 dir = ld3(dirs, e);
        for (uint32_t c = 0; c < 3; ++c)
            colors[e * 3 + c] = sh_color(degree, dir, coeffs + e * K * 3, c);
    }
    return 0;
}

// v_coeffs must be zero-filled by the caller (SphericalHarmonics.cpp:57).  v_dirs (nullable) follows
// sh_coeffs_to_color_fast_vjp's direction gradient; LichtFeld never requests it
// (Rasterization.cpp:620).  Degrees 0-4 (SphericalHarmonicsCUDA.cu:112-371), pinned by central differences of a
// float64 basis in tests/test_oracle_geometry.py.
ORC_API int orc_spherical_harmonics_bwd(uint32_t N, uint32_t K, uint32_t degree, const float* dirs,
                                        const float* coeffs, const uint8_t* masks /*nullable*/,
                                        const float* v_colors, float* v_coeffs, float* v_dirs /*nullable*/) {
    if (v_dirs != nullptr && degree > 4)
        return -2;
#pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < (int64_t)N; ++e) {
        if (masks != nullptr && !masks[e])
            continue;
        const vec3 dir = ld3(dirs, e);
        float B[25];
        const int nb = sh_basis(degree, dir, B);
        for (uint32_t c = 0; c < 3; ++c) {
            const float v = v_colors[e * 3 + c];
            for (int k = 0; k < nb; ++k)
                v_coeffs[(e * K + k) * 3 + c] = B[k] * v;
        }
        if (v_dirs != nullptr) {
            // :139-143, :178-205, :237-287 accumulate d colour / d (x,y,z), then project out the
            // normalisation (:144-152)
            float vx = 0.f, vy = 0.f, vz = 0.f;
            if (degree >= 1) {
                const float inorm = gsx::rsqrt(dir.x * dir.x + dir.y * dir.y + dir.z * dir.z);
                const float x = dir.x * inorm, y = dir.y * inorm, z = dir.z * inorm;
                for (uint32_t c = 0; c < 3; ++c) {
                    const float* co = coeffs + e * K * 3;
                    const float v = v_colors[e * 3 + c];
                    float v_x = 0.f, v_y = 0.f, v_z = 0.f;
                    v_x += -0.48860251190292f * co[3 * 3 + c] * v;
                    v_y += -0.48860251190292f * co[1 * 3 + c] * v;
                    v_z += 0.48860251190292f * co[2 * 3 + c] * v;
                    float fC1 = 0, fS1 = 0, fC1_x = 0, fC1_y = 0, fS1_x = 0, fS1_y = 0;
                    const float z2 = z * z;
                    if (degree >= 2) {
                        const float fTmp0B = -1.092548430592079f * z;
                        fC1 = x * x - y * y;
                        fS1 = 2.f * x * y;
                        const float fTmp0B_z = -1.092548430592079f;
                        fC1_x = 2.f * x;
                        fC1_y = -2.f * y;
                        fS1_x = 2.f * y;
                        fS1_y = 2.f * x;
                        const float pSH6_z = 2.f * 0.9461746957575601f * z;
                        const float pSH7_x = fTmp0B, pSH7_z = fTmp0B_z * x;
                        const float pSH5_y = fTmp0B, pSH5_z = fTmp0B_z * y;
                        const float pSH8_x = 0.5462742152960395f * fC1_x, pSH8_y = 0.5462742152960395f * fC1_y;
                        const float pSH4_x = 0.5462742152960395f * fS1_x, pSH4_y = 0.5462742152960395f * fS1_y;
                        v_x += v * (pSH4_x * co[4 * 3 + c] + pSH8_x * co[8 * 3 + c] + pSH7_x * co[7 * 3 + c]);
                        v_y += v * (pSH4_y * co[4 * 3 + c] + pSH8_y * co[8 * 3 + c] + pSH5_y * co[5 * 3 + c]);
                        v_z += v * (pSH6_z * co[6 * 3 + c] + pSH7_z * co[7 * 3 + c] + pSH5_z * co[5 * 3 + c]);
                    }
                    if (degree >= 3) {
                        const float fTmp0C = -2.285228997322329f * z2 + 0.4570457994644658f;
                        const float fTmp1B = 1.445305721320277f * z;
                        const float fTmp0C_z = -2.285228997322329f * 2.f * z;
                        const float fTmp1B_z = 1.445305721320277f;
                        const float fC2_x = fC1 + x * fC1_x - y * fS1_x;
                        const float fC2_y = x * fC1_y - fS1 - y * fS1_y;
                        const float fS2_x = fS1 + x * fS1_x + y * fC1_x;
                        const float fS2_y = x * fS1_y + fC1 + y * fC1_y;
                        const float pSH12_z = 3.f * 1.865881662950577f * z2 - 1.119528997770346f;
                        const float pSH13_x = fTmp0C, pSH13_z = fTmp0C_z * x;
                        const float pSH11_y = fTmp0C, pSH11_z = fTmp0C_z * y;
                        const float pSH14_x = fTmp1B * fC1_x, pSH14_y = fTmp1B * fC1_y, pSH14_z = fTmp1B_z * fC1;
                        const float pSH10_x = fTmp1B * fS1_x, pSH10_y = fTmp1B * fS1_y, pSH10_z = fTmp1B_z * fS1;
                        const float pSH15_x = -0.5900435899266435f * fC2_x, pSH15_y = -0.5900435899266435f * fC2_y;
                        const float pSH9_x = -0.5900435899266435f * fS2_x, pSH9_y = -0.5900435899266435f * fS2_y;
                        v_x += v * (pSH9_x * co[9 * 3 + c] + pSH15_x * co[15 * 3 + c] + pSH10_x * co[10 * 3 + c] +
                                    pSH14_x * co[14 * 3 + c] + pSH13_x * co[13 * 3 + c]);
                        v_y += v * (pSH9_y * co[9 * 3 + c] + pSH15_y * co[15 * 3 + c] + pSH10_y * co[10 * 3 + c] +
                                    pSH14_y * co[14 * 3 + c] + pSH11_y * co[11 * 3 + c]);
                        v_z += v * (pSH12_z * co[12 * 3 + c] + pSH13_z * co[13 * 3 + c] + pSH11_z * co[11 * 3 + c] +
                                    pSH14_z * co[14 * 3 + c] + pSH10_z * co[10 * 3 + c]);
                        if (degree >= 4) { // SphericalHarmonicsCUDA.cu:288-360
                            const float fC2 = x * fC1 - y * fS1, fS2 = x * fS1 + y * fC1;
                            const float pSH6 = (0.9461746957575601f * z2 - 0.3153915652525201f);
                            const float pSH6_z4 = 2.f * 0.9461746957575601f * z;
                            const float pSH12 = z * (1.865881662950577f * z2 - 1.119528997770346f);
                            const float fTmp0D = z * (-4.683325804901025f * z2 + 2.007139630671868f);
                            const float fTmp1C = 3.31161143515146f * z2 - 0.47308734787878f;
                            const float fTmp2B = -1.770130769779931f * z;
                            const float fTmp0D_z = 3.f * -4.683325804901025f * z2 + 2.007139630671868f;
                            const float fTmp1C_z = 2.f * 3.31161143515146f * z;
                            const float fTmp2B_z = -1.770130769779931f;
                            const float fC3_x = fC2 + x * fC2_x - y * fS2_x;
                            const float fC3_y = x * fC2_y - fS2 - y * fS2_y;
                            const float fS3_x = fS2 + y * fC2_x + x * fS2_x;
                            const float fS3_y = x * fS2_y + fC2 + y * fC2_y;
                            const float pSH20_z = 1.984313483298443f * (pSH12 + z * pSH12_z) + -1.006230589874905f * pSH6_z4;
                            const float pSH21_x = fTmp0D, pSH21_z = fTmp0D_z * x;
                            const float pSH19_y = fTmp0D, pSH19_z = fTmp0D_z * y;
                            const float pSH22_x = fTmp1C * fC1_x, pSH22_y = fTmp1C * fC1_y, pSH22_z = fTmp1C_z * fC1;
                            const float pSH18_x = fTmp1C * fS1_x, pSH18_y = fTmp1C * fS1_y, pSH18_z = fTmp1C_z * fS1;
                            const float pSH23_x = fTmp2B * fC2_x, pSH23_y = fTmp2B * fC2_y, pSH23_z = fTmp2B_z * fC2;
                            const float pSH17_x = fTmp2B * fS2_x, pSH17_y = fTmp2B * fS2_y, pSH17_z = fTmp2B_z * fS2;
                            const float pSH24_x = 0.6258357354491763f * fC3_x, pSH24_y = 0.6258357354491763f * fC3_y;
                            const float pSH16_x = 0.6258357354491763f * fS3_x, pSH16_y = 0.6258357354491763f * fS3_y;
                            (void)pSH6;
                            v_x += v * (pSH16_x * co[16 * 3 + c] + pSH24_x * co[24 * 3 + c] + pSH17_x * co[17 * 3 + c] +
                                        pSH23_x * co[23 * 3 + c] + pSH18_x * co[18 * 3 + c] + pSH22_x * co[22 * 3 + c] +
                                        pSH21_x * co[21 * 3 + c]);
                            v_y += v * (pSH16_y * co[16 * 3 + c] + pSH24_y * co[24 * 3 + c] + pSH17_y * co[17 * 3 + c] +
                                        pSH23_y * co[23 * 3 + c] + pSH18_y * co[18 * 3 + c] + pSH22_y * co[22 * 3 + c] +
                                        pSH19_y * co[19 * 3 + c]);
                            v_z += v * (pSH20_z * co[20 * 3 + c] + pSH21_z * co[21 * 3 + c] + pSH19_z * co[19 * 3 + c] +
                                        pSH22_z * co[22 * 3 + c] + pSH18_z * co[18 * 3 + c] + pSH23_z * co[23 * 3 + c] +
                                        pSH17_z * co[17 * 3 + c]);
                        }
                    }
                    const float d = v_x * x + v_y * y + v_z * z;
                    vx += (v_x - d * x) * inorm;
                    vy += (v_y - d * y) * inorm;
                    vz += (v_z - d * z) * inorm;
                }
            }
            v_dirs[e * 3 + 0] = vx;
            v_dirs[e * 3 + 1] = vy;
            v_dirs[e * 3 + 2] = vz;
        }
    }
    return 0;
}

// =============================================================================================
// k4  intersect_tile  gsplat/IntersectTile.cu:23-114, host Intersect.cpp:41-104
// pass 1 (isect_ids == nullptr): tiles_per_gauss ; pass 2: keys and values in emission order.
// =============================================================================================
namespace {
inline void tile_bounds(const float* means2d, const int32_t* radii, int64_t idx, uint32_t tile_size,
                        uint32_t tile_width, uint32_t tile_height, uint32_t* x0, uint32_t* y0, uint32_t* x1,
                        uint32_t* y1, bool* skip) {
    const float radius_x = (float)radii[idx * 2];
    const float radius_y = (float)radii[idx * 2 + 1];
    if (radius_x <= 0 || radius_y <= 0) {
        *skip = true;
        return;
    }
    *skip = false;
    const float ts = (float)tile_size;
    const float tile_radius_x = radius_x / ts, tile_radius_y = radius_y / ts;
    const float tile_x = means2d[2 * idx] / ts, tile_y = means2d[2 * idx + 1] / ts;
    // :72-76 the float -> uint32 casts saturate (negative -> 0) on the reference's hardware
    *x0 = std::min(gsx::sat_u32(gsx::floor(tile_x - tile_radius_x)), tile_width);
    *y0 = std::min(gsx::sat_u32(gsx::floor(tile_y - tile_radius_y)), tile_height);
    *x1 = std::min(gsx::sat_u32(gsx::ceil(tile_x + tile_radius_x)), tile_width);
    *y1 = std::min(gsx::sat_u32(gsx::ceil(tile_y + tile_radius_y)), tile_height);
}
} // namespace

// Intersect.cpp:46-47
ORC_API uint32_t orc_tile_n_bits(uint32_t n_tiles) { return (uint32_t)std::floor(std::log2((double)n_tiles)) + 1; }

ORC_API int orc_intersect_tile_count(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                     uint32_t tile_size, uint32_t tile_width, uint32_t tile_height,
                                     int32_t* tiles_per_gauss, int64_t* cum_tiles_per_gauss, int64_t* n_isects) {
    const int64_t n = (int64_t)C * N;
#pragma omp parallel for schedule(static)
    for (int64_t idx = 0; idx < n; ++idx) {
        uint32_t x0, y0, x1, y1;
        bool skip;
        tile_bounds(means2d, radii, idx, tile_size, tile_width, tile_height, &x0, &y0, &x1, &y1, &skip);
        tiles_per_gauss[idx] = skip ? 0 : (int32_t)((y1 - y0) * (x1 - x0));
    }
    int64_t acc = 0; // at::cumsum (Intersect.cpp:75)
    for (int64_t idx = 0; idx < n; ++idx) {
        acc += tiles_per_gauss[idx];
        cum_tiles_per_gauss[idx] = acc;
    }
    *n_isects = acc;
    return 0;
}

// camera_ids: null for [C, N] rows (camera = idx / N); else packed rows [nnz = C * N as passed], each naming its
// camera (IntersectTile.cu:86-94)
static int intersect_tile_emit(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                               const float* depths, const int64_t* camera_ids, const int64_t* cum_tiles_per_gauss,
                               uint32_t tile_size, uint32_t tile_width, uint32_t tile_height, int64_t* isect_ids,
                               int32_t* flatten_ids) {
    const int64_t n = (int64_t)C * N;
    const uint32_t tile_n_bits = orc_tile_n_bits(tile_width * tile_height);
#pragma omp parallel for schedule(static)
    for (int64_t idx = 0; idx < n; ++idx) {
        uint32_t x0, y0, x1, y1;
        bool skip;
        tile_bounds(means2d, radii, idx, tile_size, tile_width, tile_height, &x0, &y0, &x1, &y1, &skip);
        if (skip)
            continue;
        const int64_t cid = camera_ids != nullptr ? camera_ids[idx] : idx / N;
        const int64_t cid_enc = cid << (32 + tile_n_bits);
        uint32_t dbits;
        std::memcpy(&dbits, depths + idx, 4);
        const int64_t depth_id_enc = (int64_t)dbits; // zero-extended (:96-98)
        int64_t cur = (idx == 0) ? 0 : cum_tiles_per_gauss[idx - 1];
        for (int32_t i = (int32_t)y0; i < (int32_t)y1; ++i)
            for (int32_t j = (int32_t)x0; j < (int32_t)x1; ++j) {
                const int64_t tile_id = (int64_t)i * tile_width + j;
                isect_ids[cur] = cid_enc | (tile_id << 32) | depth_id_enc;
                flatten_ids[cur] = (int32_t)idx;
                ++cur;
            }
    }
    return 0;
}

ORC_API int orc_intersect_tile_emit(uint32_t C, uint32_t N, const float* means2d, const int32_t* radii,
                                    const float* depths, const int64_t* cum_tiles_per_gauss, uint32_t tile_size,
                                    uint32_t tile_width, uint32_t tile_height, int64_t* isect_ids,
                                    int32_t* flatten_ids) {
    return intersect_tile_emit(C, N, means2d, radii, depths, nullptr, cum_tiles_per_gauss, tile_size, tile_width,
                               tile_height, isect_ids, flatten_ids);
}

ORC_API int orc_intersect_tile_emit_packed(uint32_t nnz, const float* means2d, const int32_t* radii,
                                           const float* depths, const int64_t* camera_ids,
                                           const int64_t* cum_tiles_per_gauss, uint32_t tile_size,
                                           uint32_t tile_width, uint32_t tile_height, int64_t* isect_ids,
                                           int32_t* flatten_ids) {
    return intersect_tile_emit(1, nnz, means2d, radii, depths, camera_ids, cum_tiles_per_gauss, tile_size,
                               tile_width, tile_height, isect_ids, flatten_ids);
}

// =============================================================================================
// k5  radix_sort_double_buffer  gsplat/IntersectTile.cu:290-328
// cub::DeviceRadixSort::SortPairs on bits [0, end_bit): a stable ascending sort of the keys
// masked to those bits.  (CUB is third-party and absent from the reference tree; its documented
// contract - stable, unsigned compare on the bit range - is restated with std::stable_sort.)
// =============================================================================================
ORC_API int orc_radix_sort_pairs(int64_t n, const int64_t* keys_in, const int32_t* vals_in, uint32_t end_bit,
                                 int64_t* keys_out, int32_t* vals_out) {
    const uint64_t mask = end_bit >= 64 ? ~0ull : ((1ull << end_bit) - 1ull);
    std::vector<int64_t> order(n);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int64_t a, int64_t b) {
        return ((uint64_t)keys_in[a] & mask) < ((uint64_t)keys_in[b] & mask);
    });
    for (int64_t i = 0; i < n; ++i) {
        keys_out[i] = keys_in[order[i]];
        vals_out[i] = vals_in[order[i]];
    }
    return 0;
}

// =============================================================================================
// k6  intersect_offset  gsplat/IntersectTile.cu:206-252 (I == 0 -> zeros, :268-271)
// =============================================================================================
ORC_API int orc_intersect_offset(int64_t n_isects, const int64_t* isect_ids, uint32_t C, uint32_t tile_width,
                                 uint32_t tile_height, int32_t* offsets) {
    const uint32_t n_tiles = tile_width * tile_height;
    if (n_isects == 0) {
        std::fill(offsets, offsets + (int64_t)C * n_tiles, 0);
        return 0;
    }
    const uint32_t tile_n_bits = orc_tile_n_bits(n_tiles);
    for (int64_t idx = 0; idx < n_isects; ++idx) {
        const int64_t isect_id_curr = isect_ids[idx] >> 32;
        const int64_t cid_curr = isect_id_curr >> tile_n_bits;
        const int64_t tid_curr = isect_id_curr & ((1 << tile_n_bits) - 1);
        const int64_t id_curr = cid_curr * n_tiles + tid_curr;
        if (idx == 0)
            for (int64_t i = 0; i < id_curr + 1; ++i)
                offsets[i] = (int32_t)idx;
        if (idx == n_isects - 1)
            for (int64_t i = id_curr + 1; i < (int64_t)C * n_tiles; ++i)
                offsets[i] = (int32_t)n_isects;
        if (idx > 0) {
            const int64_t isect_id_prev = isect_ids[idx - 1] >> 32;
            if (isect_id_prev == isect_id_curr)
                continue;
            const int64_t cid_prev = isect_id_prev >> tile_n_bits;
            const int64_t tid_prev = isect_id_prev & ((1 << tile_n_bits) - 1);
            const int64_t id_prev = cid_prev * n_tiles + tid_prev;
            for (int64_t i = id_prev + 1; i < id_curr + 1; ++i)
                offsets[i] = (int32_t)idx;
        }
    }
    return 0;
}

// =============================================================================================
// k7  rasterize_to_pixels_from_world_3dgs_fwd  gsplat/RasterizeToPixelsFromWorld3DGSFwd.cu:19-285
// C == 1 (the reference indexes means[] with the flattened id, :203-210).  CDIM is a run-time
// argument here.  masks: optional per-tile bool; false tiles get the background (:147-155) and
// leave alphas / last_ids untouched.
// *pairs_evaluated (nullable) returns the number of (pixel, Gaussian) evaluations performed.
// =============================================================================================
ORC_API int orc_rasterize_to_pixels_from_world_3dgs_fwd(
    uint32_t C, uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
    const float* colors, uint32_t CDIM, const float* opacities, const float* backgrounds /*nullable*/,
    const uint8_t* masks /*nullable*/, uint32_t image_width, uint32_t image_height, uint32_t tile_size,
    const float* viewmats0, const float* Ks, const int32_t* tile_offsets, const int32_t* flatten_ids,
    float* render_colors, float* render_alphas, int32_t* last_ids, int64_t* pairs_evaluated) {
    if (C != 1 || CDIM > 513)
        return -2;
    (void)N;
    const uint32_t tile_width = (image_width + tile_size - 1) / tile_size;
    const uint32_t tile_height = (image_height + tile_size - 1) / tile_size;
    const uint32_t n_tiles = tile_width * tile_height;
    const float fx = Ks[0], fy = Ks[4], cx = Ks[2], cy = Ks[5];
    const RollingShutter rs = make_rolling_shutter(viewmats0, nullptr);
    int64_t pairs = 0;
#pragma omp parallel for schedule(dynamic, 1) reduction(+ : pairs)
    for (int64_t tile_id = 0; tile_id < (int64_t)n_tiles; ++tile_id) {
        const uint32_t ty = tile_id / tile_width, tx = tile_id % tile_width;
        const int32_t range_start = tile_offsets[tile_id];
        const int32_t range_end = (tile_id == (int64_t)n_tiles - 1) ? (int32_t)n_isects : tile_offsets[tile_id + 1];
        // stage the tile's Gaussians once (what the reference does per 256-batch in shared memory)
        const int32_t cnt = range_end - range_start;
        std::vector<mat3> Ms(cnt > 0 ? cnt : 0);
        for (int32_t t = 0; t < cnt; ++t) {
            const int32_t g = flatten_ids[range_start + t];
            Ms[t] = iscl_rot(ld4(quats, g), ld3(scales, g));
        }
        for (uint32_t ly = 0; ly < tile_size; ++ly)
            for (uint32_t lx = 0; lx < tile_size; ++lx) {
                const uint32_t i = ty * tile_size + ly, j = tx * tile_size + lx;
                if (!(i < image_height && j < image_width))
                    continue;
                const int64_t pix_id = (int64_t)i * image_width + j;
                if (masks != nullptr && !masks[tile_id]) {
                    for (uint32_t k = 0; k < CDIM; ++k)
                        render_colors[pix_id * CDIM + k] = backgrounds == nullptr ? 0.0f : backgrounds[k];
                    continue;
                }
                vec3 ray_o, ray_d;
                const bool ray_ok =
                    pixel_world_ray((float)j + 0.5f, (float)i + 0.5f, fx, fy, cx, cy, rs, &ray_o, &ray_d);
                float T = 1.0f;
                uint32_t cur_idx = 0;
                float pix_out[513] = {};
                // a pixel without a valid ray is done from the start (RasterizeToPixelsFromWorld3DGSFwd.cu:145)
                for (int32_t t = 0; t < (ray_ok ? cnt : 0); ++t) {
                    ++pairs;
                    const int32_t g = flatten_ids[range_start + t];
                    const vec3 xyz = ld3(means, g);
                    const float opac = opacities[g];
                    const mat3& M = Ms[t];
                    const vec3 gro = gsx::mul(M, gsx::sub(ray_o, xyz));
                    const vec3 grd = gsx::safe_normalize(gsx::mul(M, ray_d));
                    const vec3 gcrod = gsx::cross(grd, gro);
                    const float grayDist = gsx::dot(gcrod, gcrod);
                    const float power = -0.5f * grayDist;
                    const float alpha = gsx::min_limit(0.999f, opac * gsx::exp(power));
                    if (alpha < 1.f / 255.f)
                        continue;
                    const float next_T = T * (1.0f - alpha);
                    if (next_T <= 1e-4f)
                        break;
                    const float vis = alpha * T;
                    for (uint32_t k = 0; k < CDIM; ++k)
                        pix_out[k] = gsx::fma(colors[(int64_t)g * CDIM + k], vis, pix_out[k]);
                    cur_idx = (uint32_t)(range_start + t);
                    T = next_T;
                }
                render_alphas[pix_id] = 1.0f - T;
                for (uint32_t k = 0; k < CDIM; ++k)
                    render_colors[pix_id * CDIM + k] =
                        backgrounds == nullptr ? pix_out[k] : gsx::fma(T, backgrounds[k], pix_out[k]);
                last_ids[pix_id] = (int32_t)cur_idx;
            }
    }
    if (pairs_evaluated)
        *pairs_evaluated = pairs;
    return 0;
}

// =============================================================================================
// k8  rasterize_to_pixels_from_world_3dgs_bwd  gsplat/RasterizeToPixelsFromWorld3DGSBwd.cu:16-379
// VJP helpers: Utils.cuh:104-158 (quat/scale), :186-194 (normalize).
// Per-pixel terms are computed in fp32 exactly as a reference thread does; the per-Gaussian sums
// (warp reduce + atomicAdd in the reference, order unspecified) are formed in double and rounded
// once.  Outputs must be zero-filled by the caller (Rasterization.cpp:190-194).
// =============================================================================================
ORC_API int orc_rasterize_to_pixels_from_world_3dgs_bwd(
    uint32_t C, uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales,
    const float* colors, uint32_t CDIM, const float* opacities, const float* backgrounds /*nullable*/,
    const uint8_t* masks /*nullable*/, uint32_t image_width, uint32_t image_height, uint32_t tile_size,
    const float* viewmats0, const float* Ks, const int32_t* tile_offsets, const int32_t* flatten_ids,
    const float* render_alphas, const int32_t* last_ids, const float* v_render_colors,
    const float* v_render_alphas, float* v_means, float* v_quats, float* v_scales, float* v_colors,
    float* v_opacities) {
    constexpr uint32_t kMaxC = 513; // Rasterization.cpp:106-128
    if (C != 1 || CDIM < 1 || CDIM > kMaxC)
        return -2;
    const size_t kRow = 11 + CDIM; // mean 3, quat 4, scale 3, opacity 1, then the colour channels
    const uint32_t tile_width = (image_width + tile_size - 1) / tile_size;
    const uint32_t tile_height = (image_height + tile_size - 1) / tile_size;
    const uint32_t n_tiles = tile_width * tile_height;
    const float fx = Ks[0], fy = Ks[4], cx = Ks[2], cy = Ks[5];
    const RollingShutter rs = make_rolling_shutter(viewmats0, nullptr);
    std::vector<double> acc((size_t)N * kRow, 0.0);
    // tiles that share a Gaussian would race on acc: process tiles in parallel with per-Gaussian
    // atomic double adds (order-independent to ~1e-16, far below the fp32 comparison tolerance)
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t tile_id = 0; tile_id < (int64_t)n_tiles; ++tile_id) {
        if (masks != nullptr && !masks[tile_id])
            continue;
        const uint32_t ty = tile_id / tile_width, tx = tile_id % tile_width;
        const int32_t range_start = tile_offsets[tile_id];
        const int32_t range_end = (tile_id == (int64_t)n_tiles - 1) ? (int32_t)n_isects : tile_offsets[tile_id + 1];
        const int32_t cnt = range_end - range_start;
        if (cnt <= 0)
            continue;
        std::vector<double> local((size_t)cnt * kRow, 0.0);
        for (uint32_t ly = 0; ly < tile_size; ++ly)
            for (uint32_t lx = 0; lx < tile_size; ++lx) {
                const uint32_t i = ty * tile_size + ly, j = tx * tile_size + lx;
                if (!(i < image_height && j < image_width))
                    continue;
                const int64_t pix_id = (int64_t)i * image_width + j;
                vec3 ray_o, ray_d;
                if (!pixel_world_ray((float)j + 0.5f, (float)i + 0.5f, fx, fy, cx, cy, rs, &ray_o, &ray_d))
                    continue; // RasterizeToPixelsFromWorld3DGSBwd.cu:157
                const float T_final = 1.0f - render_alphas[pix_id];
                float T = T_final;
                float buffer[kMaxC] = {};
                const int32_t bin_final = last_ids[pix_id];
                float v_render_c[kMaxC] = {};
                for (uint32_t k = 0; k < CDIM; ++k)
                    v_render_c[k] = v_render_colors[pix_id * CDIM + k];
                const float v_render_a = v_render_alphas[pix_id];
                // back to front over the tile's list; entries behind bin_final are not valid (:236-239)
                for (int32_t idx = std::min(range_end - 1, bin_final); idx >= range_start; --idx) {
                    const int32_t g = flatten_ids[idx];
                    const vec3 xyz = ld3(means, g);
                    const float opac = opacities[g];
                    const vec3 scale = ld3(scales, g);
                    const quat q = ld4(quats, g);
                    const mat3 R = gsx::quat_to_rotmat(q);
                    const float is[3] = {1.0f / scale.x, 1.0f / scale.y, 1.0f / scale.z};
                    mat3 Mt; // transpose(R * S) = S * R^T
                    for (int a = 0; a < 3; ++a)
                        for (int b = 0; b < 3; ++b)
                            Mt.m[a][b] = R.m[b][a] * is[a];
                    const vec3 o_minus_mu = gsx::sub(ray_o, xyz);
                    const vec3 gro = gsx::mul(Mt, o_minus_mu);
                    const vec3 grd = gsx::mul(Mt, ray_d);
                    const vec3 grd_n = gsx::safe_normalize(grd);
                    const vec3 gcrod = gsx::cross(grd_n, gro);
                    const float grayDist = gsx::dot(gcrod, gcrod);
                    const float power = -0.5f * grayDist;
                    const float vis = gsx::exp(power);
                    const float alpha = gsx::min_limit(0.999f, opac * vis);
                    if (power > 0.f || alpha < 1.f / 255.f)
                        continue;

                    const float ra = 1.0f / (1.0f - alpha);
                    T *= ra;
                    const float fac = alpha * T;
                    float v_rgb_local[kMaxC] = {};
                    for (uint32_t k = 0; k < CDIM; ++k)
                        v_rgb_local[k] = fac * v_render_c[k];
                    float v_alpha = 0.f;
                    for (uint32_t k = 0; k < CDIM; ++k)
                        v_alpha += (colors[(int64_t)g * CDIM + k] * T - buffer[k] * ra) * v_render_c[k];
                    v_alpha += T_final * ra * v_render_a;
                    if (backgrounds != nullptr) {
                        float accum = 0.f;
                        for (uint32_t k = 0; k < CDIM; ++k)
                            accum += backgrounds[k] * v_render_c[k];
                        v_alpha += -T_final * ra * accum;
                    }
                    vec3 v_mean_local = gsx::mk3(0.f, 0.f, 0.f);
                    float v_scale_local[3] = {0.f, 0.f, 0.f};
                    float v_quat_local[4] = {0.f, 0.f, 0.f, 0.f}; // w, x, y, z
                    float v_opacity_local = 0.f;
                    if (opac * vis <= 0.999f) {
                        const float v_vis = opac * v_alpha;
                        const float v_gradDist = -0.5f * vis * v_vis;
                        const vec3 v_gcrod = gsx::scale(gcrod, 2.0f * v_gradDist);
                        const vec3 v_grd_n = gsx::neg(gsx::cross(v_gcrod, gro));
                        const vec3 v_gro = gsx::cross(v_gcrod, grd_n);
                        const vec3 v_grd = gsx::safe_normalize_bw(grd, v_grd_n);
                        // v_Mt(i,j) = v_grd_i ray_d_j + v_gro_i o_j   (glm::outerProduct(c, r) = c r^T)
                        const float vg[3] = {v_grd.x, v_grd.y, v_grd.z};
                        const float vo[3] = {v_gro.x, v_gro.y, v_gro.z};
                        const float rd[3] = {ray_d.x, ray_d.y, ray_d.z};
                        const float om[3] = {o_minus_mu.x, o_minus_mu.y, o_minus_mu.z};
                        float v_Mt[3][3];
                        for (int a = 0; a < 3; ++a)
                            for (int b = 0; b < 3; ++b)
                                v_Mt[a][b] = vg[a] * rd[b] + vo[a] * om[b];
                        const vec3 v_o_minus_mu = gsx::mul_t(Mt, v_gro);
                        v_mean_local = gsx::neg(v_o_minus_mu);
                        // quat_scale_to_preci_half_vjp(quat, scale, R, v_M = transpose(v_Mt)) Utils.cuh:128-158
                        // v_M(k,j) = v_Mt[j][k];  v_R(k,j) = v_M(k,j) * is[j]
                        float vr[3][3];
                        for (int k = 0; k < 3; ++k)
                            for (int jj = 0; jj < 3; ++jj)
                                vr[k][jj] = v_Mt[jj][k] * is[jj];
                        {
                            // quat_to_rotmat_vjp Utils.cuh:104-126 ; glm v_R[a][b] = vr[b][a]
                            const float inv_norm =
                                gsx::rsqrt(gsx::fma(q.w, q.w, gsx::fma(q.z, q.z, gsx::fma(q.y, q.y, q.x * q.x))));
                            const float x = q.x * inv_norm, y = q.y * inv_norm, z = q.z * inv_norm,
                                        w = q.w * inv_norm;
                            const float vq_w = 2.f * (x * (vr[2][1] - vr[1][2]) + y * (vr[0][2] - vr[2][0]) +
                                                      z * (vr[1][0] - vr[0][1]));
                            const float vq_x =
                                2.f * (-2.f * x * (vr[1][1] + vr[2][2]) + y * (vr[1][0] + vr[0][1]) +
                                       z * (vr[2][0] + vr[0][2]) + w * (vr[2][1] - vr[1][2]));
                            const float vq_y =
                                2.f * (x * (vr[1][0] + vr[0][1]) - 2.f * y * (vr[0][0] + vr[2][2]) +
                                       z * (vr[2][1] + vr[1][2]) + w * (vr[0][2] - vr[2][0]));
                            const float vq_z =
                                2.f * (x * (vr[2][0] + vr[0][2]) + y * (vr[2][1] + vr[1][2]) -
                                       2.f * z * (vr[0][0] + vr[1][1]) + w * (vr[1][0] - vr[0][1]));
                            const float d = vq_w * w + vq_x * x + vq_y * y + vq_z * z;
                            v_quat_local[0] = (vq_w - d * w) * inv_norm;
                            v_quat_local[1] = (vq_x - d * x) * inv_norm;
                            v_quat_local[2] = (vq_y - d * y) * inv_norm;
                            v_quat_local[3] = (vq_z - d * z) * inv_norm;
                        }
                        // v_scale[j] = -is_j^2 * sum_k R(k,j) v_M(k,j)   (Utils.cuh:147-157)
                        for (int jj = 0; jj < 3; ++jj)
                            v_scale_local[jj] = -is[jj] * is[jj] *
                                                (R.m[0][jj] * v_Mt[jj][0] + R.m[1][jj] * v_Mt[jj][1] +
                                                 R.m[2][jj] * v_Mt[jj][2]);
                        v_opacity_local = vis * v_alpha;
                    }
                    for (uint32_t k = 0; k < CDIM; ++k)
                        buffer[k] += colors[(int64_t)g * CDIM + k] * fac;

                    double* a = local.data() + (size_t)(idx - range_start) * kRow;
                    a[0] += v_mean_local.x;
                    a[1] += v_mean_local.y;
                    a[2] += v_mean_local.z;
                    a[3] += v_quat_local[0];
                    a[4] += v_quat_local[1];
                    a[5] += v_quat_local[2];
                    a[6] += v_quat_local[3];
                    a[7] += v_scale_local[0];
                    a[8] += v_scale_local[1];
                    a[9] += v_scale_local[2];
                    a[10] += v_opacity_local;
                    for (uint32_t k = 0; k < CDIM; ++k)
                        a[11 + k] += v_rgb_local[k];
                }
            }
        for (int32_t t = 0; t < cnt; ++t) {
            const int32_t g = flatten_ids[range_start + t];
            for (size_t k = 0; k < kRow; ++k) {
                const double v = local[(size_t)t * kRow + k];
                if (v != 0.0) {
#pragma omp atomic
                    acc[(size_t)g * kRow + k] += v;
                }
            }
        }
    }
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < (int64_t)N; ++g) {
        const double* a = acc.data() + (size_t)g * kRow;
        for (int k = 0; k < 3; ++k)
            v_means[g * 3 + k] += (float)a[k];
        for (int k = 0; k < 4; ++k)
            v_quats[g * 4 + k] += (float)a[3 + k];
        for (int k = 0; k < 3; ++k)
            v_scales[g * 3 + k] += (float)a[7 + k];
        for (uint32_t k = 0; k < CDIM; ++k)
            v_colors[g * CDIM + k] += (float)a[11 + k];
        v_opacities[g] += (float)a[10];
    }
    return 0;
}

// ---------------------------------------------------------------------------------------------
// float64 evaluation of the same backward pass, for judging fp32 results.
// Which (pixel, Gaussian) pairs take part is decided by the fp32 path above (thresholds on alpha and
// the last contributing index), the values are then evaluated in double from the same fp32 inputs.
// grads[N][14]: mean 3, quat 4 (wxyz), scale 3, colour 3, opacity 1.
// bound[N][14]: the same expressions evaluated with every product replaced by its absolute value and every
// difference by a sum (a running error-bound scale: an fp32 evaluation of depth d differs from the exact
// value by at most about d * 2^-24 * bound).
// =============================================================================================
namespace {
struct d3 {
    double x, y, z;
};
inline d3 dcross(d3 a, d3 b) { return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x}; }
inline d3 dcross_abs(d3 a, d3 b) {
    return {std::fabs(a.y * b.z) + std::fabs(a.z * b.y), std::fabs(a.z * b.x) + std::fabs(a.x * b.z),
            std::fabs(a.x * b.y) + std::fabs(a.y * b.x)};
}
inline double ddot(d3 a, d3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
inline double ddot_abs(d3 a, d3 b) { return std::fabs(a.x * b.x) + std::fabs(a.y * b.y) + std::fabs(a.z * b.z); }
} // namespace

ORC_API int orc_rasterize_bwd_f64(
    uint32_t N, int64_t n_isects, const float* means, const float* quats, const float* scales, const float* colors,
    const float* opacities, const float* backgrounds /*nullable*/, uint32_t image_width, uint32_t image_height,
    uint32_t tile_size, const float* viewmats0, const float* Ks, const int32_t* tile_offsets,
    const int32_t* flatten_ids, const float* render_alphas, const int32_t* last_ids, const float* v_render_colors,
    const float* v_render_alphas, double* grads, double* bound) {
    const uint32_t tile_width = (image_width + tile_size - 1) / tile_size;
    const uint32_t tile_height = (image_height + tile_size - 1) / tile_size;
    const uint32_t n_tiles = tile_width * tile_height;
    const float fx = Ks[0], fy = Ks[4], cx = Ks[2], cy = Ks[5];
    const RollingShutter rs = make_rolling_shutter(viewmats0, nullptr);
    std::fill(grads, grads + (size_t)N * 14, 0.0);
    std::fill(bound, bound + (size_t)N * 14, 0.0);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t tile_id = 0; tile_id < (int64_t)n_tiles; ++tile_id) {
        const uint32_t ty = tile_id / tile_width, tx = tile_id % tile_width;
        const int32_t range_start = tile_offsets[tile_id];
        const int32_t range_end = (tile_id == (int64_t)n_tiles - 1) ? (int32_t)n_isects : tile_offsets[tile_id + 1];
        const int32_t cnt = range_end - range_start;
        if (cnt <= 0)
            continue;
        std::vector<double> local((size_t)cnt * 14, 0.0), lbound((size_t)cnt * 14, 0.0);
        for (uint32_t ly = 0; ly < tile_size; ++ly)
            for (uint32_t lx = 0; lx < tile_size; ++lx) {
                const uint32_t i = ty * tile_size + ly, j = tx * tile_size + lx;
                if (!(i < image_height && j < image_width))
                    continue;
                const int64_t pix_id = (int64_t)i * image_width + j;
                vec3 ray_of, ray_df;
                if (!pixel_world_ray((float)j + 0.5f, (float)i + 0.5f, fx, fy, cx, cy, rs, &ray_of, &ray_df))
                    continue;
                const d3 ray_o = {ray_of.x, ray_of.y, ray_of.z}, ray_d = {ray_df.x, ray_df.y, ray_df.z};
                const double T_final = 1.0 - (double)render_alphas[pix_id];
                double T = T_final;
                double buffer[3] = {0, 0, 0}, buffer_abs[3] = {0, 0, 0};
                const int32_t bin_final = last_ids[pix_id];
                const double vrc[3] = {v_render_colors[pix_id * 3], v_render_colors[pix_id * 3 + 1],
                                       v_render_colors[pix_id * 3 + 2]};
                const double vra = v_render_alphas[pix_id];
                for (int32_t idx = std::min(range_end - 1, bin_final); idx >= range_start; --idx) {
                    const int32_t g = flatten_ids[idx];
                    // fp32 decision and fp32 alpha (identical to orc_rasterize_to_pixels_from_world_3dgs_bwd): the
                    // transmittance is recovered by dividing by (1 - alpha) with the alpha the forward pass used
                    float alphaf;
                    {
                        const mat3 Mf = iscl_rot(ld4(quats, g), ld3(scales, g));
                        const vec3 grof = gsx::mul(Mf, gsx::sub(ray_of, ld3(means, g)));
                        const vec3 grdf = gsx::safe_normalize(gsx::mul(Mf, ray_df));
                        const vec3 cf = gsx::cross(grdf, grof);
                        const float powerf = -0.5f * gsx::dot(cf, cf);
                        alphaf = gsx::min_limit(0.999f, opacities[g] * gsx::exp(powerf));
                        if (powerf > 0.f || alphaf < 1.f / 255.f)
                            continue;
                    }
                    // values in double
                    const double qw = quats[g * 4], qx = quats[g * 4 + 1], qy = quats[g * 4 + 2], qz = quats[g * 4 + 3];
                    const double inv_norm = 1.0 / std::sqrt(qw * qw + qx * qx + qy * qy + qz * qz);
                    const double w = qw * inv_norm, x = qx * inv_norm, y = qy * inv_norm, z = qz * inv_norm;
                    double R[3][3];
                    R[0][0] = 1 - 2 * (y * y + z * z), R[0][1] = 2 * (x * y - w * z), R[0][2] = 2 * (x * z + w * y);
                    R[1][0] = 2 * (x * y + w * z), R[1][1] = 1 - 2 * (x * x + z * z), R[1][2] = 2 * (y * z - w * x);
                    R[2][0] = 2 * (x * z - w * y), R[2][1] = 2 * (y * z + w * x), R[2][2] = 1 - 2 * (x * x + y * y);
                    const double is[3] = {1.0 / scales[g * 3], 1.0 / scales[g * 3 + 1], 1.0 / scales[g * 3 + 2]};
                    double Mt[3][3];
                    for (int a = 0; a < 3; ++a)
                        for (int b = 0; b < 3; ++b)
                            Mt[a][b] = R[b][a] * is[a];
                    const double om[3] = {ray_o.x - means[g * 3], ray_o.y - means[g * 3 + 1], ray_o.z - means[g * 3 + 2]};
                    const double rd[3] = {ray_d.x, ray_d.y, ray_d.z};
                    double gro_[3], grd_[3];
                    for (int a = 0; a < 3; ++a) {
                        gro_[a] = Mt[a][0] * om[0] + Mt[a][1] * om[1] + Mt[a][2] * om[2];
                        grd_[a] = Mt[a][0] * rd[0] + Mt[a][1] * rd[1] + Mt[a][2] * rd[2];
                    }
                    const d3 gro = {gro_[0], gro_[1], gro_[2]}, grd = {grd_[0], grd_[1], grd_[2]};
                    const double l = ddot(grd, grd);
                    const double il = 1.0 / std::sqrt(l);
                    const d3 grd_n = {grd.x * il, grd.y * il, grd.z * il};
                    const d3 gcrod = dcross(grd_n, gro);
                    const double power = -0.5 * ddot(gcrod, gcrod);
                    const double vis = std::exp(power);
                    const double opac = opacities[g];
                    const double alpha = (double)alphaf;
                    const double ra = 1.0 / (double)(1.0f - alphaf);
                    T *= ra;
                    const double fac = alpha * T;
                    const double rgb[3] = {colors[(int64_t)g * 3], colors[(int64_t)g * 3 + 1], colors[(int64_t)g * 3 + 2]};
                    double v_alpha = 0, v_alpha_abs = 0;
                    for (int k = 0; k < 3; ++k) {
                        v_alpha += (rgb[k] * T - buffer[k] * ra) * vrc[k];
                        v_alpha_abs += (std::fabs(rgb[k] * T) + buffer_abs[k] * ra) * std::fabs(vrc[k]);
                    }
                    v_alpha += T_final * ra * vra;
                    v_alpha_abs += std::fabs(T_final * ra * vra);
                    if (backgrounds != nullptr) {
                        double accum = 0, accum_abs = 0;
                        for (int k = 0; k < 3; ++k) {
                            accum += backgrounds[k] * vrc[k];
                            accum_abs += std::fabs(backgrounds[k] * vrc[k]);
                        }
                        v_alpha += -T_final * ra * accum;
                        v_alpha_abs += std::fabs(T_final * ra) * accum_abs;
                    }
                    double* a = local.data() + (size_t)(idx - range_start) * 14;
                    double* ab = lbound.data() + (size_t)(idx - range_start) * 14;
                    for (int k = 0; k < 3; ++k) {
                        a[10 + k] += fac * vrc[k];
                        ab[10 + k] += std::fabs(fac * vrc[k]);
                    }
                    if (opac * vis <= 0.999) {
                        const double v_vis = opac * v_alpha, v_vis_abs = opac * v_alpha_abs;
                        const double v_gd = -0.5 * vis * v_vis, v_gd_abs = 0.5 * vis * v_vis_abs;
                        const d3 v_gcrod = {2 * v_gd * gcrod.x, 2 * v_gd * gcrod.y, 2 * v_gd * gcrod.z};
                        const d3 gcrod_abs = dcross_abs(grd_n, gro);
                        const d3 v_gcrod_abs = {2 * v_gd_abs * gcrod_abs.x, 2 * v_gd_abs * gcrod_abs.y,
                                                2 * v_gd_abs * gcrod_abs.z};
                        d3 v_grd_n = dcross(v_gcrod, gro);
                        v_grd_n = {-v_grd_n.x, -v_grd_n.y, -v_grd_n.z};
                        const d3 v_grd_n_abs = dcross_abs(v_gcrod_abs, gro);
                        const d3 v_gro = dcross(v_gcrod, grd_n);
                        const d3 v_gro_abs = dcross_abs(v_gcrod_abs, grd_n);
                        const double il3 = il * il * il;
                        const double dd = ddot(v_grd_n, grd), dd_abs = ddot_abs(v_grd_n_abs, grd);
                        const d3 v_grd = {il * v_grd_n.x - il3 * dd * grd.x, il * v_grd_n.y - il3 * dd * grd.y,
                                          il * v_grd_n.z - il3 * dd * grd.z};
                        const d3 v_grd_abs = {il * v_grd_n_abs.x + il3 * dd_abs * std::fabs(grd.x),
                                              il * v_grd_n_abs.y + il3 * dd_abs * std::fabs(grd.y),
                                              il * v_grd_n_abs.z + il3 * dd_abs * std::fabs(grd.z)};
                        const double vg[3] = {v_grd.x, v_grd.y, v_grd.z}, vo[3] = {v_gro.x, v_gro.y, v_gro.z};
                        const double vga[3] = {v_grd_abs.x, v_grd_abs.y, v_grd_abs.z};
                        const double voa[3] = {v_gro_abs.x, v_gro_abs.y, v_gro_abs.z};
                        double v_Mt[3][3], v_Mt_abs[3][3];
                        for (int p = 0; p < 3; ++p)
                            for (int q = 0; q < 3; ++q) {
                                v_Mt[p][q] = vg[p] * rd[q] + vo[p] * om[q];
                                v_Mt_abs[p][q] = vga[p] * std::fabs(rd[q]) + voa[p] * std::fabs(om[q]);
                            }
                        for (int q = 0; q < 3; ++q) { // v_mean = -Mt^T v_gro
                            a[q] += -(Mt[0][q] * vo[0] + Mt[1][q] * vo[1] + Mt[2][q] * vo[2]);
                            ab[q] += std::fabs(Mt[0][q]) * voa[0] + std::fabs(Mt[1][q]) * voa[1] +
                                     std::fabs(Mt[2][q]) * voa[2];
                        }
                        double vr[3][3], vra_[3][3];
                        for (int k = 0; k < 3; ++k)
                            for (int jj = 0; jj < 3; ++jj) {
                                vr[k][jj] = v_Mt[jj][k] * is[jj];
                                vra_[k][jj] = v_Mt_abs[jj][k] * is[jj];
                            }
                        const double vq_w =
                            2 * (x * (vr[2][1] - vr[1][2]) + y * (vr[0][2] - vr[2][0]) + z * (vr[1][0] - vr[0][1]));
                        const double vq_x = 2 * (-2 * x * (vr[1][1] + vr[2][2]) + y * (vr[1][0] + vr[0][1]) +
                                                 z * (vr[2][0] + vr[0][2]) + w * (vr[2][1] - vr[1][2]));
                        const double vq_y = 2 * (x * (vr[1][0] + vr[0][1]) - 2 * y * (vr[0][0] + vr[2][2]) +
                                                 z * (vr[2][1] + vr[1][2]) + w * (vr[0][2] - vr[2][0]));
                        const double vq_z = 2 * (x * (vr[2][0] + vr[0][2]) + y * (vr[2][1] + vr[1][2]) -
                                                 2 * z * (vr[0][0] + vr[1][1]) + w * (vr[1][0] - vr[0][1]));
                        const double ax = std::fabs(x), ay = std::fabs(y), az = std::fabs(z), aw = std::fabs(w);
                        const double vqa_w = 2 * (ax * (vra_[2][1] + vra_[1][2]) + ay * (vra_[0][2] + vra_[2][0]) +
                                                  az * (vra_[1][0] + vra_[0][1]));
                        const double vqa_x = 2 * (2 * ax * (vra_[1][1] + vra_[2][2]) + ay * (vra_[1][0] + vra_[0][1]) +
                                                  az * (vra_[2][0] + vra_[0][2]) + aw * (vra_[2][1] + vra_[1][2]));
                        const double vqa_y = 2 * (ax * (vra_[1][0] + vra_[0][1]) + 2 * ay * (vra_[0][0] + vra_[2][2]) +
                                                  az * (vra_[2][1] + vra_[1][2]) + aw * (vra_[0][2] + vra_[2][0]));
                        const double vqa_z = 2 * (ax * (vra_[2][0] + vra_[0][2]) + ay * (vra_[2][1] + vra_[1][2]) +
                                                  2 * az * (vra_[0][0] + vra_[1][1]) + aw * (vra_[1][0] + vra_[0][1]));
                        const double dq = vq_w * w + vq_x * x + vq_y * y + vq_z * z;
                        const double dqa = vqa_w * aw + vqa_x * ax + vqa_y * ay + vqa_z * az;
                        a[3] += (vq_w - dq * w) * inv_norm;
                        a[4] += (vq_x - dq * x) * inv_norm;
                        a[5] += (vq_y - dq * y) * inv_norm;
                        a[6] += (vq_z - dq * z) * inv_norm;
                        ab[3] += (vqa_w + dqa * aw) * inv_norm;
                        ab[4] += (vqa_x + dqa * ax) * inv_norm;
                        ab[5] += (vqa_y + dqa * ay) * inv_norm;
                        ab[6] += (vqa_z + dqa * az) * inv_norm;
                        for (int jj = 0; jj < 3; ++jj) {
                            a[7 + jj] += -is[jj] * is[jj] *
                                         (R[0][jj] * v_Mt[jj][0] + R[1][jj] * v_Mt[jj][1] + R[2][jj] * v_Mt[jj][2]);
                            ab[7 + jj] += is[jj] * is[jj] *
                                          (std::fabs(R[0][jj]) * v_Mt_abs[jj][0] + std::fabs(R[1][jj]) * v_Mt_abs[jj][1] +
                                           std::fabs(R[2][jj]) * v_Mt_abs[jj][2]);
                        }
                        a[13] += vis * v_alpha;
                        ab[13] += vis * v_alpha_abs;
                    }
                    for (int k = 0; k < 3; ++k) {
                        buffer[k] += rgb[k] * fac;
                        buffer_abs[k] += std::fabs(rgb[k] * fac);
                    }
                }
            }
        for (int32_t t = 0; t < cnt; ++t) {
            const int32_t g = flatten_ids[range_start + t];
            for (int k = 0; k < 14; ++k) {
                const double v = local[(size_t)t * 14 + k], vb = lbound[(size_t)t * 14 + k];
                if (vb != 0.0) {
#pragma omp atomic
                    grads[(size_t)g * 14 + k] += v;
#pragma omp atomic
                    bound[(size_t)g * 14 + k] += vb;
                }
            }
        }
    }
    return 0;
}

// =============================================================================================
// k9/k10  fused SSIM  src/training/kernels/ssim.cu:16-27 (window), :64-276 (fwd), :284-424 (bwd)
// Images are [B, CH, H, W].  dm_* may be null (train == false).
// The reference is compiled with --use_fast_math (fused multiply-adds wherever nvcc finds them, approximate
// quotients), so the bits of its sums and quotients are not defined by its source.  This restatement fixes one
// evaluation of the same expressions: taps in the reference's order (symmetric pairs from the centre outwards, then the
// centre; rows after columns), every accumulation a fused multiply-add, and the seven quotients of a pixel as
// products with the two IEEE reciprocals 1/A and 1/B.  Pinned by the float64 definitions, not by this choice.
// =============================================================================================
namespace {
const float cGauss[11] = {0.001028380123898387f, 0.0075987582094967365f, 0.036000773310661316f,
                          0.10936068743467331f,  0.21300552785396576f,   0.26601171493530273f,
                          0.21300552785396576f,  0.10936068743467331f,   0.036000773310661316f,
                          0.0075987582094967365f, 0.001028380123898387f};

inline float pix(const float* img, int64_t plane, int y, int x, int H, int W) {
    if (x < 0 || x >= W || y < 0 || y >= H)
        return 0.0f;
    return img[plane + (int64_t)y * W + x];
}
} // namespace

ORC_API int orc_fusedssim(int B, int CH, int H, int W, float C1, float C2, const float* img1, const float* img2,
                          float* ssim_map, float* dm_dmu1, float* dm_dsigma1_sq, float* dm_dsigma12) {
#pragma omp parallel for schedule(static)
    for (int64_t bc = 0; bc < (int64_t)B * CH; ++bc) {
        const int64_t plane = bc * H * W;
        // horizontal pass for every row (rows outside the image are all-zero, as the halo is)
        std::vector<float> xconv((size_t)H * W * 5);
        for (int y = 0; y < H; ++y)
            for (int x = 0; x < W; ++x) {
                float sumX = 0.f, sumX2 = 0.f, sumY = 0.f, sumY2 = 0.f, sumXY = 0.f;
                for (int d = 1; d <= 5; ++d) {
                    const float w = cGauss[5 - d];
                    const float Xl = pix(img1, plane, y, x - d, H, W), Yl = pix(img2, plane, y, x - d, H, W);
                    const float Xr = pix(img1, plane, y, x + d, H, W), Yr = pix(img2, plane, y, x + d, H, W);
                    sumX = gsx::fma(Xl + Xr, w, sumX);
                    sumX2 = gsx::fma(gsx::fma(Xl, Xl, Xr * Xr), w, sumX2);
                    sumY = gsx::fma(Yl + Yr, w, sumY);
                    sumY2 = gsx::fma(gsx::fma(Yl, Yl, Yr * Yr), w, sumY2);
                    sumXY = gsx::fma(gsx::fma(Xl, Yl, Xr * Yr), w, sumXY);
                }
                const float cX = pix(img1, plane, y, x, H, W), cY = pix(img2, plane, y, x, H, W);
                const float wc = cGauss[5];
                sumX = gsx::fma(cX, wc, sumX);
                sumX2 = gsx::fma(cX * cX, wc, sumX2);
                sumY = gsx::fma(cY, wc, sumY);
                sumY2 = gsx::fma(cY * cY, wc, sumY2);
                sumXY = gsx::fma(cX * cY, wc, sumXY);
                float* o = &xconv[((size_t)y * W + x) * 5];
                o[0] = sumX;
                o[1] = sumX2;
                o[2] = sumY;
                o[3] = sumY2;
                o[4] = sumXY;
            }
        const float zero5[5] = {0, 0, 0, 0, 0};
        for (int y = 0; y < H; ++y)
            for (int x = 0; x < W; ++x) {
                float out[5] = {0, 0, 0, 0, 0};
                for (int d = 1; d <= 5; ++d) {
                    const float w = cGauss[5 - d];
                    const float* top = (y - d >= 0) ? &xconv[((size_t)(y - d) * W + x) * 5] : zero5;
                    const float* bot = (y + d < H) ? &xconv[((size_t)(y + d) * W + x) * 5] : zero5;
                    for (int k = 0; k < 5; ++k)
                        out[k] = gsx::fma(top[k] + bot[k], w, out[k]);
                }
                const float* ctr = &xconv[((size_t)y * W + x) * 5];
                for (int k = 0; k < 5; ++k)
                    out[k] = gsx::fma(ctr[k], cGauss[5], out[k]);
                // ssim.cu:215-274 with the quotients as products of two reciprocals
                const float mu1 = out[0], mu2 = out[2];
                const float sigma1_sq = gsx::fma(-mu1, mu1, out[1]), sigma2_sq = gsx::fma(-mu2, mu2, out[3]);
                const float sigma12 = gsx::fma(-mu1, mu2, out[4]);
                const float A = gsx::fma(mu1, mu1, gsx::fma(mu2, mu2, C1));
                const float Bv = (sigma1_sq + sigma2_sq) + C2;
                const float two_mu1 = mu1 + mu1;
                const float C_ = gsx::fma(two_mu1, mu2, C1);
                const float D_ = gsx::fma(2.f, sigma12, C2);
                const float rA = 1.0f / A, rB = 1.0f / Bv;
                const float r = rA * rB;
                const float CD = C_ * D_;
                const int64_t gi = plane + (int64_t)y * W + x;
                ssim_map[gi] = CD * r;
                if (dm_dmu1) {
                    // 2 mu2 (D - C) / (A B) + 2 mu1 C D (1 / (A B B) - 1 / (A A B))
                    const float rrB = r * rB;
                    dm_dmu1[gi] = gsx::fma(two_mu1 * CD, rrB - r * rA, ((mu2 + mu2) * (D_ - C_)) * r);
                    dm_dsigma1_sq[gi] = -(CD * rrB);
                    dm_dsigma12[gi] = (C_ + C_) * r;
                }
            }
    }
    return 0;
}

ORC_API int orc_fusedssim_backward(int B, int CH, int H, int W, float C1, float C2, const float* img1,
                                   const float* img2, const float* dL_dmap, const float* dm_dmu1,
                                   const float* dm_dsigma1_sq, const float* dm_dsigma12, float* dL_dimg1) {
    (void)C1;
    (void)C2;
#pragma omp parallel for schedule(static)
    for (int64_t bc = 0; bc < (int64_t)B * CH; ++bc) {
        const int64_t plane = bc * H * W;
        std::vector<float> sc((size_t)H * W * 3);
        for (int y = 0; y < H; ++y)
            for (int x = 0; x < W; ++x) {
                float a0 = 0.f, a1 = 0.f, a2 = 0.f;
                auto fused = [&](int xx, float* f) {
                    const float chain = pix(dL_dmap, plane, y, xx, H, W);
                    f[0] = pix(dm_dmu1, plane, y, xx, H, W) * chain;
                    f[1] = pix(dm_dsigma1_sq, plane, y, xx, H, W) * chain;
                    f[2] = pix(dm_dsigma12, plane, y, xx, H, W) * chain;
                };
                for (int d = 1; d <= 5; ++d) {
                    const float w = cGauss[5 - d];
                    float l[3], r[3];
                    fused(x - d, l);
                    fused(x + d, r);
                    a0 = gsx::fma(l[0] + r[0], w, a0);
                    a1 = gsx::fma(l[1] + r[1], w, a1);
                    a2 = gsx::fma(l[2] + r[2], w, a2);
                }
                float c[3];
                fused(x, c);
                a0 = gsx::fma(c[0], cGauss[5], a0);
                a1 = gsx::fma(c[1], cGauss[5], a1);
                a2 = gsx::fma(c[2], cGauss[5], a2);
                float* o = &sc[((size_t)y * W + x) * 3];
                o[0] = a0;
                o[1] = a1;
                o[2] = a2;
            }
        const float zero3[3] = {0, 0, 0};
        for (int y = 0; y < H; ++y)
            for (int x = 0; x < W; ++x) {
                float s[3] = {0, 0, 0};
                for (int d = 1; d <= 5; ++d) {
                    const float w = cGauss[5 - d];
                    const float* top = (y - d >= 0) ? &sc[((size_t)(y - d) * W + x) * 3] : zero3;
                    const float* bot = (y + d < H) ? &sc[((size_t)(y + d) * W + x) * 3] : zero3;
                    for (int k = 0; k < 3; ++k)
                        s[k] = gsx::fma(top[k] + bot[k], w, s[k]);
                }
                const float* ctr = &sc[((size_t)y * W + x) * 3];
                for (int k = 0; k < 3; ++k)
                    s[k] = gsx::fma(ctr[k], cGauss[5], s[k]);
                const int64_t gi = plane + (int64_t)y * W + x;
                const float p1 = img1[gi], p2 = img2[gi];
                dL_dimg1[gi] = gsx::fma(p2, s[2], gsx::fma(p1 + p1, s[1], s[0]));
            }
    }
    return 0;
}

// =============================================================================================
// k11  adam_step_cu  src/training/fastgs/optimizer/include/adam_kernels.cuh:13-36
// bias corrections are computed by the caller in double and cast (fused_adam.cpp:78-92).
// =============================================================================================
ORC_API int orc_adam_step(float* param, float* exp_avg, float* exp_avg_sq, const float* grad, int64_t n, float lr,
                          float beta1, float beta2, float eps, float bias_correction1_rcp,
                          float bias_correction2_sqrt_rcp) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const float g = grad[i];
        const float moment1 = beta1 * exp_avg[i] + (1.0f - beta1) * g;
        const float moment2 = beta2 * exp_avg_sq[i] + (1.0f - beta2) * g * g;
        const float denom = gsx::sqrt(moment2) * bias_correction2_sqrt_rcp + eps;
        const float step_size = lr * bias_correction1_rcp;
        param[i] -= step_size * moment1 / denom;
        exp_avg[i] = moment1;
        exp_avg_sq[i] = moment2;
    }
    return 0;
}

// =============================================================================================
// k12  relocation_kernel  gsplat/RelocationCUDA.cu:11-43  (MCMC Eq. 9)
// =============================================================================================
ORC_API int orc_relocation(int M, const float* opacities, const float* scales, const int32_t* ratios,
                           const float* binoms, int n_max, float* new_opacities, float* new_scales) {
#pragma omp parallel for schedule(static)
    for (int idx = 0; idx < M; ++idx) {
        const int n_idx = ratios[idx];
        float denom_sum = 0.0f;
        const float new_o = 1.0f - gsx::pow(1.0f - opacities[idx], 1.0f / (float)n_idx);
        new_opacities[idx] = new_o;
        for (int i = 1; i <= n_idx; ++i)
            for (int k = 0; k <= (i - 1); ++k) {
                const float bin_coeff = binoms[(i - 1) * n_max + k];
                const float sgn = (k & 1) ? -1.0f : 1.0f; // pow(-1, k)
                const float term = (sgn / gsx::sqrt((float)(k + 1))) * gsx::pow(new_o, (float)(k + 1));
                denom_sum += (bin_coeff * term);
            }
        const float coeff = (opacities[idx] / denom_sum);
        for (int i = 0; i < 3; ++i)
            new_scales[idx * 3 + i] = coeff * scales[idx * 3 + i];
    }
    return 0;
}

// =============================================================================================
// k13  add_noise_kernel  gsplat/RelocationCUDA.cu:88-144
// =============================================================================================
ORC_API int orc_add_noise(int N, const float* raw_opacities, const float* raw_scales, const float* raw_quats,
                          const float* noise, float* means, float current_lr) {
#pragma omp parallel for schedule(static)
    for (int idx = 0; idx < N; ++idx) {
        const vec3 rs = ld3(raw_scales, idx);
        const float s2[3] = {gsx::exp(2.f * rs.x), gsx::exp(2.f * rs.y), gsx::exp(2.f * rs.z)};
        const mat3 R = gsx::quat_to_rotmat(ld4(raw_quats, idx), 1e+12f);
        // covariance = R * S2 * R^T ; (R*S2)(i,k) = R(i,k) s2[k]
        mat3 cov;
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j) {
                float a = (R.m[i][0] * s2[0]) * R.m[j][0];
                a = gsx::fma(R.m[i][1] * s2[1], R.m[j][1], a);
                a = gsx::fma(R.m[i][2] * s2[2], R.m[j][2], a);
                cov.m[i][j] = a;
            }
        const vec3 tn = gsx::mul(cov, ld3(noise, idx));
        const float opacity = 1.0f / (1.f + gsx::exp(-raw_opacities[idx]));
        const float op_sigmoid = 1.0f / (1.f + gsx::exp(100.f * opacity - 0.5f));
        const float noise_factor = current_lr * op_sigmoid;
        means[idx * 3] += noise_factor * tn.x;
        means[idx * 3 + 1] += noise_factor * tn.y;
        means[idx * 3 + 2] += noise_factor * tn.z;
    }
    return 0;
}

// =============================================================================================
// k14  quat_to_rotmat_kernel  gsplat/QuatToRotmatCUDA.cu:14-39  (row-major output)
// =============================================================================================
ORC_API int orc_quats_to_rotmats(int N, const float* quats, float* rotmats) {
#pragma omp parallel for schedule(static)
    for (int idx = 0; idx < N; ++idx) {
        const mat3 R = gsx::quat_to_rotmat(ld4(quats, idx));
        for (int i = 0; i < 3; ++i)
            for (int j = 0; j < 3; ++j)
                rotmats[idx * 9 + i * 3 + j] = R.m[i][j];
    }
    return 0;
}

// =============================================================================================
// g1  glue inside rasterize_from_world_with_sh_fwd  gsplat/Rasterization.cpp:327,356-378
// dirs = means - campos, colours = max(SH + 0.5, 0) for Gaussians with radii > 0, 0 otherwise.
// campos is the translation column of inverse(viewmat); for the rigid [R|t] matrices LichtFeld
// passes (src/core/camera.cpp:17-24) that is -R^T t, which is what is evaluated here (at::inverse
// runs a LU factorisation whose rounding is not reproducible; "parity unpinned" at the 1e-7 level).
// =============================================================================================
ORC_API int orc_sh_colors_from_world(uint32_t N, uint32_t K, uint32_t degree, const float* means,
                                     const float* sh_coeffs, const int32_t* radii, const float* viewmat,
                                     float* colors) {
    mat3 R;
    for (int r = 0; r < 3; ++r)
        for (int c = 0; c < 3; ++c)
            R.m[r][c] = viewmat[r * 4 + c];
    const vec3 t = gsx::mk3(viewmat[3], viewmat[7], viewmat[11]);
    const vec3 campos = gsx::neg(gsx::mul_t(R, t));
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < (int64_t)N; ++g) {
        if (!(radii[g * 2] > 0 && radii[g * 2 + 1] > 0)) {
            colors[g * 3] = colors[g * 3 + 1] = colors[g * 3 + 2] = 0.f;
            continue;
        }
        const vec3 dir = gsx::sub(ld3(means, g), campos);
        for (uint32_t c = 0; c < 3; ++c)
            colors[g * 3 + c] = gsx::fmax(sh_color(degree, dir, sh_coeffs + g * K * 3, c) + 0.5f, 0.0f);
    }
    return 0;
}

// backward of the same glue (Rasterization.cpp:608-624): v_coeffs = basis * (v_colors masked where
// colours <= 0), zero for culled Gaussians and for k >= (degree+1)^2.  v_coeffs is fully written.
ORC_API int orc_sh_colors_from_world_bwd(uint32_t N, uint32_t K, uint32_t degree, const float* means,
                                         const int32_t* radii, const float* viewmat, const float* colors,
                                         const float* v_colors, float* v_coeffs) {
    mat3 R;
    for (int r = 0; r < 3; ++r)
        for (int c = 0; c < 3; ++c)
            R.m[r][c] = viewmat[r * 4 + c];
    const vec3 t = gsx::mk3(viewmat[3], viewmat[7], viewmat[11]);
    const vec3 campos = gsx::neg(gsx::mul_t(R, t));
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < (int64_t)N; ++g) {
        float* out = v_coeffs + g * K * 3;
        for (uint32_t k = 0; k < K * 3; ++k)
            out[k] = 0.f;
        if (!(radii[g * 2] > 0 && radii[g * 2 + 1] > 0))
            continue;
        const vec3 dir = gsx::sub(ld3(means, g), campos);
        float B[25];
        const int nb = sh_basis(degree, dir, B);
        for (uint32_t c = 0; c < 3; ++c) {
            const float v = colors[g * 3 + c] <= 0.0f ? 0.0f : v_colors[g * 3 + c];
            for (int k = 0; k < nb; ++k)
                out[k * 3 + c] = B[k] * v;
        }
    }
    return 0;
}

// =============================================================================================
// a15  step-driver semantics around the boundary
// activations: SplatData getters, src/core/splat_data.cpp:271-286 (torch sigmoid / exp / normalize with eps 1e-12)
// and their VJPs (what LibTorch autograd applies to the gradients Ops.h's backward returns).
// =============================================================================================
ORC_API int orc_activate_params(uint32_t N, const float* opacity_raw, const float* scaling_raw,
                                const float* rotation_raw, float* opacities, float* scales, float* quats) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)N; ++i) {
        opacities[i] = gsx::sigmoid(opacity_raw[i]);
        for (int k = 0; k < 3; ++k)
            scales[3 * i + k] = gsx::exp(scaling_raw[3 * i + k]);
        const quat q = ld4(rotation_raw, i);
        const float nrm = gsx::fmax(gsx::sqrt(gsx::qdot(q, q)), 1e-12f);
        quats[4 * i + 0] = q.w / nrm;
        quats[4 * i + 1] = q.x / nrm;
        quats[4 * i + 2] = q.y / nrm;
        quats[4 * i + 3] = q.z / nrm;
    }
    return 0;
}

// regularization.cu:20-57 (exp) / 60-90 (sigmoid): loss = weight * mean(f(x)); grads += (weight / n) f'(x).
// mode 0: f = exp; mode 1: f = sigmoid.  The sum is taken in double (the kernels' block order is not part of the
// contract; the loss value is compared with a tolerance, the gradients bit for bit).
ORC_API double orc_l1_regularization(int mode, const float* params, float* grads, int64_t n, float weight) {
    if (weight == 0.0f || n <= 0)
        return 0.0;
    const float grad_scale = weight / (float)n;
    double sum = 0.0;
    for (int64_t i = 0; i < n; ++i) {
        float value, deriv;
        if (mode == 0) {
            value = gsx::exp(params[i]);
            deriv = value;
        } else {
            value = gsx::sigmoid(params[i]);
            deriv = value * (1.0f - value);
        }
        sum += (double)value;
        if (grads)
            grads[i] += grad_scale * deriv;
    }
    return (double)weight * (sum / (double)n);
}

ORC_API int orc_activate_params_bwd(uint32_t N, const float* opacity_raw, const float* scaling_raw,
                                    const float* rotation_raw, const float* v_opacities, const float* v_scales,
                                    const float* v_quats, float* v_opacity_raw, float* v_scaling_raw,
                                    float* v_rotation_raw) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)N; ++i) {
        const float o = gsx::sigmoid(opacity_raw[i]);
        v_opacity_raw[i] = v_opacities[i] * (o * (1.0f - o));
        for (int k = 0; k < 3; ++k)
            v_scaling_raw[3 * i + k] = v_scales[3 * i + k] * gsx::exp(scaling_raw[3 * i + k]);
        const quat q = ld4(rotation_raw, i);
        const quat g = ld4(v_quats, i);
        const float len = gsx::sqrt(gsx::qdot(q, q));
        if (len > 1e-12f) {
            const float inv = 1.0f / len;
            const float yw = q.w * inv, yx = q.x * inv, yy = q.y * inv, yz = q.z * inv;
            const float d = g.w * yw + g.x * yx + g.y * yy + g.z * yz;
            v_rotation_raw[4 * i + 0] = (g.w - yw * d) * inv;
            v_rotation_raw[4 * i + 1] = (g.x - yx * d) * inv;
            v_rotation_raw[4 * i + 2] = (g.y - yy * d) * inv;
            v_rotation_raw[4 * i + 3] = (g.z - yz * d) * inv;
        } else {
            v_rotation_raw[4 * i + 0] = g.w * 1e12f;
            v_rotation_raw[4 * i + 1] = g.x * 1e12f;
            v_rotation_raw[4 * i + 2] = g.y * 1e12f;
            v_rotation_raw[4 * i + 3] = g.z * 1e12f;
        }
    }
    return 0;
}

// photometric loss of trainer.cpp:126-129 around the rasterizer output:
// image = clamp(render[0] HWC -> CHW, 0, 1) (rasterizer.cpp:205); loss = (1-l) mean|image - gt| + l (1 - mean(ssim_valid))
// with the "valid" crop of fused_ssim.cuh:59-67.  Sums are formed in double.  Returns loss, l1, ssim in out[0..2],
// the clamped image, and (when v_render != nullptr) d loss / d render [H,W,3] including the SSIM backward
// (fused_ssim.cuh:74-102) and the clamp VJP.
ORC_API int orc_photometric_loss(uint32_t H, uint32_t W, float lambda_dssim, const float* render_hwc,
                                 const float* gt_chw, float* image_chw, double* out, float* v_render_hwc) {
    const int64_t HW = (int64_t)H * W;
    double l1 = 0.0;
#pragma omp parallel for schedule(static) reduction(+ : l1)
    for (int64_t p = 0; p < HW; ++p)
        for (int c = 0; c < 3; ++c) {
            const float r = render_hwc[p * 3 + c];
            const float v = gsx::fmin(gsx::fmax(r, 0.0f), 1.0f);
            image_chw[c * HW + p] = v;
            l1 += (double)gsx::fabs(v - gt_chw[c * HW + p]);
        }
    l1 /= (double)(3 * HW);
    double ss = 0.0;
    std::vector<float> map, d1, d2, d3;
    const bool crop = H > 10 && W > 10;
    const double count = crop ? 3.0 * (H - 10) * (W - 10) : 3.0 * H * W;
    if (lambda_dssim != 0.f) {
        map.resize(3 * HW), d1.resize(3 * HW), d2.resize(3 * HW), d3.resize(3 * HW);
        orc_fusedssim(1, 3, (int)H, (int)W, 0.01f * 0.01f, 0.03f * 0.03f, image_chw, gt_chw, map.data(), d1.data(),
                      d2.data(), d3.data());
        for (int c = 0; c < 3; ++c)
            for (uint32_t y = 0; y < H; ++y)
                for (uint32_t x = 0; x < W; ++x)
                    if (!crop || (y >= 5 && y < H - 5 && x >= 5 && x < W - 5))
                        ss += map[c * HW + (int64_t)y * W + x];
        ss /= count;
    }
    out[0] = (1.0 - lambda_dssim) * l1 + lambda_dssim * (1.0 - ss);
    out[1] = l1;
    out[2] = ss;
    if (v_render_hwc == nullptr)
        return 0;
    std::vector<float> dimg;
    if (lambda_dssim != 0.f) {
        std::vector<float> dmap(3 * HW, 0.f);
        const float sc = -lambda_dssim / (float)count;
        for (int c = 0; c < 3; ++c)
            for (uint32_t y = 0; y < H; ++y)
                for (uint32_t x = 0; x < W; ++x)
                    if (!crop || (y >= 5 && y < H - 5 && x >= 5 && x < W - 5))
                        dmap[c * HW + (int64_t)y * W + x] = sc;
        dimg.resize(3 * HW);
        orc_fusedssim_backward(1, 3, (int)H, (int)W, 0.01f * 0.01f, 0.03f * 0.03f, image_chw, gt_chw, dmap.data(),
                               d1.data(), d2.data(), d3.data(), dimg.data());
    }
    const float l1_scale = (1.f - lambda_dssim) / (3.f * (float)H * (float)W);
#pragma omp parallel for schedule(static)
    for (int64_t p = 0; p < HW; ++p)
        for (int c = 0; c < 3; ++c) {
            const float r = render_hwc[p * 3 + c];
            const float d = image_chw[c * HW + p] - gt_chw[c * HW + p];
            const float sgn = d > 0.f ? 1.f : (d < 0.f ? -1.f : 0.f);
            float g = l1_scale * sgn;
            if (!dimg.empty())
                g += dimg[c * HW + p];
            v_render_hwc[p * 3 + c] = (r >= 0.f && r <= 1.f) ? g : 0.f;
        }
    return 0;
}

// ---------------------------------------------------------------------------------------------
// primitive probes (so that tests can pin gsx_math.h against libm / numpy on arrays)
// ---------------------------------------------------------------------------------------------
ORC_API void orc_math_unary(int which, int64_t n, const float* x, float* y) {
    for (int64_t i = 0; i < n; ++i) {
        switch (which) {
        case 0: y[i] = gsx::exp(x[i]); break;
        case 1: y[i] = gsx::log(x[i]); break;
        case 2: y[i] = gsx::rsqrt(x[i]); break;
        case 3: y[i] = gsx::sin(x[i]); break;
        case 4: y[i] = gsx::acos(x[i]); break;
        case 5: y[i] = gsx::sigmoid(x[i]); break;
        case 6: y[i] = (float)gsx::sat_u32(x[i]); break;
        default: y[i] = 0.f;
        }
    }
}
ORC_API void orc_math_pow(int64_t n, const float* x, const float* e, float* y) {
    for (int64_t i = 0; i < n; ++i)
        y[i] = gsx::pow(x[i], e[i]);
}
// which: 7 pow, 8 x / x2, 9 sqrt(x), 10 fma(x, x2, x), 15 min_limit(x2, x)  (same numbering as the device probe)
// probes of the camera-model primitives of gsx_camera.h: 0 atan2(x, x2), 1 cbrt(x), 2 asin(x), 3 cos(x),
// 4 fisheye_max_angle_sq(x, x2, x3)
ORC_API void orc_math_camera(int which, int64_t n, const float* x, const float* x2, const float* x3, float* y) {
    for (int64_t i = 0; i < n; ++i) {
        switch (which) {
        case 0: y[i] = gsx::atan2(x[i], x2[i]); break;
        case 1: y[i] = gsx::cbrt(x[i]); break;
        case 2: y[i] = gsx::asin(x[i]); break;
        case 3: y[i] = gsx::cos(x[i]); break;
        default: y[i] = gsx::fisheye_max_angle_sq(x[i], x2[i], x3[i]); break;
        }
    }
}

ORC_API void orc_math_binary(int which, int64_t n, const float* x, const float* x2, float* y) {
    for (int64_t i = 0; i < n; ++i) {
        switch (which) {
        case 7: y[i] = gsx::pow(x[i], x2[i]); break;
        case 8: y[i] = x[i] / x2[i]; break;
        case 9: y[i] = gsx::sqrt(x[i]); break;
        case 10: y[i] = gsx::fma(x[i], x2[i], x[i]); break;
        case 15: y[i] = gsx::min_limit(x2[i], x[i]); break;
        default: y[i] = 0.f;
        }
    }
}
// quaternion helpers: which = 0 quat_cast(R row-major 9) -> q ; 1 mat3_cast(q) -> R ; 2 quat_to_rotmat(q) -> R ;
// 3 quat_rotate(q, v) (in = q4 + v3) -> v3 ; 4 slerp(q0, q1, a) (in = 9 floats) -> q
ORC_API void orc_math_quat(int which, const float* in, float* out) {
    if (which == 0) {
        mat3 R;
        for (int i = 0; i < 9; ++i)
            R.m[i / 3][i % 3] = in[i];
        const quat q = gsx::quat_cast(R);
        out[0] = q.w, out[1] = q.x, out[2] = q.y, out[3] = q.z;
    } else if (which == 1 || which == 2) {
        const quat q = ld4(in, 0);
        const mat3 R = which == 1 ? gsx::mat3_cast(q) : gsx::quat_to_rotmat(q);
        for (int i = 0; i < 9; ++i)
            out[i] = R.m[i / 3][i % 3];
    } else if (which == 3) {
        const vec3 v = gsx::quat_rotate(ld4(in, 0), gsx::mk3(in[4], in[5], in[6]));
        out[0] = v.x, out[1] = v.y, out[2] = v.z;
    } else if (which == 4) {
        const quat q = gsx::slerp(ld4(in, 0), ld4(in + 4, 0), in[8]);
        out[0] = q.w, out[1] = q.x, out[2] = q.y, out[3] = q.z;
    }
}

ORC_API int orc_num_threads(void) {
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}
ORC_API void orc_set_num_threads(int n) {
#if defined(_OPENMP)
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

// ---- conservativeness of the rasterizers' per-Gaussian pixel bounds (csrc/gsx_record.h) ----
// For each Gaussian: the bounds as the kernels compute them, and a brute-force pass over EVERY pixel of the image
// with the per-pair arithmetic of the forward pass above (RasterizeToPixelsFromWorld3DGSFwd.cu:228-246): how many
// pixels reach alpha >= 1/255 (true_count) and how many of those lie outside the bounds (violations, must be 0).
#include "gsx_record.h"

ORC_API int orc_record_bounds_check(uint32_t N, const float* means, const float* quats, const float* scales,
                                    const float* opacities, const float* viewmat, const float* Ks, uint32_t W,
                                    uint32_t H, int32_t* bounds, int64_t* true_count, int64_t* violations,
                                    int64_t* blocks_true, int64_t* blocks_hit) {
    const float fx = Ks[0], fy = Ks[4], cx = Ks[2], cy = Ks[5];
    const RollingShutter rs = make_rolling_shutter(viewmat, nullptr);
    const uint32_t bw = (W + 7) / 8, bh = (H + 7) / 8;
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t g = 0; g < (int64_t)N; ++g) {
        vec3 ray_o, ray_d;
        pixel_world_ray(0.5f, 0.5f, fx, fy, cx, cy, rs, &ray_o, &ray_d);
        const vec3 xyz = ld3(means, g);
        const mat3 M = gsx::record_whitening(ld4(quats, g), ld3(scales, g));
        const vec3 gro = gsx::mul(M, gsx::sub(ray_o, xyz));
        const gsx::RecordRegion b = gsx::record_region(gro, M, opacities[g], xyz, viewmat, fx, fy, cx, cy, W, H);
        bounds[g * 4 + 0] = b.jmin, bounds[g * 4 + 1] = b.imin, bounds[g * 4 + 2] = b.jmax, bounds[g * 4 + 3] = b.imax;
        int64_t cnt = 0, bad = 0, bt = 0, bhit = 0;
        std::vector<uint8_t> block_has(bw * bh, 0);
        for (uint32_t i = 0; i < H; ++i)
            for (uint32_t j = 0; j < W; ++j) {
                pixel_world_ray((float)j + 0.5f, (float)i + 0.5f, fx, fy, cx, cy, rs, &ray_o, &ray_d);
                const vec3 grd = gsx::safe_normalize(gsx::mul(M, ray_d));
                const vec3 gcrod = gsx::cross(grd, gro);
                const float power = -0.5f * gsx::dot(gcrod, gcrod);
                const float alpha = gsx::min_limit(0.999f, opacities[g] * gsx::exp(power));
                if (alpha < 1.f / 255.f)
                    continue;
                ++cnt;
                block_has[(i / 8) * bw + j / 8] = 1;
                if ((int32_t)j < b.jmin || (int32_t)j > b.jmax || (int32_t)i < b.imin || (int32_t)i > b.imax)
                    ++bad;
                if (power < b.cut)
                    ++bad; // the cut-off must lie below every contributing pair's power
            }
        for (uint32_t by = 0; by < bh; ++by)
            for (uint32_t bx = 0; bx < bw; ++bx) {
                const bool hit = gsx::record_region_hits_block(b.jmin, b.imin, b.jmax, b.imax, b.a00, b.a01, b.a11,
                                                               b.pcx, b.pcy, (int32_t)(by * 8), (int32_t)(bx * 8));
                bhit += hit;
                bt += block_has[by * bw + bx];
                if (block_has[by * bw + bx] && !hit)
                    ++bad;
            }
        true_count[g] = cnt;
        violations[g] = bad;
        blocks_true[g] = bt;
        blocks_hit[g] = bhit;
    }
    return 0;
}

// ---------------------------------------------------------------------------------------------
// camera model state and probes
// ---------------------------------------------------------------------------------------------
// radial [6], tangential [2], thin_prism [4], each nullable; all null = perfect pinhole.
ORC_API void orc_set_camera_model(int model, const float* radial, const float* tangential, const float* thin_prism,
                                  uint32_t W, uint32_t H);
ORC_API void orc_set_distortion(const float* radial, const float* tangential, const float* thin_prism) {
    orc_set_camera_model(0, radial, tangential, thin_prism, 0, 0);
}

// model: 0 pinhole (coefficients: radial [6], tangential [2], thin_prism [4]), 2 fisheye (radial [4]), 3
// equirectangular.  W, H: the image size (the fisheye and equirectangular unprojections need it).
ORC_API void orc_set_camera_model(int model, const float* radial, const float* tangential, const float* thin_prism,
                                  uint32_t W, uint32_t H) {
    g_model = model;
    g_W = W, g_H = H;
    g_dist = Distortion();
    g_fisheye_has_coeffs = model == 2 && radial != nullptr;
    if (model != 0) {
        for (int i = 0; i < 4 && radial && model == 2; ++i)
            g_dist.k[i] = radial[i];
        return;
    }
    g_dist.on = radial != nullptr || tangential != nullptr || thin_prism != nullptr;
    for (int i = 0; i < 6 && radial; ++i)
        g_dist.k[i] = radial[i];
    for (int i = 0; i < 2 && tangential; ++i)
        g_dist.p[i] = tangential[i];
    for (int i = 0; i < 4 && thin_prism; ++i)
        g_dist.s[i] = thin_prism[i];
}

ORC_API void orc_set_image_size(uint32_t W, uint32_t H) { g_W = W, g_H = H; }
ORC_API uint32_t orc_get_image_size(int axis) { return axis == 0 ? g_W : g_H; }

// rs_type: gsplat/Cameras.h:16-22 (4 = GLOBAL); viewmat1: the end-of-frame pose [4,4] or null (= the start pose)
ORC_API void orc_set_rolling_shutter(int rs_type, const float* viewmat1) {
    g_rs_type = rs_type;
    g_has_end_pose = viewmat1 != nullptr;
    if (viewmat1 != nullptr)
        std::memcpy(g_end_pose, viewmat1, sizeof(g_end_pose));
}

// world points [n,3] -> image points [n,2] + valid [n] under the current camera model and shutter, viewmat [4,4]
ORC_API void orc_world_project(int64_t n, const float* pts, const float* viewmat, float fx, float fy, float cx,
                               float cy, uint32_t W, uint32_t H, float margin, float* out, uint8_t* valid) {
    const RollingShutter rs = make_rolling_shutter(viewmat, nullptr);
    for (int64_t i = 0; i < n; ++i) {
        vec2 p;
        valid[i] = project_world_point_shutter(ld3(pts, i), rs, fx, fy, cx, cy, W, H, margin, &p) ? 1 : 0;
        out[2 * i] = p.x, out[2 * i + 1] = p.y;
    }
}

// pixel positions [n,2] -> world rays (origin [n,3], direction [n,3]) + valid [n] under the current model and shutter
ORC_API void orc_pixel_world_rays(int64_t n, const float* image_points, const float* viewmat, float fx, float fy,
                                  float cx, float cy, float* origins, float* dirs, uint8_t* valid) {
    const RollingShutter rs = make_rolling_shutter(viewmat, nullptr);
    for (int64_t i = 0; i < n; ++i) {
        vec3 o, d;
        valid[i] = pixel_world_ray(image_points[2 * i], image_points[2 * i + 1], fx, fy, cx, cy, rs, &o, &d) ? 1 : 0;
        origins[3 * i] = o.x, origins[3 * i + 1] = o.y, origins[3 * i + 2] = o.z;
        dirs[3 * i] = d.x, dirs[3 * i + 1] = d.y, dirs[3 * i + 2] = d.z;
    }
}

// camera-space points [n,3] -> image points [n,2] + valid [n] under the current camera model
ORC_API void orc_camera_project(int64_t n, const float* pts, float fx, float fy, float cx, float cy, uint32_t W,
                                uint32_t H, float margin, float* out, uint8_t* valid) {
    for (int64_t i = 0; i < n; ++i) {
        vec2 p;
        valid[i] = project_point(ld3(pts, i), fx, fy, cx, cy, W, H, margin, &p) ? 1 : 0;
        out[2 * i] = p.x, out[2 * i + 1] = p.y;
    }
}

// image points [n,2] -> unit camera rays [n,3] + valid [n] (identity pose) under the current camera model
ORC_API void orc_camera_unproject(int64_t n, const float* image_points, float fx, float fy, float cx, float cy,
                                  float* rays, uint8_t* valid) {
    const float eye[16] = {1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1};
    const RollingShutter rs = make_rolling_shutter(eye, nullptr);
    for (int64_t i = 0; i < n; ++i) {
        vec3 o, d;
        valid[i] = pixel_world_ray(image_points[2 * i], image_points[2 * i + 1], fx, fy, cx, cy, rs, &o, &d) ? 1 : 0;
        rays[3 * i] = d.x, rays[3 * i + 1] = d.y, rays[3 * i + 2] = d.z;
    }
}

// ---------------------------------------------------------------------------------------------
// counter-based normal draws: Philox4x32-10 (Salmon et al., SC'11; known-answer vectors of the Random123
// distribution in tests/test_oracle_loss_opt.py) + Box-Muller.  Stands in for torch::randn_like of mcmc.cpp:358,
// whose stream no implementation outside torch reproduces: "parity unpinned" against the reference's values, pinned
// as a generator (known answers, moments, Kolmogorov-Smirnov).
// ---------------------------------------------------------------------------------------------
ORC_API void orc_philox4x32_10(const uint32_t* ctr, const uint32_t* key, uint32_t* out) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
        c0 = n0, c1 = n1, c2 = n2, c3 = n3;
        k0 += 0x9E3779B9u, k1 += 0xBB67AE85u;
    }
    out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

ORC_API void orc_philox_randn3(uint32_t N, uint64_t seed, uint64_t offset, float* out) {
    const float scale = 5.9604644775390625e-8f; // 2^-24
    for (uint32_t i = 0; i < N; ++i) {
        const uint32_t ctr[4] = {i, (uint32_t)offset, (uint32_t)(offset >> 32), 0u};
        const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
        uint32_t u[4];
        orc_philox4x32_10(ctr, key, u);
        const float ra = gsx::sqrt(-2.0f * gsx::log((float)((u[0] >> 8) + 1u) * scale));
        const float rb = gsx::sqrt(-2.0f * gsx::log((float)((u[2] >> 8) + 1u) * scale));
        const float pa = 3.14159265358979323846f * (2.0f * ((float)(u[1] >> 8) * scale) - 1.0f);
        const float pb = 3.14159265358979323846f * (2.0f * ((float)(u[3] >> 8) * scale) - 1.0f);
        out[3 * (size_t)i] = ra * gsx::cos(pa);
        out[3 * (size_t)i + 1] = ra * gsx::sin(pa);
        out[3 * (size_t)i + 2] = rb * gsx::cos(pb);
    }
}
