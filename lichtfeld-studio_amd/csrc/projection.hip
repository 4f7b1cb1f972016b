// projection.hip - per-Gaussian streaming kernels: unscented-transform projection, spherical harmonics
// forward/backward, quaternion -> rotation matrix, parameter activations.
//
// All of these touch each Gaussian once and are bound by HBM bandwidth; one lane owns one Gaussian and
// rows are read with whole-row vector loads.
#include <string.h>

#include "gsx_common.h"
#include "gsx_step.h"

namespace gsx {

static constexpr float kAlphaThreshold = 1.f / 255.f; // gsplat/Common.h:54

// ---------------------------------------------------------------------------------------------
// Unscented-transform projection of one Gaussian (gsplat/ProjectionUT3DGSFused.cu:47-210,
// gsplat/Cameras.cuh:1064-1186, 416-455).  Returns false when the Gaussian is culled.
// ---------------------------------------------------------------------------------------------
struct ProjOut {
    float rx, ry;     // radii (already ceil'ed)
    float mx, my;     // mean2d
    float depth;      // camera z of the mean under the centre-of-shutter pose
    float c0, c1, c2; // conic
    float compensation;
};

struct ProjCfg {
    uint32_t W, H;
    float eps2d, near_plane, far_plane, radius_clip;
    float ut_alpha, ut_beta, ut_kappa, ut_margin;
    int ut_require_all;
    // sigma-point spread and weights (Cameras.cuh:1070-1119), the same for every Gaussian: formed once on the host
    // from the three parameters above with correctly rounded fp32 operations (what the device would compute)
    float ut_sq, ut_w0m, ut_w0c, ut_wi;
    float fx, fy, cx, cy;
    CameraModel cam; // type 0 with cam.dist.on = false: the perfect pinhole model
};

__device__ __forceinline__ bool pinhole_project(vec3 cam, const ProjCfg& cfg, vec2* out) {
    out->x = 0.f;
    out->y = 0.f;
    if (cam.z <= 0.f)
        return false;
    out->x = (cam.x / cam.z) * cfg.fx + cfg.cx;
    out->y = (cam.y / cam.z) * cfg.fy + cfg.cy;
    const float mx = (float)cfg.W * cfg.ut_margin;
    const float my = (float)cfg.H * cfg.ut_margin;
    bool valid = true;
    valid &= (-mx) <= out->x && out->x < ((float)cfg.W + mx);
    valid &= (-my) <= out->y && out->y < ((float)cfg.H + my);
    return valid;
}

// Cameras.cuh:535-597: camera_ray_to_image_point of the distorted model
__device__ __forceinline__ bool opencv_project(vec3 cam, const ProjCfg& cfg, vec2* out) {
    out->x = 0.f;
    out->y = 0.f;
    if (cam.z <= 0.f)
        return false;
    const float u = cam.x / cam.z, v = cam.y / cam.z;
    float icD, dx, dy;
    compute_distortion(cfg.cam.dist, u, v, &icD, &dx, &dy);
    const bool valid_radial = icD > 0.8f;
    out->x = (icD * u + dx) * cfg.fx + cfg.cx;
    out->y = (icD * v + dy) * cfg.fy + cfg.cy;
    const float mx = (float)cfg.W * cfg.ut_margin;
    const float my = (float)cfg.H * cfg.ut_margin;
    bool valid = valid_radial;
    valid &= (-mx) <= out->x && out->x < ((float)cfg.W + mx);
    valid &= (-my) <= out->y && out->y < ((float)cfg.H + my);
    return valid;
}

// camera_ray_to_image_point of the configured model
template <bool GENERAL>
__device__ __forceinline__ bool project_cam_point(const ProjCfg& cfg, vec3 pc, vec2* uv) {
    if (GENERAL) {
        if (cfg.cam.type == 2)
            return fisheye_project(cfg.cam.fe, pc, cfg.ut_margin, uv);
        if (cfg.cam.type == 3) {
            equirect_project((float)cfg.W, (float)cfg.H, pc, uv);
            return true; // Cameras.cuh:1013-1025 returns valid for every point
        }
        if (cfg.cam.dist.on)
            return opencv_project(pc, cfg, uv);
    }
    return pinhole_project(pc, cfg, uv);
}

// world_point_to_image_point_shutter_pose (Cameras.cuh:346-414).  Global shutter: the start pose's projection.
// Rolling shutter: from the start-pose projection (the end-pose one if only that is valid; neither valid = invalid)
// ten passes of "exposure time of the current image point -> pose -> projection"; the last point is returned as
// valid.  One loop, one projection call site: pass 0 = start pose, 1 = end pose, 2 .. 11 = the iteration.
template <bool GENERAL>
__device__ __forceinline__ bool project_world_point(const ProjCfg& cfg, const CamPose& cp, vec3 p, vec2* uv) {
    if (!GENERAL || cp.rs_type == GSX_GLOBAL)
        return project_cam_point<GENERAL>(cfg, add(quat_rotate(cp.q_start, p), cp.t_start), uv);
    vec2 prev = {0.f, 0.f}, p_start = {0.f, 0.f};
    bool valid_start = false;
#pragma unroll 1
    for (int pass = 0; pass < 12; ++pass) {
        quat q = cp.q_start;
        vec3 t = cp.t_start;
        if (pass == 1) {
            q = cp.q_end;
            t = cp.t_end;
        } else if (pass > 1) {
            shutter_pose(cp, shutter_relative_frame_time(cp, prev.x, prev.y), &q, &t);
        }
        vec2 pt;
        const bool pv = project_cam_point<GENERAL>(cfg, add(quat_rotate(q, p), t), &pt);
        if (pass == 0) {
            p_start = pt;
            valid_start = pv;
        } else if (pass == 1) {
            if (valid_start) {
                prev = p_start;
            } else if (pv) {
                prev = pt;
            } else {
                *uv = pt;
                return false;
            }
        } else {
            prev = pt;
        }
    }
    *uv = prev;
    return true;
}

// GENERAL = false: the perfect pinhole with a global shutter (the training step's camera), decided at compile time
// Rc: mat3_cast(cp.q_start), read by the GENERAL = false instance only (its sigma points go through the pose as a
// matrix, gsx_camera.h ut_sigma_points_camera)
template <bool GENERAL>
__device__ __forceinline__ bool project_ut(const ProjCfg& cfg, const CamPose& cp, quat qc, vec3 tc, const mat3& Rc,
                                           vec3 mean, quat q_in, vec3 scl, bool has_opacity, float opacity_in,
                                           ProjOut* o) {
    // qc, tc: the centre-of-shutter pose shutter_pose(cp, 0.5) (ProjectionUT3DGSFused.cu:76-77)
    const quat q = quat_normalize(q_in);
    // one pose for the whole frame: the centre-of-shutter pose is the start pose, and the mean in camera coordinates
    // is the first sigma point
    const vec3 mean_c = GENERAL ? add(quat_rotate(qc, mean), tc) : add(mul(Rc, mean), cp.t_start);
    // the equirectangular model sees behind the camera (ProjectionUT3DGSFused.cu:78)
    if ((mean_c.z < cfg.near_plane && !(GENERAL && cfg.cam.type == 3)) || mean_c.z > cfg.far_plane)
        return false;

    const mat3 Rg = mat3_cast(q);
    const float sq = cfg.ut_sq, w0m = cfg.ut_w0m, w0c = cfg.ut_w0c, wi = cfg.ut_wi;
    const float sc[3] = {scl.x, scl.y, scl.z};

    vec2 ip[7];
    vec2 m2 = {0.f, 0.f};
    bool valid = cfg.ut_require_all != 0;
    vec3 pc[7]; // the sigma points in camera coordinates (perfect pinhole, one pose)
    if (!GENERAL)
        ut_sigma_points_camera(Rc, cp.t_start, mean, Rg, scl, sq, pc);
#pragma unroll
    for (int i = 0; i < 7; ++i) {
        vec2 uv;
        bool pv;
        if (GENERAL) {
            vec3 p;
            if (i == 0) {
                p = mean;
            } else {
                const int a = (i - 1) % 3;
                const float s = sq * sc[a];
                const vec3 delta = mk3(s * Rg.m[0][a], s * Rg.m[1][a], s * Rg.m[2][a]);
                p = (i <= 3) ? add(mean, delta) : sub(mean, delta);
            }
            pv = project_world_point<GENERAL>(cfg, cp, p, &uv);
        } else {
            pv = pinhole_project_point(pc[i], cfg.fx, cfg.fy, cfg.cx, cfg.cy, (float)cfg.W, (float)cfg.H,
                                       cfg.ut_margin, &uv);
        }
        if (cfg.ut_require_all) {
            valid &= pv;
            if (!pv)
                return false;
        } else {
            valid |= pv;
        }
        ip[i] = uv;
        const float w = (i == 0) ? w0m : wi;
        m2.x += w * uv.x;
        m2.y += w * uv.y;
    }
    if (!valid)
        return false;
    float c00 = 0.f, c01 = 0.f, c11 = 0.f;
#pragma unroll
    for (int i = 0; i < 7; ++i) {
        const float w = (i == 0) ? w0c : wi;
        const float dx = ip[i].x - m2.x, dy = ip[i].y - m2.y;
        c00 += w * (dx * dx);
        c01 += w * (dx * dy);
        c11 += w * (dy * dy);
    }
    // add_blur (gsplat/Utils.cuh:171-179)
    const float det_orig = c00 * c11 - c01 * c01;
    c00 += cfg.eps2d;
    c11 += cfg.eps2d;
    const float det = c00 * c11 - c01 * c01;
    const float compensation = gsx::sqrt(gsx::fmax(0.f, det_orig / det));
    if (det <= 0.f)
        return false;
    const float ood = 1.0f / det;

    float extend = 3.33f;
    if (has_opacity) {
        const float opacity = opacity_in * compensation;
        if (opacity < kAlphaThreshold)
            return false;
        extend = gsx::fmin(extend, gsx::sqrt(2.0f * gsx::log(opacity / kAlphaThreshold)));
    }
    const float b = 0.5f * (c00 + c11);
    const float tmp = gsx::sqrt(gsx::fmax(0.01f, b * b - det));
    const float v1 = b + tmp;
    const float r1 = extend * gsx::sqrt(v1);
    const float radius_x = gsx::ceil(gsx::fmin(extend * gsx::sqrt(c00), r1));
    const float radius_y = gsx::ceil(gsx::fmin(extend * gsx::sqrt(c11), r1));
    if (radius_x <= cfg.radius_clip && radius_y <= cfg.radius_clip)
        return false;
    if (m2.x + radius_x <= 0 || m2.x - radius_x >= (float)cfg.W || m2.y + radius_y <= 0 ||
        m2.y - radius_y >= (float)cfg.H)
        return false;
    o->rx = radius_x;
    o->ry = radius_y;
    o->mx = m2.x;
    o->my = m2.y;
    o->depth = mean_c.z;
    o->c0 = c11 * ood;
    o->c1 = -c01 * ood;
    o->c2 = c00 * ood;
    o->compensation = compensation;
    return true;
}

// The pose of the one perfect-pinhole, global-shutter camera for a whole workgroup: the first wave derives it from
// the view matrix (quaternion of its rotation, rotation matrix of that quaternion - a few hundred instructions whose
// results are the same for every lane of the launch) and every lane reads it back from LDS.  Every thread of the
// workgroup must call it.  Of `cp` only the start translation is set, and qc / tc are the identity: the plain
// instance of project_ut reads nothing else.
struct WorkgroupPose {
    CamPose cp;
    quat qc;
    vec3 tc;
    mat3 Rc;
};
__device__ __forceinline__ WorkgroupPose workgroup_pose(const float* __restrict__ viewmat) {
    __shared__ float s[12];
    if (threadIdx.x < 64u) {
        const CamPose cp = load_cam_pose(viewmat);
        const mat3 Rc = mat3_cast(cp.q_start);
        if (threadIdx.x == 0) {
            s[0] = cp.t_start.x, s[1] = cp.t_start.y, s[2] = cp.t_start.z;
#pragma unroll
            for (int r = 0; r < 3; ++r)
#pragma unroll
                for (int c = 0; c < 3; ++c)
                    s[3 + 3 * r + c] = Rc.m[r][c];
        }
    }
    __syncthreads();
    WorkgroupPose p;
    p.qc.w = 1.f, p.qc.x = 0.f, p.qc.y = 0.f, p.qc.z = 0.f;
    p.tc = mk3(0.f, 0.f, 0.f);
    p.cp.q_start = p.qc, p.cp.q_end = p.qc;
    p.cp.t_start = mk3(s[0], s[1], s[2]);
    p.cp.t_end = p.cp.t_start;
    p.cp.rs_type = GSX_GLOBAL;
    p.cp.W = 0, p.cp.H = 0;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 3; ++c)
            p.Rc.m[r][c] = s[3 + 3 * r + c];
    return p;
}

// GENERAL = false: every camera a perfect pinhole with a global shutter (no coefficient rows, no end-of-frame pose)
template <bool GENERAL>
__global__ void __launch_bounds__(256) projection_ut_kernel(
    uint32_t C, uint32_t N, const float* __restrict__ means, const float* __restrict__ quats,
    const float* __restrict__ scales, const float* __restrict__ opacities, const float* __restrict__ viewmats0,
    const float* __restrict__ viewmats1, int rs_type, const float* __restrict__ Ks, int camera_model,
    const float* __restrict__ radial, const float* __restrict__ tangential, const float* __restrict__ thin_prism,
    ProjCfg cfg,
    int32_t* __restrict__ radii, float* __restrict__ means2d,
    float* __restrict__ depths, float* __restrict__ conics, float* __restrict__ compensations) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    WorkgroupPose wp;
    if (!GENERAL)
        wp = workgroup_pose(viewmats0); // one camera (check_camera_args)
    if (idx >= C * N)
        return;
    const uint32_t cid = idx / N, gid = idx % N;
    cfg.fx = Ks[cid * 9 + 0];
    cfg.fy = Ks[cid * 9 + 4];
    cfg.cx = Ks[cid * 9 + 2];
    cfg.cy = Ks[cid * 9 + 5];
    if (GENERAL) {
        const uint32_t n_radial = camera_model == GSX_FISHEYE ? 4u : 6u; // ProjectionUT3DGSFused.cu:103, 124
        cfg.cam = load_camera_model(camera_model, radial != nullptr ? radial + cid * n_radial : nullptr,
                                    tangential != nullptr ? tangential + cid * 2 : nullptr,
                                    thin_prism != nullptr ? thin_prism + cid * 4 : nullptr, cfg.fx, cfg.fy, cfg.cx,
                                    cfg.cy, cfg.W, cfg.H);
    }
    ProjOut o;
    if (GENERAL) {
        wp.cp = load_cam_pose(viewmats0 + cid * 16, viewmats1 != nullptr ? viewmats1 + cid * 16 : nullptr, rs_type,
                              cfg.W, cfg.H);
        shutter_pose(wp.cp, 0.5f, &wp.qc, &wp.tc);
    }
    const bool ok = project_ut<GENERAL>(cfg, wp.cp, wp.qc, wp.tc, wp.Rc, ld3(means, gid), ld4q(quats, gid), ld3(scales, gid), opacities != nullptr,
                               opacities != nullptr ? opacities[gid] : 0.f, &o);
    int2* r2 = reinterpret_cast<int2*>(radii);
    if (!ok) {
        r2[idx] = make_int2(0, 0);
        return;
    }
    r2[idx] = make_int2((int32_t)o.rx, (int32_t)o.ry);
    reinterpret_cast<float2*>(means2d)[idx] = make_float2(o.mx, o.my);
    depths[idx] = o.depth;
    conics[idx * 3 + 0] = o.c0;
    conics[idx * 3 + 1] = o.c1;
    conics[idx * 3 + 2] = o.c2;
    if (compensations != nullptr)
        compensations[idx] = o.compensation;
}

// activate_params + projection in one pass (C == 1): raw parameters in, activated parameters and the projection
// outputs out - the same values as the two separate kernels.
// 512 lanes a workgroup: the pose costs one wave in eight its few hundred instructions
__global__ void __launch_bounds__(512) projection_ut_raw_kernel(
    uint32_t N, const float* __restrict__ means, const float* __restrict__ opacity_raw,
    const float* __restrict__ scaling_raw, const float* __restrict__ rotation_raw,
    const float* __restrict__ viewmat, const float* __restrict__ Ks, ProjCfg cfg, float* __restrict__ opacities,
    float* __restrict__ scales, float* __restrict__ quats, int32_t* __restrict__ radii, float* __restrict__ means2d,
    float* __restrict__ depths, float* __restrict__ conics) {
    const uint32_t idx = blockIdx.x * 512u + threadIdx.x;
    const WorkgroupPose wp = workgroup_pose(viewmat);
    if (idx >= N)
        return;
    const Activated a = activate(opacity_raw[idx], ld3(scaling_raw, idx), ld4q(rotation_raw, idx));
    opacities[idx] = a.opacity;
    scales[3 * idx + 0] = a.scales.x;
    scales[3 * idx + 1] = a.scales.y;
    scales[3 * idx + 2] = a.scales.z;
    reinterpret_cast<float4*>(quats)[idx] = make_float4(a.quat.w, a.quat.x, a.quat.y, a.quat.z);
    cfg.fx = Ks[0];
    cfg.fy = Ks[4];
    cfg.cx = Ks[2];
    cfg.cy = Ks[5];
    ProjOut o;
    const bool ok = project_ut<false>(cfg, wp.cp, wp.qc, wp.tc, wp.Rc, ld3(means, idx), a.quat, a.scales, true,
                                      a.opacity, &o);
    int2* r2 = reinterpret_cast<int2*>(radii);
    if (!ok) {
        r2[idx] = make_int2(0, 0);
        return;
    }
    r2[idx] = make_int2((int32_t)o.rx, (int32_t)o.ry);
    reinterpret_cast<float2*>(means2d)[idx] = make_float2(o.mx, o.my);
    depths[idx] = o.depth;
    if (conics != nullptr) {
        conics[idx * 3 + 0] = o.c0;
        conics[idx * 3 + 1] = o.c1;
        conics[idx * 3 + 2] = o.c2;
    }
}

// ---------------------------------------------------------------------------------------------
// Spherical harmonics (gsplat/SphericalHarmonicsCUDA.cu:20-110): basis values and the colour of one
// channel in the reference's summation order.
// ---------------------------------------------------------------------------------------------
// co: the Gaussian's coefficients, element (k, c) at co[k * 3 + c]
__device__ __forceinline__ float sh_color_channel(uint32_t degree, vec3 dir, const float* B,
                                                  const float* __restrict__ co, uint32_t c) {
    float result = 0.2820947917738781f * co[c];
    if (degree >= 1) {
        // same value as B[1..3] folded: 0.4886 * (-y k1 + z k2 - x k3), in the reference's order
        const float inorm = gsx::rsqrt(dir.x * dir.x + dir.y * dir.y + dir.z * dir.z);
        const float x = dir.x * inorm, y = dir.y * inorm, z = dir.z * inorm;
        result += 0.48860251190292f * (-y * co[1 * 3 + c] + z * co[2 * 3 + c] - x * co[3 * 3 + c]);
        if (degree >= 2) {
            result += B[4] * co[4 * 3 + c] + B[5] * co[5 * 3 + c] + B[6] * co[6 * 3 + c] + B[7] * co[7 * 3 + c] +
                      B[8] * co[8 * 3 + c];
            if (degree >= 3) {
                result += B[9] * co[9 * 3 + c] + B[10] * co[10 * 3 + c] + B[11] * co[11 * 3 + c] +
                          B[12] * co[12 * 3 + c] + B[13] * co[13 * 3 + c] + B[14] * co[14 * 3 + c] +
                          B[15] * co[15 * 3 + c];
                if (degree >= 4) {
                    result += B[16] * co[16 * 3 + c] + B[17] * co[17 * 3 + c] + B[18] * co[18 * 3 + c] +
                              B[19] * co[19 * 3 + c] + B[20] * co[20 * 3 + c] + B[21] * co[21 * 3 + c] +
                              B[22] * co[22 * 3 + c] + B[23] * co[23 * 3 + c] + B[24] * co[24 * 3 + c];
                }
            }
        }
    }
    return result;
}

// direction gradient, accumulated over the three channels
// (sh_coeffs_to_color_fast_vjp with v_dir != nullptr; the reference adds the channels with atomics, :474-478)
__global__ void __launch_bounds__(256) sh_bwd_dirs_kernel(uint32_t N, uint32_t K, uint32_t degree,
                                                           const float* __restrict__ dirs,
                                                           const float* __restrict__ coeffs,
                                                           const uint8_t* __restrict__ masks,
                                                           const float* __restrict__ v_colors,
                                                           float* __restrict__ v_dirs) {
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    if (e >= N)
        return;
    if (masks != nullptr && !masks[e])
        return;
    const vec3 dir = ld3(dirs, e);
    float vx = 0.f, vy = 0.f, vz = 0.f;
    if (degree >= 1) {
        const float inorm = gsx::rsqrt(dir.x * dir.x + dir.y * dir.y + dir.z * dir.z);
        const float x = dir.x * inorm, y = dir.y * inorm, z = dir.z * inorm;
        const float* co = coeffs + (size_t)e * K * 3;
        for (uint32_t c = 0; c < 3; ++c) {
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

__global__ void __launch_bounds__(256) quats_to_rotmats_kernel(uint32_t N, const float* __restrict__ quats,
                                                                float* __restrict__ rotmats) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= N)
        return;
    const mat3 R = quat_to_rotmat(ld4q(quats, idx));
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j)
            rotmats[(size_t)idx * 9 + i * 3 + j] = R.m[i][j];
}

// SplatData getters (src/core/splat_data.cpp:271-286) in one pass
__global__ void __launch_bounds__(256) activate_params_kernel(uint32_t N, const float* __restrict__ opacity_raw,
                                                               const float* __restrict__ scaling_raw,
                                                               const float* __restrict__ rotation_raw,
                                                               float* __restrict__ opacities,
                                                               float* __restrict__ scales, float* __restrict__ quats) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= N)
        return;
    const Activated a = activate(opacity_raw[i], ld3(scaling_raw, i), ld4q(rotation_raw, i));
    opacities[i] = a.opacity;
    scales[3 * i + 0] = a.scales.x;
    scales[3 * i + 1] = a.scales.y;
    scales[3 * i + 2] = a.scales.z;
    reinterpret_cast<float4*>(quats)[i] = make_float4(a.quat.w, a.quat.x, a.quat.y, a.quat.z);
}

// VJPs of the three activations (what autograd applies to the gradients Ops.h's backward returns)
__global__ void __launch_bounds__(256) activate_params_bwd_kernel(
    uint32_t N, const float* __restrict__ opacity_raw, const float* __restrict__ scaling_raw,
    const float* __restrict__ rotation_raw, const float* __restrict__ v_opacities, const float* __restrict__ v_scales,
    const float* __restrict__ v_quats, float* __restrict__ v_opacity_raw, float* __restrict__ v_scaling_raw,
    float* __restrict__ v_rotation_raw) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= N)
        return;
    const vec3 vs = ld3(v_scales, i);
    const ActivationVjp a = activation_vjp(opacity_raw[i], ld3(scaling_raw, i), ld4q(rotation_raw, i), v_opacities[i],
                                           vs, ld4q(v_quats, i));
    v_opacity_raw[i] = a.opacity;
    v_scaling_raw[3 * i + 0] = a.scaling.x;
    v_scaling_raw[3 * i + 1] = a.scaling.y;
    v_scaling_raw[3 * i + 2] = a.scaling.z;
    reinterpret_cast<float4*>(v_rotation_raw)[i] = make_float4(a.rotation.w, a.rotation.x, a.rotation.y, a.rotation.z);
}

// glue of the fused entry point (Rasterization.cpp:356-378): dirs, radii mask, SH, +0.5, clamp in one pass.
// WORLD: dirs = means - campos, radii mask, +0.5 and clamp; otherwise the plain operator with an optional mask.
// LDS16: K == 16 and 16-byte aligned coefficients, rows staged through LDS.
template <bool WORLD, bool LDS16>
__global__ void __launch_bounds__(256) sh_fwd_generic_kernel(uint32_t N, uint32_t K, uint32_t degree,
                                                              const float* __restrict__ dirs_or_means,
                                                              const float* __restrict__ coeffs,
                                                              const uint8_t* __restrict__ masks,
                                                              const int32_t* __restrict__ radii,
                                                              const float* __restrict__ viewmat,
                                                              float* __restrict__ colors) {
    __shared__ float4 lds[LDS16 ? 4 * 64 * kShLdsF4 : 1];
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    float4* wave_lds = lds + (LDS16 ? wave * 64 * kShLdsF4 : 0);
    if (LDS16) {
        const uint32_t row0 = blockIdx.x * 256u + wave * 64u;
        if (row0 < N)
            sh16_rows_to_lds(coeffs, row0, N, wave_lds, lane);
        __builtin_amdgcn_wave_barrier();
    }
    if (e >= N)
        return;
    bool live;
    if (WORLD) { // both radii with one 8-byte load (two loads behind `&&` are two round trips in a row)
        const int2 rad = reinterpret_cast<const int2*>(radii)[e];
        live = rad.x > 0 && rad.y > 0;
    } else {
        live = masks == nullptr || masks[e];
    }
    if (!live) {
        if (WORLD) {
            colors[e * 3 + 0] = 0.f;
            colors[e * 3 + 1] = 0.f;
            colors[e * 3 + 2] = 0.f;
        }
        return;
    }
    vec3 dir = ld3(dirs_or_means, e);
    if (WORLD)
        dir = sub(dir, campos_from_viewmat(viewmat));
    float B[25];
    sh_basis(degree, dir, B);
    float co_reg[48];
    const float* co;
    if (LDS16) {
#pragma unroll
        for (uint32_t j = 0; j < kShRowF4; ++j) {
            const float4 t = wave_lds[lane * kShLdsF4 + j];
            co_reg[4 * j + 0] = t.x;
            co_reg[4 * j + 1] = t.y;
            co_reg[4 * j + 2] = t.z;
            co_reg[4 * j + 3] = t.w;
        }
        co = co_reg;
    } else {
        co = coeffs + (size_t)e * K * 3;
    }
#pragma unroll
    for (uint32_t c = 0; c < 3; ++c) {
        float v = sh_color_channel(degree, dir, B, co, c);
        if (WORLD)
            v = gsx::fmax(v + 0.5f, 0.0f);
        colors[e * 3 + c] = v;
    }
}

template <bool WORLD, bool LDS16>
__global__ void __launch_bounds__(256) sh_bwd_generic_kernel(uint32_t N, uint32_t K, uint32_t degree,
                                                              const float* __restrict__ dirs_or_means,
                                                              const uint8_t* __restrict__ masks,
                                                              const int32_t* __restrict__ radii,
                                                              const float* __restrict__ viewmat,
                                                              const float* __restrict__ colors,
                                                              const float* __restrict__ v_colors,
                                                              float* __restrict__ v_coeffs) {
    __shared__ float4 lds[LDS16 ? 4 * 64 * kShLdsF4 : 1];
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    float4* wave_lds = lds + (LDS16 ? wave * 64 * kShLdsF4 : 0);
    float B[25];
    int nb = 0;
    float v[3] = {0.f, 0.f, 0.f};
    if (e < N) {
        bool live;
        if (WORLD) {
            const int2 rad = reinterpret_cast<const int2*>(radii)[e];
            live = rad.x > 0 && rad.y > 0;
        } else {
            live = masks == nullptr || masks[e];
        }
        if (live) {
            vec3 dir = ld3(dirs_or_means, e);
            if (WORLD)
                dir = sub(dir, campos_from_viewmat(viewmat));
            nb = sh_basis(degree, dir, B);
#pragma unroll
            for (int c = 0; c < 3; ++c) {
                v[c] = v_colors[e * 3 + c];
                if (WORLD && colors[e * 3 + c] <= 0.0f) // clamp VJP (Rasterization.cpp:609-610)
                    v[c] = 0.f;
            }
        }
    }
    if (LDS16) {
        float o[48];
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const bool used = k < nb;
            o[k * 3 + 0] = used ? B[k] * v[0] : 0.f;
            o[k * 3 + 1] = used ? B[k] * v[1] : 0.f;
            o[k * 3 + 2] = used ? B[k] * v[2] : 0.f;
        }
#pragma unroll
        for (uint32_t j = 0; j < kShRowF4; ++j)
            wave_lds[lane * kShLdsF4 + j] = make_float4(o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
        __builtin_amdgcn_wave_barrier();
        const uint32_t row0 = blockIdx.x * 256u + wave * 64u;
        if (row0 < N)
            sh16_rows_from_lds(v_coeffs, row0, N, wave_lds, lane);
        return;
    }
    if (e >= N)
        return;
    float* out = v_coeffs + (size_t)e * K * 3;
    for (uint32_t k = 0; k < K; ++k) {
        const bool used = (int)k < nb;
        const float b = B[k < 25 ? k : 24];
        out[k * 3 + 0] = used ? b * v[0] : 0.f;
        out[k * 3 + 1] = used ? b * v[1] : 0.f;
        out[k * 3 + 2] = used ? b * v[2] : 0.f;
    }
}

// A wave's 64 consecutive coefficient rows (K = 16: 48 floats each, 16-byte aligned) -> the 48 coefficients of
// every live lane's own row in registers.  Rows are read by consecutive lanes (request_coefficient_rows: the twelve
// requests per lane leave together; rows of lanes that are not live are not read) and turned through LDS 32 at a
// time (turn_coefficient_rows: half the LDS per wave, more waves per CU).  wave_lds: 32 * kShLdsF4 float4 owned by
// the wave.
__device__ __forceinline__ void request_coefficient_rows(const float* __restrict__ coeffs, uint32_t N, uint32_t row0,
                                                         uint64_t live_rows, uint32_t lane, float4* tmp) {
    const float4* src = reinterpret_cast<const float4*>(coeffs + (size_t)min(row0, N - 1) * 48);
    const uint32_t n_f4 = row0 < N ? min(64u, N - row0) * kShRowF4 : 0u;
#pragma unroll
    for (uint32_t i = 0; i < kShRowF4; ++i) {
        const uint32_t q = i * 64u + lane;
        const uint32_t r = (q * 43691u) >> 19; // q / 12 for q < 768
        tmp[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (q < n_f4 && ((live_rows >> r) & 1ull))
            tmp[i] = load_streaming(src + q); // read once per pass
    }
}
__device__ __forceinline__ void turn_coefficient_rows(const float4* tmp, uint32_t lane, float4* wave_lds,
                                                      float* co_reg) {
#pragma unroll
    for (uint32_t half = 0; half < 2; ++half) {
#pragma unroll
        for (uint32_t i = 0; i < kShRowF4 / 2; ++i) {
            const uint32_t q = i * 64u + lane;     // position inside this half's 32 rows
            const uint32_t r = (q * 43691u) >> 19; // q / 12
            wave_lds[r * kShLdsF4 + (q - r * kShRowF4)] = tmp[half * (kShRowF4 / 2) + i];
        }
        __builtin_amdgcn_wave_barrier();
        if ((lane >> 5) == half) {
#pragma unroll
            for (uint32_t k = 0; k < kShRowF4; ++k) {
                const float4 t = wave_lds[(lane & 31u) * kShLdsF4 + k];
                co_reg[4 * k + 0] = t.x;
                co_reg[4 * k + 1] = t.y;
                co_reg[4 * k + 2] = t.z;
                co_reg[4 * k + 3] = t.w;
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
}
__device__ __forceinline__ void wave_coefficient_rows(const float* __restrict__ coeffs, uint32_t N, uint32_t row0,
                                                      bool live, uint32_t lane, float4* wave_lds, float* co_reg) {
    const uint64_t live_rows = __builtin_amdgcn_ballot_w64(live);
    if (row0 >= N || !live_rows)
        return;
    float4 tmp[kShRowF4];
    request_coefficient_rows(coeffs, N, row0, live_rows, lane, tmp);
    turn_coefficient_rows(tmp, lane, wave_lds, co_reg);
}

// Gaussian e's colour (clamped SH colour of the direction camera -> mean) and, if it touches a tile, its record
__device__ __forceinline__ void color_and_record(uint32_t e, bool live, uint32_t degree, vec3 mean, float opac,
                                                 quat q_in, vec3 scl, const float* co,
                                                 const float* __restrict__ viewmat, const float* __restrict__ Kmat,
                                                 uint32_t W, uint32_t H, float* __restrict__ colors,
                                                 float4* __restrict__ records) {
    float c[3] = {0.f, 0.f, 0.f};
    if (live) {
        const vec3 dir = sub(mean, campos_from_viewmat(viewmat));
        float B[25];
        sh_basis(degree, dir, B);
#pragma unroll
        for (uint32_t ch = 0; ch < 3; ++ch)
            c[ch] = gsx::fmax(sh_color_channel(degree, dir, B, co, ch) + 0.5f, 0.0f);
    }
    colors[e * 3 + 0] = c[0];
    colors[e * 3 + 1] = c[1];
    colors[e * 3 + 2] = c[2];
    if (!live)
        return; // no tile lists this Gaussian: its record is never read
    const vec3 ray_o = camera_ray_origin(load_cam_pose(viewmat));
    const mat3 M = record_whitening(q_in, scl);
    const vec3 gro = mul(M, sub(ray_o, mean));
    const RecordRegion reg = record_region(gro, M, opac, mean, viewmat, Kmat[0], Kmat[4], Kmat[2], Kmat[5], W, H);
    store_record(records + (size_t)e * kRecordF4, gro, opac, M, c[0], c[1], c[2], reg);
}

// The same for a whole wave (lane = Gaussian row0 + lane; lanes beyond N are not live): the 96-byte records are
// turned through LDS and leave as runs of consecutive 16-byte pieces instead of 64 strided ones per store.
// wave_lds: kShWaveLdsF4 float4 owned by the wave (free again after wave_coefficient_rows).
static constexpr uint32_t kRecLdsF4 = 7; // padded record stride in LDS: conflict-free 16-byte accesses
static constexpr uint32_t kShWaveLdsF4 = 64 * kRecLdsF4 > 32 * kShLdsF4 ? 64 * kRecLdsF4 : 32 * kShLdsF4;
__device__ __forceinline__ void wave_color_and_record(uint32_t row0, uint32_t N, uint32_t lane, bool live,
                                                      uint32_t degree, vec3 mean, float opac, quat q_in, vec3 scl,
                                                      const float* co, const float* __restrict__ viewmat,
                                                      const float* __restrict__ Kmat, uint32_t W, uint32_t H,
                                                      float* __restrict__ colors, float4* __restrict__ records,
                                                      float4* wave_lds) {
    const uint32_t e = row0 + lane;
    float c[3] = {0.f, 0.f, 0.f};
    if (live) {
        const vec3 dir = sub(mean, campos_from_viewmat(viewmat));
        float B[25];
        sh_basis(degree, dir, B);
#pragma unroll
        for (uint32_t ch = 0; ch < 3; ++ch)
            c[ch] = gsx::fmax(sh_color_channel(degree, dir, B, co, ch) + 0.5f, 0.0f);
        const vec3 ray_o = camera_ray_origin(load_cam_pose(viewmat));
        const mat3 M = record_whitening(q_in, scl);
        const vec3 gro = mul(M, sub(ray_o, mean));
        const RecordRegion reg = record_region(gro, M, opac, mean, viewmat, Kmat[0], Kmat[4], Kmat[2], Kmat[5], W, H);
        store_record(wave_lds + lane * kRecLdsF4, gro, opac, M, c[0], c[1], c[2], reg);
    }
    if (e < N) {
        colors[e * 3 + 0] = c[0];
        colors[e * 3 + 1] = c[1];
        colors[e * 3 + 2] = c[2];
    }
    const uint64_t live_rows = __builtin_amdgcn_ballot_w64(live);
    __builtin_amdgcn_wave_barrier();
    float4* dst = records + (size_t)row0 * kRecordF4;
#pragma unroll
    for (uint32_t i = 0; i < kRecordF4; ++i) {
        const uint32_t q = i * 64u + lane;     // piece q of the wave's 64 * 6
        const uint32_t r = (q * 43691u) >> 18; // q / 6 for q < 384
        if ((live_rows >> r) & 1ull)           // a Gaussian no tile lists keeps its record untouched
            dst[q] = wave_lds[r * kRecLdsF4 + (q - r * kRecordF4)];
    }
}

// Colours AND raster records in one pass (what gsx_sh_colors_from_world followed by gsx_pack_raster_records
// produce, same arithmetic): the colour goes straight from the SH evaluation into the record, and the coefficient
// rows of Gaussians that touch no tile are not read at all.
template <bool LDS16>
__global__ void __launch_bounds__(256) sh_records_kernel(uint32_t N, uint32_t K, uint32_t degree,
                                                          const float* __restrict__ means,
                                                          const float* __restrict__ quats,
                                                          const float* __restrict__ scales,
                                                          const float* __restrict__ opacities,
                                                          const float* __restrict__ coeffs,
                                                          const int32_t* __restrict__ radii,
                                                          const float* __restrict__ viewmat,
                                                          const float* __restrict__ Kmat, uint32_t W, uint32_t H,
                                                          float* __restrict__ colors, float4* __restrict__ records) {
    __shared__ float4 lds[LDS16 ? 4 * kShWaveLdsF4 : 1];
    const uint32_t e = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    // (both radii with one unconditional 8-byte load: `a > 0 && b > 0` on two loads is two round trips in a row)
    const int2 rad = reinterpret_cast<const int2*>(radii)[min(e, N - 1)];
    const bool live = e < N && rad.x > 0 && rad.y > 0;
    // everything the record needs is requested now, together with the coefficient rows below: one memory round
    // trip instead of one per phase (the 44 bytes are read for Gaussians without a tile too)
    const uint32_t ec = min(e, N - 1);
    const vec3 mean = ld3(means, ec);
    const float opac = opacities[ec];
    const quat q_in = ld4q(quats, ec);
    const vec3 scl = ld3(scales, ec);
    float co_reg[48];
    if (LDS16) {
        const uint32_t row0 = blockIdx.x * 256u + wave * 64u;
        float4* wave_lds = lds + wave * kShWaveLdsF4;
        wave_coefficient_rows(coeffs, N, row0, live, lane, wave_lds, co_reg);
        wave_color_and_record(row0, N, lane, live, degree, mean, opac, q_in, scl, co_reg, viewmat, Kmat, W, H, colors,
                              records, wave_lds);
        return;
    }
    if (e >= N)
        return;
    color_and_record(e, live, degree, mean, opac, q_in, scl, coeffs + (size_t)e * K * 3, viewmat, Kmat, W, H, colors,
                     records);
}

// The whole per-Gaussian front of a training step in one pass (one camera, K = 16): activations, UT projection,
// SH colour and raster record - what projection_ut_raw_kernel followed by sh_records_kernel<true> produce, same
// arithmetic; the activated parameters, the radii and the visibility stay in registers between the two halves.
// (Requesting a chunk's coefficient rows while the next chunk is projected - a software pipeline inside the wave -
// needs about 300 live registers as the compiler schedules it and runs slower than this plain sequence.)
__global__ void __launch_bounds__(256) project_sh_records_kernel(
    uint32_t N, uint32_t degree, const float* __restrict__ means, const float* __restrict__ opacity_raw,
    const float* __restrict__ scaling_raw, const float* __restrict__ rotation_raw, const float* __restrict__ coeffs,
    const float* __restrict__ viewmat, const float* __restrict__ Ks, ProjCfg cfg, float* __restrict__ opacities,
    float* __restrict__ scales, float* __restrict__ quats, int32_t* __restrict__ radii, float* __restrict__ means2d,
    float* __restrict__ depths, float* __restrict__ conics, float* __restrict__ colors,
    float4* __restrict__ records) {
    __shared__ float4 lds[4 * kShWaveLdsF4];
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t ic = min(idx, N - 1);
    const WorkgroupPose wp = workgroup_pose(viewmat);
    const vec3 mean = ld3(means, ic);
    const Activated a = activate(opacity_raw[ic], ld3(scaling_raw, ic), ld4q(rotation_raw, ic));
    bool live = false;
    if (idx < N) {
        opacities[idx] = a.opacity;
        scales[3 * idx + 0] = a.scales.x;
        scales[3 * idx + 1] = a.scales.y;
        scales[3 * idx + 2] = a.scales.z;
        reinterpret_cast<float4*>(quats)[idx] = make_float4(a.quat.w, a.quat.x, a.quat.y, a.quat.z);
        cfg.fx = Ks[0];
        cfg.fy = Ks[4];
        cfg.cx = Ks[2];
        cfg.cy = Ks[5];
        ProjOut o;
        live = project_ut<false>(cfg, wp.cp, wp.qc, wp.tc, wp.Rc, mean, a.quat, a.scales, true, a.opacity, &o);
        int2* r2 = reinterpret_cast<int2*>(radii);
        if (!live) {
            r2[idx] = make_int2(0, 0);
        } else {
            r2[idx] = make_int2((int32_t)o.rx, (int32_t)o.ry);
            reinterpret_cast<float2*>(means2d)[idx] = make_float2(o.mx, o.my);
            depths[idx] = o.depth;
            if (conics != nullptr) {
                conics[idx * 3 + 0] = o.c0;
                conics[idx * 3 + 1] = o.c1;
                conics[idx * 3 + 2] = o.c2;
            }
            live = o.rx > 0.f && o.ry > 0.f; // what sh_records_kernel reads back from radii
        }
    }
    float co_reg[48];
    const uint32_t row0 = blockIdx.x * 256u + wave * 64u;
    float4* wave_lds = lds + wave * kShWaveLdsF4;
    wave_coefficient_rows(coeffs, N, row0, live, lane, wave_lds, co_reg);
    wave_color_and_record(row0, N, lane, live, degree, mean, a.opacity, a.quat, a.scales, co_reg, viewmat, Ks, cfg.W,
                          cfg.H, colors, records, wave_lds);
}

template <bool WORLD>
static void launch_sh_fwd(uint32_t N, uint32_t K, uint32_t degree, const float* dirs_or_means, const float* coeffs,
                          const uint8_t* masks, const int32_t* radii, const float* viewmat, float* colors,
                          hipStream_t s) {
    const bool lds16 = K == 16 && (((uintptr_t)coeffs) & 15u) == 0;
    if (lds16)
        hipLaunchKernelGGL((sh_fwd_generic_kernel<WORLD, true>), dim3(cdiv(N, 256)), dim3(256), 0, s, N, K, degree,
                           dirs_or_means, coeffs, masks, radii, viewmat, colors);
    else
        hipLaunchKernelGGL((sh_fwd_generic_kernel<WORLD, false>), dim3(cdiv(N, 256)), dim3(256), 0, s, N, K, degree,
                           dirs_or_means, coeffs, masks, radii, viewmat, colors);
}

template <bool WORLD>
static void launch_sh_bwd(uint32_t N, uint32_t K, uint32_t degree, const float* dirs_or_means, const uint8_t* masks,
                          const int32_t* radii, const float* viewmat, const float* colors, const float* v_colors,
                          float* v_coeffs, hipStream_t s) {
    const bool lds16 = K == 16 && (((uintptr_t)v_coeffs) & 15u) == 0;
    if (lds16)
        hipLaunchKernelGGL((sh_bwd_generic_kernel<WORLD, true>), dim3(cdiv(N, 256)), dim3(256), 0, s, N, K, degree,
                           dirs_or_means, masks, radii, viewmat, colors, v_colors, v_coeffs);
    else
        hipLaunchKernelGGL((sh_bwd_generic_kernel<WORLD, false>), dim3(cdiv(N, 256)), dim3(256), 0, s, N, K, degree,
                           dirs_or_means, masks, radii, viewmat, colors, v_colors, v_coeffs);
}

} // namespace gsx

using namespace gsx;

// =============================================================================================
// C ABI
// =============================================================================================

// Cameras.cuh:1070-1119: lambda = alpha^2 (D + kappa) - D, spread sqrt(D + lambda), weights; D = 3
static void set_ut_constants(ProjCfg& cfg, const gsx_ut_params& ut) {
    cfg.ut_alpha = ut.alpha, cfg.ut_beta = ut.beta, cfg.ut_kappa = ut.kappa;
    cfg.ut_margin = ut.in_image_margin_factor;
    cfg.ut_require_all = ut.require_all_sigma_points_valid;
    const float D = 3.0f;
    const float lambda = cfg.ut_alpha * cfg.ut_alpha * (D + cfg.ut_kappa) - D;
    cfg.ut_sq = gsx::sqrt(D + lambda);
    cfg.ut_w0m = lambda / (D + lambda);
    cfg.ut_w0c = lambda / (D + lambda) + (1.f - cfg.ut_alpha * cfg.ut_alpha + cfg.ut_beta);
    cfg.ut_wi = 1.f / (2.f * (D + lambda));
}

extern "C" int gsx_projection_ut_3dgs_fused(
    uint32_t C, uint32_t N, const float* means, const float* quats, const float* scales, const float* opacities,
    const float* viewmats0, const float* viewmats1, const float* Ks, uint32_t image_width, uint32_t image_height,
    float eps2d, float near_plane, float far_plane, float radius_clip, int camera_model, gsx_ut_params ut,
    int rs_type, const float* radial_coeffs, const float* tangential_coeffs, const float* thin_prism_coeffs,
    int32_t* radii, float* means2d, float* depths, float* conics, float* compensations, void* stream) {
    if ((uint64_t)C * N == 0)
        return GSX_OK; // ProjectionUT3DGSFused.cu:249-252
    GSX_REQUIRE(means && quats && scales && viewmats0 && Ks && radii && means2d && depths && conics,
                GSX_ERR_INVALID_ARGUMENT, "projection_ut_3dgs_fused: null tensor");
    GSX_REQUIRE((uint64_t)C * N < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "projection_ut_3dgs_fused: C*N >= 2^31");
    const int rc = check_camera_args(C, viewmats1, camera_model, rs_type, radial_coeffs, tangential_coeffs,
                                     thin_prism_coeffs);
    if (rc != GSX_OK)
        return rc;
    ProjCfg cfg;
    cfg.W = image_width;
    cfg.H = image_height;
    cfg.eps2d = eps2d;
    cfg.near_plane = near_plane;
    cfg.far_plane = far_plane;
    cfg.radius_clip = radius_clip;
    set_ut_constants(cfg, ut);
    cfg.fx = cfg.fy = cfg.cx = cfg.cy = 0.f;
    memset(&cfg.cam, 0, sizeof(cfg.cam));
    // the trainer's camera (rasterizer.cpp:33-35, rasterizer_autograd.cpp:59-60) takes the instance without the
    // other models' branches: same arithmetic, same results
    const bool plain = camera_model == GSX_PINHOLE && !radial_coeffs && !tangential_coeffs && !thin_prism_coeffs &&
                       viewmats1 == nullptr && rs_type == GSX_GLOBAL;
    hipLaunchKernelGGL(plain ? projection_ut_kernel<false> : projection_ut_kernel<true>,
                       dim3(cdiv((uint64_t)C * N, 256)), dim3(256), 0, (hipStream_t)stream, C, N, means, quats, scales,
                       opacities, viewmats0, viewmats1, rs_type, Ks, camera_model, radial_coeffs, tangential_coeffs,
                       thin_prism_coeffs, cfg, radii, means2d, depths, conics, compensations);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_activate_project_ut(uint32_t N, const float* means, const float* opacity_raw,
                                       const float* scaling_raw, const float* rotation_raw, const float* viewmat,
                                       const float* K, uint32_t image_width, uint32_t image_height, float eps2d,
                                       float near_plane, float far_plane, float radius_clip, gsx_ut_params ut,
                                       float* opacities, float* scales, float* quats, int32_t* radii, float* means2d,
                                       float* depths, float* conics, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && opacity_raw && scaling_raw && rotation_raw && viewmat && K && opacities && scales && quats &&
                    radii && means2d && depths,
                GSX_ERR_INVALID_ARGUMENT, "activate_project_ut: null tensor");
    GSX_REQUIRE((((uintptr_t)rotation_raw) & 15) == 0 && (((uintptr_t)quats) & 15) == 0, GSX_ERR_INVALID_ARGUMENT,
                "activate_project_ut: quaternion tensors need 16-byte alignment");
    ProjCfg cfg;
    memset(&cfg, 0, sizeof(cfg));
    cfg.W = image_width, cfg.H = image_height;
    cfg.eps2d = eps2d, cfg.near_plane = near_plane, cfg.far_plane = far_plane, cfg.radius_clip = radius_clip;
    set_ut_constants(cfg, ut);
    hipLaunchKernelGGL(projection_ut_raw_kernel, dim3(cdiv(N, 512)), dim3(512), 0, (hipStream_t)stream, N, means,
                       opacity_raw, scaling_raw, rotation_raw, viewmat, K, cfg, opacities, scales, quats, radii,
                       means2d, depths, conics);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_spherical_harmonics_fwd(uint32_t N, uint32_t K, uint32_t degrees_to_use, const float* dirs,
                                           const float* coeffs, const uint8_t* masks, float* colors, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(dirs && coeffs && colors, GSX_ERR_INVALID_ARGUMENT, "spherical_harmonics_fwd: null tensor");
    GSX_REQUIRE(degrees_to_use <= 4 && K >= (degrees_to_use + 1) * (degrees_to_use + 1), GSX_ERR_INVALID_ARGUMENT,
                "spherical_harmonics_fwd: degree %u needs K >= %u (got %u)", degrees_to_use,
                (degrees_to_use + 1) * (degrees_to_use + 1), K);
    launch_sh_fwd<false>(N, K, degrees_to_use, dirs, coeffs, masks, nullptr, nullptr, colors, (hipStream_t)stream);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_spherical_harmonics_bwd(uint32_t N, uint32_t K, uint32_t degrees_to_use, const float* dirs,
                                           const float* coeffs, const uint8_t* masks, const float* v_colors,
                                           float* v_coeffs, float* v_dirs, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(dirs && coeffs && v_colors && v_coeffs, GSX_ERR_INVALID_ARGUMENT,
                "spherical_harmonics_bwd: null tensor");
    GSX_REQUIRE(degrees_to_use <= 4 && K >= (degrees_to_use + 1) * (degrees_to_use + 1), GSX_ERR_INVALID_ARGUMENT,
                "spherical_harmonics_bwd: degree %u needs K >= %u (got %u)", degrees_to_use,
                (degrees_to_use + 1) * (degrees_to_use + 1), K);

    launch_sh_bwd<false>(N, K, degrees_to_use, dirs, masks, nullptr, nullptr, nullptr, v_colors, v_coeffs,
                         (hipStream_t)stream);
    GSX_LAUNCH_CHECK();
    if (v_dirs != nullptr) {
        hipLaunchKernelGGL(sh_bwd_dirs_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, K,
                           degrees_to_use, dirs, coeffs, masks, v_colors, v_dirs);
        GSX_LAUNCH_CHECK();
    }
    return GSX_OK;
}

extern "C" int gsx_sh_colors_from_world(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                        const float* sh_coeffs, const int32_t* radii, const float* viewmat,
                                        float* colors, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && sh_coeffs && radii && viewmat && colors, GSX_ERR_INVALID_ARGUMENT,
                "sh_colors_from_world: null tensor");
    GSX_REQUIRE(((uintptr_t)radii & 7) == 0, GSX_ERR_INVALID_ARGUMENT, "sh_colors_from_world: radii need 8-byte alignment");
    GSX_REQUIRE(sh_degree <= 4 && K >= (sh_degree + 1) * (sh_degree + 1), GSX_ERR_INVALID_ARGUMENT,
                "sh_colors_from_world: degree %u needs K >= %u (got %u)", sh_degree, (sh_degree + 1) * (sh_degree + 1),
                K);
    launch_sh_fwd<true>(N, K, sh_degree, means, sh_coeffs, nullptr, radii, viewmat, colors, (hipStream_t)stream);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_sh_colors_records_from_world(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                                const float* quats, const float* scales, const float* opacities,
                                                const float* sh_coeffs, const int32_t* radii, const float* viewmat,
                                                const float* Kmat, uint32_t image_width, uint32_t image_height,
                                                float* colors, void* records, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && quats && scales && opacities && sh_coeffs && radii && viewmat && Kmat && colors && records,
                GSX_ERR_INVALID_ARGUMENT, "sh_colors_records_from_world: null tensor");
    GSX_REQUIRE(sh_degree <= 4 && K >= (sh_degree + 1) * (sh_degree + 1), GSX_ERR_INVALID_ARGUMENT,
                "sh_colors_records_from_world: degree %u needs K >= %u (got %u)", sh_degree,
                (sh_degree + 1) * (sh_degree + 1), K);
    GSX_REQUIRE(((uintptr_t)records & 15) == 0 && ((uintptr_t)quats & 15) == 0 && ((uintptr_t)radii & 7) == 0,
                GSX_ERR_INVALID_ARGUMENT,
                "sh_colors_records_from_world: records / quats need 16-byte alignment, radii 8-byte");
    const bool lds16 = K == 16 && (((uintptr_t)sh_coeffs) & 15u) == 0;
    const dim3 grid(cdiv(N, 256)), block(256);
    if (lds16)
        hipLaunchKernelGGL((sh_records_kernel<true>), grid, block, 0, (hipStream_t)stream, N, K, sh_degree, means,
                           quats, scales, opacities, sh_coeffs, radii, viewmat, Kmat, image_width, image_height, colors,
                           (float4*)records);
    else
        hipLaunchKernelGGL((sh_records_kernel<false>), grid, block, 0, (hipStream_t)stream, N, K, sh_degree, means,
                           quats, scales, opacities, sh_coeffs, radii, viewmat, Kmat, image_width, image_height, colors,
                           (float4*)records);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

// gsx_activate_project_ut followed by gsx_sh_colors_records_from_world, as one pass over the Gaussians where the
// coefficient layout allows it (K = 16, 16-byte aligned rows), as those two launches otherwise: same outputs.
extern "C" int gsx_activate_project_sh_records(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                               const float* opacity_raw, const float* scaling_raw,
                                               const float* rotation_raw, const float* sh_coeffs,
                                               const float* viewmat, const float* Kmat, uint32_t image_width,
                                               uint32_t image_height, float eps2d, float near_plane, float far_plane,
                                               float radius_clip, gsx_ut_params ut, float* opacities, float* scales,
                                               float* quats, int32_t* radii, float* means2d, float* depths,
                                               float* conics, float* colors, void* records, void* stream) {
    if (N == 0)
        return GSX_OK;
    const bool one_pass = K == 16 && (((uintptr_t)sh_coeffs) & 15u) == 0;
    if (!one_pass) {
        const int rc = gsx_activate_project_ut(N, means, opacity_raw, scaling_raw, rotation_raw, viewmat, Kmat,
                                               image_width, image_height, eps2d, near_plane, far_plane, radius_clip,
                                               ut, opacities, scales, quats, radii, means2d, depths, conics, stream);
        if (rc != GSX_OK)
            return rc;
        return gsx_sh_colors_records_from_world(N, K, sh_degree, means, quats, scales, opacities, sh_coeffs, radii,
                                                viewmat, Kmat, image_width, image_height, colors, records, stream);
    }
    GSX_REQUIRE(means && opacity_raw && scaling_raw && rotation_raw && sh_coeffs && viewmat && Kmat && opacities &&
                    scales && quats && radii && means2d && depths && colors && records,
                GSX_ERR_INVALID_ARGUMENT, "activate_project_sh_records: null tensor");
    GSX_REQUIRE((((uintptr_t)rotation_raw) & 15) == 0 && (((uintptr_t)quats) & 15) == 0 &&
                    ((uintptr_t)records & 15) == 0,
                GSX_ERR_INVALID_ARGUMENT, "activate_project_sh_records: quaternions / records need 16-byte alignment");
    GSX_REQUIRE(sh_degree <= 3, GSX_ERR_INVALID_ARGUMENT, "activate_project_sh_records: degree %u needs K >= %u (got %u)",
                sh_degree, (sh_degree + 1) * (sh_degree + 1), K);
    ProjCfg cfg;
    memset(&cfg, 0, sizeof(cfg));
    cfg.W = image_width, cfg.H = image_height;
    cfg.eps2d = eps2d, cfg.near_plane = near_plane, cfg.far_plane = far_plane, cfg.radius_clip = radius_clip;
    set_ut_constants(cfg, ut);
    hipLaunchKernelGGL(project_sh_records_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, sh_degree,
                       means, opacity_raw, scaling_raw, rotation_raw, sh_coeffs, viewmat, Kmat, cfg, opacities, scales,
                       quats, radii, means2d, depths, conics, colors, (float4*)records);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_sh_colors_from_world_bwd(uint32_t N, uint32_t K, uint32_t sh_degree, const float* means,
                                            const int32_t* radii, const float* viewmat, const float* colors,
                                            const float* v_colors, float* v_sh_coeffs, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && radii && viewmat && colors && v_colors && v_sh_coeffs, GSX_ERR_INVALID_ARGUMENT,
                "sh_colors_from_world_bwd: null tensor");
    GSX_REQUIRE(((uintptr_t)radii & 7) == 0, GSX_ERR_INVALID_ARGUMENT,
                "sh_colors_from_world_bwd: radii need 8-byte alignment");
    GSX_REQUIRE(sh_degree <= 4 && K >= (sh_degree + 1) * (sh_degree + 1), GSX_ERR_INVALID_ARGUMENT,
                "sh_colors_from_world_bwd: degree %u needs K >= %u (got %u)", sh_degree,
                (sh_degree + 1) * (sh_degree + 1), K);
    launch_sh_bwd<true>(N, K, sh_degree, means, nullptr, radii, viewmat, colors, v_colors, v_sh_coeffs,
                        (hipStream_t)stream);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_quats_to_rotmats(int N, const float* quats, float* rotmats, void* stream) {
    if (N <= 0)
        return GSX_OK;
    GSX_REQUIRE(quats && rotmats, GSX_ERR_INVALID_ARGUMENT, "quats_to_rotmats: null tensor");
    hipLaunchKernelGGL(quats_to_rotmats_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, (uint32_t)N,
                       quats, rotmats);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_activate_params(uint32_t N, const float* opacity_raw, const float* scaling_raw,
                                   const float* rotation_raw, float* opacities, float* scales, float* quats,
                                   void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(opacity_raw && scaling_raw && rotation_raw && opacities && scales && quats, GSX_ERR_INVALID_ARGUMENT,
                "activate_params: null tensor");
    hipLaunchKernelGGL(activate_params_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, opacity_raw,
                       scaling_raw, rotation_raw, opacities, scales, quats);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_activate_params_bwd(uint32_t N, const float* opacity_raw, const float* scaling_raw,
                                       const float* rotation_raw, const float* v_opacities, const float* v_scales,
                                       const float* v_quats, float* v_opacity_raw, float* v_scaling_raw,
                                       float* v_rotation_raw, void* stream) {
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(opacity_raw && scaling_raw && rotation_raw && v_opacities && v_scales && v_quats && v_opacity_raw &&
                    v_scaling_raw && v_rotation_raw,
                GSX_ERR_INVALID_ARGUMENT, "activate_params_bwd: null tensor");
    hipLaunchKernelGGL(activate_params_bwd_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N,
                       opacity_raw, scaling_raw, rotation_raw, v_opacities, v_scales, v_quats, v_opacity_raw,
                       v_scaling_raw, v_rotation_raw);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
