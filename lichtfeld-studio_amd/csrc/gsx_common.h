// gsx_common.h - shared host/device helpers of libgsx (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define GSX_BUILD 1
#include "../../include/gsx.h"
#include "gsx_math.h"

namespace gsx {

// ---- error reporting -------------------------------------------------------------------------
void set_error(const char* fmt, ...);

#define GSX_REQUIRE(cond, status, ...)  \
    do {                                \
        if (!(cond)) {                  \
            gsx::set_error(__VA_ARGS__); \
            return (status);            \
        }                               \
    } while (0)

#define GSX_HIP_CHECK(expr)                                                                       \
    do {                                                                                          \
        hipError_t _e = (expr);                                                                   \
        if (_e != hipSuccess) {                                                                   \
            gsx::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
            return GSX_ERR_HIP;                                                                   \
        }                                                                                         \
    } while (0)

// after a kernel launch: catches launch-configuration errors without synchronising
#define GSX_LAUNCH_CHECK() GSX_HIP_CHECK(hipGetLastError())

static inline uint32_t cdiv(uint64_t a, uint64_t b) { return (uint32_t)((a + b - 1) / b); }
static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

int check_camera_args(uint32_t C, const float* viewmats1, int camera_model, int rs_type, const float* radial,
                      const float* tangential, const float* thin_prism);

// ---- camera pose (device) ---------------------------------------------------------------------
// Rotation of the row-major [4,4] world->camera matrix as a quaternion plus its translation, and the
// pose the reference interpolates from it for a global shutter (gsplat/Cameras.cuh:33-71, 268-280).
struct CamPose {
    quat q_start;
    vec3 t_start;
};

__device__ __forceinline__ CamPose load_cam_pose(const float* __restrict__ vm) {
    mat3 R;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 3; ++c)
            R.m[r][c] = vm[r * 4 + c];
    CamPose p;
    p.q_start = quat_cast(R);
    p.t_start = mk3(vm[3], vm[7], vm[11]);
    return p;
}

// interpolate_shutter_pose(rel, {start, end = start})
__device__ __forceinline__ void shutter_pose(const CamPose& cp, float rel, quat* q, vec3* t) {
    t->x = (1.f - rel) * cp.t_start.x + rel * cp.t_start.x;
    t->y = (1.f - rel) * cp.t_start.y + rel * cp.t_start.y;
    t->z = (1.f - rel) * cp.t_start.z + rel * cp.t_start.z;
    *q = slerp(cp.q_start, cp.q_start, rel);
}

// world ray through a pixel centre, perfect pinhole, global shutter
// (Cameras.cuh:457-470 unproject, :253-266 camera_ray_to_world_ray, :322-339)
__device__ __forceinline__ void pixel_world_ray(const CamPose& cp, float px, float py, float fx, float fy, float cx,
                                                float cy, vec3* ray_o, vec3* ray_d) {
    const float u = (px - cx) / fx;
    const float v = (py - cy) / fy;
    const vec3 cr = mk3(u, v, 1.f);
    const float len = gsx::sqrt(dot(cr, cr));
    const vec3 d_cam = mk3(cr.x / len, cr.y / len, cr.z / len);
    quat q;
    vec3 t;
    shutter_pose(cp, 0.f, &q, &t);
    const mat3 R_inv = mat3_cast(quat_inverse(q));
    *ray_o = neg(mul(R_inv, t));
    *ray_d = mul(R_inv, d_cam);
}

__device__ __forceinline__ vec3 ld3(const float* __restrict__ p, uint32_t i) {
    return mk3(p[3 * i], p[3 * i + 1], p[3 * i + 2]);
}
__device__ __forceinline__ quat ld4q(const float* __restrict__ p, uint32_t i) {
    const float4 v = *reinterpret_cast<const float4*>(p + 4 * (size_t)i);
    quat q;
    q.w = v.x;
    q.x = v.y;
    q.y = v.z;
    q.z = v.w;
    return q;
}

} // namespace gsx
