// gsx_common.h - shared host/device helpers of libgsx (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define GSX_BUILD 1
#include "../../include/gsx.h"
#include "../../include/gsx_debug.h"
#include "gsx_math.h"
#include "gsx_camera.h"
#include "gsx_record.h"

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

// intersect.hip: the depth-ordered tile count from ready-made keys.  ordered_keys(ws) is where the N
// (tile count << 32 | depth bits) keys go inside a gsx_intersect_tile_count_ordered workspace; the second call sorts
// them on the depth bits, scans the counts in that order into cum (inclusive) and starts the copy of the total; the
// sorted keys stay in ordered_keys(ws).  rect_keys: the high words are packed tile rectangles
// (x0 | y0 << 8 | x1 << 16 | y1 << 24, 0 = none) instead of counts.
int64_t* ordered_keys(void* workspace);
// intersect.hip: the tile visiting order of a backward pass from the forward pass's per-pixel outputs
int tile_order_from_pixels(int64_t n_isects, uint32_t image_width, uint32_t image_height, const int32_t* tile_offsets,
                           const float* render_alphas, const int32_t* last_ids, void* scratch,
                           const uint32_t** tile_order, void* stream);
int ordered_counts_from_keys(const char* who, uint32_t N, int32_t* order, int64_t* cum_tiles_per_gauss, void* workspace,
                             size_t workspace_bytes, int64_t* n_isects_host, int wait, void* stream,
                             bool rect_keys = false, bool first_hist_done = false);
// radix_sort.hip: the table of the first 8-bit pass of a 32-bit sort, for a key-writing kernel that fills it itself
struct RadixFirstPass {
    uint32_t items, nblocks; // sort block b covers keys [b * 256 * items, (b + 1) * 256 * items)
    uint32_t* table;         // [256][nblocks], digit-major
};
RadixFirstPass radix_first_pass_table(int64_t n, void* sort_workspace);
int radix_sort_pairs_32_bits(int64_t n, int64_t* keys0, int32_t* vals0, int64_t* keys1, int32_t* vals1,
                             uint32_t begin_bit, void* workspace, size_t workspace_bytes, int* selector_host,
                             void* stream, bool first_hist_done);

// radix_sort.hip: one stable 1..8-bit radix pass as ONE launch (chained look-back between the workgroups).  The
// caller provides digit_total[256] = how many of the pairs carry each digit, a status table of
// radix_chained_rows(n_max) x 256 empty (zero) words; the launch can clear the table of the pass that follows it.  n_dev (nullable): the number of pairs is min(*n_dev, n_max), read on the device.
// Limit: n_max < 2^30.  error: device word, bit 1 is set if a look-back's bounded wait ran out.
// how many empty reads a look-back waits before it gives up (gsx_lookback.h): the default, or what a test set
uint32_t lookback_spin_limit();
struct RadixChainArgs {
    const int64_t* n_dev;
    uint32_t *status, *clear_status;
    uint32_t clear_rows;
    uint32_t* error;
    uint32_t total_replicas, total_stride; // digit_total is the sum of this many tables, total_stride words apart
};
uint32_t radix_chained_rows(int64_t n_max);
int radix_chained_pass_i64(uint32_t n_max, const int64_t* kin, const int32_t* vin, int64_t* kout, int32_t* vout,
                           uint32_t shift, uint32_t bits, const uint32_t* digit_total, const RadixChainArgs& a,
                           void* stream);
int radix_chained_pass_u16(uint32_t n_max, const uint16_t* kin, const int32_t* vin, uint16_t* kout, int32_t* vout,
                           uint32_t shift, uint32_t bits, const uint32_t* digit_total, const RadixChainArgs& a,
                           bool write_keys, void* stream);

int check_camera_args(uint32_t C, const float* viewmats1, int camera_model, int rs_type, const float* radial,
                      const float* tangential, const float* thin_prism);

// ---- camera pose (device) ---------------------------------------------------------------------
// Rotation of the row-major [4,4] world->camera matrix as a quaternion plus its translation, and the
// pose the reference interpolates from it for a global shutter (gsplat/Cameras.cuh:33-71, 268-280).
struct CamPose {
    quat q_start;
    vec3 t_start;
    quat q_end; // = the start pose for a global shutter or when no end-of-frame pose is given
    vec3 t_end;
    int rs_type;   // gsx_shutter_type
    uint32_t W, H; // image size: the exposure time of a pixel is its row / column over H - 1 / W - 1
};

// RollingShutterParameters (Cameras.cuh:33-71): row-major [4,4] world->camera matrices; vm1 nullable
__device__ __forceinline__ CamPose load_cam_pose(const float* __restrict__ vm, const float* __restrict__ vm1 = nullptr,
                                                 int rs_type = 4 /*GLOBAL*/, uint32_t W = 0, uint32_t H = 0) {
    mat3 R;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 3; ++c)
            R.m[r][c] = vm[r * 4 + c];
    CamPose p;
    p.q_start = quat_cast(R);
    p.t_start = mk3(vm[3], vm[7], vm[11]);
    p.q_end = p.q_start;
    p.t_end = p.t_start;
    if (vm1 != nullptr) {
#pragma unroll
        for (int r = 0; r < 3; ++r)
#pragma unroll
            for (int c = 0; c < 3; ++c)
                R.m[r][c] = vm1[r * 4 + c];
        p.q_end = quat_cast(R);
        p.t_end = mk3(vm1[3], vm1[7], vm1[11]);
    }
    p.rs_type = rs_type;
    p.W = W, p.H = H;
    return p;
}

// interpolate_shutter_pose (Cameras.cuh:268-280)
__device__ __forceinline__ void shutter_pose(const CamPose& cp, float rel, quat* q, vec3* t) {
    t->x = (1.f - rel) * cp.t_start.x + rel * cp.t_end.x;
    t->y = (1.f - rel) * cp.t_start.y + rel * cp.t_end.y;
    t->z = (1.f - rel) * cp.t_start.z + rel * cp.t_end.z;
    *q = slerp(cp.q_start, cp.q_end, rel);
}

// shutter_relative_frame_time (Cameras.cuh:293-320): 0 for a global shutter
__device__ __forceinline__ float shutter_relative_frame_time(const CamPose& cp, float x, float y) {
    switch (cp.rs_type) {
    case 0: return gsx::floor(y) / (float)(cp.H - 1);
    case 1: return gsx::floor(x) / (float)(cp.W - 1);
    case 2: return ((float)cp.H - gsx::ceil(y)) / (float)(cp.H - 1);
    case 3: return ((float)cp.W - gsx::ceil(x)) / (float)(cp.W - 1);
    default: return 0.f;
    }
}

// ---- OpenCV pinhole distortion (gsplat/Cameras.cuh:473-815) ------------------------------------
// radial [6], tangential [2], thin prism [4]; `on` when the caller gave any of the three coefficient arrays (the
// reference's dispatch, ProjectionUT3DGSFused.cu:86-113).
struct Distortion {
    bool on;
    float k[6], p[2], s[4];
};

__device__ __forceinline__ Distortion load_distortion(const float* __restrict__ radial,
                                                      const float* __restrict__ tangential,
                                                      const float* __restrict__ thin_prism) {
    Distortion d;
    d.on = radial != nullptr || tangential != nullptr || thin_prism != nullptr;
#pragma unroll
    for (int i = 0; i < 6; ++i)
        d.k[i] = radial != nullptr ? radial[i] : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
        d.p[i] = tangential != nullptr ? tangential[i] : 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        d.s[i] = thin_prism != nullptr ? thin_prism[i] : 0.f;
    return d;
}

// Cameras.cuh:504-533
__device__ __forceinline__ void compute_distortion(const Distortion& d, float u, float v, float* icD, float* delta_x,
                                                   float* delta_y) {
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

// Cameras.cuh:635-740: Newton undistortion, at most 5 steps.  The reference's double literals make parts of the
// Jacobian double arithmetic; the expressions are kept as written there.  Returns "converged".
__device__ __forceinline__ bool opencv_undistort_newton(const Distortion& d, float xd, float yd, float* xo, float* yo) {
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

// The camera model of one call: the (distorted) pinhole, the OpenCV fisheye or the equirectangular model
// (gsx_camera_model values; the reference's dispatch, ProjectionUT3DGSFused.cu:86-136).
struct CameraModel {
    int type; // 0 pinhole (dist.on: with distortion), 2 fisheye, 3 equirectangular
    Distortion dist;
    Fisheye fe;
    float W, H;
};

__device__ __forceinline__ CameraModel load_camera_model(int type, const float* __restrict__ radial,
                                                         const float* __restrict__ tangential,
                                                         const float* __restrict__ thin_prism, float fx, float fy,
                                                         float cx, float cy, uint32_t W, uint32_t H) {
    CameraModel m;
    m.type = type;
    m.W = (float)W, m.H = (float)H;
    m.dist.on = false;
    if (type == 2)
        m.fe = fisheye_setup(radial, fx, fy, cx, cy, W, H);
    else if (type == 0)
        m.dist = load_distortion(radial, tangential, thin_prism);
    return m;
}

// world ray through a pixel centre under the pose of the pixel's exposure time (Cameras.cuh:457-470 / 742-755 / 961-1000 / 1027-1036
// unproject, :253-266 camera_ray_to_world_ray, :322-339).  Returns the ray's valid flag: false when an undistortion
// or the fisheye inverse did not converge or left the field of view (the ray is then zero, :330-333, and the pixel
// takes no part in either pass).
__device__ __forceinline__ bool pixel_world_ray(const CamPose& cp, float px, float py, float fx, float fy, float cx,
                                                float cy, const CameraModel& cam, vec3* ray_o, vec3* ray_d) {
    vec3 d_cam;
    bool ok = true;
    if (cam.type == 2) {
        ok = fisheye_unproject(cam.fe, px, py, &d_cam);
    } else if (cam.type == 3) {
        equirect_unproject(cam.W, cam.H, px, py, &d_cam);
    } else {
        float u = (px - cx) / fx;
        float v = (py - cy) / fy;
        if (cam.dist.on)
            ok = opencv_undistort_newton(cam.dist, u, v, &u, &v);
        const vec3 cr = mk3(u, v, 1.f);
        const float len = gsx::sqrt(dot(cr, cr));
        d_cam = mk3(cr.x / len, cr.y / len, cr.z / len);
    }
    if (!ok) {
        *ray_o = mk3(0.f, 0.f, 0.f);
        *ray_d = mk3(0.f, 0.f, 0.f);
        return false;
    }
    quat q;
    vec3 t;
    shutter_pose(cp, shutter_relative_frame_time(cp, px, py), &q, &t);
    const mat3 R_inv = mat3_cast(quat_inverse(q));
    *ray_o = neg(mul(R_inv, t));
    *ray_d = mul(R_inv, d_cam);
    return true;
}

// camera centre in world space exactly as the rasterizers form it (Cameras.cuh:253-266 with the start pose)
__device__ __forceinline__ vec3 camera_ray_origin(const CamPose& cp) {
    quat q;
    vec3 t;
    shutter_pose(cp, 0.f, &q, &t);
    return neg(mul(mat3_cast(quat_inverse(q)), t));
}

// ---- tile geometry shared by the forward and backward rasterizers ----------------------------
// One 256-lane workgroup per 16x16 tile; wave w owns the 8x8 pixel block (w & 1, w >> 1), lane l the pixel
// (l >> 3, l & 7) of it: compact blocks keep a wave's pixels coherent (saturation, bounds rejection).
// colour channel counts the rasterizers take (gsplat/Rasterization.cpp:106-128): up to 32 an instance each, beyond
// that one instance that takes 32 channels per launch, counted at run time
static inline bool raster_channels_built(uint32_t c) {
    return c == 1 || c == 2 || c == 3 || c == 4 || c == 5 || c == 8 || c == 9 || c == 16 || c == 17 || c == 32 ||
           c == 33 || c == 64 || c == 65 || c == 128 || c == 129 || c == 256 || c == 257 || c == 512 || c == 513;
}
static constexpr const char* kRasterChannelsText =
    "supported: 1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 64, 65, 128, 129, 256, 257, 512, 513";
static constexpr uint32_t kTile = 16;
// what (uint32_t)GSX_COUNT_IN_OFFSETS is inside the kernels
static constexpr uint32_t kCountInOffsets = 0xFFFFFFFFu;
static constexpr uint32_t kBatch = 256;

struct TilePixel {
    uint32_t i, j;     // pixel row / column
    int32_t wi0, wj0;  // first row / column of the wave's 8x8 block
};
__device__ __forceinline__ TilePixel tile_pixel(uint32_t tile_id, uint32_t tile_width, uint32_t tr) {
    const uint32_t ty = tile_id / tile_width, tx = tile_id % tile_width;
    const uint32_t wave = tr >> 6, lane = tr & 63u;
    TilePixel p;
    p.wi0 = (int32_t)(ty * kTile + (wave >> 1) * 8u);
    p.wj0 = (int32_t)(tx * kTile + (wave & 1u) * 8u);
    p.i = (uint32_t)p.wi0 + (lane >> 3);
    p.j = (uint32_t)p.wj0 + (lane & 7u);
    return p;
}

// 16-byte accesses with the non-temporal hint, for arrays a kernel streams through once (measured on a seven-stream
// Adam-like kernel over 1.8 GB: 5.75 instead of 5.32 TB/s when both the loads and the stores carry it)
typedef float gsx_float4_nt __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 load_streaming(const float4* p) {
    const gsx_float4_nt v = __builtin_nontemporal_load(reinterpret_cast<const gsx_float4_nt*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_streaming(float4* p, float4 v) {
    const gsx_float4_nt t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, reinterpret_cast<gsx_float4_nt*>(p));
}

// The record of one Gaussian as the rasterizers read it (gsx_record.h)
__device__ __forceinline__ void store_record(float4* __restrict__ r, vec3 gro, float opac, const mat3& M, float c0,
                                             float c1, float c2, const RecordRegion& g) {
    r[0] = make_float4(gro.x, gro.y, gro.z, opac);
    r[1] = make_float4(M.m[0][0], M.m[0][1], M.m[0][2], M.m[1][0]);
    r[2] = make_float4(M.m[1][1], M.m[1][2], M.m[2][0], M.m[2][1]);
    r[3] = make_float4(M.m[2][2], c0, c1, c2);
    const bool is_empty = g.jmin > g.jmax || g.imin > g.imax;
    const uint32_t jb = is_empty ? 1u : ((uint32_t)g.jmin | ((uint32_t)g.jmax << 16)); // empty: min 1 > max 0
    const uint32_t ib = is_empty ? 1u : ((uint32_t)g.imin | ((uint32_t)g.imax << 16));
    r[4] = make_float4(u2f(jb), u2f(ib), g.cut, g.a00);
    r[5] = make_float4(g.a01, g.a11, g.pcx, g.pcy);
}

// Stage one batch of records (the tile's list entries first, first + step, ... count of them) into LDS: the
// 64 bytes the per-pair arithmetic reads go to `stage`, the power cut-off to `cuts`, the region test stays in
// registers of the staging lane's wave via `region`.  Then build, per wave, the ordered list of batch slots whose
// region meets the wave's 8x8 block and whose slot index is >= t_start.  Returns the length of the wave's list.
// Contains two barriers.
template <uint32_t BATCH = kBatch>
__device__ __forceinline__ uint32_t stage_and_select(const float4* __restrict__ records,
                                                     const int32_t* __restrict__ flatten_ids, int32_t first,
                                                     int32_t step, uint32_t count, uint32_t tr, const TilePixel& px,
                                                     uint32_t t_start, bool wave_active, float4* stage, float4* region,
                                                     float* cuts, int32_t* ids, uint8_t* wave_list) {
    if (tr < count) {
        const int32_t g = flatten_ids[first + step * (int32_t)tr];
        const float4* __restrict__ r = records + (size_t)g * kRecordF4;
        const float4 r0 = r[0], r1 = r[1], r2 = r[2], r3 = r[3], r4 = r[4], r5 = r[5];
        stage[tr * 4 + 0] = r0;
        stage[tr * 4 + 1] = r1;
        stage[tr * 4 + 2] = r2;
        stage[tr * 4 + 3] = r3;
        region[tr * 2 + 0] = r4;
        region[tr * 2 + 1] = r5;
        cuts[tr] = r4.z;
        if (ids != nullptr)
            ids[tr] = g;
    }
    __syncthreads();
    uint32_t n = 0;
    if (wave_active) {
        const uint32_t lane = tr & 63u;
#pragma unroll
        for (uint32_t r = 0; r < BATCH / 64; ++r) {
            const uint32_t t = r * 64u + lane;
            bool hit = false;
            if (t < count && t >= t_start) {
                const float4 q0 = region[t * 2 + 0], q1 = region[t * 2 + 1];
                const uint32_t jb = f2u(q0.x), ib = f2u(q0.y);
                hit = record_region_hits_block((int32_t)(jb & 0xffffu), (int32_t)(ib & 0xffffu), (int32_t)(jb >> 16),
                                               (int32_t)(ib >> 16), q0.w, q1.x, q1.y, q1.z, q1.w, px.wi0, px.wj0);
            }
            const uint64_t m = __builtin_amdgcn_ballot_w64(hit);
            if (hit) {
                const uint32_t below =
                    __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                wave_list[n + below] = (uint8_t)t;
            }
            n += (uint32_t)__builtin_popcountll(m);
        }
    }
    __syncthreads();
    return n;
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
