// fastgs.hip - the reference's default ("fastgs", Jacobian-EWA) rasterization backend behind
// fast_gs::rasterization::forward_wrapper / backward_wrapper (src/training/fastgs/rasterization/include/
// rasterization_api.h:25-75; src/forward.cu:15-199; src/backward.cu:14-116; kernels in include/kernels_forward.cuh,
// include/kernels_backward.cuh, include/kernel_utils.cuh), re-designed for 64-wide wavefronts:
//
//  * preprocess: one lane per Gaussian (raw parameters in, activations fused), exact per-tile contribution test
//    with wave-cooperative counting for large footprints.  No atomic compaction: every Gaussian writes a
//    (tile count << 32 | depth bits) key and the N keys are sorted on the depth bits, which gives the visiting
//    order and the counts in that order deterministically (ties by index).
//  * instances: emitted in depth order with their 16-bit tile index as the key, which is all that is sorted
//    afterwards.
//  * blend forward / backward: one 256-lane workgroup per 16x16 tile, each wave owns an 8x8 pixel block and keeps
//    its own ordered list of the batch's Gaussians whose footprint box meets the block.  The backward walks back
//    to front from the last contributor with the final transmittance (no per-bucket checkpoints are stored: the
//    reference writes and re-reads 4 KB per 32 list entries), sums the nine per-Gaussian terms over the wave with
//    a halving butterfly, accumulates per batch in LDS and flushes with coalesced atomics.
//  * preprocess backward: one lane per Gaussian, clears the accumulator row it consumed.
#include "gsx_common.h"
#include "../../include/gsx_fastgs.h"
#include "gsx_wave.h"

namespace gsx {

static constexpr float kFgsDilation = 0.3f;          // rasterization_config.h:17
static constexpr float kFgsMinAlphaRcp = 255.0f;     // :18
static constexpr float kFgsMinAlpha = 1.0f / 255.0f; // :19
static constexpr float kFgsMaxAlpha = 0.999f;        // :20
static constexpr float kFgsMinT = 1e-4f;             // :21
// tiles of a footprint the owning lane tests itself before the wave takes over the rest; the reference takes 4 on a
// 32-lane warp (:32).  A cooperative round on 64 lanes costs a wave-wide pass per Gaussian however few tiles are left:
// 12 measured best at 1 M Gaussians (preprocess 105 -> 78 us, instances 98 -> 65 us; 4, 8, 16, 32, 64 tried)
static constexpr uint32_t kFgsSequential = 12;
static constexpr uint32_t kFgsMaxRestFloats = 45; // 15 higher-band coefficients x 3 channels (degree 3)
static constexpr uint32_t kFgsPrimF4 = 3;            // per-primitive record: 12 floats
static constexpr uint32_t kFgsAcc = 12;              // backward accumulator row (9 used)

struct FgsCam {
    float r1[4], r2[4], r3[4], cam[3];
    uint32_t active_bases, total_rest, grid_w, grid_h;
    float w, h, fx, fy, cx, cy, near_plane, far_plane;
};

struct FgsProj {
    float depth, opacity, x, y, tx, ty, j11, j22, q_norm_sq, power_threshold;
    float mean2d[2], cov2d[3], conic[3], variance[3];
    float R[9], RS[9], jw1[3], jw2[3], jwc1[3], jwc2[3];
};

__device__ __forceinline__ float fgs_clamp(float f, float a, float b) { // helper_math.h:1006-1008
    const float m = f < b ? f : b;
    return a > m ? a : m;
}

// preprocess_cu up to the conic (kernels_forward.cuh:58-163); returns false for a culled primitive.  Operation
// order is part of the contract with the CPU checker.
__device__ __forceinline__ bool fgs_project(const float* __restrict__ mean, const float* __restrict__ raw_scale,
                                            const float4 raw_rot, float raw_opacity, const FgsCam& c, FgsProj& P) {
    bool active = true;
    const float depth = c.r3[0] * mean[0] + c.r3[1] * mean[1] + c.r3[2] * mean[2] + c.r3[3];
    P.depth = depth;
    if (depth < c.near_plane || depth > c.far_plane)
        active = false;
    const float opacity = 1.0f / (1.0f + gsx::exp(-raw_opacity));
    P.opacity = opacity;
    if (opacity < kFgsMinAlpha)
        active = false;
#pragma unroll
    for (int k = 0; k < 3; ++k)
        P.variance[k] = gsx::exp(2.0f * raw_scale[k]);
    const float qr = raw_rot.x, qx = raw_rot.y, qy = raw_rot.z, qz = raw_rot.w;
    const float qrr_raw = qr * qr, qxx_raw = qx * qx, qyy_raw = qy * qy, qzz_raw = qz * qz;
    const float q_norm_sq = qrr_raw + qxx_raw + qyy_raw + qzz_raw;
    P.q_norm_sq = q_norm_sq;
    if (q_norm_sq < 1e-8f)
        active = false;
    const float qxx = 2.0f * qxx_raw / q_norm_sq, qyy = 2.0f * qyy_raw / q_norm_sq, qzz = 2.0f * qzz_raw / q_norm_sq;
    const float qxy = 2.0f * qx * qy / q_norm_sq, qxz = 2.0f * qx * qz / q_norm_sq, qyz = 2.0f * qy * qz / q_norm_sq;
    const float qrx = 2.0f * qr * qx / q_norm_sq, qry = 2.0f * qr * qy / q_norm_sq, qrz = 2.0f * qr * qz / q_norm_sq;
    float* R = P.R;
    R[0] = 1.0f - (qyy + qzz), R[1] = qxy - qrz, R[2] = qry + qxz;
    R[3] = qrz + qxy, R[4] = 1.0f - (qxx + qzz), R[5] = qyz - qrx;
    R[6] = qxz - qry, R[7] = qrx + qyz, R[8] = 1.0f - (qxx + qyy);
    float* RS = P.RS;
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int k = 0; k < 3; ++k)
            RS[i * 3 + k] = R[i * 3 + k] * P.variance[k];
    float C[6]; // m11 m12 m13 m22 m23 m33
    C[0] = RS[0] * R[0] + RS[1] * R[1] + RS[2] * R[2];
    C[1] = RS[0] * R[3] + RS[1] * R[4] + RS[2] * R[5];
    C[2] = RS[0] * R[6] + RS[1] * R[7] + RS[2] * R[8];
    C[3] = RS[3] * R[3] + RS[4] * R[4] + RS[5] * R[5];
    C[4] = RS[3] * R[6] + RS[4] * R[7] + RS[5] * R[8];
    C[5] = RS[6] * R[6] + RS[7] * R[7] + RS[8] * R[8];
    const float x = (c.r1[0] * mean[0] + c.r1[1] * mean[1] + c.r1[2] * mean[2] + c.r1[3]) / depth;
    const float y = (c.r2[0] * mean[0] + c.r2[1] * mean[1] + c.r2[2] * mean[2] + c.r2[3]) / depth;
    P.x = x, P.y = y;
    const float clip_left = (-0.15f * c.w - c.cx) / c.fx, clip_right = (1.15f * c.w - c.cx) / c.fx;
    const float clip_top = (-0.15f * c.h - c.cy) / c.fy, clip_bottom = (1.15f * c.h - c.cy) / c.fy;
    const float tx = fgs_clamp(x, clip_left, clip_right), ty = fgs_clamp(y, clip_top, clip_bottom);
    P.tx = tx, P.ty = ty;
    const float j11 = c.fx / depth, j13 = -j11 * tx, j22 = c.fy / depth, j23 = -j22 * ty;
    P.j11 = j11, P.j22 = j22;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        P.jw1[k] = j11 * c.r1[k] + j13 * c.r3[k];
        P.jw2[k] = j22 * c.r2[k] + j23 * c.r3[k];
    }
    const float* a = P.jw1;
    const float* b = P.jw2;
    P.jwc1[0] = a[0] * C[0] + a[1] * C[1] + a[2] * C[2];
    P.jwc1[1] = a[0] * C[1] + a[1] * C[3] + a[2] * C[4];
    P.jwc1[2] = a[0] * C[2] + a[1] * C[4] + a[2] * C[5];
    P.jwc2[0] = b[0] * C[0] + b[1] * C[1] + b[2] * C[2];
    P.jwc2[1] = b[0] * C[1] + b[1] * C[3] + b[2] * C[4];
    P.jwc2[2] = b[0] * C[2] + b[1] * C[4] + b[2] * C[5];
    float cov[3];
    cov[0] = P.jwc1[0] * a[0] + P.jwc1[1] * a[1] + P.jwc1[2] * a[2];
    cov[1] = P.jwc1[0] * b[0] + P.jwc1[1] * b[1] + P.jwc1[2] * b[2];
    cov[2] = P.jwc2[0] * b[0] + P.jwc2[1] * b[1] + P.jwc2[2] * b[2];
    cov[0] += kFgsDilation;
    cov[2] += kFgsDilation;
    P.cov2d[0] = cov[0], P.cov2d[1] = cov[1], P.cov2d[2] = cov[2];
    const float det = cov[0] * cov[2] - cov[1] * cov[1];
    if (det < 1e-8f)
        active = false;
    P.conic[0] = cov[2] / det, P.conic[1] = -cov[1] / det, P.conic[2] = cov[0] / det;
    P.mean2d[0] = x * c.fx + c.cx, P.mean2d[1] = y * c.fy + c.cy;
    P.power_threshold = gsx::log(opacity * kFgsMinAlphaRcp);
    return active;
}

// min(cap, (uint)max(0, __float2int_rd / _ru(v)))  (kernels_forward.cuh:168-173)
__device__ __forceinline__ uint32_t fgs_tile_lo(float v, uint32_t cap) {
    const float f = gsx::floor(v);
    const float g = f > 0.0f ? f : 0.0f; // also maps NaN to 0
    return g >= (float)cap ? cap : (uint32_t)g;
}
__device__ __forceinline__ uint32_t fgs_tile_hi(float v, uint32_t cap) {
    const float f = gsx::ceil(v);
    const float g = f > 0.0f ? f : 0.0f;
    return g >= (float)cap ? cap : (uint32_t)g;
}

// will_primitive_contribute (kernel_utils.cuh:108-143); (mx, my) is the mean shifted by -0.5
__device__ __forceinline__ bool fgs_will_contribute(float mx, float my, float c0, float c1, float c2, uint32_t tile_x,
                                                    uint32_t tile_y, float power_threshold) {
    const float rect_min_x = (float)(tile_x * kTile), rect_min_y = (float)(tile_y * kTile);
    const float rect_max_x = (float)((tile_x + 1) * kTile - 1), rect_max_y = (float)((tile_y + 1) * kTile - 1);
    const float x_min_diff = rect_min_x - mx;
    const float x_left = x_min_diff > 0.0f ? 1.0f : 0.0f;
    const float not_in_x_range = x_left + (mx > rect_max_x ? 1.0f : 0.0f);
    const float y_min_diff = rect_min_y - my;
    const float y_above = y_min_diff > 0.0f ? 1.0f : 0.0f;
    const float not_in_y_range = y_above + (my > rect_max_y ? 1.0f : 0.0f);
    if (not_in_y_range + not_in_x_range == 0.0f)
        return true;
    const float corner_x = rect_max_x + x_left * (rect_min_x - rect_max_x);
    const float corner_y = rect_max_y + y_above * (rect_min_y - rect_max_y);
    const float diff_x = mx - corner_x, diff_y = my - corner_y;
    const float dx = __builtin_copysignf((float)(kTile - 1), x_min_diff);
    const float dy = __builtin_copysignf((float)(kTile - 1), y_min_diff);
    const float qx = (dx * c0 * diff_x + dx * c1 * diff_y) / (dx * c0 * dx);
    const float qy = (dy * c1 * diff_x + dy * c2 * diff_y) / (dy * c2 * dy);
    const float sx = qx > 0.0f ? (qx < 1.0f ? qx : 1.0f) : 0.0f; // __saturatef, NaN -> 0
    const float sy = qy > 0.0f ? (qy < 1.0f ? qy : 1.0f) : 0.0f;
    const float tx = not_in_y_range * sx, ty = not_in_x_range * sy;
    const float px = corner_x + tx * dx, py = corner_y + ty * dy;
    const float ddx = mx - px, ddy = my - py;
    const float max_power = 0.5f * (c0 * ddx * ddx + c2 * ddy * ddy) + c1 * ddx * ddy;
    return max_power <= power_threshold;
}

// convert_sh_to_color (kernel_utils.cuh:15-41)
__device__ __forceinline__ void fgs_sh_to_color(const float* __restrict__ sh0, const float* __restrict__ rest,
                                                const float* __restrict__ pos, const float* cam, uint32_t active,
                                                float* out) {
#pragma unroll
    for (int ch = 0; ch < 3; ++ch)
        out[ch] = 0.5f + 0.28209479177387814f * sh0[ch];
    if (active > 1) {
        const float dx = pos[0] - cam[0], dy = pos[1] - cam[1], dz = pos[2] - cam[2];
        const float inv = gsx::rsqrt(dx * dx + dy * dy + dz * dz);
        const float x = dx * inv, y = dy * inv, z = dz * inv;
#pragma unroll
        for (int ch = 0; ch < 3; ++ch)
            out[ch] = out[ch] + (-0.48860251190291987f * y) * rest[0 * 3 + ch] + (0.48860251190291987f * z) * rest[1 * 3 + ch] +
                      (-0.48860251190291987f * x) * rest[2 * 3 + ch];
        if (active > 4) {
            const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, xz = x * z, yz = y * z;
#pragma unroll
            for (int ch = 0; ch < 3; ++ch)
                out[ch] = out[ch] + (1.0925484305920792f * xy) * rest[3 * 3 + ch] + (-1.0925484305920792f * yz) * rest[4 * 3 + ch] +
                          (0.94617469575755997f * zz - 0.31539156525251999f) * rest[5 * 3 + ch] +
                          (-1.0925484305920792f * xz) * rest[6 * 3 + ch] +
                          (0.54627421529603959f * xx - 0.54627421529603959f * yy) * rest[7 * 3 + ch];
            if (active > 9) {
#pragma unroll
                for (int ch = 0; ch < 3; ++ch)
                    out[ch] = out[ch] + (0.59004358992664352f * y * (-3.0f * xx + yy)) * rest[8 * 3 + ch] +
                              (2.8906114426405538f * xy * z) * rest[9 * 3 + ch] +
                              (0.45704579946446572f * y * (1.0f - 5.0f * zz)) * rest[10 * 3 + ch] +
                              (0.3731763325901154f * z * (5.0f * zz - 3.0f)) * rest[11 * 3 + ch] +
                              (0.45704579946446572f * x * (1.0f - 5.0f * zz)) * rest[12 * 3 + ch] +
                              (1.4453057213202769f * z * (xx - yy)) * rest[13 * 3 + ch] +
                              (0.59004358992664352f * x * (-xx + 3.0f * yy)) * rest[14 * 3 + ch];
            }
        }
    }
}

// ---- preprocess ----------------------------------------------------------------------------------
// prims [N] (3 float4): {mean2d.x, mean2d.y, conic.x, conic.y} {conic.z, opacity, colour r, g} {colour b (raw, the
// clamp at 0 happens at load as in the reference), box half-width x, y, depth}.  The box is the footprint
// |d| <= sqrt(2 ln(255 o) cov_ii), inflated so that a pixel the blend's own arithmetic lets contribute is never
// outside it.
__global__ void __launch_bounds__(256) fgs_preprocess_kernel(
    uint32_t N, const float* __restrict__ means, const float* __restrict__ scales_raw,
    const float* __restrict__ rotations_raw, const float* __restrict__ opacities_raw, const float* __restrict__ sh0,
    const float* __restrict__ shN, const FgsCam c, float4* __restrict__ prims, uint32_t* __restrict__ n_touched,
    ushort4* __restrict__ bounds_out, int64_t* __restrict__ keys, int32_t* __restrict__ order) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    bool active = i < N;
    FgsProj P = {};
    uint32_t b[4] = {0, 0, 0, 0};
    uint32_t tile_count = 0;
    float mean[3] = {0.f, 0.f, 0.f};
    if (active) {
        mean[0] = means[3 * i], mean[1] = means[3 * i + 1], mean[2] = means[3 * i + 2];
        const float rs[3] = {scales_raw[3 * i], scales_raw[3 * i + 1], scales_raw[3 * i + 2]};
        active = fgs_project(mean, rs, reinterpret_cast<const float4*>(rotations_raw)[i], opacities_raw[i], c, P);
    }
    float ext_x = 0.f, ext_y = 0.f;
    if (active) {
        const float factor = gsx::sqrt(2.0f * P.power_threshold);
        const float fx = factor * gsx::sqrt(P.cov2d[0]), fy = factor * gsx::sqrt(P.cov2d[2]);
        float ex = fx - 0.5f, ey = fy - 0.5f;
        ex = ex > 0.0f ? ex : 0.0f, ey = ey > 0.0f ? ey : 0.0f;
        b[0] = fgs_tile_lo((P.mean2d[0] - ex) / (float)kTile, c.grid_w);
        b[1] = fgs_tile_hi((P.mean2d[0] + ex) / (float)kTile, c.grid_w);
        b[2] = fgs_tile_lo((P.mean2d[1] - ey) / (float)kTile, c.grid_h);
        b[3] = fgs_tile_hi((P.mean2d[1] + ey) / (float)kTile, c.grid_h);
        tile_count = (b[1] - b[0]) * (b[3] - b[2]);
        if (tile_count == 0)
            active = false;
        ext_x = fx * 1.01f + 0.25f, ext_y = fy * 1.01f + 0.25f;
    }
    // compute_exact_n_touched_tiles (kernel_utils.cuh:146-210), 64 lanes wide
    const float mx = P.mean2d[0] - 0.5f, my = P.mean2d[1] - 0.5f;
    uint32_t cnt = 0;
    if (active) {
        const uint32_t bw = b[1] - b[0];
        for (uint32_t k = 0; k < tile_count && k < kFgsSequential; ++k)
            cnt += fgs_will_contribute(mx, my, P.conic[0], P.conic[1], P.conic[2], b[0] + k % bw, b[2] + k / bw,
                                       P.power_threshold)
                       ? 1u
                       : 0u;
    }
    uint64_t remaining = __builtin_amdgcn_ballot_w64(active && tile_count > kFgsSequential);
    while (remaining) {
        const int src = __builtin_ctzll(remaining);
        remaining &= remaining - 1;
        const uint32_t bx0 = (uint32_t)__shfl((int)b[0], src, 64), bx1 = (uint32_t)__shfl((int)b[1], src, 64);
        const uint32_t by0 = (uint32_t)__shfl((int)b[2], src, 64), by1 = (uint32_t)__shfl((int)b[3], src, 64);
        const float smx = __shfl(mx, src, 64), smy = __shfl(my, src, 64);
        const float s0 = __shfl(P.conic[0], src, 64), s1 = __shfl(P.conic[1], src, 64), s2 = __shfl(P.conic[2], src, 64);
        const float spt = __shfl(P.power_threshold, src, 64);
        const uint32_t bw = bx1 - bx0, total = bw * (by1 - by0);
        uint32_t found = 0;
        for (uint32_t base = kFgsSequential; base < total; base += 64u) {
            const uint32_t k = base + lane;
            const bool hit = k < total && fgs_will_contribute(smx, smy, s0, s1, s2, bx0 + k % bw, by0 + k / bw, spt);
            found += (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(hit));
        }
        if ((int)lane == src)
            cnt += found;
    }
    if (i >= N)
        return;
    if (!active)
        cnt = 0;
    n_touched[i] = cnt;
    keys[i] = (int64_t)(((uint64_t)cnt << 32) | (cnt ? f2u(P.depth) : 0xFFFFFFFFu));
    order[i] = (int32_t)i;
    if (cnt == 0)
        return;
    bounds_out[i] = make_ushort4((unsigned short)b[0], (unsigned short)b[1], (unsigned short)b[2], (unsigned short)b[3]);
    float col[3];
    fgs_sh_to_color(sh0 + 3 * (size_t)i, shN + (size_t)i * c.total_rest * 3, mean, c.cam, c.active_bases, col);
    float4* pr = prims + (size_t)i * kFgsPrimF4;
    pr[0] = make_float4(P.mean2d[0], P.mean2d[1], P.conic[0], P.conic[1]);
    pr[1] = make_float4(P.conic[2], P.opacity, col[0], col[1]);
    pr[2] = make_float4(col[2], ext_x, ext_y, P.depth);
}

// ---- instances (create_instances_cu, kernels_forward.cuh:220-321) -----------------------------------
// One lane per depth-ordered position; keys are the 16-bit tile index (the reference's ushort keys,
// buffer_utils.h:90), values the primitive index.
__global__ void __launch_bounds__(256) fgs_create_instances_kernel(
    uint32_t N, const int32_t* __restrict__ order, const int64_t* __restrict__ cum /*inclusive*/,
    const uint32_t* __restrict__ n_touched, const ushort4* __restrict__ bounds, const float4* __restrict__ prims,
    uint32_t grid_w, uint16_t* __restrict__ keys, int32_t* __restrict__ vals) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    const uint32_t lane = threadIdx.x & 63u;
    bool active = idx < N;
    uint32_t prim = 0, cnt = 0;
    if (active) {
        prim = (uint32_t)order[idx];
        cnt = n_touched[prim];
        active = cnt != 0;
    }
    uint32_t b[4] = {0, 0, 0, 0};
    float mx = 0.f, my = 0.f, c0 = 0.f, c1 = 0.f, c2 = 0.f, pt = 0.f;
    uint32_t write = 0, tile_count = 0;
    if (active) {
        const ushort4 sb = bounds[prim];
        b[0] = sb.x, b[1] = sb.y, b[2] = sb.z, b[3] = sb.w;
        const float4 p0 = prims[(size_t)prim * kFgsPrimF4], p1 = prims[(size_t)prim * kFgsPrimF4 + 1];
        mx = p0.x - 0.5f, my = p0.y - 0.5f, c0 = p0.z, c1 = p0.w, c2 = p1.x;
        pt = gsx::log(p1.y * kFgsMinAlphaRcp);
        write = (uint32_t)(cum[idx] - (int64_t)cnt);
        const uint32_t bw = b[1] - b[0];
        tile_count = bw * (b[3] - b[2]);
        for (uint32_t k = 0; k < tile_count && k < kFgsSequential; ++k) {
            const uint32_t tx = b[0] + k % bw, ty = b[2] + k / bw;
            if (fgs_will_contribute(mx, my, c0, c1, c2, tx, ty, pt)) {
                keys[write] = (uint16_t)(ty * grid_w + tx);
                vals[write] = (int32_t)prim;
                ++write;
            }
        }
    }
    uint64_t remaining = __builtin_amdgcn_ballot_w64(active && tile_count > kFgsSequential);
    while (remaining) {
        const int src = __builtin_ctzll(remaining);
        remaining &= remaining - 1;
        const uint32_t bx0 = (uint32_t)__shfl((int)b[0], src, 64), bx1 = (uint32_t)__shfl((int)b[1], src, 64);
        const uint32_t by0 = (uint32_t)__shfl((int)b[2], src, 64), by1 = (uint32_t)__shfl((int)b[3], src, 64);
        const float smx = __shfl(mx, src, 64), smy = __shfl(my, src, 64);
        const float s0 = __shfl(c0, src, 64), s1 = __shfl(c1, src, 64), s2 = __shfl(c2, src, 64);
        const float spt = __shfl(pt, src, 64);
        const int32_t sprim = __shfl((int)prim, src, 64);
        uint32_t at = (uint32_t)__shfl((int)write, src, 64);
        const uint32_t bw = bx1 - bx0, total = bw * (by1 - by0);
        for (uint32_t base = kFgsSequential; base < total; base += 64u) {
            const uint32_t k = base + lane;
            const uint32_t tx = bx0 + k % bw, ty = by0 + k / bw;
            const bool hit = k < total && fgs_will_contribute(smx, smy, s0, s1, s2, tx, ty, spt);
            const uint64_t m = __builtin_amdgcn_ballot_w64(hit);
            if (hit) {
                const uint32_t below =
                    __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                keys[at + below] = (uint16_t)(ty * grid_w + tx);
                vals[at + below] = sprim;
            }
            at += (uint32_t)__builtin_popcountll(m);
        }
    }
}

// ---- blend ---------------------------------------------------------------------------------------
// Stage `count` records of the tile's list (entries first, first + step, ...) and build the wave's ordered list of
// the slots >= t_start whose footprint box meets the wave's 8x8 block of pixel centres.  One barrier inside; the
// caller places one before the next staging.
__device__ __forceinline__ uint32_t fgs_stage_and_select(const float4* __restrict__ prims,
                                                         const int32_t* __restrict__ inst, int32_t first, int32_t step,
                                                         uint32_t count, uint32_t tr, const TilePixel& px,
                                                         uint32_t t_start, bool wave_active, float4* stage,
                                                         int32_t* ids, uint8_t* wave_list) {
    if (tr < count) {
        const int32_t g = inst[first + step * (int32_t)tr];
        const float4* __restrict__ r = prims + (size_t)g * kFgsPrimF4;
        const float4 r0 = r[0], r1 = r[1], r2 = r[2];
        stage[tr * 3 + 0] = r0;
        stage[tr * 3 + 1] = r1;
        stage[tr * 3 + 2] = r2;
        if (ids != nullptr)
            ids[tr] = g;
    }
    __syncthreads();
    uint32_t n = 0;
    if (wave_active) {
        const uint32_t lane = tr & 63u;
        const float bx0 = (float)px.wj0 + 0.5f, bx1 = (float)px.wj0 + 7.5f;
        const float by0 = (float)px.wi0 + 0.5f, by1 = (float)px.wi0 + 7.5f;
#pragma unroll
        for (uint32_t r = 0; r < kBatch / 64; ++r) {
            const uint32_t t = r * 64u + lane;
            bool hit = false;
            if (t < count && t >= t_start) {
                const float4 q0 = stage[t * 3 + 0], q2 = stage[t * 3 + 2];
                hit = q0.x + q2.y >= bx0 && q0.x - q2.y <= bx1 && q0.y + q2.z >= by0 && q0.y - q2.z <= by1;
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
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    return n;
}

// blend_cu (kernels_forward.cuh:356-459).  image [3,H,W] (+ T * background when given, fast_rasterizer.cpp:63),
// alpha [H,W], and for the backward the final transmittance and the list position after the last contributor.
__global__ void __launch_bounds__(256) fgs_blend_fwd_kernel(
    uint32_t n_instances, const float4* __restrict__ prims, const int32_t* __restrict__ tile_offsets,
    const int32_t* __restrict__ inst, uint32_t width, uint32_t height, uint32_t grid_w, uint32_t n_tiles,
    const float* __restrict__ background, float* __restrict__ image, float* __restrict__ alpha_map,
    float* __restrict__ t_final, uint32_t* __restrict__ n_contributions, uint32_t* __restrict__ tile_walk) {
    __shared__ float4 stage[kBatch * kFgsPrimF4];
    __shared__ uint8_t lists[4][kBatch];
    __shared__ uint32_t walk_s;
    const uint32_t tile_id = blockIdx.x;
    const uint32_t tr = threadIdx.x;
    const TilePixel px = tile_pixel(tile_id, grid_w, tr);
    const bool inside = px.i < height && px.j < width;
    const float pxf = (float)px.j + 0.5f, pyf = (float)px.i + 0.5f;
    uint8_t* wave_list = lists[tr >> 6];
    const int32_t range_start = tile_offsets[tile_id];
    const int32_t range_end = (tile_id == n_tiles - 1) ? (int32_t)n_instances : tile_offsets[tile_id + 1];
    float c0 = 0.f, c1 = 0.f, c2 = 0.f, T = 1.0f;
    uint32_t n_contrib = 0;
    bool done = !inside;
    for (int32_t first = range_start; first < range_end; first += (int32_t)kBatch) {
        if (__syncthreads_count(done) == 256) // also the barrier between this staging and the last batch's reads
            break;
        const uint32_t count = (uint32_t)min((int32_t)kBatch, range_end - first);
        const bool wave_active = __builtin_amdgcn_ballot_w64(!done) != 0;
        const uint32_t n_sel = (uint32_t)__builtin_amdgcn_readfirstlane(
            (int)fgs_stage_and_select(prims, inst, first, 1, count, tr, px, 0, wave_active, stage, nullptr, wave_list));
        // a pixel leaves the loop when it is saturated, the wave when its last pixel has (the loop's own divergence:
        // the lane mask shrinks with scalar instructions only)
        for (uint32_t s = 0; s < n_sel && !done; ++s) {
            const uint32_t t = wave_list[s];
            const float4 q0 = stage[t * 3 + 0], q1 = stage[t * 3 + 1];
            const float dx = q0.x - pxf, dy = q0.y - pyf;
            const float sigma_over_2 = 0.5f * (q0.z * dx * dx + q1.x * dy * dy) + q0.w * dx * dy;
            // beyond 87 the exponential is zero (gsx::exp) and alpha with it; up to there its restricted variant has
            // the same bits
            if (sigma_over_2 < 0.0f || sigma_over_2 > 87.0f)
                continue;
            const float gaussian = gsx::exp_nonpos(-sigma_over_2);
            const float og = q1.y * gaussian;
            const float alpha = og < kFgsMaxAlpha ? og : kFgsMaxAlpha;
            if (alpha < kFgsMinAlpha)
                continue;
            const float next = T * (1.0f - alpha);
            if (next < kFgsMinT) {
                done = true;
                continue;
            }
            const float4 q2 = stage[t * 3 + 2];
            const float w = T * alpha;
            c0 += w * (q1.z > 0.0f ? q1.z : 0.0f);
            c1 += w * (q1.w > 0.0f ? q1.w : 0.0f);
            c2 += w * (q2.x > 0.0f ? q2.x : 0.0f);
            T = next;
            n_contrib = (uint32_t)(first - range_start) + t + 1u;
        }
    }
    if (inside) {
        const size_t p = (size_t)px.i * width + px.j, n = (size_t)width * height;
        if (background != nullptr) {
            c0 += T * background[0];
            c1 += T * background[1];
            c2 += T * background[2];
        }
        image[p] = c0;
        image[p + n] = c1;
        image[p + 2 * n] = c2;
        alpha_map[p] = 1.0f - T;
        t_final[p] = T;
        n_contributions[p] = n_contrib;
    }
    // how far into its list the tile's pixels went: what the tile costs the backward pass
    if (tr == 0)
        walk_s = 0;
    __syncthreads();
    uint32_t w = inside ? n_contrib : 0u;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        w = max(w, (uint32_t)__shfl_xor((int)w, m, 64));
    if ((tr & 63u) == 0)
        atomicMax(&walk_s, w);
    __syncthreads();
    if (tr == 0)
        tile_walk[tile_id] = walk_s;
}

// blend_backward_cu (kernels_backward.cuh:240-449) as a back-to-front walk per pixel; per Gaussian and wave the
// nine terms (mean2d 2, conic 3, opacity 1, colour 3) are summed over the 64 pixels, accumulated per batch in LDS
// and flushed to gacc [N, 12] with coalesced atomics.
__global__ void __launch_bounds__(256) fgs_blend_bwd_kernel(
    uint32_t n_instances, const float4* __restrict__ prims, const int32_t* __restrict__ tile_offsets,
    const int32_t* __restrict__ inst, uint32_t width, uint32_t height, uint32_t grid_w, uint32_t n_tiles,
    const float* __restrict__ background, const float* __restrict__ t_final, const uint32_t* __restrict__ n_contributions,
    const float* __restrict__ grad_image, const float* __restrict__ grad_alpha,
    const uint32_t* __restrict__ tile_order, float* __restrict__ gacc) {
    __shared__ float4 stage[kBatch * kFgsPrimF4];
    __shared__ uint8_t lists[4][kBatch];
    __shared__ int32_t id_batch[kBatch];
    __shared__ float acc[kBatch * kFgsAcc];
    __shared__ int32_t block_max;
    const uint32_t tile_id = tile_order[blockIdx.x]; // dearest tiles first
    const uint32_t tr = threadIdx.x, lane = tr & 63u;
    // which of the 9 per-Gaussian sums this lane ends up with after the wave reduction (15: none)
    const uint32_t sum_index = (lane & 3u) == 0 ? wave_reduce9_index(lane) : 15u;
    const TilePixel px = tile_pixel(tile_id, grid_w, tr);
    const bool inside = px.i < height && px.j < width;
    const float pxf = (float)px.j + 0.5f, pyf = (float)px.i + 0.5f;
    uint8_t* wave_list = lists[tr >> 6];
    const int32_t range_start = tile_offsets[tile_id];
    int32_t range_end = (tile_id == n_tiles - 1) ? (int32_t)n_instances : tile_offsets[tile_id + 1];
    const size_t p = inside ? (size_t)px.i * width + px.j : 0, n = (size_t)width * height;
    const int32_t last = inside ? (int32_t)n_contributions[p] : 0; // list positions < last are replayed
    const float T_final = inside ? t_final[p] : 1.0f;
    const float g0 = inside ? grad_image[p] : 0.f, g1 = inside ? grad_image[p + n] : 0.f,
                g2 = inside ? grad_image[p + 2 * n] : 0.f;
    float ga = inside ? grad_alpha[p] : 0.f;
    if (background != nullptr) // image = blend + T * background: the same path as alpha = 1 - T, opposite sign
        ga -= background[0] * g0 + background[1] * g1 + background[2] * g2;
    const float ga_common = ga * T_final; // grad_alpha * (1 - alpha_pixel), kernels_backward.cuh:330

    int32_t wave_last = last;
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
        wave_last = max(wave_last, __shfl_xor(wave_last, m, 64));
    wave_last = __builtin_amdgcn_readfirstlane(wave_last);
    if (tr == 0)
        block_max = 0;
    __syncthreads();
    if (lane == 0)
        atomicMax(&block_max, wave_last);
#pragma unroll
    for (uint32_t k = 0; k < kFgsAcc; ++k)
        acc[tr * kFgsAcc + k] = 0.f;
    __syncthreads();
    range_end = min(range_end, range_start + block_max);
    if (range_end <= range_start)
        return;
    float T = T_final, adot = 0.f; // adot: colour behind the current Gaussian, dotted with the pixel's colour gradient
    const uint32_t num_batches = (uint32_t)(range_end - range_start + (int32_t)kBatch - 1) / kBatch;
    for (uint32_t b = 0; b < num_batches; ++b) {
        const int32_t batch_end = range_end - 1 - (int32_t)(kBatch * b); // slot 0: the farthest entry
        const int32_t batch_size = min((int32_t)kBatch, batch_end + 1 - range_start);
        // slots in front of t_start lie behind every last contributor of this wave
        const uint32_t t_start = (uint32_t)max(0, batch_end - (range_start + wave_last - 1));
        const uint32_t n_sel = (uint32_t)__builtin_amdgcn_readfirstlane(
            (int)fgs_stage_and_select(prims, inst, batch_end, -1, (uint32_t)batch_size, tr, px, t_start,
                                      t_start < (uint32_t)batch_size, stage, id_batch, wave_list));
        for (uint32_t s = 0; s < n_sel; ++s) {
            const int32_t t = (int32_t)wave_list[s];
            bool valid = inside && (batch_end - t - range_start < last);
            const float4 q0 = stage[t * 3 + 0], q1 = stage[t * 3 + 1], q2 = stage[t * 3 + 2];
            const float dx = q0.x - pxf, dy = q0.y - pyf;
            const float sigma_over_2 = 0.5f * (q0.z * dx * dx + q1.x * dy * dy) + q0.w * dx * dy;
            if (sigma_over_2 < 0.0f || sigma_over_2 > 87.0f) // beyond 87: exp = 0 and alpha below the threshold
                valid = false;
            if (__builtin_amdgcn_ballot_w64(valid) == 0)
                continue;
            const float gaussian = gsx::exp_nonpos(-(valid ? sigma_over_2 : 0.0f)); // gsx::exp's bits on [-87, 0]
            const float og = q1.y * gaussian;
            const float alpha = og < kFgsMaxAlpha ? og : kFgsMaxAlpha;
            if (alpha < kFgsMinAlpha)
                valid = false;
            if (__builtin_amdgcn_ballot_w64(valid) == 0)
                continue;
            // branch-free from here: a lane that is not valid carries ra = 1 and zero weights
            const float ra = valid ? gsx::rcp_refined(1.0f - alpha) : 1.0f;
            T *= ra; // transmittance in front of this Gaussian
            const float w = valid ? T * alpha : 0.f;
            const float col0 = q1.z > 0.0f ? q1.z : 0.0f, col1 = q1.w > 0.0f ? q1.w : 0.0f,
                        col2 = q2.x > 0.0f ? q2.x : 0.0f;
            // sum_k (T c_k - a_k ra) g_k with the colour sums folded: cdot = sum_k c_k g_k, and since a_k grows by
            // w c_k per Gaussian, adot = sum_k a_k g_k grows by w cdot (one running scalar instead of three)
            const float cdot = fma(col2, g2, fma(col1, g1, col0 * g0));
            const float dL_dalpha = fma(T, cdot, ra * (ga_common - adot));
            adot = fma(w, cdot, adot);
            const float ad = valid ? alpha * dL_dalpha : 0.f;
            const float helper = -ad;
            float v[9];
            v[0] = helper * (q0.z * dx + q0.w * dy);
            v[1] = helper * (q0.w * dx + q1.x * dy);
            v[2] = 0.5f * helper * dx * dx;
            v[3] = 0.5f * helper * dx * dy;
            v[4] = 0.5f * helper * dy * dy;
            v[5] = ad;
            v[6] = q1.z >= 0.0f ? w * g0 : 0.f; // zero where the colour was clamped (:286-291)
            v[7] = q1.w >= 0.0f ? w * g1 : 0.f;
            v[8] = q2.x >= 0.0f ? w * g2 : 0.f;
            const float total = wave_reduce9(v, lane);
            if (sum_index < 9u)
                atomicAdd(&acc[(uint32_t)t * kFgsAcc + sum_index], total); // LDS: ds_add_f32
        }
        __syncthreads();
#pragma unroll 4
        for (uint32_t s = 0; s < kFgsAcc; ++s) {
            const uint32_t e = s * 256u + tr, gi = e / kFgsAcc, k = e % kFgsAcc;
            if ((int32_t)gi < batch_size && k < 9u) {
                const float val = acc[e];
                acc[e] = 0.f;
                if (val != 0.f)
                    unsafeAtomicAdd(&gacc[(size_t)id_batch[gi] * kFgsAcc + k], val);
            }
        }
        __syncthreads();
    }
}

// ---- preprocess backward (kernels_backward.cuh:17-237, kernel_utils.cuh:43-105) ------------------
__global__ void __launch_bounds__(256) fgs_preprocess_bwd_kernel(
    uint32_t N, const float* __restrict__ means, const float* __restrict__ scales_raw,
    const float* __restrict__ rotations_raw, const float* __restrict__ shN, const FgsCam c,
    const uint32_t* __restrict__ n_touched, const float4* __restrict__ prims, float* __restrict__ gacc,
    float* __restrict__ grad_means, float* __restrict__ grad_scales_raw, float* __restrict__ grad_rotations_raw,
    float* __restrict__ grad_opacities_raw, float* __restrict__ grad_sh0, float* __restrict__ grad_shN,
    float* __restrict__ grad_w2c_partial /*nullable: [12] accumulated with atomics*/,
    float* __restrict__ densification_info /*nullable [2,N]*/) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const bool in = i < N;
    const bool live = in && n_touched[i] != 0;
    const uint32_t B = c.total_rest;
    // The gradient rows of the higher SH bands (180 bytes a Gaussian at degree 3) leave through LDS: a lane fills its
    // own row there and the workgroup then writes its 256 rows, which are one contiguous piece of grad_shN, with
    // 16-byte stores by consecutive lanes (a lane storing its row itself touches 64 cache lines per instruction:
    // 202 us against 121 us at 1 M Gaussians).  Reading the coefficient rows the same way gains nothing here, and in
    // the forward kernel the 46 KB of LDS cost more occupancy than the loads save (78 -> 122 us): not done.
    __shared__ __align__(16) float g_stage[256 * kFgsMaxRestFloats];
    const bool staged = 3u * B <= kFgsMaxRestFloats; // more stored bands than degree 3 has: every lane stores its own row
    float* const gco = staged ? g_stage + threadIdx.x * 3u * B : grad_shN + (size_t)(in ? i : 0u) * 3u * B;
    float dcam[3] = {0.f, 0.f, 0.f}, mean[3] = {0.f, 0.f, 0.f};
    if (in && !live) {
#pragma unroll
        for (int k = 0; k < 3; ++k)
            grad_means[3 * (size_t)i + k] = 0.f, grad_scales_raw[3 * (size_t)i + k] = 0.f, grad_sh0[3 * (size_t)i + k] = 0.f;
        reinterpret_cast<float4*>(grad_rotations_raw)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        grad_opacities_raw[i] = 0.f;
        for (uint32_t k = 0; k < 3 * B; ++k)
            gco[k] = 0.f;
    }
    if (live) {
        float4* row = reinterpret_cast<float4*>(gacc + (size_t)i * kFgsAcc);
        const float4 ra = row[0], rb = row[1], rc = row[2];
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        row[0] = z, row[1] = z, row[2] = z; // ready for the next backward pass
        const float gm2[2] = {ra.x, ra.y};
        const float gk[3] = {ra.z, ra.w, rb.x};
        const float gcol[3] = {rb.z, rb.w, rc.x};
        const float opacity = prims[(size_t)i * kFgsPrimF4 + 1].y;
        grad_opacities_raw[i] = rb.y * (1.0f - opacity); // kernels_backward.cuh:443
        mean[0] = means[3 * (size_t)i], mean[1] = means[3 * (size_t)i + 1], mean[2] = means[3 * (size_t)i + 2];
        // ---- SH backward ----
#pragma unroll
        for (int ch = 0; ch < 3; ++ch)
            grad_sh0[3 * (size_t)i + ch] = 0.28209479177387814f * gcol[ch];
        float dpos[3] = {0.f, 0.f, 0.f};
        const uint32_t active = c.active_bases;
        const uint32_t written = active > 9 ? 15u : (active > 4 ? 8u : (active > 1 ? 3u : 0u));
        for (uint32_t k = 3 * written; k < 3 * B; ++k)
            gco[k] = 0.f; // inactive bases
        if (active > 1) {
            const float* co = shN + (size_t)i * B * 3;
            const float x_raw = mean[0] - c.cam[0], y_raw = mean[1] - c.cam[1], z_raw = mean[2] - c.cam[2];
            const float inv = gsx::rsqrt(x_raw * x_raw + y_raw * y_raw + z_raw * z_raw);
            const float x = x_raw * inv, y = y_raw * inv, zz_ = z_raw * inv;
            const float z = zz_;
            float gdx[3], gdy[3], gdz[3];
#define FGS_SETG(k, basis)                      \
    {                                           \
        const float bb_ = (basis);              \
        gco[(k) * 3 + 0] = bb_ * gcol[0];       \
        gco[(k) * 3 + 1] = bb_ * gcol[1];       \
        gco[(k) * 3 + 2] = bb_ * gcol[2];       \
    }
            FGS_SETG(0, -0.48860251190291987f * y);
            FGS_SETG(1, 0.48860251190291987f * z);
            FGS_SETG(2, -0.48860251190291987f * x);
#pragma unroll
            for (int ch = 0; ch < 3; ++ch) {
                gdx[ch] = -0.48860251190291987f * co[2 * 3 + ch];
                gdy[ch] = -0.48860251190291987f * co[0 * 3 + ch];
                gdz[ch] = 0.48860251190291987f * co[1 * 3 + ch];
            }
            if (active > 4) {
                const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, xz = x * z, yz = y * z;
                FGS_SETG(3, 1.0925484305920792f * xy);
                FGS_SETG(4, -1.0925484305920792f * yz);
                FGS_SETG(5, 0.94617469575755997f * zz - 0.31539156525251999f);
                FGS_SETG(6, -1.0925484305920792f * xz);
                FGS_SETG(7, 0.54627421529603959f * xx - 0.54627421529603959f * yy);
#pragma unroll
                for (int ch = 0; ch < 3; ++ch) {
                    gdx[ch] = gdx[ch] + (1.0925484305920792f * y) * co[3 * 3 + ch] + (-1.0925484305920792f * z) * co[6 * 3 + ch] +
                              (1.0925484305920792f * x) * co[7 * 3 + ch];
                    gdy[ch] = gdy[ch] + (1.0925484305920792f * x) * co[3 * 3 + ch] + (-1.0925484305920792f * z) * co[4 * 3 + ch] +
                              (-1.0925484305920792f * y) * co[7 * 3 + ch];
                    gdz[ch] = gdz[ch] + (-1.0925484305920792f * y) * co[4 * 3 + ch] + (1.8923493915151202f * z) * co[5 * 3 + ch] +
                              (-1.0925484305920792f * x) * co[6 * 3 + ch];
                }
                if (active > 9) {
                    FGS_SETG(8, 0.59004358992664352f * y * (-3.0f * xx + yy));
                    FGS_SETG(9, 2.8906114426405538f * xy * z);
                    FGS_SETG(10, 0.45704579946446572f * y * (1.0f - 5.0f * zz));
                    FGS_SETG(11, 0.3731763325901154f * z * (5.0f * zz - 3.0f));
                    FGS_SETG(12, 0.45704579946446572f * x * (1.0f - 5.0f * zz));
                    FGS_SETG(13, 1.4453057213202769f * z * (xx - yy));
                    FGS_SETG(14, 0.59004358992664352f * x * (-xx + 3.0f * yy));
#pragma unroll
                    for (int ch = 0; ch < 3; ++ch) {
                        gdx[ch] = gdx[ch] + (-3.5402615395598609f * xy) * co[8 * 3 + ch] + (2.8906114426405538f * yz) * co[9 * 3 + ch] +
                                  (0.45704579946446572f - 2.2852289973223288f * zz) * co[12 * 3 + ch] +
                                  (2.8906114426405538f * xz) * co[13 * 3 + ch] +
                                  (-1.7701307697799304f * xx + 1.7701307697799304f * yy) * co[14 * 3 + ch];
                        gdy[ch] = gdy[ch] + (-1.7701307697799304f * xx + 1.7701307697799304f * yy) * co[8 * 3 + ch] +
                                  (2.8906114426405538f * xz) * co[9 * 3 + ch] +
                                  (0.45704579946446572f - 2.2852289973223288f * zz) * co[10 * 3 + ch] +
                                  (-2.8906114426405538f * yz) * co[13 * 3 + ch] + (3.5402615395598609f * xy) * co[14 * 3 + ch];
                        gdz[ch] = gdz[ch] + (2.8906114426405538f * xy) * co[9 * 3 + ch] + (-4.5704579946446566f * yz) * co[10 * 3 + ch] +
                                  (5.597644988851731f * zz - 1.1195289977703462f) * co[11 * 3 + ch] +
                                  (-4.5704579946446566f * xz) * co[12 * 3 + ch] +
                                  (1.4453057213202769f * xx - 1.4453057213202769f * yy) * co[13 * 3 + ch];
                    }
                }
            }
#undef FGS_SETG
            const float gx = gdx[0] * gcol[0] + gdx[1] * gcol[1] + gdx[2] * gcol[2];
            const float gy = gdy[0] * gcol[0] + gdy[1] * gcol[1] + gdy[2] * gcol[2];
            const float gz = gdz[0] * gcol[0] + gdz[1] * gcol[1] + gdz[2] * gcol[2];
            const float xx_raw = x_raw * x_raw, yy_raw = y_raw * y_raw, zz_raw = z_raw * z_raw;
            const float xy_raw = x_raw * y_raw, xz_raw = x_raw * z_raw, yz_raw = y_raw * z_raw;
            const float norm_sq = xx_raw + yy_raw + zz_raw;
            const float s = gsx::rsqrt(norm_sq * norm_sq * norm_sq);
            dpos[0] = ((yy_raw + zz_raw) * gx - xy_raw * gy - xz_raw * gz) * s;
            dpos[1] = (-xy_raw * gx + (xx_raw + zz_raw) * gy - yz_raw * gz) * s;
            dpos[2] = (-xz_raw * gx - yz_raw * gy + (xx_raw + yy_raw) * gz) * s;
        }
        // ---- EWA chain ----
        FgsProj P;
        const float rs[3] = {scales_raw[3 * (size_t)i], scales_raw[3 * (size_t)i + 1], scales_raw[3 * (size_t)i + 2]};
        const float4 q4 = reinterpret_cast<const float4*>(rotations_raw)[i];
        fgs_project(mean, rs, q4, 0.0f, c, P);
        const float a = P.cov2d[0], b = P.cov2d[1], cc_ = P.cov2d[2];
        const float aa = a * a, bb = b * b, cc = cc_ * cc_, ac = a * cc_, ab = a * b, bc = b * cc_;
        const float determinant = ac - bb;
        const float determinant_rcp = 1.0f / determinant;
        const float determinant_rcp_sq = determinant_rcp * determinant_rcp;
        const float dcov[3] = {determinant_rcp_sq * (2.0f * bc * gk[1] - cc * gk[0] - bb * gk[2]),
                               determinant_rcp_sq * (bc * gk[0] - (ac + bb) * gk[1] + ab * gk[2]),
                               determinant_rcp_sq * (2.0f * ab * gk[1] - bb * gk[0] - aa * gk[2])};
        const float* j1 = P.jw1;
        const float* j2 = P.jw2;
        float d3[6];
        d3[0] = (j1[0] * j1[0]) * dcov[0] + 2.0f * (j1[0] * j2[0]) * dcov[1] + (j2[0] * j2[0]) * dcov[2];
        d3[1] = (j1[0] * j1[1]) * dcov[0] + (j1[0] * j2[1] + j1[1] * j2[0]) * dcov[1] + (j2[0] * j2[1]) * dcov[2];
        d3[2] = (j1[0] * j1[2]) * dcov[0] + (j1[0] * j2[2] + j1[2] * j2[0]) * dcov[1] + (j2[0] * j2[2]) * dcov[2];
        d3[3] = (j1[1] * j1[1]) * dcov[0] + 2.0f * (j1[1] * j2[1]) * dcov[1] + (j2[1] * j2[1]) * dcov[2];
        d3[4] = (j1[1] * j1[2]) * dcov[0] + (j1[1] * j2[2] + j1[2] * j2[1]) * dcov[1] + (j2[1] * j2[2]) * dcov[2];
        d3[5] = (j1[2] * j1[2]) * dcov[0] + 2.0f * (j1[2] * j2[2]) * dcov[1] + (j2[2] * j2[2]) * dcov[2];
        float djw1[3], djw2[3];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            djw1[k] = 2.0f * (P.jwc1[k] * dcov[0] + P.jwc2[k] * dcov[1]);
            djw2[k] = 2.0f * (P.jwc1[k] * dcov[1] + P.jwc2[k] * dcov[2]);
        }
        const float dj11 = c.r1[0] * djw1[0] + c.r1[1] * djw1[1] + c.r1[2] * djw1[2];
        const float dj22 = c.r2[0] * djw2[0] + c.r2[1] * djw2[1] + c.r2[2] * djw2[2];
        const float dj13 = c.r3[0] * djw1[0] + c.r3[1] * djw1[1] + c.r3[2] * djw1[2];
        const float dj23 = c.r3[0] * djw2[0] + c.r3[1] * djw2[1] + c.r3[2] * djw2[2];
        const float h1 = dj11 - 2.0f * P.tx * dj13, h2 = dj22 - 2.0f * P.ty * dj23;
        dcam[0] = P.j11 * (gm2[0] - dj13 / P.depth);
        dcam[1] = P.j22 * (gm2[1] - dj23 / P.depth);
        dcam[2] = -P.j11 * (P.x * gm2[0] + h1 / P.depth) - P.j22 * (P.y * gm2[1] + h2 / P.depth);
#pragma unroll
        for (int k = 0; k < 3; ++k)
            grad_means[3 * (size_t)i + k] = (c.r1[k] * dcam[0] + c.r2[k] * dcam[1] + c.r3[k] * dcam[2]) + dpos[k];
        const float* R = P.R;
        const float* RS = P.RS;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const float dvar = R[0 + k] * R[0 + k] * d3[0] + R[3 + k] * R[3 + k] * d3[3] + R[6 + k] * R[6 + k] * d3[5] +
                               2.0f * (R[0 + k] * R[3 + k] * d3[1] + R[0 + k] * R[6 + k] * d3[2] + R[3 + k] * R[6 + k] * d3[4]);
            grad_scales_raw[3 * (size_t)i + k] = 2.0f * P.variance[k] * dvar;
        }
        float dR[9];
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            dR[0 + k] = 2.0f * (RS[0 + k] * d3[0] + RS[3 + k] * d3[1] + RS[6 + k] * d3[2]);
            dR[3 + k] = 2.0f * (RS[0 + k] * d3[1] + RS[3 + k] * d3[3] + RS[6 + k] * d3[4]);
            dR[6 + k] = 2.0f * (RS[0 + k] * d3[2] + RS[3 + k] * d3[4] + RS[6 + k] * d3[5]);
        }
        const float qr = q4.x, qx = q4.y, qy = q4.z, qz = q4.w, qn = P.q_norm_sq;
        const float qxx = 2.0f * (qx * qx) / qn, qyy = 2.0f * (qy * qy) / qn, qzz = 2.0f * (qz * qz) / qn;
        const float qxy = 2.0f * qx * qy / qn, qxz = 2.0f * qx * qz / qn, qyz = 2.0f * qy * qz / qn;
        const float qrx = 2.0f * qr * qx / qn, qry = 2.0f * qr * qy / qn, qrz = 2.0f * qr * qz / qn;
        const float dqxx = -dR[4] - dR[8], dqyy = -dR[0] - dR[8], dqzz = -dR[0] - dR[4];
        const float dqxy = dR[1] + dR[3], dqxz = dR[2] + dR[6], dqyz = dR[5] + dR[7];
        const float dqrx = dR[7] - dR[5], dqry = dR[2] - dR[6], dqrz = dR[3] - dR[1];
        const float helper = qxx * dqxx + qyy * dqyy + qzz * dqzz + qxy * dqxy + qxz * dqxz + qyz * dqyz + qrx * dqrx +
                             qry * dqry + qrz * dqrz;
        reinterpret_cast<float4*>(grad_rotations_raw)[i] =
            make_float4(2.0f * (qx * dqrx + qy * dqry + qz * dqrz - qr * helper) / qn,
                        2.0f * (2.0f * qx * dqxx + qy * dqxy + qz * dqxz + qr * dqrx - qx * helper) / qn,
                        2.0f * (2.0f * qy * dqyy + qx * dqxy + qz * dqyz + qr * dqry - qy * helper) / qn,
                        2.0f * (2.0f * qz * dqzz + qx * dqxz + qy * dqyz + qr * dqrz - qz * helper) / qn);
        if (densification_info != nullptr) {
            densification_info[i] += 1.0f;
            const float sx = gm2[0] * (0.5f * c.w), sy = gm2[1] * (0.5f * c.h);
            densification_info[(size_t)N + i] += gsx::sqrt(sx * sx + sy * sy);
        }
    }
    if (staged && B != 0) {
        __syncthreads();
        const size_t first_row = (size_t)blockIdx.x * 256u;
        const uint32_t floats = (uint32_t)min((size_t)256, (size_t)N - first_row) * 3u * B;
        float* const dst = grad_shN + first_row * 3u * B; // 16-byte aligned: 256 rows are a multiple of four floats
        for (uint32_t k = threadIdx.x; k < floats / 4u; k += 256u)
            reinterpret_cast<float4*>(dst)[k] = reinterpret_cast<const float4*>(g_stage)[k];
        for (uint32_t k = (floats & ~3u) + threadIdx.x; k < floats; k += 256u)
            dst[k] = g_stage[k];
    }
    if (grad_w2c_partial != nullptr) { // kernels_backward.cuh:177-190; uniform branch, every lane takes part
        const uint32_t lane = threadIdx.x & 63u;
#pragma unroll
        for (int r = 0; r < 3; ++r) {
            float t[4] = {dcam[r] * mean[0], dcam[r] * mean[1], dcam[r] * mean[2], dcam[r]};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                float v = t[k];
#pragma unroll
                for (int m = 32; m >= 1; m >>= 1)
                    v += __shfl_xor(v, m, 64);
                if (lane == 0 && v != 0.f)
                    unsafeAtomicAdd(&grad_w2c_partial[r * 4 + k], v);
            }
        }
    }
}

__global__ void __launch_bounds__(64) fgs_fill_kernel(uint32_t n, float v, float* __restrict__ out) {
    if (threadIdx.x < n)
        out[threadIdx.x] = v;
}

struct FgsPrimLayout {
    size_t n_touched_off, bounds_off, order_off, cum_off, ws_off, total;
};
static FgsPrimLayout fgs_prim_layout(uint32_t N) {
    FgsPrimLayout L;
    size_t at = align_up((size_t)N * kFgsPrimF4 * 16, 256);
    L.n_touched_off = at, at += align_up((size_t)N * 4, 256);
    L.bounds_off = at, at += align_up((size_t)N * 8, 256);
    L.order_off = at, at += align_up((size_t)N * 4, 256);
    L.cum_off = at, at += align_up((size_t)N * 8, 256);
    L.ws_off = at, at += align_up(gsx_intersect_tile_count_ordered_workspace_bytes(N), 256);
    L.total = at;
    return L;
}

struct FgsInstLayout {
    size_t keys1_off, vals0_off, vals1_off, offsets_off, sel_off, ws_off, total;
};
// bits of the tile index the instance sort looks at (at most 65 536 tiles)
static uint32_t fgs_tile_bits(uint32_t n_tiles) {
    const uint32_t b = gsx_n_bits(n_tiles);
    return b < 16u ? b : 16u;
}
static FgsInstLayout fgs_inst_layout(int64_t n, uint32_t n_tiles) {
    FgsInstLayout L;
    const size_t m = (size_t)(n > 0 ? n : 1);
    size_t at = align_up(m * 2, 256);
    L.keys1_off = at, at += align_up(m * 2, 256);
    L.vals0_off = at, at += align_up(m * 4, 256);
    L.vals1_off = at, at += align_up(m * 4, 256);
    L.offsets_off = at, at += align_up((size_t)n_tiles * 4, 256);
    L.sel_off = at, at += 256;
    L.ws_off = at, at += align_up(gsx_radix_sort_pairs_workspace_bytes((int64_t)m), 256);
    L.total = at;
    return L;
}

static int fgs_make_cam(const char* who, const gsx_fastgs_settings* S, const float* w2c_host, const float* cam_host,
                        FgsCam* c) {
    GSX_REQUIRE(S && w2c_host && cam_host, GSX_ERR_INVALID_ARGUMENT, "%s: null settings / camera", who);
    GSX_REQUIRE(S->width > 0 && S->height > 0 && S->width < 65536u * kTile && S->height < 65536u * kTile,
                GSX_ERR_INVALID_ARGUMENT, "%s: image %u x %u", who, S->width, S->height);
    const uint32_t gw = (S->width + kTile - 1) / kTile, gh = (S->height + kTile - 1) / kTile;
    // the reference's u16 tile keys hold 65536 tiles (kernels_forward.cuh:262); the same limit is kept
    GSX_REQUIRE((uint64_t)gw * gh <= 65536, GSX_ERR_UNSUPPORTED, "%s: %u x %u tiles exceed 65536", who, gw, gh);
    GSX_REQUIRE(S->active_sh_bases == 1 || S->active_sh_bases == 4 || S->active_sh_bases == 9 || S->active_sh_bases == 16,
                GSX_ERR_INVALID_ARGUMENT, "%s: active_sh_bases = %u", who, S->active_sh_bases);
    GSX_REQUIRE(S->active_sh_bases <= S->total_bases_sh_rest + 1, GSX_ERR_INVALID_ARGUMENT,
                "%s: %u active SH bases but only %u stored", who, S->active_sh_bases, S->total_bases_sh_rest + 1);
    for (int k = 0; k < 4; ++k)
        c->r1[k] = w2c_host[k], c->r2[k] = w2c_host[4 + k], c->r3[k] = w2c_host[8 + k];
    for (int k = 0; k < 3; ++k)
        c->cam[k] = cam_host[k];
    c->active_bases = S->active_sh_bases, c->total_rest = S->total_bases_sh_rest, c->grid_w = gw, c->grid_h = gh;
    c->w = (float)S->width, c->h = (float)S->height, c->fx = S->fx, c->fy = S->fy, c->cx = S->cx, c->cy = S->cy;
    c->near_plane = S->near_plane, c->far_plane = S->far_plane;
    return GSX_OK;
}

} // namespace gsx

using namespace gsx;

extern "C" size_t gsx_fastgs_primitive_state_bytes(uint32_t N) { return fgs_prim_layout(N).total; }
extern "C" size_t gsx_fastgs_instance_state_bytes(int64_t n_instances, uint32_t width, uint32_t height) {
    return fgs_inst_layout(n_instances, ((width + kTile - 1) / kTile) * ((height + kTile - 1) / kTile)).total;
}
// final transmittance, number of list entries replayed per pixel; per tile how far its pixels went into the list
// and the order in which the backward visits the tiles (dearest first)
extern "C" size_t gsx_fastgs_pixel_state_bytes(uint32_t width, uint32_t height) {
    const size_t n_tiles = (size_t)((width + kTile - 1) / kTile) * ((height + kTile - 1) / kTile);
    return 2 * align_up((size_t)width * height * 4, 256) + 2 * align_up(n_tiles * 4, 256);
}
extern "C" size_t gsx_fastgs_accum_bytes(uint32_t N) { return align_up((size_t)N * kFgsAcc * 4, 256) + 256; }

extern "C" int gsx_fastgs_preprocess(uint32_t N, const float* means, const float* scales_raw, const float* rotations_raw,
                                     const float* opacities_raw, const float* sh_coefficients_0,
                                     const float* sh_coefficients_rest, const float* w2c_host,
                                     const float* cam_position_host, const gsx_fastgs_settings* settings,
                                     void* primitive_state, size_t primitive_state_bytes, int64_t* n_instances_host,
                                     int wait, void* stream) {
    GSX_REQUIRE(n_instances_host != nullptr, GSX_ERR_INVALID_ARGUMENT, "fastgs_preprocess: n_instances_host is null");
    *n_instances_host = 0;
    FgsCam c;
    int rc = fgs_make_cam("fastgs_preprocess", settings, w2c_host, cam_position_host, &c);
    if (rc != GSX_OK)
        return rc;
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && scales_raw && rotations_raw && opacities_raw && sh_coefficients_0 &&
                    (sh_coefficients_rest || settings->total_bases_sh_rest == 0),
                GSX_ERR_INVALID_ARGUMENT, "fastgs_preprocess: null tensor");
    GSX_REQUIRE(N < (1u << 31), GSX_ERR_INVALID_ARGUMENT, "fastgs_preprocess: N >= 2^31");
    const FgsPrimLayout L = fgs_prim_layout(N);
    GSX_REQUIRE(primitive_state && ((uintptr_t)primitive_state & 255) == 0 && primitive_state_bytes >= L.total,
                GSX_ERR_WORKSPACE, "fastgs_preprocess: primitive state needs %zu bytes, 256-byte aligned", L.total);
    char* ps = (char*)primitive_state;
    void* ws = ps + L.ws_off;
    hipLaunchKernelGGL(fgs_preprocess_kernel, dim3(cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream, N, means, scales_raw,
                       rotations_raw, opacities_raw, sh_coefficients_0, sh_coefficients_rest, c, (float4*)ps,
                       (uint32_t*)(ps + L.n_touched_off), (ushort4*)(ps + L.bounds_off), ordered_keys(ws),
                       (int32_t*)(ps + L.order_off));
    GSX_LAUNCH_CHECK();
    return ordered_counts_from_keys("fastgs_preprocess", N, (int32_t*)(ps + L.order_off), (int64_t*)(ps + L.cum_off), ws,
                                    gsx_intersect_tile_count_ordered_workspace_bytes(N), n_instances_host, wait, stream);
}

extern "C" int gsx_fastgs_render(uint32_t N, const gsx_fastgs_settings* settings, const void* primitive_state,
                                 size_t primitive_state_bytes, int64_t n_instances, void* instance_state,
                                 size_t instance_state_bytes, const float* background, float* image, float* alpha,
                                 void* pixel_state, size_t pixel_state_bytes, void* stream) {
    GSX_REQUIRE(settings && image && alpha && pixel_state, GSX_ERR_INVALID_ARGUMENT, "fastgs_render: null argument");
    const uint32_t W = settings->width, H = settings->height;
    const uint32_t gw = (W + kTile - 1) / kTile, gh = (H + kTile - 1) / kTile, n_tiles = gw * gh;
    GSX_REQUIRE(W > 0 && H > 0 && (uint64_t)gw * gh <= 65536, GSX_ERR_INVALID_ARGUMENT, "fastgs_render: image %u x %u", W, H);
    GSX_REQUIRE(n_instances >= 0 && n_instances < (1ll << 31), GSX_ERR_OVERFLOW,
                "fastgs_render: %lld instances do not fit int32 indices", (long long)n_instances);
    GSX_REQUIRE(N == 0 || (primitive_state && primitive_state_bytes >= fgs_prim_layout(N).total), GSX_ERR_WORKSPACE,
                "fastgs_render: primitive state of %zu bytes, %zu needed", primitive_state_bytes,
                fgs_prim_layout(N).total);
    GSX_REQUIRE(pixel_state_bytes >= gsx_fastgs_pixel_state_bytes(W, H) && ((uintptr_t)pixel_state & 255) == 0,
                GSX_ERR_WORKSPACE, "fastgs_render: pixel state needs %zu bytes, 256-byte aligned",
                gsx_fastgs_pixel_state_bytes(W, H));
    const FgsInstLayout IL = fgs_inst_layout(n_instances, n_tiles);
    GSX_REQUIRE(instance_state && ((uintptr_t)instance_state & 255) == 0 && instance_state_bytes >= IL.total,
                GSX_ERR_WORKSPACE, "fastgs_render: instance state needs %zu bytes, 256-byte aligned", IL.total);
    const FgsPrimLayout L = fgs_prim_layout(N);
    const char* ps = (const char*)primitive_state;
    char* is = (char*)instance_state;
    uint16_t* keys0 = (uint16_t*)is;
    uint16_t* keys1 = (uint16_t*)(is + IL.keys1_off);
    int32_t* vals0 = (int32_t*)(is + IL.vals0_off);
    int32_t* vals1 = (int32_t*)(is + IL.vals1_off);
    int32_t* offsets = (int32_t*)(is + IL.offsets_off);
    hipStream_t s = (hipStream_t)stream;
    int sel = 0, rc;
    if (n_instances > 0) {
        hipLaunchKernelGGL(fgs_create_instances_kernel, dim3(cdiv(N, 256)), dim3(256), 0, s, N,
                           (const int32_t*)(ps + L.order_off), (const int64_t*)(ps + L.cum_off),
                           (const uint32_t*)(ps + L.n_touched_off), (const ushort4*)(ps + L.bounds_off),
                           (const float4*)ps, gw, keys0, vals0);
        GSX_LAUNCH_CHECK();
        if ((rc = gsx_radix_sort_tile_pairs(n_instances, keys0, vals0, keys1, vals1, fgs_tile_bits(n_tiles),
                                            is + IL.ws_off, gsx_radix_sort_pairs_workspace_bytes(n_instances), &sel,
                                            stream)) != GSX_OK)
            return rc;
    }
    // which buffer holds the sorted list: kept in the state for the backward (a host-side int in the first bytes
    // of a slot the kernels never touch would not survive a device buffer; it is recomputed there instead)
    if ((rc = gsx_intersect_tile_pairs_offset(n_instances, sel ? keys1 : keys0, gw, gh, offsets, stream)) != GSX_OK)
        return rc;
    char* px = (char*)pixel_state;
    const size_t plane = align_up((size_t)W * H * 4, 256);
    float* t_final = (float*)px;
    uint32_t* n_contrib = (uint32_t*)(px + plane);
    uint32_t* tile_walk = (uint32_t*)(px + 2 * plane);
    uint32_t* tile_order = (uint32_t*)(px + 2 * plane + align_up((size_t)n_tiles * 4, 256));
    hipLaunchKernelGGL(fgs_blend_fwd_kernel, dim3(n_tiles), dim3(256), 0, s, (uint32_t)n_instances, (const float4*)ps,
                       offsets, sel ? vals1 : vals0, W, H, gw, n_tiles, background, image, alpha, t_final, n_contrib,
                       tile_walk);
    GSX_LAUNCH_CHECK();
    // the backward's visiting order: tiles whose pixels went furthest into their lists first
    return gsx_tile_order(n_instances, nullptr, tile_walk, gw, gh, tile_order, stream);
}

extern "C" int gsx_fastgs_primitive_records(uint32_t N, const void* primitive_state, const float** records,
                                            const uint32_t** n_touched_tiles) {
    GSX_REQUIRE(primitive_state && records && n_touched_tiles, GSX_ERR_INVALID_ARGUMENT,
                "fastgs_primitive_records: null argument");
    *records = (const float*)primitive_state;
    *n_touched_tiles = (const uint32_t*)((const char*)primitive_state + fgs_prim_layout(N).n_touched_off);
    return GSX_OK;
}

extern "C" int gsx_fastgs_instance_list(const gsx_fastgs_settings* settings, int64_t n_instances,
                                        const void* instance_state, const int32_t** instance_primitive,
                                        const int32_t** tile_offsets) {
    GSX_REQUIRE(settings && instance_state && instance_primitive && tile_offsets, GSX_ERR_INVALID_ARGUMENT,
                "fastgs_instance_list: null argument");
    const uint32_t gw = (settings->width + kTile - 1) / kTile, gh = (settings->height + kTile - 1) / kTile;
    const FgsInstLayout IL = fgs_inst_layout(n_instances, gw * gh);
    // the pair sorter ping-pongs once per digit pass; its pass count for this bit range fixes the final buffer
    const int sel = n_instances > 0 ? gsx_radix_sort_pairs_selector(n_instances, 0, fgs_tile_bits(gw * gh)) : 0;
    const char* is = (const char*)instance_state;
    *instance_primitive = (const int32_t*)(is + (sel ? IL.vals1_off : IL.vals0_off));
    *tile_offsets = (const int32_t*)(is + IL.offsets_off);
    return GSX_OK;
}

extern "C" int gsx_fastgs_backward(uint32_t N, const float* means, const float* scales_raw, const float* rotations_raw,
                                   const float* sh_coefficients_rest, const float* w2c_host,
                                   const float* cam_position_host, const gsx_fastgs_settings* settings,
                                   const void* primitive_state, size_t primitive_state_bytes, int64_t n_instances,
                                   const void* instance_state, size_t instance_state_bytes, const void* pixel_state,
                                   size_t pixel_state_bytes, const float* background, const float* grad_image,
                                   const float* grad_alpha, void* accum, size_t accum_bytes, float* grad_means,
                                   float* grad_scales_raw, float* grad_rotations_raw, float* grad_opacities_raw,
                                   float* grad_sh_coefficients_0, float* grad_sh_coefficients_rest, float* grad_w2c,
                                   float* densification_info, void* stream) {
    FgsCam c;
    int rc = fgs_make_cam("fastgs_backward", settings, w2c_host, cam_position_host, &c);
    if (rc != GSX_OK)
        return rc;
    hipStream_t s = (hipStream_t)stream;
    if (grad_w2c != nullptr) {
        hipLaunchKernelGGL(fgs_fill_kernel, dim3(1), dim3(64), 0, s, 16u, 0.0f, grad_w2c);
        GSX_LAUNCH_CHECK();
    }
    if (N == 0)
        return GSX_OK;
    GSX_REQUIRE(means && scales_raw && rotations_raw && (sh_coefficients_rest || settings->total_bases_sh_rest == 0) &&
                    primitive_state && instance_state && pixel_state && grad_image && grad_alpha && grad_means &&
                    grad_scales_raw && grad_rotations_raw && grad_opacities_raw && grad_sh_coefficients_0 &&
                    (grad_sh_coefficients_rest || settings->total_bases_sh_rest == 0),
                GSX_ERR_INVALID_ARGUMENT, "fastgs_backward: null tensor");
    // rows of up to 45 floats leave the workgroups as 16-byte stores
    GSX_REQUIRE(((uintptr_t)grad_sh_coefficients_rest & 15) == 0, GSX_ERR_INVALID_ARGUMENT,
                "fastgs_backward: grad_sh_coefficients_rest needs 16-byte alignment");
    GSX_REQUIRE(accum && ((uintptr_t)accum & 255) == 0 && accum_bytes >= gsx_fastgs_accum_bytes(N), GSX_ERR_WORKSPACE,
                "fastgs_backward: accumulator needs %zu bytes, 256-byte aligned, zeroed", gsx_fastgs_accum_bytes(N));
    GSX_REQUIRE(n_instances >= 0 && n_instances < (1ll << 31), GSX_ERR_OVERFLOW, "fastgs_backward: %lld instances",
                (long long)n_instances);
    const uint32_t W = settings->width, H = settings->height, n_tiles = c.grid_w * c.grid_h;
    const FgsPrimLayout L = fgs_prim_layout(N);
    GSX_REQUIRE(primitive_state_bytes >= L.total && instance_state_bytes >= fgs_inst_layout(n_instances, n_tiles).total &&
                    pixel_state_bytes >= gsx_fastgs_pixel_state_bytes(W, H),
                GSX_ERR_WORKSPACE,
                "fastgs_backward: state buffers of %zu / %zu / %zu bytes, %zu / %zu / %zu needed (primitive / instance / "
                "pixel): not the ones the forward filled for this N, instance count and image size",
                primitive_state_bytes, instance_state_bytes, pixel_state_bytes, L.total,
                fgs_inst_layout(n_instances, n_tiles).total, gsx_fastgs_pixel_state_bytes(W, H));
    const char* ps = (const char*)primitive_state;
    const int32_t *inst, *offsets;
    if ((rc = gsx_fastgs_instance_list(settings, n_instances, instance_state, &inst, &offsets)) != GSX_OK)
        return rc;
    const char* px = (const char*)pixel_state;
    if (n_instances > 0) {
        hipLaunchKernelGGL(fgs_blend_bwd_kernel, dim3(n_tiles), dim3(256), 0, s, (uint32_t)n_instances, (const float4*)ps,
                           offsets, inst, W, H, c.grid_w, n_tiles, background, (const float*)px,
                           (const uint32_t*)(px + align_up((size_t)W * H * 4, 256)), grad_image, grad_alpha,
                           (const uint32_t*)(px + 2 * align_up((size_t)W * H * 4, 256) +
                                             align_up((size_t)n_tiles * 4, 256)),
                           (float*)accum);
        GSX_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(fgs_preprocess_bwd_kernel, dim3(cdiv(N, 256)), dim3(256), 0, s, N, means, scales_raw, rotations_raw,
                       sh_coefficients_rest, c, (const uint32_t*)(ps + L.n_touched_off), (const float4*)ps, (float*)accum,
                       grad_means, grad_scales_raw, grad_rotations_raw, grad_opacities_raw, grad_sh_coefficients_0,
                       grad_sh_coefficients_rest, grad_w2c, densification_info);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}
