// gsx_step.h - device functions shared by the per-Gaussian passes of a training step (spherical harmonics,
// activations and their VJPs, the rasterizer-backward epilogue, the Adam update), so that the separate kernels and
// the fused update kernel run the same arithmetic.
#pragma once

#include "gsx_common.h"

namespace gsx {

// ---------------------------------------------------------------------------------------------
// Spherical harmonics basis (gsplat/SphericalHarmonicsCUDA.cu:20-110).  Returns the number of bases filled.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int sh_basis(uint32_t degree, vec3 dir, float* B) {
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

// campos = translation column of inverse([R|t]) = -R^T t (Rasterization.cpp:358-359 uses at::inverse; for the
// rigid matrices LichtFeld passes the two agree).  Evaluated per lane from the uniform matrix: the matrix
// lives in device memory and a host copy would cost a synchronisation.
__device__ __forceinline__ vec3 campos_from_viewmat(const float* __restrict__ vm) {
    mat3 R;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int c = 0; c < 3; ++c)
            R.m[r][c] = vm[r * 4 + c];
    return neg(mul_t(R, mk3(vm[3], vm[7], vm[11])));
}

// ---- coefficient rows through LDS (K = 16) -----------------------------------------------------
// A lane owns one Gaussian, whose 16x3 coefficients are a 192-byte row; lanes reading or writing their own rows
// directly touch 64 different cache lines per instruction.  Instead a wave moves its 64 rows (12 KiB, contiguous in
// memory) with fully coalesced 16-byte accesses and transposes through LDS; rows are padded to 13 x 16 bytes so
// that the per-lane 16-byte LDS accesses are conflict-free.
static constexpr uint32_t kShRowF4 = 12;   // float4 per row (K = 16)
static constexpr uint32_t kShLdsF4 = 13;   // padded row stride in float4

__device__ __forceinline__ void sh16_rows_to_lds(const float* __restrict__ coeffs, uint32_t row0, uint32_t N,
                                                 float4* wave_lds, uint32_t lane) {
    const float4* src = reinterpret_cast<const float4*>(coeffs + (size_t)row0 * 48);
    const uint32_t n_f4 = min(64u, N - row0) * kShRowF4;
#pragma unroll
    for (uint32_t i = 0; i < kShRowF4; ++i) {
        const uint32_t q = i * 64u + lane;
        if (q < n_f4) {
            const uint32_t r = (q * 43691u) >> 19; // q / 12 for q < 768
            wave_lds[r * kShLdsF4 + (q - r * kShRowF4)] = src[q];
        }
    }
}

__device__ __forceinline__ void sh16_rows_from_lds(float* __restrict__ v_coeffs, uint32_t row0, uint32_t N,
                                                   const float4* wave_lds, uint32_t lane) {
    float4* dst = reinterpret_cast<float4*>(v_coeffs + (size_t)row0 * 48);
    const uint32_t n_f4 = min(64u, N - row0) * kShRowF4;
#pragma unroll
    for (uint32_t i = 0; i < kShRowF4; ++i) {
        const uint32_t q = i * 64u + lane;
        if (q < n_f4) {
            const uint32_t r = (q * 43691u) >> 19;
            dst[q] = wave_lds[r * kShLdsF4 + (q - r * kShRowF4)];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Activations of the raw parameters (SplatData getters, src/core/splat_data.cpp:271-286) and their VJPs
// ---------------------------------------------------------------------------------------------
struct Activated {
    float opacity;
    vec3 scales;
    quat quat;
};
__device__ __forceinline__ Activated activate(float opacity_raw, vec3 s, quat q) {
    Activated a;
    a.opacity = gsx::sigmoid(opacity_raw);
    a.scales = mk3(gsx::exp(s.x), gsx::exp(s.y), gsx::exp(s.z));
    // torch::nn::functional::normalize: x / max(||x||_2, eps), eps = 1e-12
    const float nrm = gsx::fmax(gsx::sqrt(qdot(q, q)), 1e-12f);
    a.quat.w = q.w / nrm;
    a.quat.x = q.x / nrm;
    a.quat.y = q.y / nrm;
    a.quat.z = q.z / nrm;
    return a;
}

struct ActivationVjp {
    float opacity;
    vec3 scaling;
    quat rotation;
};
__device__ __forceinline__ ActivationVjp activation_vjp(float opacity_raw, vec3 s, quat q, float v_opacity,
                                                        vec3 v_scales, quat g) {
    ActivationVjp r;
    const float o = gsx::sigmoid(opacity_raw);
    r.opacity = v_opacity * (o * (1.0f - o));
    r.scaling = mk3(v_scales.x * gsx::exp(s.x), v_scales.y * gsx::exp(s.y), v_scales.z * gsx::exp(s.z));
    const float len = gsx::sqrt(qdot(q, q));
    if (len > 1e-12f) {
        // y = x / len : v_x = (g - y (y . g)) / len
        const float inv = 1.0f / len;
        const float yw = q.w * inv, yx = q.x * inv, yy = q.y * inv, yz = q.z * inv;
        const float d = g.w * yw + g.x * yx + g.y * yy + g.z * yz;
        r.rotation.w = (g.w - yw * d) * inv;
        r.rotation.x = (g.x - yx * d) * inv;
        r.rotation.y = (g.y - yy * d) * inv;
        r.rotation.z = (g.z - yz * d) * inv;
    } else {
        r.rotation.w = g.w * 1e12f;
        r.rotation.x = g.x * 1e12f;
        r.rotation.y = g.y * 1e12f;
        r.rotation.z = g.z * 1e12f;
    }
    return r;
}

// ---------------------------------------------------------------------------------------------
// Adam (fastgs/optimizer/include/adam_kernels.cuh:13-36)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void adam_one(float& p, float& m, float& v, float g, float lr, float beta1, float beta2,
                                         float eps, float bc1_rcp, float bc2_sqrt_rcp) {
    const float moment1 = beta1 * m + (1.0f - beta1) * g;
    const float moment2 = beta2 * v + (1.0f - beta2) * g * g;
    const float denom = gsx::sqrt(moment2) * bc2_sqrt_rcp + eps;
    const float step_size = lr * bc1_rcp;
    p -= step_size * moment1 / denom;
    m = moment1;
    v = moment2;
}

// ---------------------------------------------------------------------------------------------
// Rasterizer-backward epilogue: the linear map from one Gaussian's accumulated vo = sum k q and S = sum k q (x) q
// (symmetric) to (v_mean, v_quat, v_scale).  d L / d M^T = S M^-T with M^-1 = R diag(s), then
// quat_scale_to_preci_half_vjp / quat_to_rotmat_vjp of gsplat/Utils.cuh:104-158.  Because R is orthonormal the scale
// gradient collapses to v_scale_j = -S_jj / s_j.
// Accumulator row: r0 = rgb.xyz, vo.x ; r1 = vo.y, vo.z, Sxx, Sxy ; r2 = Sxz, Syy, Syz, Szz ; r3 = -, -, -,
// v_opacity.  quats / scales are the ACTIVATED ones the rasterizer saw.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ void epilogue_geometry_grads(float4 r0, float4 r1, float4 r2, quat q, vec3 s,
                                                        float (&vm)[3], float (&vq)[4], float (&vs)[3]) {
    const mat3 R = quat_to_rotmat(q);
    const float sv[3] = {s.x, s.y, s.z};
    const float is[3] = {1.0f / s.x, 1.0f / s.y, 1.0f / s.z};
    mat3 Mt;
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int b = 0; b < 3; ++b)
            Mt.m[a][b] = is[a] * R.m[b][a];
    const vec3 Vo = mk3(r0.w, r1.x, r1.y);
    const float S[3][3] = {{r1.z, r1.w, r2.x}, {r1.w, r2.y, r2.z}, {r2.x, r2.z, r2.w}};
    // v_Mt[a][b] = sum_c S[a][c] s_c R[b][c]
    float v_Mt[3][3];
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int b = 0; b < 3; ++b)
            v_Mt[a][b] = fma(S[a][2], sv[2] * R.m[b][2], fma(S[a][1], sv[1] * R.m[b][1], S[a][0] * (sv[0] * R.m[b][0])));
    const vec3 v_o = mul_t(Mt, Vo);
    vm[0] = -v_o.x;
    vm[1] = -v_o.y;
    vm[2] = -v_o.z;
    float vr[3][3]; // v_R(k,j) = v_M(k,j) / s_j, v_M = v_Mt^T
#pragma unroll
    for (int k = 0; k < 3; ++k)
#pragma unroll
        for (int jj = 0; jj < 3; ++jj)
            vr[k][jj] = v_Mt[jj][k] * is[jj];
    const float inv_norm = gsx::rsqrt(fma(q.w, q.w, fma(q.z, q.z, fma(q.y, q.y, q.x * q.x))));
    const float x = q.x * inv_norm, y = q.y * inv_norm, z = q.z * inv_norm, w = q.w * inv_norm;
    const float vq_w = 2.f * (x * (vr[2][1] - vr[1][2]) + y * (vr[0][2] - vr[2][0]) + z * (vr[1][0] - vr[0][1]));
    const float vq_x = 2.f * (-2.f * x * (vr[1][1] + vr[2][2]) + y * (vr[1][0] + vr[0][1]) +
                              z * (vr[2][0] + vr[0][2]) + w * (vr[2][1] - vr[1][2]));
    const float vq_y = 2.f * (x * (vr[1][0] + vr[0][1]) - 2.f * y * (vr[0][0] + vr[2][2]) +
                              z * (vr[2][1] + vr[1][2]) + w * (vr[0][2] - vr[2][0]));
    const float vq_z = 2.f * (x * (vr[2][0] + vr[0][2]) + y * (vr[2][1] + vr[1][2]) -
                              2.f * z * (vr[0][0] + vr[1][1]) + w * (vr[1][0] - vr[0][1]));
    const float d = vq_w * w + vq_x * x + vq_y * y + vq_z * z;
    vq[0] = (vq_w - d * w) * inv_norm;
    vq[1] = (vq_x - d * x) * inv_norm;
    vq[2] = (vq_y - d * y) * inv_norm;
    vq[3] = (vq_z - d * z) * inv_norm;
    // v_scale_j = -is_j^2 sum_k R(k,j) v_M(k,j) (Utils.cuh:147-157) = -S_jj / s_j, the columns of R being orthonormal
#pragma unroll
    for (int jj = 0; jj < 3; ++jj)
        vs[jj] = -(S[jj][jj] * is[jj]);
}

} // namespace gsx
