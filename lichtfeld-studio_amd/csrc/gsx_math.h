// gsx_math.h - deterministic fp32 primitives used by the gfx950 kernels and by the CPU checker.
//
// Every function here is written so that a host build (g++ or clang, -ffp-contract=off) and a
// device build (hipcc --offload-arch=gfx950 -ffp-contract=off) produce the same bits for the same
// inputs: fused multiply-adds are spelled out with gsx::fma, nothing relies on libm or on
// hardware approximations (v_exp_f32, v_rsq_f32, v_rcp_f32), divisions and square roots are the
// IEEE correctly rounded ones, and the transcendental functions are fixed polynomial evaluations.
// That is what makes tile keys (which embed float bits of depth), radii (a ceil of a float), the
// alpha thresholds of the rasterizer and therefore whole images reproducible between the CPU
// checker and the GPU.
//
// The reference is built with --use_fast_math (gsplat/CMakeLists.txt:76,80), whose bit patterns
// cannot be reproduced off an NVIDIA GPU; these primitives replace its __expf/__logf/rsqrtf/
// __frcp_rn intrinsics and the glm routines it calls (glm is not vendored in the reference tree).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define GSX_HD __host__ __device__ __forceinline__
#else
#define GSX_HD inline
#endif

namespace gsx {

// ---------------------------------------------------------------------------------------------
// scalar primitives
// ---------------------------------------------------------------------------------------------

GSX_HD float fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
GSX_HD float fmin(float a, float b) { return a < b ? a : b; } // operand order matters for NaN only
GSX_HD float fmax(float a, float b) { return a > b ? a : b; }
// min(limit, x) for a limit that is a number: the other operand if that is a number too and smaller, else the limit
// (what CUDA's min / fminf gives: a NaN x yields the limit).  One v_min_f32 on the device; the same values on the host.
GSX_HD float min_limit(float limit, float x) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_fminf(limit, x);
#else
    return x < limit ? x : limit;
#endif
}
GSX_HD float fabs(float a) { return __builtin_fabsf(a); }
GSX_HD float floor(float a) { return __builtin_floorf(a); }
GSX_HD float ceil(float a) { return __builtin_ceilf(a); }
GSX_HD float sqrt(float a) { return __builtin_sqrtf(a); } // IEEE, correctly rounded
GSX_HD float rcp(float a) { return 1.0f / a; }            // IEEE, correctly rounded
// 1 / a to one unit in the last place on the GPU (v_rcp_f32), correctly rounded on the host: only for heuristics
// whose outcome may differ between the two without changing a result (the rasterizers' conservative block test)
GSX_HD float rcp_approx(float a) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_rcpf(a);
#else
    return 1.0f / a;
#endif
}
// The hardware reciprocal with one Newton step: on [0.001, 1] within half a unit in the last place with a mean signed
// error of 0.0002 units, where v_rcp_f32 alone reaches 0.9 units with a mean of -0.07.  For the gradient chains, which
// are not bit-compared: the backward rasterizers rebuild a pixel's transmittance by multiplying with 1 / (1 - alpha)
// entry by entry, and an error of one sign adds up along the list and over the pixels of a Gaussian alike (colour
// gradients of 127 faint, stacked Gaussians: 6e-7 relative with the bare instruction, 5e-8 with the step, at the
// same speed).
GSX_HD float rcp_refined(float a) {
#if defined(__HIP_DEVICE_COMPILE__)
    const float r = __builtin_amdgcn_rcpf(a);
    return __builtin_fmaf(__builtin_fmaf(-a, r, 1.0f), r, r);
#else
    return 1.0f / a;
#endif
}

GSX_HD uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
GSX_HD float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// 1/sqrt(x) for normal positive x: integer seed + three Newton steps (<= 2 ulp, the accuracy class
// of the rsqrtf the reference uses in Utils.cuh:83,181-184).  Exact same bits on host and device.
GSX_HD float rsqrt(float x) {
    float y = u2f(0x5f375a86u - (f2u(x) >> 1));
    const float h = 0.5f * x;
    y = y * fma(-(h * y), y, 1.5f);
    y = y * fma(-(h * y), y, 1.5f);
    y = y * fma(-(h * y), y, 1.5f);
    return y;
}

// e^x.  n = round(x log2 e) through the 1.5 * 2^23 addition (the integer is then also the low mantissa bits of t),
// Cody-Waite reduction r = x - n ln 2 in two exact-product steps, a degree-6 polynomial in Horner form (minimax on
// |r| <= ln 2 / 2 with the constant and linear coefficients fixed at 1: 3.4e-9 relative), scaling by 2^n.
// Below 1 unit in the last place on the whole range (all 2.1e9 arguments compared with the double-precision
// exponential).  x < -87 returns 0 (the true value is below 1.7e-38), x > 88.7 returns +inf.
GSX_HD float exp_core(float x, float* t_out) {
    const float t = fma(x, 1.44269504088896341f, 12582912.0f);
    const float n = t - 12582912.0f;
    float r = fma(n, -0.693359375f, x);
    r = fma(n, 2.12194440e-4f, r);
    float p = 1.3855284778e-3f;
    p = fma(p, r, 8.3686923608e-3f);
    p = fma(p, r, 4.1667662561e-2f);
    p = fma(p, r, 1.6666521132e-1f);
    p = fma(p, r, 4.9999997020e-1f);
    p = fma(p, r, 1.0f);
    *t_out = t;
    return fma(p, r, 1.0f); // in (0.70, 1.42)
}
GSX_HD float exp(float x) {
    if (x < -87.0f)
        return 0.0f;
    if (x > 88.7f)
        return u2f(0x7f800000u);
    float t;
    const float y = exp_core(x, &t);
    return __builtin_ldexpf(y, (int)(f2u(t) - 0x4B400000u)); // exact scaling by 2^n, n in [-126, 128]
}

// gsx::exp restricted to -87 <= x <= 0, where its two range tests never fire and the result is a normal number, so
// that the scaling is an addition of n to the exponent field (t's low bits, shifted): the same bits for fewer
// instructions.
GSX_HD float exp_nonpos(float x) {
    float t;
    const float y = exp_core(x, &t);
    return u2f((f2u(t) << 23) + f2u(y));
}

// natural log of a positive normal float (Cephes logf scheme).
GSX_HD float log(float x) {
    uint32_t ix = f2u(x);
    int e = (int)(ix >> 23) - 126;                      // x = m * 2^e, m in [0.5, 1)
    float m = u2f((ix & 0x007fffffu) | 0x3f000000u);
    if (m < 0.707106781186547524f) {
        e -= 1;
        m = m + m - 1.0f;
    } else {
        m = m - 1.0f;
    }
    const float z = m * m;
    float p = 7.0376836292e-2f;
    p = fma(p, m, -1.1514610310e-1f);
    p = fma(p, m, 1.1676998740e-1f);
    p = fma(p, m, -1.2420140846e-1f);
    p = fma(p, m, 1.4249322787e-1f);
    p = fma(p, m, -1.6668057665e-1f);
    p = fma(p, m, 2.0000714765e-1f);
    p = fma(p, m, -2.4999993993e-1f);
    p = fma(p, m, 3.3333331174e-1f);
    float y = (m * z) * p;
    const float fe = (float)e;
    y = fma(fe, -2.12194440e-4f, y);
    y = fma(-0.5f, z, y);
    float r = m + y;
    r = fma(fe, 0.693359375f, r);
    return r;
}

// x^y for x > 0.
GSX_HD float pow(float x, float y) { return gsx::exp(y * gsx::log(x)); }

// logistic function 1/(1+e^-x)
GSX_HD float sigmoid(float x) { return 1.0f / (1.0f + gsx::exp(-x)); }

// sin on [-pi, pi] (Cephes sinf/cosf cores after an exact quadrant fold); only the camera-pose
// interpolation uses it.
GSX_HD float sin_core(float x) { // |x| <= pi/4
    const float z = x * x;
    float p = -1.9515295891e-4f;
    p = fma(p, z, 8.3321608736e-3f);
    p = fma(p, z, -1.6666654611e-1f);
    return fma(p * z, x, x);
}
GSX_HD float cos_core(float x) { // |x| <= pi/4
    const float z = x * x;
    float p = 2.443315711809948e-5f;
    p = fma(p, z, -1.388731625493765e-3f);
    p = fma(p, z, 4.166664568298827e-2f);
    return fma(p, z * z, fma(-0.5f, z, 1.0f));
}
GSX_HD float sin(float x) {
    const float ax = gsx::fabs(x);
    const float sgn = x < 0.0f ? -1.0f : 1.0f;
    const float pio2 = 1.57079632679489661923f;
    float r;
    if (ax <= 0.785398163397448309f) {
        r = sin_core(ax);
    } else if (ax <= 2.35619449019234492f) {
        r = cos_core(ax - pio2);
    } else {
        r = sin_core(3.14159265358979323846f - ax);
    }
    return sgn * r;
}

// cos on [-pi, pi] through the same cores: cos(x) = sin(pi/2 - |x|), whose argument stays inside [-pi/2, pi/2].
GSX_HD float cos(float x) { return gsx::sin(1.57079632679489661923f - gsx::fabs(x)); }

// acos on [-1, 1] (Cephes asinf core).
GSX_HD float asin_core(float a) { // 0 <= a <= 0.5
    const float z = a * a;
    float p = 4.2163199048e-2f;
    p = fma(p, z, 2.4181311049e-2f);
    p = fma(p, z, 4.5470025998e-2f);
    p = fma(p, z, 7.4953002686e-2f);
    p = fma(p, z, 1.6666752422e-1f);
    return fma(p * z, a, a);
}
GSX_HD float acos(float x) {
    const float pio2 = 1.57079632679489661923f;
    if (x > 0.5f) {
        return 2.0f * asin_core(gsx::sqrt(0.5f * (1.0f - x)));
    } else if (x < -0.5f) {
        return 3.14159265358979323846f - 2.0f * asin_core(gsx::sqrt(0.5f * (1.0f + x)));
    }
    const float ax = gsx::fabs(x);
    const float s = asin_core(ax);
    return x < 0.0f ? pio2 + s : pio2 - s;
}

// float -> uint32 with the saturating semantics the reference's kernels rely on
// (gsplat/IntersectTile.cu:72-76 casts possibly negative floats; PTX cvt.rzi.u32.f32 saturates).
GSX_HD uint32_t sat_u32(float f) {
    if (!(f > 0.0f))
        return 0u; // negative, zero and NaN
    if (f >= 4294967296.0f)
        return 0xffffffffu;
    return (uint32_t)f;
}

// ---------------------------------------------------------------------------------------------
// small vectors / matrices.  mat3 is row-major: m[r][c].
// ---------------------------------------------------------------------------------------------

struct vec2 {
    float x, y;
};
struct vec3 {
    float x, y, z;
};
struct quat { // w, x, y, z like the reference's tensors
    float w, x, y, z;
};
struct mat3 {
    float m[3][3];
};

GSX_HD vec3 mk3(float x, float y, float z) {
    vec3 r;
    r.x = x;
    r.y = y;
    r.z = z;
    return r;
}
GSX_HD vec3 add(vec3 a, vec3 b) { return mk3(a.x + b.x, a.y + b.y, a.z + b.z); }
GSX_HD vec3 sub(vec3 a, vec3 b) { return mk3(a.x - b.x, a.y - b.y, a.z - b.z); }
GSX_HD vec3 scale(vec3 a, float s) { return mk3(a.x * s, a.y * s, a.z * s); }
GSX_HD vec3 neg(vec3 a) { return mk3(-a.x, -a.y, -a.z); }
GSX_HD float dot(vec3 a, vec3 b) { return fma(a.z, b.z, fma(a.y, b.y, a.x * b.x)); }
GSX_HD vec3 cross(vec3 a, vec3 b) {
    return mk3(
        fma(a.y, b.z, -(a.z * b.y)),
        fma(a.z, b.x, -(a.x * b.z)),
        fma(a.x, b.y, -(a.y * b.x)));
}
GSX_HD vec3 mul(const mat3& A, vec3 v) { // A * v
    return mk3(
        fma(A.m[0][2], v.z, fma(A.m[0][1], v.y, A.m[0][0] * v.x)),
        fma(A.m[1][2], v.z, fma(A.m[1][1], v.y, A.m[1][0] * v.x)),
        fma(A.m[2][2], v.z, fma(A.m[2][1], v.y, A.m[2][0] * v.x)));
}
GSX_HD vec3 mul_t(const mat3& A, vec3 v) { // A^T * v
    return mk3(
        fma(A.m[2][0], v.z, fma(A.m[1][0], v.y, A.m[0][0] * v.x)),
        fma(A.m[2][1], v.z, fma(A.m[1][1], v.y, A.m[0][1] * v.x)),
        fma(A.m[2][2], v.z, fma(A.m[1][2], v.y, A.m[0][2] * v.x)));
}

// v / |v| when |v| > 0 (gsplat/Utils.cuh:181-184)
GSX_HD vec3 safe_normalize(vec3 v) {
    const float l = dot(v, v);
    return l > 0.0f ? scale(v, gsx::rsqrt(l)) : v;
}
// VJP of safe_normalize (gsplat/Utils.cuh:186-194)
GSX_HD vec3 safe_normalize_bw(vec3 v, vec3 d_out) {
    const float l = dot(v, v);
    if (l > 0.0f) {
        const float il = gsx::rsqrt(l);
        const float il3 = il * il * il;
        const float s = il3 * dot(d_out, v);
        return mk3(fma(il, d_out.x, -(s * v.x)), fma(il, d_out.y, -(s * v.y)), fma(il, d_out.z, -(s * v.z)));
    }
    return d_out;
}

// Rotation matrix of a quaternion that is normalised first with rsqrt (gsplat/Utils.cuh:80-102).
// inv_norm_cap < 0 means no cap; the MCMC noise kernel caps it at 1e12 (RelocationCUDA.cu:88-110).
GSX_HD mat3 quat_to_rotmat(quat q, float inv_norm_cap = -1.0f) {
    float inv_norm = gsx::rsqrt(fma(q.w, q.w, fma(q.z, q.z, fma(q.y, q.y, q.x * q.x))));
    if (inv_norm_cap > 0.0f)
        inv_norm = gsx::fmin(inv_norm, inv_norm_cap);
    const float x = q.x * inv_norm, y = q.y * inv_norm, z = q.z * inv_norm, w = q.w * inv_norm;
    const float x2 = x * x, y2 = y * y, z2 = z * z;
    const float xy = x * y, xz = x * z, yz = y * z;
    const float wx = w * x, wy = w * y, wz = w * z;
    mat3 R;
    R.m[0][0] = 1.f - 2.f * (y2 + z2);
    R.m[1][0] = 2.f * (xy + wz);
    R.m[2][0] = 2.f * (xz - wy);
    R.m[0][1] = 2.f * (xy - wz);
    R.m[1][1] = 1.f - 2.f * (x2 + z2);
    R.m[2][1] = 2.f * (yz + wx);
    R.m[0][2] = 2.f * (xz + wy);
    R.m[1][2] = 2.f * (yz - wx);
    R.m[2][2] = 1.f - 2.f * (x2 + y2);
    return R;
}

// ---- the glm routines the reference calls (glm 1.0.x, gtc/quaternion.inl, gtx/quaternion.inl) ----

// glm::mat3_cast: rotation matrix of q without normalising it.
GSX_HD mat3 mat3_cast(quat q) {
    const float qxx = q.x * q.x, qyy = q.y * q.y, qzz = q.z * q.z;
    const float qxz = q.x * q.z, qxy = q.x * q.y, qyz = q.y * q.z;
    const float qwx = q.w * q.x, qwy = q.w * q.y, qwz = q.w * q.z;
    mat3 R;
    R.m[0][0] = 1.f - 2.f * (qyy + qzz);
    R.m[1][0] = 2.f * (qxy + qwz);
    R.m[2][0] = 2.f * (qxz - qwy);
    R.m[0][1] = 2.f * (qxy - qwz);
    R.m[1][1] = 1.f - 2.f * (qxx + qzz);
    R.m[2][1] = 2.f * (qyz + qwx);
    R.m[0][2] = 2.f * (qxz + qwy);
    R.m[1][2] = 2.f * (qyz - qwx);
    R.m[2][2] = 1.f - 2.f * (qxx + qyy);
    return R;
}

// glm::quat_cast of a rotation matrix (row-major R here; glm's m[c][r] = R.m[r][c]).
GSX_HD quat quat_cast(const mat3& R) {
    const float m00 = R.m[0][0], m11 = R.m[1][1], m22 = R.m[2][2];
    const float fourXSquaredMinus1 = m00 - m11 - m22;
    const float fourYSquaredMinus1 = m11 - m00 - m22;
    const float fourZSquaredMinus1 = m22 - m00 - m11;
    const float fourWSquaredMinus1 = m00 + m11 + m22;
    int biggestIndex = 0;
    float fourBiggestSquaredMinus1 = fourWSquaredMinus1;
    if (fourXSquaredMinus1 > fourBiggestSquaredMinus1) {
        fourBiggestSquaredMinus1 = fourXSquaredMinus1;
        biggestIndex = 1;
    }
    if (fourYSquaredMinus1 > fourBiggestSquaredMinus1) {
        fourBiggestSquaredMinus1 = fourYSquaredMinus1;
        biggestIndex = 2;
    }
    if (fourZSquaredMinus1 > fourBiggestSquaredMinus1) {
        fourBiggestSquaredMinus1 = fourZSquaredMinus1;
        biggestIndex = 3;
    }
    const float biggestVal = gsx::sqrt(fourBiggestSquaredMinus1 + 1.0f) * 0.5f;
    const float mult = 0.25f / biggestVal;
    // glm m[a][b] = column a, row b = R.m[b][a]
    const float g01 = R.m[1][0], g10 = R.m[0][1];
    const float g02 = R.m[2][0], g20 = R.m[0][2];
    const float g12 = R.m[2][1], g21 = R.m[1][2];
    quat q;
    switch (biggestIndex) {
    case 0:
        q.w = biggestVal;
        q.x = (g12 - g21) * mult;
        q.y = (g20 - g02) * mult;
        q.z = (g01 - g10) * mult;
        break;
    case 1:
        q.w = (g12 - g21) * mult;
        q.x = biggestVal;
        q.y = (g01 + g10) * mult;
        q.z = (g20 + g02) * mult;
        break;
    case 2:
        q.w = (g20 - g02) * mult;
        q.x = (g01 + g10) * mult;
        q.y = biggestVal;
        q.z = (g12 + g21) * mult;
        break;
    default:
        q.w = (g01 - g10) * mult;
        q.x = (g20 + g02) * mult;
        q.y = (g12 + g21) * mult;
        q.z = biggestVal;
        break;
    }
    return q;
}

GSX_HD float qdot(quat a, quat b) { return fma(a.w, b.w, fma(a.z, b.z, fma(a.y, b.y, a.x * b.x))); }

// glm::normalize(quat)
GSX_HD quat quat_normalize(quat q) {
    const float len = gsx::sqrt(qdot(q, q));
    quat r;
    if (len <= 0.0f) {
        r.w = 1.f;
        r.x = 0.f;
        r.y = 0.f;
        r.z = 0.f;
        return r;
    }
    const float inv = 1.0f / len;
    r.w = q.w * inv;
    r.x = q.x * inv;
    r.y = q.y * inv;
    r.z = q.z * inv;
    return r;
}

// glm::inverse(quat) = conjugate / dot
GSX_HD quat quat_inverse(quat q) {
    const float d = qdot(q, q);
    quat r;
    r.w = q.w / d;
    r.x = -q.x / d;
    r.y = -q.y / d;
    r.z = -q.z / d;
    return r;
}

// glm::rotate(quat, vec3) = v + 2 (w (u x v) + u x (u x v))
GSX_HD vec3 quat_rotate(quat q, vec3 v) {
    const vec3 u = mk3(q.x, q.y, q.z);
    const vec3 uv = cross(u, v);
    const vec3 uuv = cross(u, uv);
    return mk3(
        fma(2.0f, fma(uv.x, q.w, uuv.x), v.x),
        fma(2.0f, fma(uv.y, q.w, uuv.y), v.y),
        fma(2.0f, fma(uv.z, q.w, uuv.z), v.z));
}

// glm::slerp(x, y, a): shortest path; falls back to a component-wise lerp when cos > 1 - eps.
GSX_HD quat slerp(quat x, quat y, float a) {
    quat z = y;
    float cosTheta = qdot(x, y);
    if (cosTheta < 0.0f) {
        z.w = -y.w;
        z.x = -y.x;
        z.y = -y.y;
        z.z = -y.z;
        cosTheta = -cosTheta;
    }
    quat r;
    if (cosTheta > 1.0f - 1.1920928955078125e-07f) {
        // glm::mix(x, y, a) = x * (1 - a) + y * a, component-wise
        r.w = x.w * (1.0f - a) + z.w * a;
        r.x = x.x * (1.0f - a) + z.x * a;
        r.y = x.y * (1.0f - a) + z.y * a;
        r.z = x.z * (1.0f - a) + z.z * a;
        return r;
    }
    const float angle = gsx::acos(cosTheta);
    const float s0 = gsx::sin((1.0f - a) * angle);
    const float s1 = gsx::sin(a * angle);
    const float sd = gsx::sin(angle);
    r.w = (s0 * x.w + s1 * z.w) / sd;
    r.x = (s0 * x.x + s1 * z.x) / sd;
    r.y = (s0 * x.y + s1 * z.y) / sd;
    r.z = (s0 * x.z + s1 * z.z) / sd;
    return r;
}

} // namespace gsx
