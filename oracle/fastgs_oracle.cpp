// fastgs_oracle.cpp - CPU restatement of the reference's default ("fastgs", Jacobian-EWA) rasterization backend:
// fast_gs::rasterization::forward / backward (src/training/fastgs/rasterization/src/forward.cu:15-199,
// src/backward.cu:14-116) and their kernels (include/kernels_forward.cuh, include/kernels_backward.cuh,
// include/kernel_utils.cuh).
//
// TEST INFRASTRUCTURE ONLY.  The shipped library never links, loads or calls this file; only tests/ use it.
//
// One "thread" at a time, in the reference's operation order and with its thresholds.  expf / logf / rsqrtf of the
// reference (compiled with fast math) are replaced by the fixed fp32 primitives of gsx_math.h, as in gsx_oracle.cpp.
// The reference's order among Gaussians of EQUAL depth bits depends on its atomic compaction (kernels_forward.cuh:
// 198-202) and is not defined; here, and in the kernels, ties go by primitive index.
//
// The projection and the blend are templates over the scalar type: the float instance is the checker, the double
// instance (std:: functions) is the smooth model whose central differences pin the analytic backward in
// tests/test_oracle_fastgs.py.  Sums over pixels are taken in double in the backward.
//
// Pinning status (tests/test_oracle_fastgs.py): projection by the closed form of an isotropic Gaussian on the
// optical axis and by the small-Gaussian limit against the UT projection of gsx_oracle.cpp; colours against the
// second SH implementation (orc_spherical_harmonics_fwd, Sloan form); tile lists by brute force over pixels; blend
// by the single-Gaussian analytic image and the compositing identities; both backward kernels by central
// differences of the double model.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <numeric>
#include <vector>

#include "gsx_math.h"

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

constexpr float kDilation = 0.3f;              // rasterization_config.h:17
constexpr float kMinAlphaRcp = 255.0f;         // :18
constexpr float kMaxAlpha = 0.999f;            // :20
constexpr float kTransmittanceMin = 1e-4f;     // :21
constexpr uint32_t kTileW = 16, kTileH = 16;   // :29-30
constexpr uint32_t kSequential = 4;            // :32 (only the scan ORDER of the tiles matters here)

template <typename T>
struct Num;
template <>
struct Num<float> {
    static float exp(float x) { return gsx::exp(x); }
    static float log(float x) { return gsx::log(x); }
    static float sqrt(float x) { return gsx::sqrt(x); }
    static float rsqrt(float x) { return gsx::rsqrt(x); }
};
template <>
struct Num<double> {
    static double exp(double x) { return std::exp(x); }
    static double log(double x) { return std::log(x); }
    static double sqrt(double x) { return std::sqrt(x); }
    static double rsqrt(double x) { return 1.0 / std::sqrt(x); }
};

template <typename T>
T clampT(T f, T a, T b) { // helper_math.h:1006-1008
    const T m = f < b ? f : b;
    return a > m ? a : m;
}

struct Settings {
    uint32_t active_sh_bases, total_bases_sh_rest, width, height;
    float fx, fy, cx, cy, near_plane, far_plane;
};

template <typename T>
struct Projected {
    bool active;
    T depth, mean2d[2], cov2d[3], conic[3], opacity, power_threshold, color[3];
    uint32_t bounds[4]; // x_min, x_max, y_min, y_max in tiles
    // intermediates the backward needs
    T x, y, rot[9], rot_scaled[9], cov3d[6], jw1[3], jw2[3], jwc1[3], jwc2[3], variance[3], q_norm_sq, j11, j22, tx, ty;
};

// convert_sh_to_color (kernel_utils.cuh:15-41): tcnn form, colour = 0.5 + sum, NOT clamped here
template <typename T>
void sh_to_color(const T* sh0, const T* rest, const T* pos, const T* cam, uint32_t active, T* out) {
    for (int c = 0; c < 3; ++c)
        out[c] = T(0.5f) + T(0.28209479177387814f) * sh0[c];
    if (active > 1) {
        const T dx = pos[0] - cam[0], dy = pos[1] - cam[1], dz = pos[2] - cam[2];
        const T inv = Num<T>::rsqrt(dx * dx + dy * dy + dz * dz);
        const T x = dx * inv, y = dy * inv, z = dz * inv;
        for (int c = 0; c < 3; ++c)
            out[c] = out[c] + (T(-0.48860251190291987f) * y) * rest[0 * 3 + c] + (T(0.48860251190291987f) * z) * rest[1 * 3 + c] +
                     (T(-0.48860251190291987f) * x) * rest[2 * 3 + c];
        if (active > 4) {
            const T xx = x * x, yy = y * y, zz = z * z, xy = x * y, xz = x * z, yz = y * z;
            for (int c = 0; c < 3; ++c)
                out[c] = out[c] + (T(1.0925484305920792f) * xy) * rest[3 * 3 + c] + (T(-1.0925484305920792f) * yz) * rest[4 * 3 + c] +
                         (T(0.94617469575755997f) * zz - T(0.31539156525251999f)) * rest[5 * 3 + c] +
                         (T(-1.0925484305920792f) * xz) * rest[6 * 3 + c] +
                         (T(0.54627421529603959f) * xx - T(0.54627421529603959f) * yy) * rest[7 * 3 + c];
            if (active > 9) {
                for (int c = 0; c < 3; ++c)
                    out[c] = out[c] + (T(0.59004358992664352f) * y * (T(-3.0f) * xx + yy)) * rest[8 * 3 + c] +
                             (T(2.8906114426405538f) * xy * z) * rest[9 * 3 + c] +
                             (T(0.45704579946446572f) * y * (T(1.0f) - T(5.0f) * zz)) * rest[10 * 3 + c] +
                             (T(0.3731763325901154f) * z * (T(5.0f) * zz - T(3.0f))) * rest[11 * 3 + c] +
                             (T(0.45704579946446572f) * x * (T(1.0f) - T(5.0f) * zz)) * rest[12 * 3 + c] +
                             (T(1.4453057213202769f) * z * (xx - yy)) * rest[13 * 3 + c] +
                             (T(0.59004358992664352f) * x * (-xx + T(3.0f) * yy)) * rest[14 * 3 + c];
            }
        }
    }
}

// the per-primitive part of preprocess_cu up to the tile bounds (kernels_forward.cuh:48-177)
template <typename T>
Projected<T> project(const T* mean, const T* raw_scale, const T* raw_rot, T raw_opacity, const T* w2c, const Settings& S,
                     uint32_t grid_w, uint32_t grid_h) {
    Projected<T> P;
    std::memset(&P, 0, sizeof(P));
    P.active = true;
    const T w = (T)(float)S.width, h = (T)(float)S.height, fx = S.fx, fy = S.fy, cx = S.cx, cy = S.cy;
    const T* r1 = w2c;
    const T* r2 = w2c + 4;
    const T* r3 = w2c + 8;
    const T depth = r3[0] * mean[0] + r3[1] * mean[1] + r3[2] * mean[2] + r3[3];
    P.depth = depth;
    if (depth < (T)S.near_plane || depth > (T)S.far_plane)
        P.active = false;
    const T opacity = T(1.0f) / (T(1.0f) + Num<T>::exp(-raw_opacity));
    P.opacity = opacity;
    if (opacity < T(1.0f / kMinAlphaRcp))
        P.active = false;
    for (int k = 0; k < 3; ++k)
        P.variance[k] = Num<T>::exp(T(2.0f) * raw_scale[k]);
    const T qr = raw_rot[0], qx = raw_rot[1], qy = raw_rot[2], qz = raw_rot[3];
    const T qrr_raw = qr * qr, qxx_raw = qx * qx, qyy_raw = qy * qy, qzz_raw = qz * qz;
    const T q_norm_sq = qrr_raw + qxx_raw + qyy_raw + qzz_raw;
    P.q_norm_sq = q_norm_sq;
    if (q_norm_sq < T(1e-8f))
        P.active = false;
    const T qxx = T(2.0f) * qxx_raw / q_norm_sq, qyy = T(2.0f) * qyy_raw / q_norm_sq, qzz = T(2.0f) * qzz_raw / q_norm_sq;
    const T qxy = T(2.0f) * qx * qy / q_norm_sq, qxz = T(2.0f) * qx * qz / q_norm_sq, qyz = T(2.0f) * qy * qz / q_norm_sq;
    const T qrx = T(2.0f) * qr * qx / q_norm_sq, qry = T(2.0f) * qr * qy / q_norm_sq, qrz = T(2.0f) * qr * qz / q_norm_sq;
    T* R = P.rot;
    R[0] = T(1.0f) - (qyy + qzz), R[1] = qxy - qrz, R[2] = qry + qxz;
    R[3] = qrz + qxy, R[4] = T(1.0f) - (qxx + qzz), R[5] = qyz - qrx;
    R[6] = qxz - qry, R[7] = qrx + qyz, R[8] = T(1.0f) - (qxx + qyy);
    T* RS = P.rot_scaled;
    for (int i = 0; i < 3; ++i)
        for (int k = 0; k < 3; ++k)
            RS[i * 3 + k] = R[i * 3 + k] * P.variance[k];
    T* C = P.cov3d; // m11 m12 m13 m22 m23 m33
    C[0] = RS[0] * R[0] + RS[1] * R[1] + RS[2] * R[2];
    C[1] = RS[0] * R[3] + RS[1] * R[4] + RS[2] * R[5];
    C[2] = RS[0] * R[6] + RS[1] * R[7] + RS[2] * R[8];
    C[3] = RS[3] * R[3] + RS[4] * R[4] + RS[5] * R[5];
    C[4] = RS[3] * R[6] + RS[4] * R[7] + RS[5] * R[8];
    C[5] = RS[6] * R[6] + RS[7] * R[7] + RS[8] * R[8];
    const T x = (r1[0] * mean[0] + r1[1] * mean[1] + r1[2] * mean[2] + r1[3]) / depth;
    const T y = (r2[0] * mean[0] + r2[1] * mean[1] + r2[2] * mean[2] + r2[3]) / depth;
    P.x = x, P.y = y;
    const T clip_left = (T(-0.15f) * w - cx) / fx, clip_right = (T(1.15f) * w - cx) / fx;
    const T clip_top = (T(-0.15f) * h - cy) / fy, clip_bottom = (T(1.15f) * h - cy) / fy;
    const T tx = clampT(x, clip_left, clip_right), ty = clampT(y, clip_top, clip_bottom);
    P.tx = tx, P.ty = ty;
    const T j11 = fx / depth, j13 = -j11 * tx, j22 = fy / depth, j23 = -j22 * ty;
    P.j11 = j11, P.j22 = j22;
    for (int k = 0; k < 3; ++k) {
        P.jw1[k] = j11 * r1[k] + j13 * r3[k];
        P.jw2[k] = j22 * r2[k] + j23 * r3[k];
    }
    const T* a = P.jw1;
    const T* b = P.jw2;
    P.jwc1[0] = a[0] * C[0] + a[1] * C[1] + a[2] * C[2];
    P.jwc1[1] = a[0] * C[1] + a[1] * C[3] + a[2] * C[4];
    P.jwc1[2] = a[0] * C[2] + a[1] * C[4] + a[2] * C[5];
    P.jwc2[0] = b[0] * C[0] + b[1] * C[1] + b[2] * C[2];
    P.jwc2[1] = b[0] * C[1] + b[1] * C[3] + b[2] * C[4];
    P.jwc2[2] = b[0] * C[2] + b[1] * C[4] + b[2] * C[5];
    T cov[3];
    cov[0] = P.jwc1[0] * a[0] + P.jwc1[1] * a[1] + P.jwc1[2] * a[2];
    cov[1] = P.jwc1[0] * b[0] + P.jwc1[1] * b[1] + P.jwc1[2] * b[2];
    cov[2] = P.jwc2[0] * b[0] + P.jwc2[1] * b[1] + P.jwc2[2] * b[2];
    cov[0] += T(kDilation);
    cov[2] += T(kDilation);
    for (int k = 0; k < 3; ++k)
        P.cov2d[k] = cov[k];
    const T det = cov[0] * cov[2] - cov[1] * cov[1];
    if (det < T(1e-8f))
        P.active = false;
    P.conic[0] = cov[2] / det, P.conic[1] = -cov[1] / det, P.conic[2] = cov[0] / det;
    P.mean2d[0] = x * fx + cx, P.mean2d[1] = y * fy + cy;
    P.power_threshold = Num<T>::log(opacity * T(kMinAlphaRcp));
    if (!P.active)
        return P; // what follows may be NaN for a culled primitive and is never used
    const T factor = Num<T>::sqrt(T(2.0f) * P.power_threshold);
    T ex = factor * Num<T>::sqrt(cov[0]) - T(0.5f), ey = factor * Num<T>::sqrt(cov[2]) - T(0.5f);
    ex = ex > T(0) ? ex : T(0), ey = ey > T(0) ? ey : T(0);
    auto lo = [](T v, uint32_t cap) { // min(cap, (uint)max(0, __float2int_rd(v)))
        const double f = std::floor((double)v);
        const int64_t i = f < -2147483648.0 ? -2147483648ll : (f > 2147483647.0 ? 2147483647ll : (int64_t)f);
        return (uint32_t)std::min<int64_t>(cap, std::max<int64_t>(0, i));
    };
    auto hi = [](T v, uint32_t cap) {
        const double f = std::ceil((double)v);
        const int64_t i = f < -2147483648.0 ? -2147483648ll : (f > 2147483647.0 ? 2147483647ll : (int64_t)f);
        return (uint32_t)std::min<int64_t>(cap, std::max<int64_t>(0, i));
    };
    P.bounds[0] = lo((P.mean2d[0] - ex) / T((float)kTileW), grid_w);
    P.bounds[1] = hi((P.mean2d[0] + ex) / T((float)kTileW), grid_w);
    P.bounds[2] = lo((P.mean2d[1] - ey) / T((float)kTileH), grid_h);
    P.bounds[3] = hi((P.mean2d[1] + ey) / T((float)kTileH), grid_h);
    if ((P.bounds[1] - P.bounds[0]) * (P.bounds[3] - P.bounds[2]) == 0)
        P.active = false;
    return P;
}

// will_primitive_contribute (kernel_utils.cuh:108-143); mean is shifted by -0.5 by the callers
bool will_contribute(float mx, float my, const float* conic, uint32_t tile_x, uint32_t tile_y, float power_threshold) {
    const float rect_min_x = (float)(tile_x * kTileW), rect_min_y = (float)(tile_y * kTileH);
    const float rect_max_x = (float)((tile_x + 1) * kTileW - 1), rect_max_y = (float)((tile_y + 1) * kTileH - 1);
    const float x_min_diff = rect_min_x - mx;
    const float x_left = (float)(x_min_diff > 0.0f);
    const float not_in_x_range = x_left + (float)(mx > rect_max_x);
    const float y_min_diff = rect_min_y - my;
    const float y_above = (float)(y_min_diff > 0.0f);
    const float not_in_y_range = y_above + (float)(my > rect_max_y);
    if (not_in_y_range + not_in_x_range == 0.0f)
        return true;
    const float corner_x = rect_max_x + x_left * (rect_min_x - rect_max_x); // fast_lerp(a, b, t) = a + t (b - a)
    const float corner_y = rect_max_y + y_above * (rect_min_y - rect_max_y);
    const float diff_x = mx - corner_x, diff_y = my - corner_y;
    const float dx = __builtin_copysignf((float)(kTileW - 1), x_min_diff);
    const float dy = __builtin_copysignf((float)(kTileH - 1), y_min_diff);
    auto saturate = [](float v) { return v > 0.0f ? (v < 1.0f ? v : 1.0f) : 0.0f; }; // NaN -> 0 as __saturatef
    const float tx = not_in_y_range * saturate((dx * conic[0] * diff_x + dx * conic[1] * diff_y) / (dx * conic[0] * dx));
    const float ty = not_in_x_range * saturate((dy * conic[1] * diff_x + dy * conic[2] * diff_y) / (dy * conic[2] * dy));
    const float px = corner_x + tx * dx, py = corner_y + ty * dy;
    const float ddx = mx - px, ddy = my - py;
    const float max_power = 0.5f * (conic[0] * ddx * ddx + conic[2] * ddy * ddy) + conic[1] * ddx * ddy;
    return max_power <= power_threshold;
}

} // namespace

// preprocess_cu (kernels_forward.cuh:17-203) without the compaction: per primitive, in primitive order.
// n_touched [N] (0 = culled), bounds [N,4] u16, mean2d [N,2], conic_opacity [N,4], color [N,3] (unclamped),
// depth [N].  Entries of culled primitives other than n_touched are unspecified.
ORC_API int orc_fgs_preprocess(uint32_t N, const float* means, const float* scales_raw, const float* rotations_raw,
                               const float* opacities_raw, const float* sh0, const float* shN, const float* w2c,
                               const float* cam_position, const Settings* S, uint32_t* n_touched, uint16_t* bounds,
                               float* mean2d, float* conic_opacity, float* color, float* depth) {
    const uint32_t grid_w = (S->width + kTileW - 1) / kTileW, grid_h = (S->height + kTileH - 1) / kTileH;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)N; ++i) {
        n_touched[i] = 0;
        const Projected<float> P = project<float>(means + 3 * i, scales_raw + 3 * i, rotations_raw + 4 * i,
                                                  opacities_raw[i], w2c, *S, grid_w, grid_h);
        depth[i] = P.depth;
        if (!P.active)
            continue;
        // compute_exact_n_touched_tiles (kernel_utils.cuh:146-210): every tile of the bounds, row-major
        const float mx = P.mean2d[0] - 0.5f, my = P.mean2d[1] - 0.5f;
        uint32_t cnt = 0;
        for (uint32_t ty = P.bounds[2]; ty < P.bounds[3]; ++ty)
            for (uint32_t tx = P.bounds[0]; tx < P.bounds[1]; ++tx)
                cnt += will_contribute(mx, my, P.conic, tx, ty, P.power_threshold) ? 1u : 0u;
        if (cnt == 0)
            continue;
        n_touched[i] = cnt;
        for (int k = 0; k < 4; ++k)
            bounds[4 * i + k] = (uint16_t)P.bounds[k];
        mean2d[2 * i] = P.mean2d[0], mean2d[2 * i + 1] = P.mean2d[1];
        conic_opacity[4 * i] = P.conic[0], conic_opacity[4 * i + 1] = P.conic[1], conic_opacity[4 * i + 2] = P.conic[2];
        conic_opacity[4 * i + 3] = P.opacity;
        sh_to_color<float>(sh0 + 3 * i, shN + (size_t)i * S->total_bases_sh_rest * 3, means + 3 * i, cam_position,
                           S->active_sh_bases, color + 3 * i);
    }
    return 0;
}

// depth sort (forward.cu:103-108), create_instances_cu (kernels_forward.cuh:220-321), tile sort (forward.cu:141-
// 146) and extract_instance_ranges_cu (:323-343): the instance list in (tile, depth bits, primitive index) order
// and the [start, end) range of every tile.  n_instances = sum(n_touched).
ORC_API int orc_fgs_instances(uint32_t N, const uint32_t* n_touched, const uint16_t* bounds, const float* mean2d,
                              const float* conic_opacity, const float* depth, uint32_t grid_w, uint32_t grid_h,
                              uint32_t n_instances, uint32_t* instance_primitive, uint32_t* tile_ranges /*[T,2]*/) {
    std::vector<uint32_t> order;
    for (uint32_t i = 0; i < N; ++i)
        if (n_touched[i])
            order.push_back(i);
    std::stable_sort(order.begin(), order.end(),
                     [&](uint32_t a, uint32_t b) { return gsx::f2u(depth[a]) < gsx::f2u(depth[b]); });
    std::vector<uint16_t> keys;
    std::vector<uint32_t> prims;
    for (uint32_t i : order) {
        const uint16_t* b = bounds + 4 * i;
        const float mx = mean2d[2 * i] - 0.5f, my = mean2d[2 * i + 1] - 0.5f;
        const float pt = gsx::log(conic_opacity[4 * i + 3] * kMinAlphaRcp);
        uint32_t cnt = 0;
        for (uint32_t ty = b[2]; ty < b[3]; ++ty)
            for (uint32_t tx = b[0]; tx < b[1]; ++tx)
                if (will_contribute(mx, my, conic_opacity + 4 * i, tx, ty, pt)) {
                    keys.push_back((uint16_t)(ty * grid_w + tx));
                    prims.push_back(i);
                    ++cnt;
                }
        if (cnt != n_touched[i])
            return -2; // the two passes of the reference must agree
    }
    if (keys.size() != n_instances)
        return -1;
    std::vector<uint32_t> perm(keys.size());
    std::iota(perm.begin(), perm.end(), 0u);
    std::stable_sort(perm.begin(), perm.end(), [&](uint32_t a, uint32_t b) { return keys[a] < keys[b]; });
    const uint32_t T = grid_w * grid_h;
    std::fill(tile_ranges, tile_ranges + 2 * (size_t)T, 0u); // forward.cu:47-58
    for (size_t k = 0; k < perm.size(); ++k) {
        instance_primitive[k] = prims[perm[k]];
        const uint16_t t = keys[perm[k]];
        if (k == 0 || keys[perm[k - 1]] != t)
            tile_ranges[2 * t] = (uint32_t)k;
        tile_ranges[2 * t + 1] = (uint32_t)k + 1;
    }
    return 0;
}

namespace {
// the per-pixel loop of blend_cu (kernels_forward.cuh:392-436)
// decisions (nullable): one byte per list entry of this pixel - 0 skipped, 1 blended, 2 stopped here.  record =
// true writes them, false replays them (the double model differentiates the blend for FIXED decisions).
template <typename T>
void blend_pixel(T px, T py, const uint32_t* inst, uint32_t begin, uint32_t end, const T* mean2d, const T* conic_opacity,
                 const T* color, T* rgb, T* transmittance_out, uint32_t* n_contrib_out, uint8_t* decisions = nullptr,
                 bool record = false) {
    T c[3] = {0, 0, 0}, transmittance = 1;
    uint32_t possible = 0, n_contrib = 0;
    const bool replay = decisions != nullptr && !record;
    for (uint32_t k = begin; k < end; ++k) {
        const uint32_t g = inst[k];
        ++possible;
        if (record)
            decisions[k - begin] = 0;
        if (replay && decisions[k - begin] == 2)
            break;
        if (replay && decisions[k - begin] == 0)
            continue;
        const T* co = conic_opacity + 4 * g;
        const T dx = mean2d[2 * g] - px, dy = mean2d[2 * g + 1] - py;
        const T sigma_over_2 = T(0.5f) * (co[0] * dx * dx + co[2] * dy * dy) + co[1] * dx * dy;
        if (!replay && sigma_over_2 < T(0))
            continue;
        const T gaussian = Num<T>::exp(-sigma_over_2);
        const T og = co[3] * gaussian;
        const T alpha = og < T(kMaxAlpha) ? og : T(kMaxAlpha);
        if (!replay && alpha < T(1.0f / kMinAlphaRcp))
            continue;
        const T next = transmittance * (T(1.0f) - alpha);
        if (!replay && next < T(kTransmittanceMin)) {
            if (record)
                decisions[k - begin] = 2;
            break; // done: this and all later primitives are skipped
        }
        if (record)
            decisions[k - begin] = 1;
        for (int ch = 0; ch < 3; ++ch) {
            const T col = color[3 * g + ch] > T(0) ? color[3 * g + ch] : T(0); // fmaxf(color, 0) at load (:409)
            c[ch] += transmittance * alpha * col;
        }
        transmittance = next;
        n_contrib = possible;
    }
    rgb[0] = c[0], rgb[1] = c[1], rgb[2] = c[2];
    *transmittance_out = transmittance;
    *n_contrib_out = n_contrib;
}
} // namespace

// blend_cu (kernels_forward.cuh:356-459): image [3,H,W] (no background), alpha [H,W] = 1 - T, final
// transmittance [H,W] and n_contributions [H,W].  extent_violations (nullable): number of contributing
// (pixel, primitive) pairs whose pixel centre lies outside the box mean2d +- (extents + 0.01) given in
// extents [N,2] - zero when the kernels' per-wave selection by that box is conservative.
ORC_API int orc_fgs_blend(uint32_t W, uint32_t H, const uint32_t* instance_primitive, const uint32_t* tile_ranges,
                          const float* mean2d, const float* conic_opacity, const float* color, float* image,
                          float* alpha, float* transmittance, uint32_t* n_contributions, const float* extents,
                          int64_t* extent_violations) {
    const uint32_t grid_w = (W + kTileW - 1) / kTileW;
    int64_t violations = 0;
#pragma omp parallel for schedule(dynamic, 4) reduction(+ : violations)
    for (int64_t py = 0; py < (int64_t)H; ++py)
        for (uint32_t px = 0; px < W; ++px) {
            const uint32_t tile = (uint32_t)(py / kTileH) * grid_w + px / kTileW;
            float rgb[3], t;
            uint32_t nc;
            const float fx = (float)px + 0.5f, fy = (float)py + 0.5f;
            blend_pixel<float>(fx, fy, instance_primitive, tile_ranges[2 * tile], tile_ranges[2 * tile + 1], mean2d,
                               conic_opacity, color, rgb, &t, &nc);
            const size_t p = (size_t)py * W + px, n = (size_t)W * H;
            image[p] = rgb[0], image[p + n] = rgb[1], image[p + 2 * n] = rgb[2];
            alpha[p] = 1.0f - t;
            transmittance[p] = t;
            n_contributions[p] = nc;
            if (extents != nullptr) {
                for (uint32_t k = 0; k < nc; ++k) {
                    const uint32_t g = instance_primitive[tile_ranges[2 * tile] + k];
                    const float* co = conic_opacity + 4 * g;
                    const float dx = mean2d[2 * g] - fx, dy = mean2d[2 * g + 1] - fy;
                    const float s = 0.5f * (co[0] * dx * dx + co[2] * dy * dy) + co[1] * dx * dy;
                    if (s < 0.0f)
                        continue;
                    const float og = co[3] * gsx::exp(-s);
                    if ((og < kMaxAlpha ? og : kMaxAlpha) < 1.0f / kMinAlphaRcp)
                        continue;
                    if (std::fabs(dx) > extents[2 * g] + 0.01f || std::fabs(dy) > extents[2 * g + 1] + 0.01f)
                        ++violations;
                }
            }
        }
    if (extent_violations)
        *extent_violations = violations;
    return 0;
}

// blend_backward_cu (kernels_backward.cuh:240-449) as a per-pixel walk, back to front from the last contributor
// (the reference replays front to back from per-bucket checkpoints; the per-pair terms are the same):
// grad_mean2d [N,2], grad_conic [N,3], grad_raw_opacity [N] (with the (1 - opacity) factor of :443), grad_color
// [N,3] (zero where the colour was clamped, :286-291).  Doubles: the sum over pixels has no defined order.
ORC_API int orc_fgs_blend_bwd(uint32_t N, uint32_t W, uint32_t H, const uint32_t* instance_primitive,
                              const uint32_t* tile_ranges, const float* mean2d, const float* conic_opacity,
                              const float* color, const float* transmittance, const uint32_t* n_contributions,
                              const float* grad_image, const float* grad_alpha, double* grad_mean2d, double* grad_conic,
                              double* grad_raw_opacity, double* grad_color) {
    const uint32_t grid_w = (W + kTileW - 1) / kTileW;
    std::fill(grad_mean2d, grad_mean2d + 2 * (size_t)N, 0.0);
    std::fill(grad_conic, grad_conic + 3 * (size_t)N, 0.0);
    std::fill(grad_raw_opacity, grad_raw_opacity + (size_t)N, 0.0);
    std::fill(grad_color, grad_color + 3 * (size_t)N, 0.0);
    const size_t n = (size_t)W * H;
    for (uint32_t py = 0; py < H; ++py)
        for (uint32_t px = 0; px < W; ++px) {
            const uint32_t tile = (py / kTileH) * grid_w + px / kTileW;
            const size_t p = (size_t)py * W + px;
            const float fx = (float)px + 0.5f, fy = (float)py + 0.5f;
            const float gc[3] = {grad_image[p], grad_image[p + n], grad_image[p + 2 * n]};
            const float t_final = transmittance[p];
            const float grad_alpha_common = grad_alpha[p] * t_final; // grad_alpha * (1 - alpha_pixel), :330
            float T = t_final, after[3] = {0.f, 0.f, 0.f};
            for (int32_t k = (int32_t)n_contributions[p] - 1; k >= 0; --k) {
                const uint32_t g = instance_primitive[tile_ranges[2 * tile] + (uint32_t)k];
                const float* co = conic_opacity + 4 * g;
                const float dx = mean2d[2 * g] - fx, dy = mean2d[2 * g + 1] - fy;
                const float sigma_over_2 = 0.5f * (co[0] * dx * dx + co[2] * dy * dy) + co[1] * dx * dy;
                if (sigma_over_2 < 0.0f)
                    continue;
                const float gaussian = gsx::exp(-sigma_over_2);
                const float og = co[3] * gaussian;
                const float alpha = og < kMaxAlpha ? og : kMaxAlpha;
                if (alpha < 1.0f / kMinAlphaRcp)
                    continue;
                const float one_minus_alpha_rcp = 1.0f / (1.0f - alpha);
                T *= one_minus_alpha_rcp; // transmittance in front of this primitive
                const float weight = T * alpha;
                float dL_dalpha = grad_alpha_common * one_minus_alpha_rcp;
                for (int ch = 0; ch < 3; ++ch) {
                    const float raw = color[3 * g + ch];
                    const float col = raw > 0.0f ? raw : 0.0f;
                    if (raw >= 0.0f)
                        grad_color[3 * g + ch] += (double)(weight * gc[ch]);
                    dL_dalpha += (T * col - after[ch] * one_minus_alpha_rcp) * gc[ch];
                    after[ch] += weight * col;
                }
                grad_raw_opacity[g] += (double)(alpha * dL_dalpha * (1.0f - co[3]));
                const float helper = -alpha * dL_dalpha;
                grad_conic[3 * g + 0] += (double)(0.5f * helper * dx * dx);
                grad_conic[3 * g + 1] += (double)(0.5f * helper * dx * dy);
                grad_conic[3 * g + 2] += (double)(0.5f * helper * dy * dy);
                grad_mean2d[2 * g + 0] += (double)(helper * (co[0] * dx + co[1] * dy));
                grad_mean2d[2 * g + 1] += (double)(helper * (co[1] * dx + co[2] * dy));
            }
        }
    return 0;
}

// preprocess_backward_cu (kernels_backward.cuh:17-237) with convert_sh_to_color_backward (kernel_utils.cuh:
// 43-105).  In: per-primitive grad_mean2d [N,2], grad_conic [N,3], grad_color [N,3] (what the blend backward
// accumulated; the reference keeps the colour gradient in the sh0 gradient buffer).  Out (zero for culled
// primitives): grad_means [N,3], grad_scales_raw [N,3], grad_rotations_raw [N,4], grad_sh0 [N,3], grad_shN
// [N,B,3]; grad_w2c [16] (nullable; rows 0-2 only, :177-190); densification_info [2,N] (nullable; += as :233-236).
ORC_API int orc_fgs_preprocess_bwd(uint32_t N, const float* means, const float* scales_raw, const float* rotations_raw,
                                   const float* shN, const float* w2c, const float* cam_position, const Settings* S,
                                   const uint32_t* n_touched, const float* grad_mean2d, const float* grad_conic,
                                   const float* grad_color, float* grad_means, float* grad_scales_raw,
                                   float* grad_rotations_raw, float* grad_sh0, float* grad_shN, double* grad_w2c,
                                   float* densification_info) {
    const uint32_t B = S->total_bases_sh_rest, active = S->active_sh_bases;
    const uint32_t grid_w = (S->width + kTileW - 1) / kTileW, grid_h = (S->height + kTileH - 1) / kTileH;
    std::fill(grad_means, grad_means + 3 * (size_t)N, 0.f);
    std::fill(grad_scales_raw, grad_scales_raw + 3 * (size_t)N, 0.f);
    std::fill(grad_rotations_raw, grad_rotations_raw + 4 * (size_t)N, 0.f);
    std::fill(grad_sh0, grad_sh0 + 3 * (size_t)N, 0.f);
    std::fill(grad_shN, grad_shN + 3 * (size_t)N * B, 0.f);
    if (grad_w2c)
        std::fill(grad_w2c, grad_w2c + 16, 0.0);
    const float w = (float)S->width, h = (float)S->height;
    for (uint32_t i = 0; i < N; ++i) {
        if (n_touched[i] == 0)
            continue;
        const float* mean = means + 3 * i;
        // ---- SH backward ----
        const float gcol[3] = {grad_color[3 * i], grad_color[3 * i + 1], grad_color[3 * i + 2]};
        for (int c = 0; c < 3; ++c)
            grad_sh0[3 * i + c] = 0.28209479177387814f * gcol[c];
        float dcolor_dposition[3] = {0.f, 0.f, 0.f};
        if (active > 1) {
            const float* co = shN + (size_t)i * B * 3;
            float* gco = grad_shN + (size_t)i * B * 3;
            const float x_raw = mean[0] - cam_position[0], y_raw = mean[1] - cam_position[1], z_raw = mean[2] - cam_position[2];
            const float inv = gsx::rsqrt(x_raw * x_raw + y_raw * y_raw + z_raw * z_raw);
            const float x = x_raw * inv, y = y_raw * inv, z = z_raw * inv;
            float gdx[3], gdy[3], gdz[3];
            auto setg = [&](int k, float basis) {
                for (int c = 0; c < 3; ++c)
                    gco[k * 3 + c] = basis * gcol[c];
            };
            setg(0, -0.48860251190291987f * y);
            setg(1, 0.48860251190291987f * z);
            setg(2, -0.48860251190291987f * x);
            for (int c = 0; c < 3; ++c) {
                gdx[c] = -0.48860251190291987f * co[2 * 3 + c];
                gdy[c] = -0.48860251190291987f * co[0 * 3 + c];
                gdz[c] = 0.48860251190291987f * co[1 * 3 + c];
            }
            if (active > 4) {
                const float xx = x * x, yy = y * y, zz = z * z, xy = x * y, xz = x * z, yz = y * z;
                setg(3, 1.0925484305920792f * xy);
                setg(4, -1.0925484305920792f * yz);
                setg(5, 0.94617469575755997f * zz - 0.31539156525251999f);
                setg(6, -1.0925484305920792f * xz);
                setg(7, 0.54627421529603959f * xx - 0.54627421529603959f * yy);
                for (int c = 0; c < 3; ++c) {
                    gdx[c] = gdx[c] + (1.0925484305920792f * y) * co[3 * 3 + c] + (-1.0925484305920792f * z) * co[6 * 3 + c] +
                             (1.0925484305920792f * x) * co[7 * 3 + c];
                    gdy[c] = gdy[c] + (1.0925484305920792f * x) * co[3 * 3 + c] + (-1.0925484305920792f * z) * co[4 * 3 + c] +
                             (-1.0925484305920792f * y) * co[7 * 3 + c];
                    gdz[c] = gdz[c] + (-1.0925484305920792f * y) * co[4 * 3 + c] + (1.8923493915151202f * z) * co[5 * 3 + c] +
                             (-1.0925484305920792f * x) * co[6 * 3 + c];
                }
                if (active > 9) {
                    setg(8, 0.59004358992664352f * y * (-3.0f * xx + yy));
                    setg(9, 2.8906114426405538f * xy * z);
                    setg(10, 0.45704579946446572f * y * (1.0f - 5.0f * zz));
                    setg(11, 0.3731763325901154f * z * (5.0f * zz - 3.0f));
                    setg(12, 0.45704579946446572f * x * (1.0f - 5.0f * zz));
                    setg(13, 1.4453057213202769f * z * (xx - yy));
                    setg(14, 0.59004358992664352f * x * (-xx + 3.0f * yy));
                    for (int c = 0; c < 3; ++c) {
                        gdx[c] = gdx[c] + (-3.5402615395598609f * xy) * co[8 * 3 + c] + (2.8906114426405538f * yz) * co[9 * 3 + c] +
                                 (0.45704579946446572f - 2.2852289973223288f * zz) * co[12 * 3 + c] +
                                 (2.8906114426405538f * xz) * co[13 * 3 + c] +
                                 (-1.7701307697799304f * xx + 1.7701307697799304f * yy) * co[14 * 3 + c];
                        gdy[c] = gdy[c] + (-1.7701307697799304f * xx + 1.7701307697799304f * yy) * co[8 * 3 + c] +
                                 (2.8906114426405538f * xz) * co[9 * 3 + c] +
                                 (0.45704579946446572f - 2.2852289973223288f * zz) * co[10 * 3 + c] +
                                 (-2.8906114426405538f * yz) * co[13 * 3 + c] + (3.5402615395598609f * xy) * co[14 * 3 + c];
                        gdz[c] = gdz[c] + (2.8906114426405538f * xy) * co[9 * 3 + c] + (-4.5704579946446566f * yz) * co[10 * 3 + c] +
                                 (5.597644988851731f * zz - 1.1195289977703462f) * co[11 * 3 + c] +
                                 (-4.5704579946446566f * xz) * co[12 * 3 + c] +
                                 (1.4453057213202769f * xx - 1.4453057213202769f * yy) * co[13 * 3 + c];
                    }
                }
            }
            const float gx = gdx[0] * gcol[0] + gdx[1] * gcol[1] + gdx[2] * gcol[2];
            const float gy = gdy[0] * gcol[0] + gdy[1] * gcol[1] + gdy[2] * gcol[2];
            const float gz = gdz[0] * gcol[0] + gdz[1] * gcol[1] + gdz[2] * gcol[2];
            const float xx_raw = x_raw * x_raw, yy_raw = y_raw * y_raw, zz_raw = z_raw * z_raw;
            const float xy_raw = x_raw * y_raw, xz_raw = x_raw * z_raw, yz_raw = y_raw * z_raw;
            const float norm_sq = xx_raw + yy_raw + zz_raw;
            const float s = gsx::rsqrt(norm_sq * norm_sq * norm_sq);
            dcolor_dposition[0] = ((yy_raw + zz_raw) * gx - xy_raw * gy - xz_raw * gz) * s;
            dcolor_dposition[1] = (-xy_raw * gx + (xx_raw + zz_raw) * gy - yz_raw * gz) * s;
            dcolor_dposition[2] = (-xz_raw * gx - yz_raw * gy + (xx_raw + yy_raw) * gz) * s;
        }
        // ---- EWA chain ----
        const Projected<float> P = project<float>(mean, scales_raw + 3 * i, rotations_raw + 4 * i, 0.0f, w2c, *S, grid_w, grid_h);
        const float* r1 = w2c;
        const float* r2 = w2c + 4;
        const float* r3 = w2c + 8;
        const float a = P.cov2d[0], b = P.cov2d[1], c = P.cov2d[2];
        const float aa = a * a, bb = b * b, cc = c * c, ac = a * c, ab = a * b, bc = b * c;
        const float determinant = ac - bb;
        const float determinant_rcp = 1.0f / determinant;
        const float determinant_rcp_sq = determinant_rcp * determinant_rcp;
        const float gk[3] = {grad_conic[3 * i], grad_conic[3 * i + 1], grad_conic[3 * i + 2]};
        const float dcov[3] = {determinant_rcp_sq * (2.0f * bc * gk[1] - cc * gk[0] - bb * gk[2]),
                               determinant_rcp_sq * (bc * gk[0] - (ac + bb) * gk[1] + ab * gk[2]),
                               determinant_rcp_sq * (2.0f * ab * gk[1] - bb * gk[0] - aa * gk[2])};
        const float* j1 = P.jw1;
        const float* j2 = P.jw2;
        float d3[6]; // dL_dcov3d: m11 m12 m13 m22 m23 m33
        d3[0] = (j1[0] * j1[0]) * dcov[0] + 2.0f * (j1[0] * j2[0]) * dcov[1] + (j2[0] * j2[0]) * dcov[2];
        d3[1] = (j1[0] * j1[1]) * dcov[0] + (j1[0] * j2[1] + j1[1] * j2[0]) * dcov[1] + (j2[0] * j2[1]) * dcov[2];
        d3[2] = (j1[0] * j1[2]) * dcov[0] + (j1[0] * j2[2] + j1[2] * j2[0]) * dcov[1] + (j2[0] * j2[2]) * dcov[2];
        d3[3] = (j1[1] * j1[1]) * dcov[0] + 2.0f * (j1[1] * j2[1]) * dcov[1] + (j2[1] * j2[1]) * dcov[2];
        d3[4] = (j1[1] * j1[2]) * dcov[0] + (j1[1] * j2[2] + j1[2] * j2[1]) * dcov[1] + (j2[1] * j2[2]) * dcov[2];
        d3[5] = (j1[2] * j1[2]) * dcov[0] + 2.0f * (j1[2] * j2[2]) * dcov[1] + (j2[2] * j2[2]) * dcov[2];
        float djw1[3], djw2[3];
        for (int k = 0; k < 3; ++k) {
            djw1[k] = 2.0f * (P.jwc1[k] * dcov[0] + P.jwc2[k] * dcov[1]);
            djw2[k] = 2.0f * (P.jwc1[k] * dcov[1] + P.jwc2[k] * dcov[2]);
        }
        const float dj11 = r1[0] * djw1[0] + r1[1] * djw1[1] + r1[2] * djw1[2];
        const float dj22 = r2[0] * djw2[0] + r2[1] * djw2[1] + r2[2] * djw2[2];
        const float dj13 = r3[0] * djw1[0] + r3[1] * djw1[1] + r3[2] * djw1[2];
        const float dj23 = r3[0] * djw2[0] + r3[1] * djw2[1] + r3[2] * djw2[2];
        const float h1 = dj11 - 2.0f * P.tx * dj13, h2 = dj22 - 2.0f * P.ty * dj23;
        const float gm2[2] = {grad_mean2d[2 * i], grad_mean2d[2 * i + 1]};
        const float dcam[3] = {P.j11 * (gm2[0] - dj13 / P.depth), P.j22 * (gm2[1] - dj23 / P.depth),
                               -P.j11 * (P.x * gm2[0] + h1 / P.depth) - P.j22 * (P.y * gm2[1] + h2 / P.depth)};
        if (grad_w2c) {
            for (int r = 0; r < 3; ++r) {
                grad_w2c[4 * r + 3] += (double)dcam[r];
                for (int k = 0; k < 3; ++k)
                    grad_w2c[4 * r + k] += (double)(dcam[r] * mean[k]);
            }
        }
        for (int k = 0; k < 3; ++k)
            grad_means[3 * i + k] = (r1[k] * dcam[0] + r2[k] * dcam[1] + r3[k] * dcam[2]) + dcolor_dposition[k];
        const float* R = P.rot;
        const float* RS = P.rot_scaled;
        for (int k = 0; k < 3; ++k) {
            const float dvar = R[0 + k] * R[0 + k] * d3[0] + R[3 + k] * R[3 + k] * d3[3] + R[6 + k] * R[6 + k] * d3[5] +
                               2.0f * (R[0 + k] * R[3 + k] * d3[1] + R[0 + k] * R[6 + k] * d3[2] + R[3 + k] * R[6 + k] * d3[4]);
            grad_scales_raw[3 * i + k] = 2.0f * P.variance[k] * dvar;
        }
        float dR[9];
        for (int k = 0; k < 3; ++k) {
            dR[0 + k] = 2.0f * (RS[0 + k] * d3[0] + RS[3 + k] * d3[1] + RS[6 + k] * d3[2]);
            dR[3 + k] = 2.0f * (RS[0 + k] * d3[1] + RS[3 + k] * d3[3] + RS[6 + k] * d3[4]);
            dR[6 + k] = 2.0f * (RS[0 + k] * d3[2] + RS[3 + k] * d3[4] + RS[6 + k] * d3[5]);
        }
        const float* q = rotations_raw + 4 * i;
        const float qr = q[0], qx = q[1], qy = q[2], qz = q[3], qn = P.q_norm_sq;
        const float qxx = 2.0f * (qx * qx) / qn, qyy = 2.0f * (qy * qy) / qn, qzz = 2.0f * (qz * qz) / qn;
        const float qxy = 2.0f * qx * qy / qn, qxz = 2.0f * qx * qz / qn, qyz = 2.0f * qy * qz / qn;
        const float qrx = 2.0f * qr * qx / qn, qry = 2.0f * qr * qy / qn, qrz = 2.0f * qr * qz / qn;
        const float dqxx = -dR[4] - dR[8], dqyy = -dR[0] - dR[8], dqzz = -dR[0] - dR[4];
        const float dqxy = dR[1] + dR[3], dqxz = dR[2] + dR[6], dqyz = dR[5] + dR[7];
        const float dqrx = dR[7] - dR[5], dqry = dR[2] - dR[6], dqrz = dR[3] - dR[1];
        const float helper = qxx * dqxx + qyy * dqyy + qzz * dqzz + qxy * dqxy + qxz * dqxz + qyz * dqyz + qrx * dqrx +
                             qry * dqry + qrz * dqrz;
        grad_rotations_raw[4 * i + 0] = 2.0f * (qx * dqrx + qy * dqry + qz * dqrz - qr * helper) / qn;
        grad_rotations_raw[4 * i + 1] = 2.0f * (2.0f * qx * dqxx + qy * dqxy + qz * dqxz + qr * dqrx - qx * helper) / qn;
        grad_rotations_raw[4 * i + 2] = 2.0f * (2.0f * qy * dqyy + qx * dqxy + qz * dqyz + qr * dqry - qy * helper) / qn;
        grad_rotations_raw[4 * i + 3] = 2.0f * (2.0f * qz * dqzz + qx * dqxz + qy * dqyz + qr * dqrz - qz * helper) / qn;
        if (densification_info) {
            densification_info[i] += 1.0f;
            const float sx = gm2[0] * (0.5f * w), sy = gm2[1] * (0.5f * h);
            densification_info[N + i] += gsx::sqrt(sx * sx + sy * sy);
        }
    }
    return 0;
}

// The double model: loss = sum(weight_image * image) + sum(weight_alpha * alpha) for FIXED tile lists (those of
// the float run) and, with `decisions`, fixed skip / stop decisions per (pixel, list entry) - recorded by a call
// with record = 1 at the base point, replayed by the perturbed calls.  Every parameter in double.  Central
// differences of this pin the analytic backward.  max_list >= the longest tile list.
ORC_API double orc_fgs_loss_f64(uint32_t N, const double* means, const double* scales_raw, const double* rotations_raw,
                                const double* opacities_raw, const double* sh0, const double* shN, const double* w2c,
                                const double* cam_position, const Settings* S, const uint32_t* instance_primitive,
                                const uint32_t* tile_ranges, const float* weight_image, const float* weight_alpha,
                                uint8_t* decisions /*[H*W*max list length]*/, uint32_t max_list, int record) {
    const uint32_t W = S->width, H = S->height;
    const uint32_t grid_w = (W + kTileW - 1) / kTileW, grid_h = (H + kTileH - 1) / kTileH;
    std::vector<double> mean2d(2 * (size_t)N), co(4 * (size_t)N), color(3 * (size_t)N);
    for (uint32_t i = 0; i < N; ++i) {
        const Projected<double> P = project<double>(means + 3 * i, scales_raw + 3 * i, rotations_raw + 4 * i,
                                                    opacities_raw[i], w2c, *S, grid_w, grid_h);
        mean2d[2 * i] = P.mean2d[0], mean2d[2 * i + 1] = P.mean2d[1];
        co[4 * i] = P.conic[0], co[4 * i + 1] = P.conic[1], co[4 * i + 2] = P.conic[2], co[4 * i + 3] = P.opacity;
        sh_to_color<double>(sh0 + 3 * i, shN + (size_t)i * S->total_bases_sh_rest * 3, means + 3 * i, cam_position,
                            S->active_sh_bases, color.data() + 3 * i);
    }
    double loss = 0.0;
    const size_t n = (size_t)W * H;
    for (uint32_t py = 0; py < H; ++py)
        for (uint32_t px = 0; px < W; ++px) {
            const uint32_t tile = (py / kTileH) * grid_w + px / kTileW;
            double rgb[3], t;
            uint32_t nc;
            blend_pixel<double>((double)px + 0.5, (double)py + 0.5, instance_primitive, tile_ranges[2 * tile],
                                tile_ranges[2 * tile + 1], mean2d.data(), co.data(), color.data(), rgb, &t, &nc,
                                decisions ? decisions + ((size_t)py * W + px) * max_list : nullptr, record != 0);
            const size_t p = (size_t)py * W + px;
            loss += weight_image[p] * rgb[0] + weight_image[p + n] * rgb[1] + weight_image[p + 2 * n] * rgb[2];
            loss += weight_alpha[p] * (1.0 - t);
        }
    return loss;
}
