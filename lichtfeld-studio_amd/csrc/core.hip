// core.hip - error reporting, version, argument checks shared by the entry points.
#include <stdarg.h>

#include <algorithm>
#include <atomic>

#include "gsx_common.h"
#include "gsx_lookback.h"

namespace gsx {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

// One camera per call (the reference's rasterizer indexes per-Gaussian arrays with the flattened [C*N] id,
// RasterizeToPixelsFromWorld3DGSFwd.cu:203-210, so C > 1 is not usable there either); the pinhole model with or
// without OpenCV distortion coefficients (radial [6], tangential [2], thin prism [4]), the OpenCV fisheye model
// (radial [4]) and the equirectangular model; global or rolling shutter (viewmats1 = the end-of-frame pose, null =
// the start pose).
int check_camera_args(uint32_t C, const float* viewmats1, int camera_model, int rs_type, const float* radial,
                      const float* tangential, const float* thin_prism) {
    GSX_REQUIRE(C == 1, GSX_ERR_UNSUPPORTED, "C = %u cameras: only C == 1 is supported", C);
    GSX_REQUIRE(camera_model == GSX_PINHOLE || camera_model == GSX_FISHEYE || camera_model == GSX_EQUIRECTANGULAR,
                GSX_ERR_UNSUPPORTED, "camera model %d: PINHOLE, FISHEYE and EQUIRECTANGULAR are supported", camera_model);
    (void)radial, (void)tangential, (void)thin_prism;
    (void)viewmats1;
    GSX_REQUIRE(rs_type >= GSX_ROLLING_TOP_TO_BOTTOM && rs_type <= GSX_GLOBAL, GSX_ERR_INVALID_ARGUMENT,
                "shutter type %d: must be 0 .. 4 (gsx_shutter_type)", rs_type);
    return GSX_OK;
}

// probe of the shared math primitives on the device (lets a test compare them bit for bit with a host build)
__global__ void __launch_bounds__(256) math_unary_kernel(int which, uint32_t n, const float* __restrict__ x,
                                                          const float* __restrict__ x2, float* __restrict__ y) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= n)
        return;
    const float a = x[i];
    float r = 0.f;
    switch (which) {
    case 0: r = gsx::exp(a); break;
    case 1: r = gsx::log(a); break;
    case 2: r = gsx::rsqrt(a); break;
    case 3: r = gsx::sin(a); break;
    case 4: r = gsx::acos(a); break;
    case 5: r = gsx::sigmoid(a); break;
    case 6: r = (float)gsx::sat_u32(a); break;
    case 7: r = gsx::pow(a, x2[i]); break;
    case 8: r = a / x2[i]; break;
    case 9: r = gsx::sqrt(a); break;
    case 10: r = gsx::fma(a, x2[i], a); break;
    case 11: r = gsx::exp_nonpos(a); break;
    case 12: r = gsx::rcp_refined(a); break;
    case 13: r = gsx::rcp_approx(a); break;
    case 15: r = gsx::min_limit(x2[i], a); break;
    default: break;
    }
    y[i] = r;
}

// streaming copy of known size: the yardstick that HBM byte counters and achieved bandwidths are scaled by.  One
// 16-byte element per lane, loads and stores with the non-temporal hint: the fastest copy found on this GPU.
__global__ void __launch_bounds__(256) copy_probe_kernel(const float4* __restrict__ src, float4* __restrict__ dst,
                                                          size_t n16) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16)
        store_streaming(dst + i, load_streaming(src + i));
}

} // namespace gsx

namespace gsx {
static std::atomic<int64_t> g_spin_limit{-1};
uint32_t lookback_spin_limit() {
    const int64_t v = g_spin_limit.load(std::memory_order_relaxed);
    return v < 0 ? kLbSpinLimit : (uint32_t)v;
}
} // namespace gsx

extern "C" int gsx_debug_set_lookback_spin_limit(int64_t limit) {
    gsx::g_spin_limit.store(limit < 0 ? -1 : std::min<int64_t>(limit, gsx::kLbSpinLimit), std::memory_order_relaxed);
    return GSX_OK;
}

extern "C" int gsx_debug_copy(const void* src, void* dst, size_t bytes, void* stream) {
    if (bytes == 0)
        return GSX_OK;
    GSX_REQUIRE(src && dst && bytes % 16 == 0 && ((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0,
                GSX_ERR_INVALID_ARGUMENT, "debug_copy: null / unaligned buffers or size %zu not a multiple of 16", bytes);
    const size_t n16 = bytes / 16;
    const size_t blocks = (n16 + 255) / 256;
    GSX_REQUIRE(blocks < (1ull << 31), GSX_ERR_INVALID_ARGUMENT, "debug_copy: %zu bytes in one call", bytes);
    hipLaunchKernelGGL(gsx::copy_probe_kernel, dim3((uint32_t)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const float4*)src, (float4*)dst, n16);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_debug_math(int which, uint32_t n, const float* x, const float* x2, float* y, void* stream) {
    if (n == 0)
        return GSX_OK;
    GSX_REQUIRE(x && y, GSX_ERR_INVALID_ARGUMENT, "debug_math: null tensor");
    GSX_REQUIRE(which < 7 || (which >= 11 && which != 15) || x2 != nullptr, GSX_ERR_INVALID_ARGUMENT,
                "debug_math: second operand is null");
    hipLaunchKernelGGL(gsx::math_unary_kernel, dim3(gsx::cdiv(n, 256)), dim3(256), 0, (hipStream_t)stream, which, n, x,
                       x2, y);
    GSX_LAUNCH_CHECK();
    return GSX_OK;
}

extern "C" int gsx_version(void) { return 100; }

extern "C" const char* gsx_last_error(void) { return gsx::g_err; }

extern "C" const char* gsx_status_string(int status) {
    switch (status) {
    case GSX_OK: return "ok";
    case GSX_ERR_INVALID_ARGUMENT: return "invalid argument";
    case GSX_ERR_UNSUPPORTED: return "unsupported configuration";
    case GSX_ERR_WORKSPACE: return "workspace too small or misaligned";
    case GSX_ERR_HIP: return "HIP runtime error";
    case GSX_ERR_OVERFLOW: return "intersection count overflows int32";
    default: return "unknown status";
    }
}

extern "C" gsx_ut_params gsx_ut_defaults(void) {
    gsx_ut_params p;
    p.alpha = 0.1f;
    p.beta = 2.f;
    p.kappa = 0.f;
    p.in_image_margin_factor = 0.1f;
    p.require_all_sigma_points_valid = 1;
    return p;
}

extern "C" uint32_t gsx_n_bits(uint32_t n) {
    // (uint32_t)floor(log2(n)) + 1 for n >= 1 (gsplat/Intersect.cpp:46-47)
    uint32_t b = 0;
    while (n) {
        ++b;
        n >>= 1;
    }
    return b;
}
