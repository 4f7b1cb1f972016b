// fastgs_api.cpp - fast_gs::rasterization::forward_wrapper / backward_wrapper over at::Tensor with the allocation and
// return conventions of LichtFeld-Studio's src/training/fastgs/rasterization/src/rasterization_api.cu:16-181, calling
// the gfx950 kernels through the C ABI of gsx_fastgs.h on torch's current stream.
#include "fastgs_api.h"

#include <ATen/Functions.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <c10/util/Exception.h>

#include "gsx_fastgs.h"

namespace {

// torch_utils.h CHECK_INPUT (the reference compiles it out unless config::debug; kept on here: a host tensor or a
// strided view handed to a kernel is a memory fault, not an error message)
#define FGS_CHECK_INPUT(x) \
    TORCH_CHECK((x).is_cuda() && (x).is_contiguous() && (x).scalar_type() == at::kFloat, #x " must be a contiguous CUDA float tensor")

inline void* cur_stream(const at::Tensor& t) { return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }
inline void gsx_check(int status) { TORCH_CHECK(status == GSX_OK, "gsx (", gsx_status_string(status), "): ", gsx_last_error()); }
inline at::Tensor bytes(size_t n, const at::Tensor& like) {
    return at::empty({(int64_t)(n < 256 ? 256 : n)}, like.options().dtype(at::kByte));
}
inline float* opt_ptr(const at::Tensor& t) { return t.defined() && t.numel() > 0 ? t.data_ptr<float>() : nullptr; }

struct HostCamera {
    at::Tensor w2c, cam; // host, float, contiguous
    HostCamera(const at::Tensor& w2c_in, const at::Tensor& cam_in)
        : w2c(w2c_in.detach().to(at::kCPU, at::kFloat).contiguous()), cam(cam_in.detach().to(at::kCPU, at::kFloat).contiguous()) {
        TORCH_CHECK(w2c.numel() == 16, "w2c must hold 16 values");
        TORCH_CHECK(cam.numel() == 3, "cam_position must hold 3 values");
    }
};

gsx_fastgs_settings make_settings(int active_sh_bases, int64_t total_rest, int width, int height, float fx, float fy, float cx,
                                  float cy, float near_plane, float far_plane) {
    TORCH_CHECK(width > 0 && height > 0 && active_sh_bases > 0, "fastgs: bad image size / SH base count");
    gsx_fastgs_settings S;
    S.active_sh_bases = (uint32_t)active_sh_bases, S.total_bases_sh_rest = (uint32_t)total_rest;
    S.width = (uint32_t)width, S.height = (uint32_t)height;
    S.fx = fx, S.fy = fy, S.cx = cx, S.cy = cy, S.near_plane = near_plane, S.far_plane = far_plane;
    return S;
}

} // namespace

namespace fast_gs::rasterization {

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, int, int, int, int, int>
forward_wrapper(const at::Tensor& means, const at::Tensor& scales_raw, const at::Tensor& rotations_raw,
                const at::Tensor& opacities_raw, const at::Tensor& sh_coefficients_0,
                const at::Tensor& sh_coefficients_rest, const at::Tensor& w2c, const at::Tensor& cam_position,
                const int active_sh_bases, const int width, const int height, const float focal_x, const float focal_y,
                const float center_x, const float center_y, const float near_plane, const float far_plane) {
    FGS_CHECK_INPUT(means);
    FGS_CHECK_INPUT(scales_raw);
    FGS_CHECK_INPUT(rotations_raw);
    FGS_CHECK_INPUT(opacities_raw);
    FGS_CHECK_INPUT(sh_coefficients_0);
    FGS_CHECK_INPUT(sh_coefficients_rest);
    const c10::DeviceGuard guard(means.device());
    const uint32_t N = (uint32_t)means.size(0);
    const gsx_fastgs_settings S = make_settings(active_sh_bases, sh_coefficients_rest.size(1), width, height, focal_x,
                                                focal_y, center_x, center_y, near_plane, far_plane);
    const HostCamera cam(w2c, cam_position);
    void* stream = cur_stream(means);
    const auto fopt = means.options().dtype(at::kFloat);
    at::Tensor image = at::empty({3, height, width}, fopt);
    at::Tensor alpha = at::empty({1, height, width}, fopt);
    at::Tensor prim = bytes(gsx_fastgs_primitive_state_bytes(N), means);
    int64_t n_instances = 0;
    gsx_check(gsx_fastgs_preprocess(N, means.data_ptr<float>(), scales_raw.data_ptr<float>(), rotations_raw.data_ptr<float>(),
                                    opacities_raw.data_ptr<float>(), sh_coefficients_0.data_ptr<float>(),
                                    opt_ptr(sh_coefficients_rest), cam.w2c.data_ptr<float>(), cam.cam.data_ptr<float>(), &S,
                                    prim.data_ptr(), (size_t)prim.numel(), &n_instances, /*wait=*/1, stream));
    at::Tensor inst = bytes(gsx_fastgs_instance_state_bytes(n_instances, S.width, S.height), means);
    at::Tensor pix = bytes(gsx_fastgs_pixel_state_bytes(S.width, S.height), means);
    gsx_check(gsx_fastgs_render(N, &S, prim.data_ptr(), (size_t)prim.numel(), n_instances, inst.data_ptr(),
                                (size_t)inst.numel(), nullptr, image.data_ptr<float>(), alpha.data_ptr<float>(),
                                pix.data_ptr(), (size_t)pix.numel(), stream));
    at::Tensor bucket = at::empty({0}, means.options().dtype(at::kByte));
    return {image, alpha, prim, pix, inst, bucket, -1, (int)n_instances, 0, 0, 0};
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor>
backward_wrapper(at::Tensor& densification_info, const at::Tensor& grad_image, const at::Tensor& grad_alpha,
                 const at::Tensor& image, const at::Tensor& alpha, const at::Tensor& means, const at::Tensor& scales_raw,
                 const at::Tensor& rotations_raw, const at::Tensor& sh_coefficients_rest,
                 const at::Tensor& per_primitive_buffers, const at::Tensor& per_tile_buffers,
                 const at::Tensor& per_instance_buffers, const at::Tensor& per_bucket_buffers, const at::Tensor& w2c,
                 const at::Tensor& cam_position, const int active_sh_bases, const int width, const int height,
                 const float focal_x, const float focal_y, const float center_x, const float center_y,
                 const float near_plane, const float far_plane, const int n_visible_primitives, const int n_instances,
                 const int n_buckets, const int primitive_primitive_indices_selector,
                 const int instance_primitive_indices_selector) {
    (void)image, (void)alpha, (void)per_bucket_buffers, (void)n_visible_primitives, (void)n_buckets;
    (void)primitive_primitive_indices_selector, (void)instance_primitive_indices_selector;
    FGS_CHECK_INPUT(means);
    FGS_CHECK_INPUT(scales_raw);
    FGS_CHECK_INPUT(rotations_raw);
    FGS_CHECK_INPUT(sh_coefficients_rest);
    const c10::DeviceGuard guard(means.device());
    const int64_t n = means.size(0), B = sh_coefficients_rest.size(1);
    const gsx_fastgs_settings S = make_settings(active_sh_bases, B, width, height, focal_x, focal_y, center_x, center_y,
                                                near_plane, far_plane);
    const HostCamera cam(w2c, cam_position);
    const auto fopt = means.options().dtype(at::kFloat);
    // rasterization_api.cu:123-133 zero-fills these; here the kernels write every element
    at::Tensor grad_means = at::empty({n, 3}, fopt), grad_scales_raw = at::empty({n, 3}, fopt);
    at::Tensor grad_rotations_raw = at::empty({n, 4}, fopt), grad_opacities_raw = at::empty({n, 1}, fopt);
    at::Tensor grad_sh0 = at::empty({n, 1, 3}, fopt), grad_shN = at::empty({n, B, 3}, fopt);
    at::Tensor grad_w2c;
    if (w2c.requires_grad())
        grad_w2c = at::empty({4, 4}, fopt);
    const bool update_info = densification_info.defined() && densification_info.size(0) > 0; // rasterization_api.cu:130
    if (update_info) {
        TORCH_CHECK(densification_info.is_cuda() && densification_info.is_contiguous() &&
                        densification_info.numel() == 2 * n,
                    "densification_info must be a contiguous CUDA tensor [2, N]");
    }
    for (const at::Tensor* t : {&per_primitive_buffers, &per_tile_buffers, &per_instance_buffers})
        TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == at::kByte,
                    "the state buffers must be the byte tensors forward_wrapper returned");
    TORCH_CHECK(grad_image.is_cuda() && grad_image.scalar_type() == at::kFloat && grad_image.numel() == 3ll * width * height,
                "grad_image must be a CUDA float tensor [3, H, W]");
    TORCH_CHECK(grad_alpha.is_cuda() && grad_alpha.scalar_type() == at::kFloat && grad_alpha.numel() == 1ll * width * height,
                "grad_alpha must be a CUDA float tensor [1, H, W]");
    const at::Tensor gi = grad_image.contiguous(), ga = grad_alpha.contiguous();
    at::Tensor accum = at::zeros({(int64_t)gsx_fastgs_accum_bytes((uint32_t)n)}, means.options().dtype(at::kByte));
    gsx_check(gsx_fastgs_backward((uint32_t)n, means.data_ptr<float>(), scales_raw.data_ptr<float>(),
                                  rotations_raw.data_ptr<float>(), opt_ptr(sh_coefficients_rest), cam.w2c.data_ptr<float>(),
                                  cam.cam.data_ptr<float>(), &S, per_primitive_buffers.data_ptr(),
                                  (size_t)per_primitive_buffers.numel(), n_instances, per_instance_buffers.data_ptr(),
                                  (size_t)per_instance_buffers.numel(), per_tile_buffers.data_ptr(),
                                  (size_t)per_tile_buffers.numel(), nullptr, gi.data_ptr<float>(),
                                  ga.data_ptr<float>(), accum.data_ptr(), (size_t)accum.numel(), grad_means.data_ptr<float>(),
                                  grad_scales_raw.data_ptr<float>(), grad_rotations_raw.data_ptr<float>(),
                                  grad_opacities_raw.data_ptr<float>(), grad_sh0.data_ptr<float>(), opt_ptr(grad_shN),
                                  grad_w2c.defined() ? grad_w2c.data_ptr<float>() : nullptr,
                                  update_info ? densification_info.data_ptr<float>() : nullptr, cur_stream(means)));
    return {grad_means, grad_scales_raw, grad_rotations_raw, grad_opacities_raw, grad_sh0, grad_shN, grad_w2c};
}

} // namespace fast_gs::rasterization
