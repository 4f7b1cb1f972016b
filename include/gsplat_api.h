// gsplat_api.h - the C++ host interface of the path, with the names, namespaces, argument order and
// by-value at::Tensor conventions of LichtFeld-Studio's gsplat/Ops.h:9-272 (+ gsplat/Cameras.h:16-61,
// gsplat/Common.h:46-54, include/kernels/ssim.cuh:11-28, fastgs/optimizer/include/adam_api.h), implemented in
// lichtfeld-studio_amd/csrc/host/gsplat_ops.cpp on top of the C ABI of gsx.h.  A LichtFeld build keeps its own
// headers; this one exists so that the implementation can be compiled and tested without the reference tree.
#pragma once

#include <ATen/core/Tensor.h>
#include <c10/util/Optional.h>

#include <cstdint>
#include <string>
#include <tuple>

// global namespace, as in gsplat/Cameras.h
enum class ShutterType { ROLLING_TOP_TO_BOTTOM, ROLLING_LEFT_TO_RIGHT, ROLLING_BOTTOM_TO_TOP, ROLLING_RIGHT_TO_LEFT, GLOBAL };

struct UnscentedTransformParameters {
    float alpha = 0.1f, beta = 2.f, kappa = 0.f;
    float in_image_margin_factor = 0.1f;
    bool require_all_sigma_points_valid = true;
};

namespace gsplat {

    enum CameraModelType { PINHOLE = 0, ORTHO = 1, FISHEYE = 2, EQUIRECTANGULAR = 3 };

    using OptT = at::optional<at::Tensor>;

    at::Tensor spherical_harmonics_fwd(const uint32_t degrees_to_use, const at::Tensor dirs, const at::Tensor coeffs,
                                       const OptT masks);
    std::tuple<at::Tensor, at::Tensor> spherical_harmonics_bwd(const uint32_t K, const uint32_t degrees_to_use,
                                                               const at::Tensor dirs, const at::Tensor coeffs,
                                                               const OptT masks, const at::Tensor v_colors,
                                                               bool compute_v_dirs);

    std::tuple<at::Tensor, at::Tensor, at::Tensor> intersect_tile(const at::Tensor means2d, const at::Tensor radii,
                                                                  const at::Tensor depths, const OptT camera_ids,
                                                                  const OptT gaussian_ids, const uint32_t C,
                                                                  const uint32_t tile_size, const uint32_t tile_width,
                                                                  const uint32_t tile_height, const bool sort);
    at::Tensor intersect_offset(const at::Tensor isect_ids, const uint32_t C, const uint32_t tile_width,
                                const uint32_t tile_height);
    void radix_sort_double_buffer(const int64_t n_isects, const uint32_t tile_n_bits, const uint32_t cam_n_bits,
                                  at::Tensor isect_ids, at::Tensor flatten_ids, at::Tensor isect_ids_sorted,
                                  at::Tensor flatten_ids_sorted);

    at::Tensor quats_to_rotmats(const at::Tensor quats);

    std::tuple<at::Tensor, at::Tensor> relocation(at::Tensor opacities, at::Tensor scales, at::Tensor ratios,
                                                  at::Tensor binoms, const int n_max);
    void add_noise(at::Tensor raw_opacities, at::Tensor raw_scales, at::Tensor raw_quats, at::Tensor noise,
                   at::Tensor means, const float current_lr);

    std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> projection_ut_3dgs_fused(
        const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const OptT opacities,
        const at::Tensor viewmats0, const OptT viewmats1, const at::Tensor Ks, const uint32_t image_width,
        const uint32_t image_height, const float eps2d, const float near_plane, const float far_plane,
        const float radius_clip, const bool calc_compensations, const CameraModelType camera_model,
        const UnscentedTransformParameters ut_params, ShutterType rs_type, const OptT radial_coeffs,
        const OptT tangential_coeffs, const OptT thin_prism_coeffs);

    std::tuple<at::Tensor, at::Tensor, at::Tensor> rasterize_to_pixels_from_world_3dgs_fwd(
        const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const at::Tensor colors,
        const at::Tensor opacities, const OptT backgrounds, const OptT masks, const uint32_t image_width,
        const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0, const OptT viewmats1,
        const at::Tensor Ks, const CameraModelType camera_model, const UnscentedTransformParameters ut_params,
        ShutterType rs_type, const OptT radial_coeffs, const OptT tangential_coeffs, const OptT thin_prism_coeffs,
        const at::Tensor tile_offsets, const at::Tensor flatten_ids);

    std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> rasterize_to_pixels_from_world_3dgs_bwd(
        const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const at::Tensor colors,
        const at::Tensor opacities, const OptT backgrounds, const OptT masks, const uint32_t image_width,
        const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0, const OptT viewmats1,
        const at::Tensor Ks, const CameraModelType camera_model, const UnscentedTransformParameters ut_params,
        ShutterType rs_type, const OptT radial_coeffs, const OptT tangential_coeffs, const OptT thin_prism_coeffs,
        const at::Tensor tile_offsets, const at::Tensor flatten_ids, const at::Tensor render_alphas,
        const at::Tensor last_ids, const at::Tensor v_render_colors, const at::Tensor v_render_alphas);

    // -> (render_colors, render_alphas, radii, means2d, depths, colors, tile_offsets, flatten_ids, last_ids, compensations)
    std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor,
               at::Tensor>
    rasterize_from_world_with_sh_fwd(const at::Tensor means, const at::Tensor quats, const at::Tensor scales,
                                     const at::Tensor opacities, const at::Tensor sh_coeffs, const uint32_t sh_degree,
                                     const OptT backgrounds, const OptT masks, const uint32_t image_width,
                                     const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0,
                                     const OptT viewmats1, const at::Tensor Ks, const CameraModelType camera_model,
                                     const float eps2d, const float near_plane, const float far_plane,
                                     const float radius_clip, const float scaling_modifier,
                                     const bool calc_compensations, const int render_mode,
                                     const UnscentedTransformParameters ut_params, ShutterType rs_type,
                                     const OptT radial_coeffs, const OptT tangential_coeffs,
                                     const OptT thin_prism_coeffs);

    // -> (v_means, v_quats, v_scales, v_opacities, v_sh_coeffs)
    std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> rasterize_from_world_with_sh_bwd(
        const at::Tensor means, const at::Tensor quats, const at::Tensor scales, const at::Tensor opacities,
        const at::Tensor sh_coeffs, const uint32_t sh_degree, const OptT backgrounds, const OptT masks,
        const uint32_t image_width, const uint32_t image_height, const uint32_t tile_size, const at::Tensor viewmats0,
        const OptT viewmats1, const at::Tensor Ks, const CameraModelType camera_model, const float eps2d,
        const float near_plane, const float far_plane, const float radius_clip, const float scaling_modifier,
        const bool calc_compensations, const int render_mode, const UnscentedTransformParameters ut_params,
        ShutterType rs_type, const OptT radial_coeffs, const OptT tangential_coeffs, const OptT thin_prism_coeffs,
        const at::Tensor render_alphas, const at::Tensor last_ids, const at::Tensor tile_offsets,
        const at::Tensor flatten_ids, const at::Tensor colors, const at::Tensor radii, const at::Tensor means2d,
        const at::Tensor depths, const at::Tensor compensations, const at::Tensor v_render_colors,
        const at::Tensor v_render_alphas);

} // namespace gsplat

// include/kernels/ssim.cuh:11-28
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> fusedssim(float C1, float C2, at::Tensor& img1,
                                                                     at::Tensor& img2, bool train);
at::Tensor fusedssim_backward(float C1, float C2, at::Tensor& img1, at::Tensor& img2, at::Tensor& dL_dmap,
                              at::Tensor& dm_dmu1, at::Tensor& dm_dsigma1_sq, at::Tensor& dm_dsigma12);
// include/kernels/fused_ssim.cuh:117-122 without the autograd node: mean SSIM ("same" or "valid" crop)
at::Tensor fused_ssim_value(at::Tensor img1, at::Tensor img2, const std::string& padding);

// src/training/fastgs/optimizer/include/adam_api.h
namespace fast_gs::optimizer {
    void adam_step_wrapper(at::Tensor& param, at::Tensor& exp_avg, at::Tensor& exp_avg_sq, const at::Tensor& param_grad,
                           const float lr, const float beta1, const float beta2, const float eps,
                           const float bias_correction1_rcp, const float bias_correction2_sqrt_rcp);
}
