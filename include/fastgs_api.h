// fastgs_api.h - the C++ host interface of the fastgs backend with the names, namespace, argument order and return
// tuples of LichtFeld-Studio's src/training/fastgs/rasterization/include/rasterization_api.h:12-75, implemented in
// lichtfeld-studio_amd/csrc/host/fastgs_api.cpp on top of the C ABI of gsx_fastgs.h.  A LichtFeld build keeps its own
// header; this one exists so that the implementation can be compiled and tested without the reference tree.
#pragma once

#include <ATen/core/Tensor.h>

#include <tuple>

namespace fast_gs::rasterization {

    // rasterization_api.h:12-23: the camera and image parameters of one view, as LichtFeld's fast_rasterize gathers
    // them before it spreads them over the wrappers' arguments (fast_rasterizer.cpp:35-45, fast_rasterizer_autograd.cpp:19)
    struct FastGSSettings {
        at::Tensor cam_position;
        int active_sh_bases;
        int width;
        int height;
        float focal_x;
        float focal_y;
        float center_x;
        float center_y;
        float near_plane;
        float far_plane;
    };

    // (image [3,H,W], alpha [1,H,W], per_primitive_buffers, per_tile_buffers, per_instance_buffers,
    //  per_bucket_buffers, n_visible_primitives, n_instances, n_buckets, primitive selector, instance selector).
    // The four byte tensors are this library's state (per_tile holds the per-pixel state; per_bucket is empty: no
    // checkpoints are stored); n_visible_primitives is -1, n_buckets and the selectors are 0.  A caller only hands
    // them back to backward_wrapper, as FastGSRasterize does (fast_rasterizer_autograd.cpp:44-91).
    std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, int, int, int, int, int>
    forward_wrapper(const at::Tensor& means, const at::Tensor& scales_raw, const at::Tensor& rotations_raw,
                    const at::Tensor& opacities_raw, const at::Tensor& sh_coefficients_0,
                    const at::Tensor& sh_coefficients_rest, const at::Tensor& w2c, const at::Tensor& cam_position,
                    const int active_sh_bases, const int width, const int height, const float focal_x,
                    const float focal_y, const float center_x, const float center_y, const float near_plane,
                    const float far_plane);

    // (grad_means, grad_scales_raw, grad_rotations_raw, grad_opacities_raw [N,1], grad_sh_coefficients_0 [N,1,3],
    //  grad_sh_coefficients_rest [N,B,3], grad_w2c (undefined unless w2c.requires_grad()))
    std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor>
    backward_wrapper(at::Tensor& densification_info, const at::Tensor& grad_image, const at::Tensor& grad_alpha,
                     const at::Tensor& image, const at::Tensor& alpha, const at::Tensor& means,
                     const at::Tensor& scales_raw, const at::Tensor& rotations_raw,
                     const at::Tensor& sh_coefficients_rest, const at::Tensor& per_primitive_buffers,
                     const at::Tensor& per_tile_buffers, const at::Tensor& per_instance_buffers,
                     const at::Tensor& per_bucket_buffers, const at::Tensor& w2c, const at::Tensor& cam_position,
                     const int active_sh_bases, const int width, const int height, const float focal_x,
                     const float focal_y, const float center_x, const float center_y, const float near_plane,
                     const float far_plane, const int n_visible_primitives, const int n_instances, const int n_buckets,
                     const int primitive_primitive_indices_selector, const int instance_primitive_indices_selector);

} // namespace fast_gs::rasterization
