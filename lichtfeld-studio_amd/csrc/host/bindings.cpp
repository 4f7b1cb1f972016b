// Python module over the C++ host layer (gsplat_api.h) so that the same tests that drive the ctypes binding can
// drive the functions a LichtFeld build would link.  Names and argument order are those of gsplat/Ops.h.
#include <torch/extension.h>

#include "fastgs_api.h"
#include "gsplat_api.h"

namespace py = pybind11;

PYBIND11_MODULE(gsx_torch_ext, m) {
    py::enum_<ShutterType>(m, "ShutterType")
        .value("ROLLING_TOP_TO_BOTTOM", ShutterType::ROLLING_TOP_TO_BOTTOM)
        .value("ROLLING_LEFT_TO_RIGHT", ShutterType::ROLLING_LEFT_TO_RIGHT)
        .value("ROLLING_BOTTOM_TO_TOP", ShutterType::ROLLING_BOTTOM_TO_TOP)
        .value("ROLLING_RIGHT_TO_LEFT", ShutterType::ROLLING_RIGHT_TO_LEFT)
        .value("GLOBAL", ShutterType::GLOBAL);
    py::enum_<gsplat::CameraModelType>(m, "CameraModelType")
        .value("PINHOLE", gsplat::PINHOLE)
        .value("ORTHO", gsplat::ORTHO)
        .value("FISHEYE", gsplat::FISHEYE)
        .value("EQUIRECTANGULAR", gsplat::EQUIRECTANGULAR);
    py::class_<UnscentedTransformParameters>(m, "UnscentedTransformParameters")
        .def(py::init<>())
        .def_readwrite("alpha", &UnscentedTransformParameters::alpha)
        .def_readwrite("beta", &UnscentedTransformParameters::beta)
        .def_readwrite("kappa", &UnscentedTransformParameters::kappa)
        .def_readwrite("in_image_margin_factor", &UnscentedTransformParameters::in_image_margin_factor)
        .def_readwrite("require_all_sigma_points_valid", &UnscentedTransformParameters::require_all_sigma_points_valid);

    m.def("spherical_harmonics_fwd", &gsplat::spherical_harmonics_fwd);
    m.def("spherical_harmonics_bwd", &gsplat::spherical_harmonics_bwd);
    m.def("intersect_tile", &gsplat::intersect_tile);
    m.def("intersect_offset", &gsplat::intersect_offset);
    m.def("quats_to_rotmats", &gsplat::quats_to_rotmats);
    m.def("relocation", &gsplat::relocation);
    m.def("add_noise", &gsplat::add_noise);
    m.def("projection_ut_3dgs_fused", &gsplat::projection_ut_3dgs_fused);
    m.def("rasterize_to_pixels_from_world_3dgs_fwd", &gsplat::rasterize_to_pixels_from_world_3dgs_fwd);
    m.def("rasterize_to_pixels_from_world_3dgs_bwd", &gsplat::rasterize_to_pixels_from_world_3dgs_bwd);
    m.def("rasterize_from_world_with_sh_fwd", &gsplat::rasterize_from_world_with_sh_fwd);
    m.def("rasterize_from_world_with_sh_bwd", &gsplat::rasterize_from_world_with_sh_bwd);
    m.def("fusedssim", [](float C1, float C2, at::Tensor img1, at::Tensor img2, bool train) {
        return fusedssim(C1, C2, img1, img2, train);
    });
    m.def("fusedssim_backward", [](float C1, float C2, at::Tensor img1, at::Tensor img2, at::Tensor dL_dmap,
                                   at::Tensor dm_dmu1, at::Tensor dm_dsigma1_sq, at::Tensor dm_dsigma12) {
        return fusedssim_backward(C1, C2, img1, img2, dL_dmap, dm_dmu1, dm_dsigma1_sq, dm_dsigma12);
    });
    m.def("fused_ssim_value", &fused_ssim_value);
    m.def("adam_step_wrapper", [](at::Tensor param, at::Tensor exp_avg, at::Tensor exp_avg_sq, at::Tensor param_grad,
                                  float lr, float beta1, float beta2, float eps, float bc1_rcp, float bc2_sqrt_rcp) {
        fast_gs::optimizer::adam_step_wrapper(param, exp_avg, exp_avg_sq, param_grad, lr, beta1, beta2, eps, bc1_rcp,
                                              bc2_sqrt_rcp);
    });
    m.def("fastgs_forward_wrapper", &fast_gs::rasterization::forward_wrapper);
    m.def("fastgs_backward_wrapper", &fast_gs::rasterization::backward_wrapper);
}
