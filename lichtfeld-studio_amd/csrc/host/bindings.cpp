// Python module over the C++ host layer (gsplat_api.h) so that the same tests that drive the ctypes binding can
// drive the functions a LichtFeld build would link.  Names and argument order are those of gsplat/Ops.h.
#include <torch/extension.h>

#include "fastgs_api.h"
#include "gsplat_api.h"
#include "gsx_training.h"

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
    // the step as LichtFeld's trainer issues it (ops_path.cpp)
    namespace gt = gsx::training;
    py::class_<gt::OpsPathTrainer>(m, "OpsPathTrainer")
        .def(py::init([](at::Tensor means, at::Tensor sh0, at::Tensor shN, at::Tensor scaling_raw,
                         at::Tensor rotation_raw, at::Tensor opacity_raw, int active_sh_degree,
                         std::array<double, 6> lrs, float lambda_dssim, bool skip_shN_early) {
            gt::SplatData d{means, sh0, shN, scaling_raw, rotation_raw, opacity_raw, active_sh_degree};
            return std::make_unique<gt::OpsPathTrainer>(std::move(d), lrs, lambda_dssim, skip_shN_early);
        }))
        .def("train_step", &gt::OpsPathTrainer::train_step, py::call_guard<py::gil_scoped_release>())
        .def("parameters", [](gt::OpsPathTrainer& t) {
            auto& d = t.model();
            return std::vector<at::Tensor>{d.means, d.sh0, d.shN, d.scaling_raw, d.rotation_raw, d.opacity_raw};
        })
        .def("moments", [](gt::OpsPathTrainer& t) {
            std::vector<std::pair<at::Tensor, at::Tensor>> out;
            for (auto& g : t.optimizer().groups())
                out.emplace_back(g.exp_avg, g.exp_avg_sq);
            return out;
        });
    // the step over the fused entry points (train_step.cpp)
    py::class_<gsx::TrainStep>(m, "TrainStep")
        .def(py::init([](at::Tensor means, at::Tensor shs, at::Tensor scaling_raw, at::Tensor rotation_raw,
                         at::Tensor opacity_raw, std::array<double, 6> lrs, float lambda_dssim, int sh_degree,
                         bool freeze_shN_early, bool overlap, bool order_tiles, float scale_reg, float opacity_reg,
                         int64_t initial_pair_capacity) {
                 gsx::TrainStep::Options o;
                 o.lrs = lrs, o.lambda_dssim = lambda_dssim, o.sh_degree = sh_degree;
                 o.freeze_shN_early = freeze_shN_early, o.overlap = overlap, o.order_tiles = order_tiles;
                 o.scale_reg = scale_reg, o.opacity_reg = opacity_reg;
                 o.initial_pair_capacity = initial_pair_capacity;
                 return std::make_unique<gsx::TrainStep>(means, shs, scaling_raw, rotation_raw, opacity_raw, o);
             }),
             py::arg("means"), py::arg("shs"), py::arg("scaling_raw"), py::arg("rotation_raw"), py::arg("opacity_raw"),
             py::arg("lrs"), py::arg("lambda_dssim") = 0.2f, py::arg("sh_degree") = 3,
             py::arg("freeze_shN_early") = false, py::arg("overlap") = true, py::arg("order_tiles") = true,
             py::arg("scale_reg") = 0.f, py::arg("opacity_reg") = 0.f, py::arg("initial_pair_capacity") = 0)
        .def("step", &gsx::TrainStep::step, py::call_guard<py::gil_scoped_release>())
        .def("steps", [](gsx::TrainStep& t, std::vector<at::Tensor> viewmats, at::Tensor K, int W, int H, at::Tensor gt,
                         int n) {
            // n steps back to back without returning to the interpreter: viewmats are taken in turn
            py::gil_scoped_release release;
            at::Tensor loss;
            for (int i = 0; i < n; ++i)
                loss = t.step(viewmats[i % viewmats.size()], K, W, H, gt);
            return loss;
        })
        .def_readonly("means", &gsx::TrainStep::means)
        .def_readonly("shs", &gsx::TrainStep::shs)
        .def_readonly("scaling_raw", &gsx::TrainStep::scaling_raw)
        .def_readonly("rotation_raw", &gsx::TrainStep::rotation_raw)
        .def_readonly("opacity_raw", &gsx::TrainStep::opacity_raw)
        .def_property_readonly("exp_avg", [](gsx::TrainStep& t) {
            return std::vector<at::Tensor>(t.exp_avg.begin(), t.exp_avg.end());
        })
        .def_property_readonly("exp_avg_sq", [](gsx::TrainStep& t) {
            return std::vector<at::Tensor>(t.exp_avg_sq.begin(), t.exp_avg_sq.end());
        })
        .def_readonly("render", &gsx::TrainStep::render)
        .def_readonly("alpha", &gsx::TrainStep::alpha)
        .def_readonly("last_ids", &gsx::TrainStep::last_ids)
        .def_readonly("loss_out", &gsx::TrainStep::loss_out)
        .def_readonly("iteration", &gsx::TrainStep::iteration)
        .def_readonly("step_count", &gsx::TrainStep::step_count)
        .def_readonly("steps_held", &gsx::TrainStep::steps_held)
        .def("pair_capacity", &gsx::TrainStep::pair_capacity)
        .def("n_isects", &gsx::TrainStep::n_isects)
        .def("lists_error", &gsx::TrainStep::lists_error)
        .def("clear_lists_error", &gsx::TrainStep::clear_lists_error)
        .def("debug_set_lists_error", &gsx::TrainStep::debug_set_lists_error);
    m.def("fastgs_forward_wrapper", &fast_gs::rasterization::forward_wrapper);
    m.def("fastgs_backward_wrapper", &fast_gs::rasterization::backward_wrapper);
}
