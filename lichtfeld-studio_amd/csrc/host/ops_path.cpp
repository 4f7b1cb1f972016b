// ops_path.cpp - one training iteration issued operator by operator, the way LichtFeld-Studio's trainer issues it
// (src/training/trainer.cpp:599-875): ATen activations, the autograd Function around
// gsplat::rasterize_from_world_with_sh_fwd / _bwd, clamp / permute, torch::l1_loss + fused_ssim, loss.backward(),
// one adam_step_wrapper launch per parameter group, zero_grad(set_to_none).  Everything behind gsplat_api.h is this
// library; everything in this file is LibTorch, used as the reference uses it.
#include "gsx_training.h"

#include <cmath>

namespace gsx::training {

    using torch::indexing::None;
    using torch::indexing::Slice;

    // src/core/splat_data.cpp:270-286
    torch::Tensor SplatData::get_opacity() const { return torch::sigmoid(opacity_raw).squeeze(-1); }
    torch::Tensor SplatData::get_rotation() const {
        return torch::nn::functional::normalize(rotation_raw, torch::nn::functional::NormalizeFuncOptions().dim(-1));
    }
    torch::Tensor SplatData::get_scaling() const { return torch::exp(scaling_raw); }
    torch::Tensor SplatData::get_shs() const { return torch::cat({sh0, shN}, 1); }

    namespace {

        // rasterizer_autograd.cpp:10-227
        class FusedRasterizationWithSHFunction : public torch::autograd::Function<FusedRasterizationWithSHFunction> {
        public:
            static torch::autograd::tensor_list forward(torch::autograd::AutogradContext* ctx, torch::Tensor means,
                                                        torch::Tensor quats, torch::Tensor scales,
                                                        torch::Tensor opacities, torch::Tensor sh_coeffs, int sh_degree,
                                                        torch::Tensor bg_color, torch::Tensor viewmat, torch::Tensor K,
                                                        FusedRasterizationSettings settings) {
                std::optional<torch::Tensor> bg_opt;
                if (bg_color.defined() && bg_color.numel() > 0)
                    bg_opt = bg_color.view({1, -1}).contiguous();
                const UnscentedTransformParameters ut_params{};
                auto results = gsplat::rasterize_from_world_with_sh_fwd(
                    means.contiguous(), quats.contiguous(), scales.contiguous(), opacities.contiguous(),
                    sh_coeffs.contiguous(), static_cast<uint32_t>(sh_degree), bg_opt, std::nullopt, settings.width,
                    settings.height, settings.tile_size, viewmat.contiguous(), std::nullopt, K.contiguous(),
                    settings.camera_model, settings.eps2d, settings.near_plane, settings.far_plane,
                    settings.radius_clip, settings.scaling_modifier, settings.calc_compensations, settings.render_mode,
                    ut_params, ShutterType::GLOBAL, std::nullopt, std::nullopt, std::nullopt);
                auto render_colors = std::get<0>(results).contiguous();
                auto render_alphas = std::get<1>(results).contiguous();
                auto radii = std::get<2>(results).contiguous();
                auto means2d = std::get<3>(results).contiguous();
                auto depths = std::get<4>(results).contiguous();
                auto colors = std::get<5>(results).contiguous();
                auto tile_offsets = std::get<6>(results).contiguous();
                auto flatten_ids = std::get<7>(results).contiguous();
                auto last_ids = std::get<8>(results).contiguous();
                auto compensations = std::get<9>(results);
                ctx->save_for_backward({means, quats, scales, opacities, sh_coeffs, bg_color, viewmat, K, render_alphas,
                                        radii, means2d, depths, colors, tile_offsets, flatten_ids, last_ids,
                                        compensations});
                ctx->saved_data["sh_degree"] = sh_degree;
                ctx->saved_data["width"] = settings.width;
                ctx->saved_data["height"] = settings.height;
                ctx->saved_data["tile_size"] = settings.tile_size;
                ctx->saved_data["eps2d"] = (double)settings.eps2d;
                ctx->saved_data["near_plane"] = (double)settings.near_plane;
                ctx->saved_data["far_plane"] = (double)settings.far_plane;
                ctx->saved_data["radius_clip"] = (double)settings.radius_clip;
                ctx->saved_data["scaling_modifier"] = (double)settings.scaling_modifier;
                ctx->saved_data["calc_compensations"] = settings.calc_compensations;
                ctx->saved_data["camera_model"] = static_cast<int>(settings.camera_model);
                ctx->saved_data["render_mode"] = settings.render_mode;
                return {render_colors, render_alphas, radii, means2d, depths};
            }

            static torch::autograd::tensor_list backward(torch::autograd::AutogradContext* ctx,
                                                         torch::autograd::tensor_list grad_outputs) {
                auto v_render_colors = grad_outputs[0].contiguous();
                auto v_render_alphas = grad_outputs[1].contiguous();
                auto saved = ctx->get_saved_variables();
                const auto& bg_color = saved[5];
                std::optional<torch::Tensor> bg_opt;
                if (bg_color.defined() && bg_color.numel() > 0)
                    bg_opt = bg_color.view({1, -1});
                const UnscentedTransformParameters ut_params{};
                auto grads = gsplat::rasterize_from_world_with_sh_bwd(
                    saved[0], saved[1], saved[2], saved[3], saved[4],
                    static_cast<uint32_t>(ctx->saved_data["sh_degree"].toInt()), bg_opt, std::nullopt,
                    (uint32_t)ctx->saved_data["width"].toInt(), (uint32_t)ctx->saved_data["height"].toInt(),
                    (uint32_t)ctx->saved_data["tile_size"].toInt(), saved[6], std::nullopt, saved[7],
                    static_cast<gsplat::CameraModelType>(ctx->saved_data["camera_model"].toInt()),
                    (float)ctx->saved_data["eps2d"].toDouble(), (float)ctx->saved_data["near_plane"].toDouble(),
                    (float)ctx->saved_data["far_plane"].toDouble(), (float)ctx->saved_data["radius_clip"].toDouble(),
                    (float)ctx->saved_data["scaling_modifier"].toDouble(), ctx->saved_data["calc_compensations"].toBool(),
                    (int)ctx->saved_data["render_mode"].toInt(), ut_params, ShutterType::GLOBAL, std::nullopt,
                    std::nullopt, std::nullopt, saved[8], saved[15], saved[13], saved[14], saved[12], saved[9],
                    saved[10], saved[11], saved[16], v_render_colors, v_render_alphas);
                auto v_bg_color = torch::Tensor();
                if (ctx->needs_input_grad(6))
                    v_bg_color = (v_render_colors * (1.0f - saved[8])).toType(torch::kFloat32).sum({-3, -2});
                return {std::get<0>(grads), std::get<1>(grads), std::get<2>(grads), std::get<3>(grads),
                        std::get<4>(grads), torch::Tensor(), v_bg_color, torch::Tensor(), torch::Tensor(),
                        torch::Tensor()};
            }
        };

        // fused_ssim.cuh:22-107
        class FusedSSIMFunction : public torch::autograd::Function<FusedSSIMFunction> {
        public:
            static torch::Tensor forward(torch::autograd::AutogradContext* ctx, torch::Tensor img1, torch::Tensor img2,
                                         const std::string& padding, bool train) {
                TORCH_CHECK(padding == "same" || padding == "valid",
                            "fused_ssim: padding must be \"same\" or \"valid\" (got \"", padding, "\")");
                img1 = img1.contiguous();
                img2 = img2.contiguous();
                if (img1.dim() == 3)
                    img1 = img1.unsqueeze(0);
                if (img2.dim() == 3)
                    img2 = img2.unsqueeze(0);
                TORCH_CHECK(img1.dim() == 4 && img2.dim() == 4, "fused_ssim expects 4D tensors [N,C,H,W], got img1: ",
                            img1.dim(), "D, img2: ", img2.dim(), "D");
                TORCH_CHECK(img1.sizes() == img2.sizes(), "img1 and img2 must have the same shape");
                auto out = fusedssim(0.01f * 0.01f, 0.03f * 0.03f, img1, img2, train);
                auto map = std::get<0>(out);
                if (padding == "valid") {
                    const int64_t h = map.size(2), w = map.size(3);
                    if (h > 10 && w > 10)
                        map = map.index({Slice(), Slice(), Slice(5, h - 5), Slice(5, w - 5)});
                }
                ctx->save_for_backward({img1.detach(), img2, std::get<1>(out), std::get<2>(out), std::get<3>(out)});
                ctx->saved_data["padding"] = padding;
                return map;
            }

            static std::vector<torch::Tensor> backward(torch::autograd::AutogradContext* ctx,
                                                       std::vector<torch::Tensor> grad_out) {
                auto vars = ctx->get_saved_variables();
                auto img1 = vars[0], img2 = vars[1], dm1 = vars[2], ds1sq = vars[3], ds12 = vars[4];
                auto dL_dmap = grad_out[0];
                if (ctx->saved_data["padding"].toStringRef() == "valid") {
                    auto full = torch::zeros_like(img1);
                    const int64_t h = full.size(2), w = full.size(3);
                    if (h > 10 && w > 10)
                        full.index_put_({Slice(), Slice(), Slice(5, h - 5), Slice(5, w - 5)}, dL_dmap);
                    dL_dmap = full;
                }
                auto grad_img1 = fusedssim_backward(0.01f * 0.01f, 0.03f * 0.03f, img1, img2, dL_dmap, dm1, ds1sq, ds12);
                return {grad_img1, torch::Tensor(), torch::Tensor(), torch::Tensor()};
            }
        };

    }  // namespace

    torch::Tensor fused_ssim(torch::Tensor img1, torch::Tensor img2, const std::string& padding, bool train) {
        img1 = img1.contiguous();
        return FusedSSIMFunction::apply(img1, img2, padding, train).mean();
    }

    RenderOutput rasterize(const torch::Tensor& viewmat, const torch::Tensor& K, int image_width, int image_height,
                           const SplatData& model, const torch::Tensor& bg_color, float scaling_modifier,
                           bool antialiased, int render_mode, gsplat::CameraModelType camera_model) {
        TORCH_CHECK(viewmat.dim() == 3 && viewmat.size(0) == 1 && viewmat.size(1) == 4 && viewmat.size(2) == 4,
                    "viewmat must be [1, 4, 4], got ", viewmat.sizes());
        TORCH_CHECK(viewmat.is_cuda() && K.is_cuda(), "viewmat and K must be on the GPU");
        auto means3D = model.get_means();
        auto opacities = model.get_opacity();
        if (opacities.dim() == 2 && opacities.size(1) == 1)
            opacities = opacities.squeeze(-1);
        auto scales = model.get_scaling();
        auto rotations = model.get_rotation();
        auto sh_coeffs = model.get_shs();
        const int sh_degree = model.active_sh_degree;
        const int64_t N = means3D.size(0);
        TORCH_CHECK(means3D.dim() == 2 && means3D.size(1) == 3, "means3D must be [N, 3], got ", means3D.sizes());
        TORCH_CHECK(opacities.dim() == 1 && opacities.size(0) == N, "opacities must be [N], got ", opacities.sizes());
        TORCH_CHECK(scales.dim() == 2 && scales.size(0) == N && scales.size(1) == 3, "scales must be [N, 3]");
        TORCH_CHECK(rotations.dim() == 2 && rotations.size(0) == N && rotations.size(1) == 4, "rotations must be [N, 4]");
        TORCH_CHECK(sh_coeffs.dim() == 3 && sh_coeffs.size(0) == N && sh_coeffs.size(2) == 3,
                    "sh_coeffs must be [N, K, 3], got ", sh_coeffs.sizes());
        const int required = (sh_degree + 1) * (sh_degree + 1);
        TORCH_CHECK(sh_coeffs.size(1) >= required, "Not enough SH coefficients. Expected at least ", required,
                    " but got ", sh_coeffs.size(1));
        torch::Tensor prepared_bg;
        if (bg_color.defined() && bg_color.numel() > 0) {
            prepared_bg = bg_color.view({1, -1});
            TORCH_CHECK(prepared_bg.size(1) == 3, "bg_color must be reshapeable to [1, 3], got ", prepared_bg.sizes());
        }
        const FusedRasterizationSettings settings{image_width, image_height, 16, 0.3f, 0.01f, 10000.0f, 0.0f,
                                                  scaling_modifier, antialiased, camera_model, render_mode};
        auto outs = FusedRasterizationWithSHFunction::apply(
            means3D, rotations, scales, opacities, sh_coeffs, sh_degree,
            prepared_bg.defined() ? prepared_bg : torch::zeros({3}, means3D.options()), viewmat, K, settings);
        auto rendered_image = outs[0], rendered_alpha = outs[1], radii = outs[2];
        auto means2d_with_grad = outs[3].contiguous();
        torch::Tensor final_image, final_depth;
        switch (render_mode) {  // rasterizer.cpp:172-200
        case 0: final_image = rendered_image; break;
        case 1: final_depth = rendered_image; break;
        case 2: final_depth = rendered_image / rendered_alpha.clamp_min(1e-10); break;
        case 3:
            final_image = rendered_image.index({Slice(), Slice(), Slice(), Slice(None, -1)});
            final_depth = rendered_image.index({Slice(), Slice(), Slice(), Slice(-1, None)});
            break;
        default:
            final_image = rendered_image.index({Slice(), Slice(), Slice(), Slice(None, -1)});
            final_depth = rendered_image.index({Slice(), Slice(), Slice(), Slice(-1, None)}) /
                          rendered_alpha.clamp_min(1e-10);
        }
        RenderOutput r;
        if (final_image.defined() && final_image.numel() > 0)
            r.image = torch::clamp(final_image.squeeze(0).permute({2, 0, 1}), 0.0f, 1.0f);
        r.alpha = rendered_alpha.squeeze(0).permute({2, 0, 1});
        if (final_depth.defined() && final_depth.numel() > 0)
            r.depth = final_depth.squeeze(0).permute({2, 0, 1});
        r.means2d = means2d_with_grad;
        r.depths = outs[4].squeeze(0);
        r.radii = std::get<0>(radii.squeeze(0).max(-1));
        r.visibility = (r.radii > 0);
        r.width = image_width;
        r.height = image_height;
        return r;
    }

    // fused_adam.cpp:22-95
    void FusedAdam::step(int iteration) {
        torch::NoGradGuard no_grad;
        int i = 0;
        for (auto& g : groups_) {
            ++i;
            if (!g.param.grad().defined())
                continue;
            if (!g.exp_avg.defined()) {
                g.exp_avg = torch::zeros_like(g.param, torch::MemoryFormat::Preserve);
                g.exp_avg_sq = torch::zeros_like(g.param, torch::MemoryFormat::Preserve);
            }
            g.step_count++;
            if (skip_shN_early && i == 3 && iteration <= 1000)
                continue;
            const double bc1_rcp = 1.0 / (1.0 - std::pow(g.beta1, (double)g.step_count));
            const double bc2_sqrt_rcp = 1.0 / std::sqrt(1.0 - std::pow(g.beta2, (double)g.step_count));
            fast_gs::optimizer::adam_step_wrapper(g.param, g.exp_avg, g.exp_avg_sq, g.param.grad(), (float)g.lr,
                                                  (float)g.beta1, (float)g.beta2, (float)g.eps, (float)bc1_rcp,
                                                  (float)bc2_sqrt_rcp);
        }
    }

    // fused_adam.cpp:98-122
    void FusedAdam::zero_grad(bool set_to_none) {
        for (auto& g : groups_) {
            if (!g.param.grad().defined())
                continue;
            if (set_to_none) {
                g.param.mutable_grad().reset();
            } else {
                g.param.mutable_grad().detach_();
                g.param.mutable_grad().zero_();
            }
        }
    }

    OpsPathTrainer::OpsPathTrainer(SplatData model, std::array<double, 6> lrs, float lambda_dssim,
                                   bool skip_shN_early)
        : model_(std::move(model)), lambda_dssim_(lambda_dssim) {
        // mcmc.cpp:487-492: means, sh0, shN, scaling, rotation, opacity
        torch::Tensor* params[6] = {&model_.means,       &model_.sh0,          &model_.shN,
                                    &model_.scaling_raw, &model_.rotation_raw, &model_.opacity_raw};
        std::vector<FusedAdam::Group> groups;
        for (int i = 0; i < 6; ++i) {
            params[i]->set_requires_grad(true);
            FusedAdam::Group g;
            g.param = *params[i];
            g.lr = lrs[i];
            groups.push_back(std::move(g));
        }
        optimizer_ = std::make_unique<FusedAdam>(std::move(groups));
        optimizer_->skip_shN_early = skip_shN_early;
        background_ = torch::zeros({3}, model_.means.options().requires_grad(false));  // trainer.cpp:383-384
    }

    torch::Tensor OpsPathTrainer::train_step(int iter, const torch::Tensor& viewmat, const torch::Tensor& K,
                                             int image_width, int image_height, const torch::Tensor& gt_image) {
        RenderOutput r = rasterize(viewmat, K, image_width, image_height, model_, background_);
        // trainer.cpp:107-134
        torch::Tensor rendered = r.image.dim() == 3 ? r.image.unsqueeze(0) : r.image;
        torch::Tensor gt = gt_image.dim() == 3 ? gt_image.unsqueeze(0) : gt_image;
        TORCH_CHECK(rendered.sizes() == gt.sizes(), "ERROR: size mismatch - rendered ", rendered.sizes(),
                    " vs. ground truth ", gt.sizes());
        auto l1_loss = torch::l1_loss(rendered, gt);
        auto ssim_loss = 1.f - fused_ssim(rendered, gt, "valid", /*train=*/true);
        torch::Tensor loss = (1.f - lambda_dssim_) * l1_loss + lambda_dssim_ * ssim_loss;
        loss.backward();
        {
            torch::NoGradGuard no_grad;
            optimizer_->step(iter);  // mcmc.cpp:410-417
            optimizer_->zero_grad(true);
        }
        return loss.detach();
    }

}  // namespace gsx::training
