// gsx_training.h - the two C++ drivers of one training iteration over the gfx950 kernels.
//
// (1) gsx::training::* - the callers of gsplat/Ops.h as LichtFeld-Studio's trainer has them, restated over
//     gsplat_api.h so that the step can be issued, timed and tested the way a LichtFeld build issues it:
//       SplatData getters                    src/core/splat_data.cpp:266-286
//       FusedRasterizationWithSHFunction     src/training/rasterization/rasterizer_autograd.cpp:10-227
//       rasterize()                          src/training/rasterization/rasterizer.cpp:15-232
//       fused_ssim() / _FusedSSIM            include/kernels/fused_ssim.cuh:16-122
//       photometric loss                     src/training/trainer.cpp:107-134
//       FusedAdam::step / zero_grad          src/training/optimizers/fused_adam.cpp:22-122
//       the iteration                        src/training/trainer.cpp:599-875, strategies/mcmc.cpp:410-417
//     Autograd, the ATen activations / concatenation / clamp / permute / loss ops and one Adam launch per group are
//     all there; only what sits behind Ops.h, fusedssim and adam_step_wrapper is this library.
//
// (2) gsx::TrainStep - the same iteration over the fused entry points of gsx.h (gsx_activate_project_ut,
//     gsx_sh_colors_records_from_world, gsx_tile_lists, gsx_rasterize_records_fwd, gsx_photometric_loss_*,
//     gsx_rasterize_bwd_accumulate, gsx_backward_update_fused): no autograd graph, no per-step allocation, no host
//     wait; sh0 | shN in one [N,K,3] tensor.  What a trainer switches to when it gives up the operator-by-operator
//     sequence; same parameters and moments after a step (to the gradient tolerance of the backward rasterizer).
#pragma once

#include <torch/torch.h>

#include <array>
#include <memory>
#include <optional>
#include <vector>

#include "gsplat_api.h"

namespace gsx::training {

    // include/core/splat_data.hpp:68-79 (raw trainable tensors) with the computed getters of splat_data.cpp:266-286
    struct SplatData {
        torch::Tensor means, sh0, shN, scaling_raw, rotation_raw, opacity_raw;  // [N,3] [N,1,3] [N,K-1,3] [N,3] [N,4] [N,1]
        int active_sh_degree = 0;
        torch::Tensor get_means() const { return means; }
        torch::Tensor get_opacity() const;
        torch::Tensor get_rotation() const;
        torch::Tensor get_scaling() const;
        torch::Tensor get_shs() const;
        int64_t size() const { return means.size(0); }
    };

    // rasterizer.hpp: what rasterize() returns
    struct RenderOutput {
        torch::Tensor image, alpha, depth, means2d, depths, radii, visibility;
        int width = 0, height = 0;
    };

    // rasterizer_autograd.hpp
    struct FusedRasterizationSettings {
        int width, height, tile_size;
        float eps2d, near_plane, far_plane, radius_clip, scaling_modifier;
        bool calc_compensations;
        gsplat::CameraModelType camera_model;
        int render_mode;
    };

    // rasterizer.cpp:15-232; viewmat [1,4,4], K [1,3,3]; bg_color [3] or undefined
    RenderOutput rasterize(const torch::Tensor& viewmat, const torch::Tensor& K, int image_width, int image_height,
                           const SplatData& model, const torch::Tensor& bg_color, float scaling_modifier = 1.0f,
                           bool antialiased = false, int render_mode = 0,
                           gsplat::CameraModelType camera_model = gsplat::PINHOLE);

    // fused_ssim.cuh:117-122
    torch::Tensor fused_ssim(torch::Tensor img1, torch::Tensor img2, const std::string& padding = "same",
                             bool train = true);

    // fused_adam.hpp / fused_adam.cpp:22-122: one group per tensor, lazily created state, one kernel launch per group
    class FusedAdam {
    public:
        struct Group {
            torch::Tensor param;
            double lr, beta1 = 0.9, beta2 = 0.999, eps = 1e-15;
            torch::Tensor exp_avg, exp_avg_sq;
            int64_t step_count = 0;
        };
        explicit FusedAdam(std::vector<Group> groups) : groups_(std::move(groups)) {}
        void step(int iteration);
        void zero_grad(bool set_to_none);
        std::vector<Group>& groups() { return groups_; }
        bool skip_shN_early = true;  // fused_adam.cpp:69-70; BASELINE's step updates every tensor: set false there

    private:
        std::vector<Group> groups_;
    };

    // Trainer::train_step for the --gut backend without bilateral grid, pose optimisation or sparsity
    // (trainer.cpp:599-875) + MCMC::step (mcmc.cpp:410-417).  The loss stays on the device (the reference's
    // loss.item() of trainer.cpp:708 is the caller's choice here).
    class OpsPathTrainer {
    public:
        OpsPathTrainer(SplatData model, std::array<double, 6> lrs, float lambda_dssim, bool skip_shN_early);
        torch::Tensor train_step(int iter, const torch::Tensor& viewmat, const torch::Tensor& K, int image_width,
                                 int image_height, const torch::Tensor& gt_image);
        SplatData& model() { return model_; }
        FusedAdam& optimizer() { return *optimizer_; }

    private:
        SplatData model_;
        std::unique_ptr<FusedAdam> optimizer_;
        torch::Tensor background_;
        float lambda_dssim_;
    };

}  // namespace gsx::training

namespace gsx {

    // One training iteration over the fused entry points of gsx.h - what Trainer::train_step (trainer.cpp:599-875)
    // + MCMC::step (mcmc.cpp:410-417) + FusedAdam::step (fused_adam.cpp:22-95) do for the --gut backend, as 17 kernel
    // launches on two streams with every buffer allocated once and no host wait inside a step.  The caller keeps
    // the tensors (they are updated in place); `shs` holds sh0 | shN as one [N,K,3] tensor - sh0() / shN() are the
    // views a SplatData keeps instead of its two tensors.
    class TrainStep {
    public:
        struct Options {
            // mcmc.cpp:487-492: means, sh0, shN, scaling, rotation, opacity (include/core/parameters.hpp:19-23)
            std::array<double, 6> lrs{1.6e-4, 2.5e-3, 2.5e-3 / 20.0, 5e-3, 1e-3, 5e-2};
            double beta1 = 0.9, beta2 = 0.999, eps = 1e-15;
            float lambda_dssim = 0.2f;             // parameters.hpp:24
            float scale_reg = 0.f, opacity_reg = 0.f;  // trainer.cpp:136-174; 0 = off
            int sh_degree = 3;                     // active degree
            bool freeze_shN_early = false;         // fused_adam.cpp:69-70 (true: the product's schedule)
            bool overlap = true;                   // SH / record pass, tile table and list-length tile order on a second stream
            bool order_tiles = true;               // rasterize the dearest tiles first
            int64_t initial_pair_capacity = 0;     // room for (Gaussian, tile) pairs before the first count; 0 = auto
        };
        TrainStep(torch::Tensor means, torch::Tensor shs, torch::Tensor scaling_raw, torch::Tensor rotation_raw,
                  torch::Tensor opacity_raw, Options options);
        ~TrainStep();
        TrainStep(const TrainStep&) = delete;
        TrainStep& operator=(const TrainStep&) = delete;

        // viewmat [1,4,4], K [1,3,3], gt_chw [1,3,H,W] or [3,H,W]; returns the device tensor [3] = (loss, L1, SSIM)
        // that the step's last loss kernel writes.  Throws c10::Error when a tile-list pass reported a failed wait.
        torch::Tensor step(const torch::Tensor& viewmat, const torch::Tensor& K, int image_width, int image_height,
                           const torch::Tensor& gt_chw);

        torch::Tensor means, shs, scaling_raw, rotation_raw, opacity_raw;  // parameters (updated in place)
        std::array<torch::Tensor, 5> exp_avg, exp_avg_sq;                 // same order as above
        torch::Tensor sh0() const { return shs.narrow(1, 0, 1); }
        torch::Tensor shN() const { return shs.narrow(1, 1, shs.size(1) - 1); }
        torch::Tensor render, alpha, last_ids, loss_out;                  // of the last step
        int64_t iteration = 0, step_count = 0, steps_held = 0;
        int64_t pair_capacity() const { return cap_; }
        // the last pair count that has reached the host (synchronise first for the last step's)
        int64_t n_isects() const;
        // (error bits, optimiser calls held back) of the tile lists; synchronises
        std::pair<uint32_t, uint32_t> lists_error();
        void clear_lists_error();
        // test hook: overwrite the device's sticky error word (what a failed look-back would leave there)
        void debug_set_lists_error(uint32_t bits);

    private:
        struct Impl;
        std::unique_ptr<Impl> impl_;
        Options opt_;
        int64_t cap_ = 0;
        void forward(const torch::Tensor& viewmat, const torch::Tensor& K, int W, int H);
        void ensure_image(int H, int W);
        void ensure_lists();
        void check_capacity();
    };

}  // namespace gsx
