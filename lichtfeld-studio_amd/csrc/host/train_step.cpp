// train_step.cpp - gsx::TrainStep: one training iteration of the --gut backend (Trainer::train_step,
// src/training/trainer.cpp:599-875; MCMC::step, strategies/mcmc.cpp:410-417; FusedAdam::step,
// optimizers/fused_adam.cpp:22-95) driven from C++ over the fused entry points of gsx.h.  LibTorch provides the
// tensors, the current stream and a second stream; every kernel is this library's.  Launch order per step:
//   activations + UT projection | SH colours + raster records (second stream) | tile lists (9 launches) |
//   tile order | rasterize forward | photometric loss forward |
//   photometric loss backward (+ loss value, + tile order by cost) | rasterize backward |
//   epilogue + SH backward + activation VJPs + Adam
#include "gsx_training.h"

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cmath>

#include "gsx.h"

namespace gsx {

    namespace {
        inline void ok(int status) {
            TORCH_CHECK(status == GSX_OK, "gsx (", gsx_status_string(status), "): ", gsx_last_error());
        }
        inline void hip_ok(hipError_t e) { TORCH_CHECK(e == hipSuccess, "gsx: ", hipGetErrorString(e)); }
        inline float* f(const torch::Tensor& t) { return t.data_ptr<float>(); }
        inline int32_t* i32(const torch::Tensor& t) { return t.data_ptr<int32_t>(); }
        inline uint32_t* u32(const torch::Tensor& t) { return reinterpret_cast<uint32_t*>(t.data_ptr<int32_t>()); }
    }  // namespace

    struct TrainStep::Impl {
        c10::Device device{c10::kCUDA, 0};
        uint32_t N = 0, K = 0;
        int W = 0, H = 0;
        uint32_t tw = 0, th = 0;
        hipStream_t side = nullptr;
        hipEvent_t ev_fork = nullptr, ev_join = nullptr;
        // per Gaussian
        torch::Tensor opacities, scales, quats, radii, means2d, depths, colors, records, accum;
        // per image
        torch::Tensor offsets_full, tile_order, tile_walk, v_render, v_alpha, dm1, dm2, dm3, l1_partials, ssim_partials;
        // tile lists
        torch::Tensor lists_ws, flat_out, n_pinned, hold_pinned;
        uint32_t* lists_error = nullptr;  // device u32 [2] inside lists_ws
        bool cap_confirmed = false, have_walk = false, order_due = false;
        const void *walk_viewmat = nullptr, *walk_K = nullptr;
        int walk_W = 0, walk_H = 0;
        const float* gt = nullptr;
        const float *viewmat = nullptr, *Kmat = nullptr;
        torch::Tensor bg;

        hipStream_t main() const { return c10::hip::getCurrentHIPStream(device.index()).stream(); }
        volatile int64_t* n_slot() const { return n_pinned.data_ptr<int64_t>(); }
        volatile uint64_t* hold_slot() const { return reinterpret_cast<uint64_t*>(hold_pinned.data_ptr<int64_t>()); }
    };

    TrainStep::TrainStep(torch::Tensor means_, torch::Tensor shs_, torch::Tensor scaling_raw_,
                         torch::Tensor rotation_raw_, torch::Tensor opacity_raw_, Options options)
        : means(std::move(means_)), shs(std::move(shs_)), scaling_raw(std::move(scaling_raw_)),
          rotation_raw(std::move(rotation_raw_)), opacity_raw(std::move(opacity_raw_)), impl_(new Impl),
          opt_(options) {
        Impl& m = *impl_;
        const int64_t N = means.size(0);
        TORCH_CHECK(means.is_cuda() && means.dim() == 2 && means.size(1) == 3, "means must be a GPU tensor [N, 3]");
        TORCH_CHECK(shs.dim() == 3 && shs.size(0) == N && shs.size(2) == 3, "shs must be [N, K, 3], got ", shs.sizes());
        TORCH_CHECK(scaling_raw.dim() == 2 && scaling_raw.size(0) == N && scaling_raw.size(1) == 3,
                    "scaling_raw must be [N, 3]");
        TORCH_CHECK(rotation_raw.dim() == 2 && rotation_raw.size(0) == N && rotation_raw.size(1) == 4,
                    "rotation_raw must be [N, 4]");
        TORCH_CHECK(opacity_raw.numel() == N, "opacity_raw must hold N values, got ", opacity_raw.sizes());
        const int need = (opt_.sh_degree + 1) * (opt_.sh_degree + 1);
        TORCH_CHECK(shs.size(1) >= need, "Not enough SH coefficients. Expected at least ", need, " but got ",
                    shs.size(1));  // rasterizer.cpp:66-69
        for (const torch::Tensor* t : {&means, &shs, &scaling_raw, &rotation_raw, &opacity_raw})
            TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->scalar_type() == torch::kFloat32 &&
                            t->device() == means.device(),
                        "parameters must be contiguous float32 tensors on one GPU");
        m.device = means.device();
        m.N = (uint32_t)N, m.K = (uint32_t)shs.size(1);
        const c10::DeviceGuard guard(m.device);
        const torch::Tensor* params[5] = {&means, &shs, &scaling_raw, &rotation_raw, &opacity_raw};
        for (int i = 0; i < 5; ++i) {
            exp_avg[i] = torch::zeros_like(*params[i]);
            exp_avg_sq[i] = torch::zeros_like(*params[i]);
        }
        const auto fo = means.options().requires_grad(false);
        const auto io = fo.dtype(torch::kInt);
        m.opacities = torch::empty({N}, fo), m.scales = torch::empty({N, 3}, fo), m.quats = torch::empty({N, 4}, fo);
        m.radii = torch::empty({1, N, 2}, io), m.means2d = torch::empty({1, N, 2}, fo);
        m.depths = torch::empty({1, N}, fo), m.colors = torch::empty({1, N, 3}, fo);
        m.records = torch::empty({(int64_t)gsx_raster_records_bytes(m.N)}, fo.dtype(torch::kByte));
        // zeroed once: the update leaves every accumulator row it read zeroed for the next backward pass
        m.accum = torch::zeros({(int64_t)gsx_rasterize_bwd_accum_bytes(m.N)}, fo.dtype(torch::kByte));
        m.bg = torch::zeros({1, 3}, fo);  // trainer.cpp:383-384
        loss_out = torch::empty({3}, fo);
        m.n_pinned = torch::zeros({1}, torch::TensorOptions().dtype(torch::kLong).pinned_memory(true));
        m.hold_pinned = torch::zeros({1}, torch::TensorOptions().dtype(torch::kLong).pinned_memory(true));
        m.side = c10::hip::getStreamFromPool(/*isHighPriority=*/false, m.device.index()).stream();
        for (hipEvent_t* e : {&m.ev_fork, &m.ev_join})
            hip_ok(hipEventCreateWithFlags(e, hipEventDisableTiming));
    }

    TrainStep::~TrainStep() {
        if (!impl_)
            return;
        // the buffers were allocated for the current stream: what the second stream still has queued on them must be
        // over before the allocator hands them to somebody else
        if (impl_->side != nullptr)
            (void)hipStreamSynchronize(impl_->side);
        for (hipEvent_t e : {impl_->ev_fork, impl_->ev_join})
            if (e != nullptr)
                (void)hipEventDestroy(e);
    }

    void TrainStep::ensure_image(int H, int W) {
        Impl& m = *impl_;
        if (m.H == H && m.W == W)
            return;
        TORCH_CHECK(H > 0 && W > 0, "image size must be positive");
        m.tw = (uint32_t)(W + 15) / 16, m.th = (uint32_t)(H + 15) / 16;
        TORCH_CHECK(gsx_intersect_tile_pairs_fit(m.tw, m.th), "TrainStep: a grid of ", m.tw, " x ", m.th,
                    " tiles is beyond the 16-bit tile indices of gsx_tile_lists");
        const auto fo = means.options().requires_grad(false);
        const auto io = fo.dtype(torch::kInt);
        const int64_t tiles = (int64_t)m.tw * m.th;
        m.offsets_full = torch::empty({tiles + 1}, io);  // the last entry: the pair count
        m.tile_order = torch::empty({tiles}, io), m.tile_walk = torch::empty({tiles}, io);
        m.have_walk = false, m.order_due = false;
        render = torch::empty({1, H, W, 3}, fo), alpha = torch::empty({1, H, W, 1}, fo);
        last_ids = torch::empty({1, H, W}, io);
        m.v_render = torch::empty({1, H, W, 3}, fo), m.v_alpha = torch::zeros({1, H, W, 1}, fo);
        const int64_t nb = std::max<int64_t>(gsx_image_loss_blocks((uint32_t)H, (uint32_t)W),
                                             gsx_photometric_partials((uint32_t)H, (uint32_t)W));
        m.l1_partials = torch::empty({nb}, fo), m.ssim_partials = torch::empty({nb}, fo);
        m.dm1 = torch::empty({1, 3, H, W}, fo), m.dm2 = torch::empty({1, 3, H, W}, fo);
        m.dm3 = torch::empty({1, 3, H, W}, fo);
        m.H = H, m.W = W;
        m.lists_ws = torch::Tensor();  // the workspace depends on the grid
    }

    void TrainStep::ensure_lists() {
        Impl& m = *impl_;
        if (m.lists_ws.defined())
            return;
        if (cap_ == 0)
            cap_ = opt_.initial_pair_capacity > 0 ? opt_.initial_pair_capacity
                                                  : std::max<int64_t>(1 << 20, 6 * (int64_t)m.N);
        const size_t bytes = gsx_tile_lists_workspace_bytes(m.N, cap_, m.tw, m.th);
        const auto bo = means.options().requires_grad(false).dtype(torch::kByte);
        m.lists_ws = torch::empty({(int64_t)bytes}, bo);
        ok(gsx_tile_lists_init(m.N, cap_, m.tw, m.th, m.lists_ws.data_ptr(), bytes, m.main()));
        m.lists_error = gsx_tile_lists_error(m.N, cap_, m.tw, m.th, m.lists_ws.data_ptr());
        m.flat_out = torch::empty({cap_}, bo.dtype(torch::kInt));
        *m.hold_slot() = 0;
    }

    int64_t TrainStep::n_isects() const { return *impl_->n_slot(); }

    std::pair<uint32_t, uint32_t> TrainStep::lists_error() {
        Impl& m = *impl_;
        if (!m.lists_ws.defined())
            return {0u, 0u};
        hip_ok(hipDeviceSynchronize());
        uint32_t w[2] = {0, 0};
        hip_ok(hipMemcpy(w, m.lists_error, sizeof(w), hipMemcpyDeviceToHost));
        return {w[0], w[1]};
    }

    void TrainStep::debug_set_lists_error(uint32_t bits) {
        Impl& m = *impl_;
        TORCH_CHECK(m.lists_ws.defined(), "no tile lists yet: run a step first");
        hip_ok(hipDeviceSynchronize());
        hip_ok(hipMemcpy(m.lists_error, &bits, sizeof(bits), hipMemcpyHostToDevice));
    }

    void TrainStep::clear_lists_error() {
        Impl& m = *impl_;
        if (!m.lists_ws.defined())
            return;
        const c10::DeviceGuard guard(m.device);
        const auto e = lists_error();
        steps_held += e.second, step_count -= e.second, iteration -= e.second;
        hip_ok(hipMemset(m.lists_error, 0, 8));
        hip_ok(hipDeviceSynchronize());
        *m.hold_slot() = 0;
    }

    // Start of a step: the last count and the last error report that reached the host decide whether the buffers
    // grow.  More pairs than the buffers held means that step (and every step queued behind it) rendered nothing and
    // was held back from the optimiser: those are counted back out of the iteration counters.
    void TrainStep::check_capacity() {
        Impl& m = *impl_;
        if (!m.lists_ws.defined() || !m.cap_confirmed)
            return;
        if (*m.hold_slot() & 2u) {
            const auto e = lists_error();
            TORCH_CHECK(false, "gsx::TrainStep: a look-back of the tile lists gave up waiting (error bits ", e.first,
                        "); ", e.second, " optimiser call(s) were held back.  clear_lists_error() re-arms the lists");
        }
        const int64_t n = *m.n_slot();
        if (n <= cap_ - cap_ / 10)
            return;
        if (n > cap_) {
            const auto e = lists_error();
            steps_held += e.second, step_count -= e.second, iteration -= e.second;
        } else {
            hip_ok(hipDeviceSynchronize());  // kernels in flight still use the buffers that are about to go
        }
        TORCH_CHECK(n < (1ll << 30), "gsx::TrainStep: ", n, " intersections are beyond the tile lists' limit");
        {
            const int64_t latest = *m.n_slot();
            cap_ = std::max<int64_t>(n, latest);
        }
        cap_ = cap_ + cap_ / 4 + 1024;
        m.lists_ws = torch::Tensor();
        ensure_lists();
    }

    void TrainStep::forward(const torch::Tensor& viewmat, const torch::Tensor& Kmat, int W, int H) {
        Impl& m = *impl_;
        hipStream_t s = m.main();
        const bool two = opt_.overlap;
        ensure_image(H, W);
        ensure_lists();
        m.viewmat = f(viewmat), m.Kmat = f(Kmat);
        gsx_ut_params ut = gsx_ut_defaults();
        ok(gsx_activate_project_ut(m.N, f(means), f(opacity_raw), f(scaling_raw), f(rotation_raw), m.viewmat, m.Kmat,
                                   (uint32_t)W, (uint32_t)H, 0.3f, 0.01f, 1e4f, 0.0f, ut, f(m.opacities), f(m.scales),
                                   f(m.quats), i32(m.radii), f(m.means2d), f(m.depths), nullptr, s));
        hipStream_t sh_stream = s;
        if (two) {
            hip_ok(hipEventRecord(m.ev_fork, s));
            hip_ok(hipStreamWaitEvent(m.side, m.ev_fork, 0));
            sh_stream = m.side;
        }
        // queued before the tile lists: the tile table goes behind it on the second stream
        ok(gsx_sh_colors_records_from_world(m.N, m.K, (uint32_t)opt_.sh_degree, f(means), f(m.quats), f(m.scales),
                                            f(m.opacities), f(shs), i32(m.radii), m.viewmat, m.Kmat, (uint32_t)W,
                                            (uint32_t)H, f(m.colors), m.records.data_ptr(), sh_stream));
        if (two)
            hip_ok(hipEventRecord(m.ev_join, m.side));
        ok(gsx_tile_lists(m.N, f(m.means2d), i32(m.radii), f(m.depths), 16, m.tw, m.th, cap_, m.lists_ws.data_ptr(),
                          (size_t)m.lists_ws.numel(), i32(m.flat_out), i32(m.offsets_full),
                          const_cast<int64_t*>(m.n_slot()), s, two ? m.side : nullptr));
        // Dearest tiles first: both rasterizers then end with cheap tiles instead of a long tail.  What a tile costs
        // is how far its pixels go into its list, which the forward pass itself reports: the forward pass uses the
        // previous step's costs if that step saw the same camera tensors, else the list lengths; the backward pass
        // this step's costs.
        const uint32_t* order = nullptr;
        if (opt_.order_tiles) {
            const bool same_cam = m.have_walk && m.walk_viewmat == viewmat.data_ptr() && m.walk_K == Kmat.data_ptr() &&
                                  m.walk_W == W && m.walk_H == H;
            if (!same_cam) {
                // by list length: the offsets are complete when the tile table is, long before the pair passes end
                ok(gsx_tile_order(GSX_COUNT_IN_OFFSETS, i32(m.offsets_full), nullptr, m.tw, m.th, u32(m.tile_order),
                                  two ? m.side : s));
                if (two)
                    hip_ok(hipEventRecord(m.ev_join, m.side));
            }
            order = u32(m.tile_order);
        }
        if (two)
            hip_ok(hipStreamWaitEvent(s, m.ev_join, 0));  // colours, records and the order are ready
        ok(gsx_rasterize_records_fwd(GSX_COUNT_IN_OFFSETS, m.records.data_ptr(), nullptr, 3, f(m.bg), nullptr,
                                     (uint32_t)W, (uint32_t)H, m.viewmat, m.Kmat, i32(m.offsets_full), i32(m.flat_out),
                                     order, opt_.order_tiles ? u32(m.tile_walk) : nullptr, f(render), f(alpha),
                                     i32(last_ids), s));
        if (opt_.order_tiles) {
            m.order_due = true;
            m.have_walk = true, m.walk_viewmat = viewmat.data_ptr(), m.walk_K = Kmat.data_ptr();
            m.walk_W = W, m.walk_H = H;
        }
    }

    torch::Tensor TrainStep::step(const torch::Tensor& viewmat, const torch::Tensor& Kmat, int W, int H,
                                  const torch::Tensor& gt_chw) {
        Impl& m = *impl_;
        const c10::DeviceGuard guard(m.device);
        TORCH_CHECK(viewmat.is_cuda() && viewmat.is_contiguous() && viewmat.numel() == 16 &&
                        viewmat.scalar_type() == torch::kFloat32,
                    "viewmat must be a contiguous float32 GPU tensor [1, 4, 4]");
        TORCH_CHECK(Kmat.is_cuda() && Kmat.is_contiguous() && Kmat.numel() == 9 && Kmat.scalar_type() == torch::kFloat32,
                    "K must be a contiguous float32 GPU tensor [1, 3, 3]");
        TORCH_CHECK(gt_chw.is_cuda() && gt_chw.is_contiguous() && gt_chw.numel() == 3ll * H * W &&
                        gt_chw.scalar_type() == torch::kFloat32,
                    "gt image must be a contiguous float32 GPU tensor [3, H, W], got ", gt_chw.sizes());
        check_capacity();
        iteration += 1;
        if (!m.cap_confirmed)
            *m.n_slot() = -1;
        forward(viewmat, Kmat, W, H);
        if (!m.cap_confirmed) {
            // the first pass with these buffers: wait for its pair count once and size them by it
            int64_t n = -1;
            for (int i = 0; i < 4000000 && (n = *m.n_slot()) < 0; ++i) {
            }
            if (n < 0) {
                hip_ok(hipStreamSynchronize(m.main()));
                n = *m.n_slot();
            }
            TORCH_CHECK(n < (1ll << 30), "gsx::TrainStep: ", n, " intersections are beyond the tile lists' limit");
            if (n > cap_ - cap_ / 10) {
                hip_ok(hipDeviceSynchronize());
                cap_ = n + n / 4 + 1024;
                m.lists_ws = torch::Tensor();
                m.order_due = false;
                forward(viewmat, Kmat, W, H);
            }
            m.cap_confirmed = true;
        }
        hipStream_t s = m.main();
        const uint32_t Hu = (uint32_t)H, Wu = (uint32_t)W;
        // loss = (1 - lambda) L1 + lambda (1 - SSIM_valid) on clamp(render) (rasterizer.cpp:205, trainer.cpp:107-134)
        ok(gsx_photometric_loss_forward(Hu, Wu, 0.01f * 0.01f, 0.03f * 0.03f, f(render), f(gt_chw), f(m.dm1), f(m.dm2),
                                        f(m.dm3), f(m.l1_partials), f(m.ssim_partials), s));
        if (m.order_due) {
            // the order for the backward pass rides on the loss kernel (one workgroup more): a fork and a join of the
            // second stream would cost this one ~14 us of idle time
            ok(gsx_photometric_loss_backward_order(Hu, Wu, opt_.lambda_dssim, f(render), f(gt_chw), f(m.dm1), f(m.dm2),
                                                   f(m.dm3), f(m.l1_partials), f(m.ssim_partials), f(loss_out),
                                                   f(m.v_render), m.tw, m.th, u32(m.tile_walk), u32(m.tile_order), s));
            m.order_due = false;
        } else {
            ok(gsx_photometric_loss_backward_finish(Hu, Wu, opt_.lambda_dssim, f(render), f(gt_chw), f(m.dm1),
                                                    f(m.dm2), f(m.dm3), f(m.l1_partials), f(m.ssim_partials),
                                                    f(loss_out), f(m.v_render), s));
        }
        ok(gsx_rasterize_bwd_accumulate(1, m.N, GSX_COUNT_IN_OFFSETS, m.records.data_ptr(), nullptr, 3, f(m.bg),
                                        nullptr, Wu, Hu, 16, m.viewmat, m.Kmat, i32(m.offsets_full), i32(m.flat_out),
                                        opt_.order_tiles ? u32(m.tile_order) : nullptr, f(alpha), i32(last_ids),
                                        f(m.v_render), f(m.v_alpha), m.accum.data_ptr(), (size_t)m.accum.numel(), s));
        // FusedAdam::step (fused_adam.cpp:78-92): bias corrections in double, cast to float
        step_count += 1;
        gsx_update_args a{};
        a.N = m.N, a.K = m.K, a.sh_degree = (uint32_t)opt_.sh_degree;
        a.means = f(means), a.opacity_raw = f(opacity_raw), a.scaling_raw = f(scaling_raw);
        a.rotation_raw = f(rotation_raw), a.shs = f(shs);
        a.m_means = f(exp_avg[0]), a.m_shs = f(exp_avg[1]), a.m_scaling = f(exp_avg[2]);
        a.m_rotation = f(exp_avg[3]), a.m_opacity = f(exp_avg[4]);
        a.v_means = f(exp_avg_sq[0]), a.v_shs = f(exp_avg_sq[1]), a.v_scaling = f(exp_avg_sq[2]);
        a.v_rotation = f(exp_avg_sq[3]), a.v_opacity = f(exp_avg_sq[4]);
        a.radii = i32(m.radii), a.colors = f(m.colors), a.viewmat = m.viewmat, a.accumulators = m.accum.data_ptr();
        a.lr_means = (float)opt_.lrs[0], a.lr_sh0 = (float)opt_.lrs[1], a.lr_shN = (float)opt_.lrs[2];
        a.lr_scaling = (float)opt_.lrs[3], a.lr_rotation = (float)opt_.lrs[4], a.lr_opacity = (float)opt_.lrs[5];
        a.beta1 = (float)opt_.beta1, a.beta2 = (float)opt_.beta2, a.eps = (float)opt_.eps;
        a.bias_correction1_rcp = (float)(1.0 / (1.0 - std::pow(opt_.beta1, (double)step_count)));
        a.bias_correction2_sqrt_rcp = (float)(1.0 / std::sqrt(1.0 - std::pow(opt_.beta2, (double)step_count)));
        a.skip_shN = (opt_.freeze_shN_early && iteration <= 1000) ? 1 : 0;
        // weight / element count in float32, as the separate regularisation kernels form it
        a.reg_scaling = opt_.scale_reg > 0.f ? opt_.scale_reg / (float)(3 * (int64_t)m.N) : 0.f;
        a.reg_opacity = opt_.opacity_reg > 0.f ? opt_.opacity_reg / (float)m.N : 0.f;
        a.hold = m.lists_error;
        a.step_scalars = nullptr;
        a.hold_report = const_cast<uint64_t*>(m.hold_slot());
        ok(gsx_backward_update_fused(&a, s));
        return loss_out;
    }

}  // namespace gsx
