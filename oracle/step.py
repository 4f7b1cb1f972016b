"""CPU restatement of one training iteration (Trainer::train_step, src/training/trainer.cpp:599-875, `--gut` path
with the MCMC strategy's optimiser, mcmc.cpp:479-497), built from the checker's kernels.

TEST INFRASTRUCTURE ONLY (tests/, __graft_entry__.smoke(), bench.py's cpu_baseline leg).
"""
import math

import numpy as np

from . import oracle as orc

DEFAULT_LRS = dict(means=1.6e-4, sh0=2.5e-3, shN=2.5e-3 / 20.0, scaling=5e-3, rotation=1e-3, opacity=5e-2)


class OracleTrainStep:
    def __init__(self, scene, lrs=None, lambda_dssim=0.2, betas=(0.9, 0.999), eps=1e-15, sh_degree=None,
                 scale_reg=0.0, opacity_reg=0.0):
        c = lambda a: np.ascontiguousarray(a, dtype=np.float32).copy()
        self.params = dict(means=c(scene.means), shs=c(np.concatenate([scene.sh0, scene.shN], 1)),
                           scaling=c(scene.scaling_raw), rotation=c(scene.rotation_raw),
                           opacity=c(scene.opacity_raw.reshape(-1)))
        self.exp_avg = {k: np.zeros_like(v) for k, v in self.params.items()}
        self.exp_avg_sq = {k: np.zeros_like(v) for k, v in self.params.items()}
        self.K = self.params["shs"].shape[1]
        self.sh_degree = scene.sh_degree if sh_degree is None else sh_degree
        self.lrs = dict(DEFAULT_LRS, **(lrs or {}))
        self.lambda_dssim, self.betas, self.eps = lambda_dssim, betas, eps
        self.step_count = 0
        self.scale_reg, self.opacity_reg = scale_reg, opacity_reg
        self.bg = np.zeros((1, 3), np.float32)

    def forward(self, viewmat, K, W, H):
        P = self.params
        self.cam = (viewmat, K, W, H)
        self.act = orc.activate_params(P["opacity"], P["scaling"], P["rotation"])
        op, scales, quats = self.act
        self.fwd = orc.rasterize_from_world_with_sh_fwd(P["means"], quats, scales, op, P["shs"], self.sh_degree,
                                                        self.bg, W, H, 16, viewmat[None], K[None])
        return self.fwd[0]

    def loss_and_backward(self, gt_chw):
        P = self.params
        viewmat, K, W, H = self.cam
        op, scales, quats = self.act
        renders, alphas, radii, means2d, depths, colors, offsets, flat, last_ids, comp, ids = self.fwd
        loss, l1, ss, image, v_render = orc.photometric_loss(renders[0], gt_chw, self.lambda_dssim, True)
        self.loss, self.image, self.v_render = (loss, l1, ss), image, v_render
        v_alpha = np.zeros_like(alphas)
        v_means, v_quats, v_scales, v_op, v_sh = orc.rasterize_from_world_with_sh_bwd(
            P["means"], quats, scales, op, P["shs"], self.sh_degree, self.bg, W, H, 16, viewmat[None], K[None], 1.0,
            False, alphas, last_ids, offsets, flat, colors, radii, comp, v_render[None], v_alpha)
        g_op, g_sc, g_rot = orc.activate_params_bwd(P["opacity"], P["scaling"], P["rotation"], v_op, v_scales,
                                                    v_quats)
        self.grads = dict(means=v_means, shs=v_sh, scaling=g_sc, rotation=g_rot, opacity=g_op)
        # trainer.cpp:136-174: the two L1 terms add their gradients onto the finished ones
        self.reg_losses = (orc.l1_regularization("exp", P["scaling"], g_sc, self.scale_reg) if self.scale_reg > 0 else 0.0,
                           orc.l1_regularization("sigmoid", P["opacity"], g_op, self.opacity_reg)
                           if self.opacity_reg > 0 else 0.0)
        return loss

    def adam(self):
        self.step_count += 1
        t = self.step_count
        b1, b2 = self.betas
        bc1 = 1.0 / (1.0 - math.pow(b1, t))
        bc2 = 1.0 / math.sqrt(1.0 - math.pow(b2, t))
        for k in ("means", "scaling", "rotation", "opacity"):
            lr = self.lrs[{"means": "means", "scaling": "scaling", "rotation": "rotation", "opacity": "opacity"}[k]]
            orc.adam_step(self.params[k], self.exp_avg[k], self.exp_avg_sq[k], self.grads[k], lr, b1, b2, self.eps,
                          bc1, bc2)
        # sh0 and shN are separate parameter groups in the reference (mcmc.cpp:488-489): same arithmetic, two lrs
        for sl, lr in ((slice(0, 1), self.lrs["sh0"]), (slice(1, self.K), self.lrs["shN"])):
            if sl.stop <= sl.start:
                continue
            p = np.ascontiguousarray(self.params["shs"][:, sl])
            m = np.ascontiguousarray(self.exp_avg["shs"][:, sl])
            v = np.ascontiguousarray(self.exp_avg_sq["shs"][:, sl])
            g = np.ascontiguousarray(self.grads["shs"][:, sl])
            orc.adam_step(p, m, v, g, lr, b1, b2, self.eps, bc1, bc2)
            self.params["shs"][:, sl], self.exp_avg["shs"][:, sl], self.exp_avg_sq["shs"][:, sl] = p, m, v

    def relocate(self, sampled_idxs, dead_idxs, binoms, min_opacity=0.005):
        """MCMC::relocate_gs (mcmc.cpp:112-190) line by line, with the caller's index sets."""
        P = self.params
        n_max = binoms.shape[0]
        if sampled_idxs.size == 0:
            return 0
        op, scales, _ = orc.activate_params(P["opacity"], P["scaling"], P["rotation"])
        ratios = np.ones(op.shape[0], np.int32)                                   # :141
        np.add.at(ratios, sampled_idxs, 1)                                        # :142-143
        ratios = np.minimum(ratios[sampled_idxs], n_max).astype(np.int32)         # :144-148
        new_op, new_sc = orc.relocation(op[sampled_idxs], scales[sampled_idxs], ratios, binoms, n_max)  # :151-156
        new_op = np.clip(new_op, np.float32(min_opacity), np.float32(1.0 - 1e-7))  # :160
        P["opacity"][sampled_idxs] = orc.math_unary("log", new_op / (np.float32(1.0) - new_op))  # logit, :165-169
        P["scaling"][sampled_idxs] = orc.math_unary("log", new_sc.reshape(-1)).reshape(-1, 3)    # log, :171
        for k in ("means", "shs", "scaling", "rotation", "opacity"):               # :175-180
            P[k][dead_idxs] = P[k][sampled_idxs]
        for k in P:                                                                # :100-104
            self.exp_avg[k][sampled_idxs] = 0
            self.exp_avg_sq[k][sampled_idxs] = 0
        return sampled_idxs.size

    def add_new_gs(self, sampled_idxs, binoms, min_opacity=0.005):
        """MCMC::add_new_gs (mcmc.cpp:192-347) line by line, with the caller's sampled sources."""
        P = self.params
        n_max = binoms.shape[0]
        if sampled_idxs.size == 0:
            return 0
        op, scales, _ = orc.activate_params(P["opacity"], P["scaling"], P["rotation"])
        ratios = np.zeros(op.shape[0], np.float32)                                 # :217
        np.add.at(ratios, sampled_idxs, 1.0)                                       # :218
        ratios = np.clip(ratios[sampled_idxs] + 1, 1, n_max).astype(np.int32)      # :219-224
        new_op, new_sc = orc.relocation(op[sampled_idxs], scales[sampled_idxs], ratios, binoms, n_max)
        new_op = np.clip(new_op, np.float32(min_opacity), np.float32(1.0 - 1e-7))  # :236
        P["opacity"][sampled_idxs] = orc.math_unary("log", new_op / (np.float32(1.0) - new_op))
        P["scaling"][sampled_idxs] = orc.math_unary("log", new_sc.reshape(-1)).reshape(-1, 3)
        for k in list(P):                                                          # :247-260, 285-291
            P[k] = np.ascontiguousarray(np.concatenate([P[k], P[k][sampled_idxs]], 0))
            zeros = np.zeros((sampled_idxs.size,) + P[k].shape[1:], np.float32)
            self.exp_avg[k] = np.ascontiguousarray(np.concatenate([self.exp_avg[k], zeros], 0))
            self.exp_avg_sq[k] = np.ascontiguousarray(np.concatenate([self.exp_avg_sq[k], zeros], 0))
        return sampled_idxs.size

    def inject_noise(self, noise=None, noise_lr=5e5, seed=0, iteration=0):
        """MCMC::inject_noise (mcmc.cpp:349-367); noise = None: the counter-based draws for (seed, iteration)"""
        P = self.params
        if noise is None:
            noise = orc.philox_randn3(P["means"].shape[0], seed, iteration)
        orc.add_noise(P["opacity"], P["scaling"], P["rotation"], noise, P["means"],
                      np.float32(self.lrs["means"] * noise_lr))

    def step(self, viewmat, K, W, H, gt_chw):
        self.forward(viewmat, K, W, H)
        loss = self.loss_and_backward(gt_chw)
        self.adam()
        return loss
