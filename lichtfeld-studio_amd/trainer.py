"""One training iteration of LichtFeld's `--gut` path (Trainer::train_step, src/training/trainer.cpp:599-875) on
the gfx950 kernels: activations -> fused rasterization with SH (Rasterization.cpp:279-467) -> photometric loss
(trainer.cpp:126-129) -> backward (Rasterization.cpp:469-642 + the autograd of the activations and of the loss)
-> fused Adam over the six parameter groups (mcmc.cpp:479-497, fused_adam.cpp:22-95).

Differences in organisation (not in arithmetic): every buffer is allocated once and reused; sh0 and shN live in
one [N,K,3] tensor (no 192 B/Gaussian concatenation per step, splat_data.cpp:285) whose two learning rates the Adam
kernel applies by element index; all parameter groups are updated by one launch; the ATen glue passes are fused
into the kernels that produce or consume their data.
"""
import ctypes
import math

import numpy as np
import torch

from . import _lib as L
from ._lib import UTParams, c_f, c_i, c_i64, c_p, c_sz, c_u32, check, lib

# mcmc.cpp:487-492 / include/core/parameters.hpp:19-23
DEFAULT_LRS = dict(means=1.6e-4, sh0=2.5e-3, shN=2.5e-3 / 20.0, scaling=5e-3, rotation=1e-3, opacity=5e-2)


def _p(t):
    return c_p(None) if t is None else c_p(t.data_ptr())


class TrainStep:
    def __init__(self, scene, device="cuda:0", lrs=None, lambda_dssim=0.2, betas=(0.9, 0.999), eps=1e-15,
                 scene_scale=1.0, sh_degree=None, use_ssim=True, fused_update=False, fused_loss=False,
                 scale_reg=0.0, opacity_reg=0.0, overlap=False, tile_pairs=True, one_front_pass=False,
                 device_count=False):
        self.dev = torch.device(device)
        self.lib = lib()
        self.one_front_pass = one_front_pass  # activations + projection + SH colours + records as one launch
        self.tile_pairs = tile_pairs  # sort (u16 tile index, id) pairs where the tile grid allows it
        # True (needs fused_update and a grid of at most 255 x 255 tiles): after the first step, which sizes the
        # buffers, the tile lists come from gsx_tile_lists and the pair count stays on the device - no host wait
        # inside a step; a step whose pairs outgrow the buffers renders nothing, is held back from the optimiser
        # and is made up for by _check_capacity at the start of the next one
        self.device_count = bool(device_count and fused_update)
        self.lists_ws, self._lists_dims, self._lists_active = None, None, False
        self.steps_held = 0
        # the fused update stores (calls held back << 32 | sticky error bits of the tile lists) here after every launch
        self.hold_report = torch.zeros(1, dtype=torch.int64, pin_memory=True)
        self._hold_slot = ctypes.c_uint64.from_address(self.hold_report.data_ptr())
        f = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(self.dev)
        self.N = scene.means.shape[0]
        self.K = 1 + scene.shN.shape[1]
        self.sh_degree = scene.sh_degree if sh_degree is None else sh_degree
        # raw trainable tensors (include/core/splat_data.hpp:68-79); sh0 | shN share one [N,K,3] tensor
        self.params = dict(
            means=f(scene.means), shs=f(np.concatenate([scene.sh0, scene.shN], 1)), scaling=f(scene.scaling_raw),
            rotation=f(scene.rotation_raw), opacity=f(scene.opacity_raw.reshape(-1)))
        self.grads = {k: torch.zeros_like(v) for k, v in self.params.items()}
        self.exp_avg = {k: torch.zeros_like(v) for k, v in self.params.items()}
        self.exp_avg_sq = {k: torch.zeros_like(v) for k, v in self.params.items()}
        self.step_count = 0
        self.iteration = 0
        lrs = dict(DEFAULT_LRS, **(lrs or {}))
        lrs["means"] = lrs["means"] * scene_scale
        self.lrs = lrs
        self.betas, self.eps = betas, eps
        self.lambda_dssim = lambda_dssim if use_ssim else 0.0
        self.use_ssim = use_ssim
        # True: epilogue + SH backward + activation VJPs + Adam run as one pass and the raw-parameter gradients
        # (self.grads) are never materialised; False: separate kernels (what the parity tests inspect)
        self.fused_update = fused_update
        # True (needs use_ssim): the loss runs as two kernels and neither the clamped image nor the SSIM map exist
        self.fused_loss = fused_loss and use_ssim
        self.ut = UTParams()
        # trainer.cpp:136-174 (weights of the L1 terms on exp(scaling_raw) and sigmoid(opacity_raw); 0 = off)
        self.scale_reg, self.opacity_reg = float(scale_reg), float(opacity_reg)
        self.reg_partials = torch.empty(self.lib.gsx_l1_regularization_partials(), dtype=torch.float32,
                                        device=self.dev)
        self.reg_losses = torch.zeros(2, dtype=torch.float32, device=self.dev)  # [scale term, opacity term]
        self._allocate_per_gaussian(self.N)
        self.cap = 0
        self.compact = False
        self.img_shape = None
        self._n_host = 0
        self.bg = torch.zeros((1, 3), dtype=torch.float32, device=self.dev)  # trainer.cpp:383-384
        # A second stream (default priority) for work that is independent of the launch-latency-bound sort chain:
        # the SH / record pass runs beside the depth-ordered count, the loss reduction beside the backward rasterizer.
        self.overlap = overlap
        self.side = torch.cuda.Stream(self.dev) if overlap else None
        self.ev_fork, self.ev_join = torch.cuda.Event(), torch.cuda.Event()
        self.ev_loss_fork, self.ev_loss_join = torch.cuda.Event(), torch.cuda.Event()
        self.ev_order_join = torch.cuda.Event()
        self.order_pending, self._order_due = False, None
        self.loss_out = torch.empty(3, dtype=torch.float32, device=self.dev)

    def __del__(self):
        # the buffers were allocated for the current stream: what the second stream still has queued on them must be
        # over before the allocator hands them to somebody else
        side = getattr(self, "side", None)
        if side is not None:
            try:
                side.synchronize()
            except Exception:
                pass

    def _allocate_per_gaussian(self, N):
        """every buffer whose size follows the number of Gaussians"""
        self.N = N
        e = lambda *s, dt=torch.float32: torch.empty(s, dtype=dt, device=self.dev)
        self.act = dict(opacities=e(N), scales=e(N, 3), quats=e(N, 4))
        self.v_act = dict(opacities=e(N), scales=e(N, 3), quats=e(N, 4))
        self.proj = dict(radii=e(1, N, 2, dt=torch.int32), means2d=e(1, N, 2), depths=e(1, N), conics=e(1, N, 3))
        self.colors = e(1, N, 3)
        self.v_colors = e(1, N, 3)
        self.tiles_per_gauss = e(N, dt=torch.int32)
        self.cum = e(N, dt=torch.int64)
        self.ws_count = e(self.lib.gsx_intersect_tile_count_ordered_workspace_bytes(c_u32(N)), dt=torch.uint8)
        self.order = e(N, dt=torch.int32)
        self.n_isects_pinned = torch.zeros(1, dtype=torch.int64, pin_memory=True)
        self._n_slot = ctypes.c_int64.from_address(self.n_isects_pinned.data_ptr())
        self.count_done = torch.cuda.Event()
        self.ws_bwd = torch.zeros(self.lib.gsx_rasterize_bwd_accum_bytes(c_u32(N)), dtype=torch.uint8,
                                  device=self.dev)  # the backward's epilogue leaves it zeroed for the next pass
        self.records = e(self.lib.gsx_raster_records_bytes(c_u32(N)), dt=torch.uint8)

    # -- buffers that depend on n_isects / image size --------------------------------------------
    def _await_count(self):
        """The intersection total: the pinned slot reads -1 until the device's copy has landed.  Watching the slot
        costs the host no driver call on the way out of the wait (the kernels behind it are queued sooner)."""
        slot = self._n_slot
        for _ in range(2_000_000):
            n = slot.value
            if n >= 0:
                break
        else:
            self.count_done.synchronize()
            n = slot.value
        self._n_host = n
        return n

    @property
    def n_isects(self):
        """pairs of the last forward pass (with the count on the device: the last value that has landed in the pinned
        slot - synchronise first to be sure it is the last pass's)"""
        return self._n_slot.value if self._lists_active else self._n_host

    # -- tile lists with the count on the device -----------------------------------------------------
    def _lists_ready(self):
        dims = (self.N, self.cap, self.tw, self.th)
        if self._lists_dims == dims:
            return
        a = (c_u32(self.N), c_i64(self.cap), c_u32(self.tw), c_u32(self.th))
        nbytes = self.lib.gsx_tile_lists_workspace_bytes(*a)
        self.lists_ws = torch.empty(nbytes, dtype=torch.uint8, device=self.dev)
        check(self.lib.gsx_tile_lists_init(*a, _p(self.lists_ws), c_sz(nbytes), self._stream()))
        base = self.lists_ws.data_ptr()
        self._lists_error = self.lib.gsx_tile_lists_error(*a, c_p(base))  # device address of u32 [2]
        self._lists_error_at = self._lists_error - base
        self.flat_out = torch.empty(self.cap, dtype=torch.int32, device=self.dev)
        self._lists_dims = dims

    def lists_counts(self):
        """(pairs in the lists, pairs there are, Gaussians that touch a tile, (super-tile, Gaussian) entries) of the
        last gsx_tile_lists call; synchronises"""
        if self.lists_ws is None:
            return 0, 0, 0, 0
        a = (c_u32(self.N), c_i64(self.cap), c_u32(self.tw), c_u32(self.th))
        at = self.lib.gsx_tile_lists_counts(*a, c_p(self.lists_ws.data_ptr())) - self.lists_ws.data_ptr()
        torch.cuda.synchronize(self.dev)
        w = self.lists_ws[at:at + 32].cpu().numpy().view(np.int64)
        return tuple(int(x) for x in w)

    def lists_error(self):
        """(error bits, optimiser calls held back) of the tile lists so far; synchronises"""
        if self.lists_ws is None:
            return 0, 0
        torch.cuda.synchronize(self.dev)
        w = self.lists_ws[self._lists_error_at:self._lists_error_at + 8].cpu().numpy().view(np.uint32)
        return int(w[0]), int(w[1])

    def clear_lists_error(self):
        """after a raised look-back error: zero the sticky error word and the held-call counter"""
        torch.cuda.synchronize(self.dev)
        _, held = self.lists_error()
        self.steps_held += held
        self.step_count -= held
        self.iteration -= held
        self.lists_ws[self._lists_error_at:self._lists_error_at + 8].zero_()
        torch.cuda.synchronize(self.dev)
        self._hold_slot.value = 0

    def _check_capacity(self):
        """Start of a step with the count on the device: the last count that reached the host decides whether the
        buffers grow.  More pairs than the buffers held means that step (and every step queued behind it) rendered
        nothing and was held back from the optimiser: they are counted back out of the iteration counters."""
        if not self._lists_active:
            return
        if self._hold_slot.value & 2:
            # a chained pass gave up waiting for its predecessor: the lists of that step (and the renders since) are
            # invalid and the optimiser has been held since - not a condition to train through
            bits, held = self.lists_error()
            raise L.GsxError(-4, f"tile lists: a look-back's bounded wait ran out (error bits {bits}); {held} "
                                 "optimiser call(s) were held back.  clear_lists_error() re-arms the lists")
        n = self._n_slot.value
        if n <= int(self.cap * 0.9):
            return
        if n > self.cap:
            bits, held = self.lists_error()
            self.steps_held += held
            self.step_count -= held
            self.iteration -= held
        else:
            torch.cuda.synchronize(self.dev)  # kernels in flight still use the buffers that are about to go
        self.cap = 0
        self._ensure_isect_capacity(max(n, self._n_slot.value))
        self._lists_ready()

    def _ensure_isect_capacity(self, n):
        if n <= self.cap and self.cap:
            return
        cap = max(int(n * 1.25) + 1024, 1 << 16)
        e = lambda *s, dt: torch.empty(s, dtype=dt, device=self.dev)
        kt = torch.int16 if self.compact else torch.int64
        self.keys = [e(cap, dt=kt), e(cap, dt=kt)]
        self.vals = [e(cap, dt=torch.int32), e(cap, dt=torch.int32)]
        self.ws_sort = e(self.lib.gsx_radix_sort_pairs_workspace_bytes(c_i64(cap)), dt=torch.uint8)
        self.cap = cap

    def _ensure_image(self, H, W):
        if self.img_shape == (H, W):
            return
        e = lambda *s, dt=torch.float32: torch.empty(s, dtype=dt, device=self.dev)
        self.tw, self.th = (W + 15) // 16, (H + 15) // 16
        self._tile_bits = self.lib.gsx_n_bits(c_u32(self.tw * self.th))
        self._end_bit = 32 + self.lib.gsx_n_bits(c_u32(self.tw * self.th)) + self.lib.gsx_n_bits(c_u32(1))
        compact = bool(self.tile_pairs and self.lib.gsx_intersect_tile_pairs_fit(c_u32(self.tw), c_u32(self.th)))
        if compact != self.compact:  # the key buffers change their element type
            self.compact, self.cap = compact, 0
        self.offsets_full = e(self.th * self.tw + 1, dt=torch.int32)  # the last entry: room for the pair count
        self.offsets = self.offsets_full[:-1].view(1, self.th, self.tw)
        self.tile_order = e(self.th * self.tw, dt=torch.int32)  # the rasterizers' tile visiting order
        self.tile_walk = e(self.th * self.tw, dt=torch.int32)   # per tile: entries up to its last contributor
        self.have_walk, self._walk_cam = False, None
        self.render = e(1, H, W, 3)
        self.alpha = e(1, H, W, 1)
        self.last_ids = e(1, H, W, dt=torch.int32)
        self.image = e(1, 3, H, W)
        self.v_render = e(1, H, W, 3)
        self.v_alpha = torch.zeros((1, H, W, 1), dtype=torch.float32, device=self.dev)
        nb = max(self.lib.gsx_image_loss_blocks(c_u32(H), c_u32(W)), self.lib.gsx_photometric_partials(c_u32(H), c_u32(W)))
        self.n_partials = self.lib.gsx_image_loss_blocks(c_u32(H), c_u32(W))
        self.n_partials_fused = self.lib.gsx_photometric_partials(c_u32(H), c_u32(W))
        self.l1_partials, self.ssim_partials = e(nb), e(nb)
        self.ssim_map, self.dm1, self.dm2, self.dm3 = e(1, 3, H, W), e(1, 3, H, W), e(1, 3, H, W), e(1, 3, H, W)
        self.dL_dmap, self.dL_dimg = e(1, 3, H, W), e(1, 3, H, W)
        crop = H > 10 and W > 10
        count = 3 * (H - 10) * (W - 10) if crop else 3 * H * W
        # d loss / d map = lambda * d(1 - mean(map_valid)) / d map ; constant per resolution
        check(self.lib.gsx_ssim_valid_grad_map(c_u32(3), c_u32(H), c_u32(W), c_f(-self.lambda_dssim / count),
                                               _p(self.dL_dmap), self._stream()))
        self.img_shape = (H, W)

    def _join_tile_order(self):
        """The tile order from the last forward pass's costs is in place for what the current stream runs next."""
        if self._order_due is not None:  # nobody has queued it yet
            self._run("tile_order", self.lib.gsx_tile_order, *self._order_due, self._stream())
            self._order_due = None
        if self.order_pending:  # it was formed on the second stream
            torch.cuda.current_stream(self.dev).wait_event(self.ev_order_join)
            self.order_pending = False

    def _order_on_side_stream(self):
        """Called with the second stream current and already waiting for the forward pass."""
        if self._order_due is not None:
            self._run("tile_order", self.lib.gsx_tile_order, *self._order_due, self._stream())
            self.ev_order_join.record(self.side)
            self._order_due, self.order_pending = None, True

    def _stream(self):
        return c_p(torch.cuda.current_stream(self.dev).cuda_stream)

    # per-stage HIP-event timing (events are recorded on the stream the kernels are launched on)
    timing = None  # None, or a dict name -> list of (start_event, stop_event)

    def _run(self, name, fn, *args):
        if self.timing is None or (self.timed_names is not None and name not in self.timed_names):
            check(fn(*args))
            return
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(torch.cuda.current_stream(self.dev))
        check(fn(*args))
        e1.record(torch.cuda.current_stream(self.dev))
        self.timing.setdefault(name, []).append((e0, e1))

    timed_names = None  # None = every stage; or a set of stage names

    def start_timing(self, names=None):
        self.timing, self.timed_names = {}, (None if names is None else set(names))

    def stop_timing(self):
        """-> dict name -> list of milliseconds (synchronises)"""
        torch.cuda.synchronize(self.dev)
        out = {k: [a.elapsed_time(b) for a, b in v] for k, v in (self.timing or {}).items()}
        self.timing = None
        return out

    # -- forward ----------------------------------------------------------------------------------
    def forward(self, viewmat, K, W, H):
        """activations + rasterize_from_world_with_sh_fwd; returns the [1,H,W,3] render (not clamped)."""
        lb, s, N = self.lib, self._stream(), self.N
        self._join_tile_order()  # a forward pass with no backward after it leaves the order kernel unjoined
        self._ensure_image(H, W)
        self.viewmat, self.Kmat, self.W, self.H = viewmat, K, W, H
        P, A, J = self.params, self.act, self.proj
        sh_args = (c_u32(N), c_u32(self.K), c_u32(self.sh_degree), _p(P["means"]), _p(A["quats"]), _p(A["scales"]),
                   _p(A["opacities"]), _p(P["shs"]), _p(J["radii"]), _p(viewmat), _p(K), c_u32(W), c_u32(H),
                   _p(self.colors), _p(self.records))
        if self.one_front_pass:
            # activations, projection, SH colours and records in one pass over the Gaussians: nothing runs beside
            # the latency-bound sort chain
            self._run("activate_project_sh_records", lb.gsx_activate_project_sh_records, c_u32(N), c_u32(self.K),
                      c_u32(self.sh_degree), _p(P["means"]), _p(P["opacity"]), _p(P["scaling"]), _p(P["rotation"]),
                      _p(P["shs"]), _p(viewmat), _p(K), c_u32(W), c_u32(H), c_f(0.3), c_f(0.01), c_f(1e4), c_f(0.0),
                      self.ut, _p(A["opacities"]), _p(A["scales"]), _p(A["quats"]), _p(J["radii"]), _p(J["means2d"]),
                      _p(J["depths"]), _p(J["conics"]), _p(self.colors), _p(self.records), s)
        else:
            self._run("activate_project_ut", lb.gsx_activate_project_ut, c_u32(N), _p(P["means"]), _p(P["opacity"]),
                      _p(P["scaling"]), _p(P["rotation"]), _p(viewmat), _p(K), c_u32(W), c_u32(H), c_f(0.3),
                      c_f(0.01), c_f(1e4), c_f(0.0), self.ut, _p(A["opacities"]), _p(A["scales"]), _p(A["quats"]),
                      _p(J["radii"]), _p(J["means2d"]), _p(J["depths"]), _p(J["conics"]), s)
        side_sh = self.side is not None and not self.one_front_pass
        if side_sh:
            self.ev_fork.record(torch.cuda.current_stream(self.dev))

        def sh_pass():
            if self.one_front_pass:
                return
            if not side_sh:
                self._run("sh_colors_records_from_world", lb.gsx_sh_colors_records_from_world, *sh_args, s)
                return
            self.side.wait_event(self.ev_fork)  # recorded after the activation / projection pass
            with torch.cuda.stream(self.side):
                self._run("sh_colors_records_from_world", lb.gsx_sh_colors_records_from_world, *sh_args,
                          self._stream())
                self.ev_join.record(self.side)

        self._lists_active = self.device_count and self.compact and self.cap > 0
        if self._lists_active:
            # every launch sized by the buffers, the count read on the device: nothing waits for the host
            self._lists_ready()
            sh_pass()  # queued first: the tile table goes behind it on the second stream
            self._run("tile_lists", lb.gsx_tile_lists, c_u32(N), _p(J["means2d"]), _p(J["radii"]), _p(J["depths"]),
                      c_u32(16), c_u32(self.tw), c_u32(self.th), c_i64(self.cap), _p(self.lists_ws),
                      c_sz(self.lists_ws.numel()), _p(self.flat_out), _p(self.offsets_full),
                      c_p(self.n_isects_pinned.data_ptr()), s,
                      c_p(self.side.cuda_stream if self.side is not None else None))
            self.flatten_ids = self.flat_out
            n = -1  # GSX_COUNT_IN_OFFSETS
        else:
            n = self._host_counted_lists(sh_pass)
        self._n_arg = n
        # Dearest tiles first: both rasterizers then end with cheap tiles instead of a long tail.  What a tile costs is
        # how far its pixels go into the list, which the forward pass itself reports; the forward pass therefore
        # uses the order of the previous step (the first one: by list length), the backward pass this step's.
        order = c_p(None)
        if self.order_tiles:
            # the previous pass's costs say something about this one only for the same camera (the same tensors)
            cam_key = (viewmat.data_ptr(), K.data_ptr(), W, H)
            if not self.have_walk or cam_key != self._walk_cam:
                order_args = (c_i64(n), _p(self.offsets), c_p(None), c_u32(self.tw), c_u32(self.th),
                              _p(self.tile_order))
                if self._lists_active and side_sh:
                    # by list length: the offsets are complete when the tile table is, long before the pair passes
                    # end - the order goes behind the table on the second stream, off the chain's critical path
                    with torch.cuda.stream(self.side):
                        self._run("tile_order", lb.gsx_tile_order, *order_args, self._stream())
                        self.ev_join.record(self.side)
                else:
                    self._run("tile_order", lb.gsx_tile_order, *order_args, s)
            order = _p(self.tile_order)
        self._tile_order_arg = order
        if side_sh:
            torch.cuda.current_stream(self.dev).wait_event(self.ev_join)  # colours and records are ready
        self._run("rasterize_to_pixels_from_world_3dgs_fwd", lb.gsx_rasterize_records_fwd, c_i64(n),
                  _p(self.records), c_p(None), c_u32(3), _p(self.bg), c_p(None), c_u32(W), c_u32(H), _p(viewmat),
                  _p(K), _p(self.offsets), _p(self.flatten_ids), order, _p(self.tile_walk) if self.order_tiles else
                  c_p(None), _p(self.render), _p(self.alpha), _p(self.last_ids), s)
        if self.order_tiles:
            # the order for the backward pass (and for the next forward pass from this camera): queued by the loss
            # pass on the second stream, or by whoever needs it first
            self._order_due = (c_i64(n), c_p(None), _p(self.tile_walk), c_u32(self.tw), c_u32(self.th),
                               _p(self.tile_order))
            self.have_walk, self._walk_cam = True, (viewmat.data_ptr(), K.data_ptr(), W, H)
        return self.render

    def _host_counted_lists(self, sh_pass):
        """intersect_tile (depth-ordered count, emission) + pair sort + intersect_offset with the pair count crossing
        to the host, which sizes the buffers and the launches by it; returns the count"""
        lb, s, N, J = self.lib, self._stream(), self.N, self.proj
        # Tile counts in depth order; the total comes back through pinned memory without blocking, and the SH /
        # record passes (which do not need it) run while the host waits for it.
        self._run("intersect_tile_count_ordered", lb.gsx_intersect_tile_count_ordered, c_u32(N), _p(J["means2d"]),
                  _p(J["radii"]), _p(J["depths"]), c_u32(16), c_u32(self.tw), c_u32(self.th), _p(self.order),
                  _p(self.tiles_per_gauss), _p(self.cum), _p(self.ws_count), c_sz(self.ws_count.numel()),
                  c_p(self.n_isects_pinned.data_ptr()), c_i(0), s)
        self.count_done.record(torch.cuda.current_stream(self.dev))
        sh_pass()
        # The emission does not need the total, only room for it: with buffers from an earlier step it is queued now
        # (writes bounded to the buffers) and the host's wake-up from the wait below hides behind it.
        if self.compact:  # pairs in depth order sort on their tile bits only: 16-bit tile indices as keys
            emit = lambda cap: self._run(
                "intersect_tile_emit", lb.gsx_intersect_tile_emit_pairs, c_u32(N), _p(self.cum), _p(self.order),
                _p(self.ws_count), c_u32(16), c_u32(self.tw), c_u32(self.th), c_i64(cap), _p(self.keys[0]),
                _p(self.vals[0]), s)
        else:
            emit = lambda cap: self._run(
                "intersect_tile_emit", lb.gsx_intersect_tile_emit_ordered, c_u32(N), _p(J["means2d"]),
                _p(J["radii"]), _p(J["depths"]), _p(self.cum), _p(self.order), _p(self.ws_count), c_u32(16),
                c_u32(self.tw), c_u32(self.th), c_i64(cap), _p(self.keys[0]), _p(self.vals[0]), s)
        emitted_cap = self.cap
        if emitted_cap:
            emit(emitted_cap)
        n = self._await_count()
        if n >= 1 << 31:
            raise L.GsxError(-5, f"{n} intersections do not fit int32 indices")
        self._ensure_isect_capacity(n)
        sel = c_i(0)
        if n:
            if n > emitted_cap:  # first step, or the buffers had to grow
                emit(self.cap)
            end_bit = self._end_bit  # 32 + tile bits + camera bits, fixed with the image size
            if self.compact:
                self._run("radix_sort_pairs", lb.gsx_radix_sort_tile_pairs, c_i64(n), _p(self.keys[0]),
                          _p(self.vals[0]), _p(self.keys[1]), _p(self.vals[1]), c_u32(self._tile_bits),
                          _p(self.ws_sort), c_sz(self.ws_sort.numel()), ctypes.byref(sel), s)
            else:
                self._run("radix_sort_pairs", lb.gsx_radix_sort_pairs, c_i64(n), _p(self.keys[0]),
                          _p(self.vals[0]), _p(self.keys[1]), _p(self.vals[1]), c_u32(32), c_u32(end_bit),
                          _p(self.ws_sort), c_sz(self.ws_sort.numel()), ctypes.byref(sel), s)
        self.sel = sel.value
        self.flatten_ids = self.vals[self.sel]
        if self.compact:
            self._run("intersect_offset", lb.gsx_intersect_tile_pairs_offset, c_i64(n), _p(self.keys[self.sel]),
                      c_u32(self.tw), c_u32(self.th), _p(self.offsets), s)
        else:
            self._run("intersect_offset", lb.gsx_intersect_offset, c_i64(n), _p(self.keys[self.sel]), c_u32(1),
                      c_u32(self.tw), c_u32(self.th), _p(self.offsets), s)
        return n

    @property
    def isect_ids(self):
        """The sorted 64-bit keys (tile << 32 | depth bits) of the last forward pass.  On the 16-bit path they are not
        formed by the step: rebuilt here, for inspection, from the sorted tile indices and the depths."""
        if not self.compact:
            return self.keys[self.sel]
        n = self.n_isects
        if self._lists_active:  # no sorted keys either: an entry's tile is the list it lies in
            bounds = self.offsets_full[1:].to(torch.int64).contiguous()
            tiles = torch.searchsorted(bounds, torch.arange(n, dtype=torch.int64, device=self.dev), right=True)
        else:
            tiles = self.keys[self.sel][:n].to(torch.int64) & 0xFFFF
        depth = self.proj["depths"].view(torch.int32).reshape(-1)[self.flatten_ids[:n].long()]
        return (tiles << 32) | (depth.to(torch.int64) & 0xFFFFFFFF)

    # -- loss ---------------------------------------------------------------------------------------
    def loss_forward(self, gt_chw, finish=True):
        """image = clamp(render, 0, 1) CHW; loss = (1-l) L1 + l (1 - SSIM_valid); result stays on the device.
        finish = False (fused loss only): the loss value is left to backward(), whose loss kernel adds the partial
        sums up on the way."""
        lb, s, H, W = self.lib, self._stream(), self.H, self.W
        self.gt = gt_chw
        self._loss_due = False
        if self.fused_loss:
            self._run("photometric_loss_forward", lb.gsx_photometric_loss_forward, c_u32(H), c_u32(W),
                      c_f(0.01 ** 2), c_f(0.03 ** 2), _p(self.render), _p(gt_chw), _p(self.dm1), _p(self.dm2),
                      _p(self.dm3), _p(self.l1_partials), _p(self.ssim_partials), s)
            fin = (c_u32(3), c_u32(H), c_u32(W), c_f(self.lambda_dssim), _p(self.l1_partials), _p(self.ssim_partials),
                   c_u32(self.n_partials_fused), _p(self.loss_out))
            self._loss_due = not finish
            if self.side is None:
                if finish:
                    self._run("photometric_loss_finish", lb.gsx_photometric_loss_finish, *fin, s)
            elif finish:  # the value is only reported: its reduction runs beside the backward pass
                self.ev_loss_fork.record(torch.cuda.current_stream(self.dev))
                self.side.wait_event(self.ev_loss_fork)
                with torch.cuda.stream(self.side):
                    self._order_on_side_stream()  # the backward pass waits for this one, not for the reduction
                    self._run("photometric_loss_finish", lb.gsx_photometric_loss_finish, *fin, self._stream())
                    self.ev_loss_join.record(self.side)
                self.loss_pending = True
            # (finish = False: the loss kernel of backward() forms the value and the tile order on its way - a fork
            # and a join of the second stream cost the current one ~14 us of idle time, more than either is worth)
            return self.loss_out
        self._run("image_from_render", lb.gsx_image_from_render, c_u32(H), c_u32(W), _p(self.render), _p(gt_chw), _p(self.image),
                                       _p(self.l1_partials), s)
        if self.use_ssim:
            self._run("fusedssim", lb.gsx_fusedssim, c_i(1), c_i(3), c_i(H), c_i(W), c_f(0.01 ** 2), c_f(0.03 ** 2), _p(self.image),
                                   _p(gt_chw), _p(self.ssim_map), _p(self.dm1), _p(self.dm2), _p(self.dm3), s)
            self._run("ssim_valid_partials", lb.gsx_ssim_valid_partials, c_u32(3), c_u32(H), c_u32(W), _p(self.ssim_map), _p(self.ssim_partials),
                                             s)
        else:
            self.ssim_partials.zero_()
        self._run("photometric_loss_finish", lb.gsx_photometric_loss_finish, c_u32(3), c_u32(H), c_u32(W), c_f(self.lambda_dssim),
                                             _p(self.l1_partials), _p(self.ssim_partials), c_u32(self.n_partials),
                                             _p(self.loss_out), s)
        return self.loss_out

    # -- backward -----------------------------------------------------------------------------------
    def backward(self):
        lb, s, N, H, W = self.lib, self._stream(), self.N, self.H, self.W
        P, A, J, G, V = self.params, self.act, self.proj, self.grads, self.v_act
        dimg = None
        if self.fused_loss and getattr(self, "_loss_due", False):
            loss_args = (c_u32(H), c_u32(W), c_f(self.lambda_dssim), _p(self.render), _p(self.gt), _p(self.dm1),
                         _p(self.dm2), _p(self.dm3), _p(self.l1_partials), _p(self.ssim_partials), _p(self.loss_out),
                         _p(self.v_render))
            if self._order_due is not None:  # one workgroup more sorts the tiles for the backward rasterizer
                self._run("photometric_loss_backward", lb.gsx_photometric_loss_backward_order, *loss_args,
                          c_u32(self.tw), c_u32(self.th), _p(self.tile_walk), _p(self.tile_order), s)
                self._order_due = None
            else:
                self._run("photometric_loss_backward", lb.gsx_photometric_loss_backward_finish, *loss_args, s)
            self._loss_due = False
        elif self.fused_loss:
            self._run("photometric_loss_backward", lb.gsx_photometric_loss_backward, c_u32(H), c_u32(W),
                      c_f(self.lambda_dssim), _p(self.render), _p(self.gt), _p(self.dm1), _p(self.dm2), _p(self.dm3),
                      _p(self.v_render), s)
        elif self.use_ssim:
            self._run("fusedssim_backward", lb.gsx_fusedssim_backward, c_i(1), c_i(3), c_i(H), c_i(W), c_f(0.01 ** 2), c_f(0.03 ** 2),
                                            _p(self.image), _p(self.gt), _p(self.dL_dmap), _p(self.dm1), _p(self.dm2),
                                            _p(self.dm3), _p(self.dL_dimg), s)
            dimg = self.dL_dimg
        if not self.fused_loss:
            self._run("render_grad_from_loss", lb.gsx_render_grad_from_loss, c_u32(H), c_u32(W),
                      c_f(self.lambda_dssim), _p(self.render), _p(self.image), _p(self.gt), _p(dimg),
                      _p(self.v_render), s)
        ws, wsn = _p(self.ws_bwd), c_sz(self.ws_bwd.numel())
        self._join_tile_order()
        self._run("rasterize_bwd_accumulate", lb.gsx_rasterize_bwd_accumulate,
                  c_u32(1), c_u32(N), c_i64(self._n_arg), _p(self.records), c_p(None), c_u32(3), _p(self.bg),
                  c_p(None), c_u32(W), c_u32(H), c_u32(16),
                  _p(self.viewmat), _p(self.Kmat), _p(self.offsets), _p(self.flatten_ids), self._tile_order_arg,
                  _p(self.alpha), _p(self.last_ids), _p(self.v_render), _p(self.v_alpha), ws, wsn, s)
        if self.fused_update:
            return
        self._run("rasterize_bwd_finish", lb.gsx_rasterize_bwd_finish, c_u32(N), _p(P["means"]), _p(A["quats"]),
                  _p(A["scales"]), _p(self.viewmat), ws, wsn, c_i(1), c_u32(3), _p(G["means"]), _p(V["quats"]),
                  _p(V["scales"]),
                  _p(self.v_colors), _p(V["opacities"]), s)
        self._run("sh_colors_from_world_bwd", lb.gsx_sh_colors_from_world_bwd, c_u32(N), c_u32(self.K), c_u32(self.sh_degree), _p(P["means"]),
                                              _p(J["radii"]), _p(self.viewmat), _p(self.colors), _p(self.v_colors),
                                              _p(G["shs"]), s)
        self._run("activate_params_bwd", lb.gsx_activate_params_bwd, c_u32(N), _p(P["opacity"]), _p(P["scaling"]), _p(P["rotation"]),
                                         _p(V["opacities"]), _p(V["scales"]), _p(V["quats"]), _p(G["opacity"]),
                                         _p(G["scaling"]), _p(G["rotation"]), s)
        self.regularization_losses(with_grads=True)

    def regularization_losses(self, with_grads=False):
        """Trainer::compute_scale_reg_loss / compute_opacity_reg_loss (trainer.cpp:136-174): the two loss values land
        in self.reg_losses (device); with_grads adds their gradients onto self.grads (the fused update adds them
        itself and only needs this call when the loss values are wanted)."""
        s = self._stream()
        P, G = self.params, self.grads
        if self.scale_reg > 0.0:
            self._run("exp_l1_regularization", self.lib.gsx_exp_l1_regularization, _p(P["scaling"]),
                      _p(G["scaling"]) if with_grads else c_p(None), c_i64(P["scaling"].numel()),
                      c_f(self.scale_reg), _p(self.reg_partials), c_p(self.reg_losses.data_ptr()), s)
        if self.opacity_reg > 0.0:
            self._run("sigmoid_l1_regularization", self.lib.gsx_sigmoid_l1_regularization, _p(P["opacity"]),
                      _p(G["opacity"]) if with_grads else c_p(None), c_i64(P["opacity"].numel()),
                      c_f(self.opacity_reg), _p(self.reg_partials), c_p(self.reg_losses.data_ptr() + 4), s)
        return self.reg_losses

    # -- optimiser ------------------------------------------------------------------------------------
    def adam(self):
        """FusedAdam::step (fused_adam.cpp:22-95): all groups share the step count here (all have gradients every
        iteration); the shN part of the SH tensor is frozen while iteration <= 1000 (:69-70)."""
        self.step_count += 1
        t = self.step_count
        b1, b2 = self.betas
        bc1 = 1.0 / (1.0 - math.pow(b1, t))
        bc2 = 1.0 / math.sqrt(1.0 - math.pow(b2, t))
        if self.fused_update:
            P, M, V = self.params, self.exp_avg, self.exp_avg_sq
            skip = 1 if self.iteration <= 1000 and self.freeze_shN_early else 0
            a = L.UpdateArgs(
                self.N, self.K, self.sh_degree, P["means"].data_ptr(), P["opacity"].data_ptr(),
                P["scaling"].data_ptr(), P["rotation"].data_ptr(), P["shs"].data_ptr(), M["means"].data_ptr(),
                M["opacity"].data_ptr(), M["scaling"].data_ptr(), M["rotation"].data_ptr(), M["shs"].data_ptr(),
                V["means"].data_ptr(), V["opacity"].data_ptr(), V["scaling"].data_ptr(), V["rotation"].data_ptr(),
                V["shs"].data_ptr(), self.proj["radii"].data_ptr(), self.colors.data_ptr(), self.viewmat.data_ptr(),
                self.ws_bwd.data_ptr(), self.lrs["means"], self.lrs["sh0"], self.lrs["shN"], self.lrs["scaling"],
                self.lrs["rotation"], self.lrs["opacity"], b1, b2, self.eps, bc1, bc2, skip,
                # weight / element count in float32, as the separate regularisation kernels form it
                float(np.float32(self.scale_reg) / np.float32(3 * self.N)) if self.scale_reg > 0.0 else 0.0,
                float(np.float32(self.opacity_reg) / np.float32(self.N)) if self.opacity_reg > 0.0 else 0.0,
                self._lists_error if self._lists_active else None, None,
                self.hold_report.data_ptr() if self._lists_active else None)
            self._run("backward_update_fused", self.lib.gsx_backward_update_fused, ctypes.byref(a), self._stream())
            return
        names = ["means", "shs", "scaling", "rotation", "opacity"]
        lr_of = dict(means=self.lrs["means"], shs=self.lrs["sh0"], scaling=self.lrs["scaling"],
                     rotation=self.lrs["rotation"], opacity=self.lrs["opacity"])
        arr = (L.AdamGroup * len(names))()
        for i, k in enumerate(names):
            p = self.params[k]
            g = L.AdamGroup(p.data_ptr(), self.exp_avg[k].data_ptr(), self.exp_avg_sq[k].data_ptr(),
                            self.grads[k].data_ptr(), p.numel(), lr_of[k], b1, b2, self.eps, bc1, bc2)
            if k == "shs" and self.K > 1:
                g.period, g.split = self.K * 3, 3
                g.lr2 = self.lrs["shN"]
                g.skip2 = 1 if self.iteration <= 1000 and self.freeze_shN_early else 0
            arr[i] = g
        self._run("adam_step_multi", self.lib.gsx_adam_step_multi, arr, c_i(len(names)), self._stream())

    order_tiles = True  # visit the tiles longest list first (gsx_tile_order)
    freeze_shN_early = False  # BASELINE's step updates all parameter tensors; set True for the product schedule

    # -- MCMC strategy steps that touch the parameters ------------------------------------------------
    def add_new_gs(self, sampled_idxs, binoms, min_opacity=0.005):
        """MCMC::add_new_gs (mcmc.cpp:192-347) for sampled sources chosen by the caller: the tensors grow by
        len(sampled_idxs) rows (copies of the sampled Gaussians after the Eq. 9 rebalancing, zero moments)."""
        n_new = int(sampled_idxs.numel())
        if n_new == 0:
            return 0
        old_n = self.N
        grow = lambda t: torch.cat([t, torch.zeros((n_new,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)])
        for d in (self.params, self.exp_avg, self.exp_avg_sq, self.grads):
            for k in d:
                d[k] = grow(d[k])
        self._allocate_per_gaussian(old_n + n_new)
        new_rows = torch.arange(old_n, old_n + n_new, dtype=torch.int64, device=self.dev)
        return self.relocate(sampled_idxs, new_rows, binoms, min_opacity, state_role=2)

    def relocate(self, sampled_idxs, dead_idxs, binoms, min_opacity=0.005, state_role=1):
        """MCMC::relocate_gs (mcmc.cpp:112-190) for index sets chosen by the caller (the multinomial draw of :132 is
        the caller's): sampled Gaussians get the Eq. 9 opacity / scales, dead ones become copies of them, the Adam
        moments of the sampled ones are cleared.  sampled_idxs / dead_idxs: int64 device tensors of equal length."""
        n = int(sampled_idxs.numel())
        assert n == int(dead_idxs.numel()) and sampled_idxs.dtype == dead_idxs.dtype == torch.int64
        if n == 0:
            return 0
        names = ["means", "shs", "scaling", "rotation", "opacity"]
        tensors = [(self.params[k], 0) for k in names]
        tensors += [(self.exp_avg[k], state_role) for k in names] + [(self.exp_avg_sq[k], state_role) for k in names]
        arr = (L.RowTensor * len(tensors))()
        for i, (t, is_state) in enumerate(tensors):
            arr[i] = L.RowTensor(t.data_ptr(), t.numel() // self.N, is_state)
        nbytes = self.lib.gsx_mcmc_relocate_workspace_bytes(c_u32(self.N), c_u32(n))
        if getattr(self, "ws_mcmc", None) is None or self.ws_mcmc.numel() < nbytes:
            self.ws_mcmc = torch.empty(nbytes, dtype=torch.uint8, device=self.dev)
        self._run("mcmc_relocate", self.lib.gsx_mcmc_relocate, c_u32(self.N), c_u32(n), _p(sampled_idxs),
                  _p(dead_idxs), _p(binoms), c_i(binoms.shape[0]), c_f(min_opacity), _p(self.params["opacity"]),
                  _p(self.params["scaling"]), arr, c_i(len(tensors)), _p(self.ws_mcmc), c_sz(self.ws_mcmc.numel()),
                  self._stream())
        return n

    def inject_noise(self, noise=None, noise_lr=5e5, seed=0):
        """MCMC::inject_noise (mcmc.cpp:349-367): with the caller's N(0,1) draws [N,3], or (noise = None) with draws
        generated inside the kernel from (seed, iteration, row) - no [N,3] tensor is written and read back."""
        P = self.params
        if noise is None:
            self._run("add_noise_philox", self.lib.gsx_add_noise_philox, c_i(self.N), _p(P["opacity"]),
                      _p(P["scaling"]), _p(P["rotation"]), _p(P["means"]), c_f(self.lrs["means"] * noise_lr),
                      ctypes.c_uint64(seed), ctypes.c_uint64(self.iteration), self._stream())
            return
        self._run("add_noise", self.lib.gsx_add_noise, c_i(self.N), _p(P["opacity"]), _p(P["scaling"]),
                  _p(P["rotation"]), _p(noise), _p(P["means"]), c_f(self.lrs["means"] * noise_lr), self._stream())

    loss_pending = False

    def step(self, viewmat, K, W, H, gt_chw):
        self._check_capacity()
        self.iteration += 1
        self.forward(viewmat, K, W, H)
        self.loss_forward(gt_chw, finish=not self.fused_loss)
        self.backward()
        self.adam()
        if self.loss_pending:  # the next step's loss pass overwrites the partial sums: rejoin the side stream
            torch.cuda.current_stream(self.dev).wait_event(self.ev_loss_join)
            self.loss_pending = False
        return self.loss_out
