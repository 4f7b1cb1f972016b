"""GPU parity of the whole training iteration (activations -> fused forward -> loss -> backward -> Adam) against
the CPU restatement of the same iteration, on a reduced-size instance of the measured configuration."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


from step_checks import check_first_step, check_forward_bit_exact, check_loss, check_params_close  # noqa: E402


@pytest.mark.parametrize("cfg,n,use_ssim,reg", [(1, 10_000, False, 0.0), (3, 30_000, True, 0.0),
                                                (3, 20_000, True, 0.01)])
def test_train_step_matches_oracle(gsx, orc, cuda, cfg, n, use_ssim, reg):
    from lichtfeld_studio_amd.trainer import TrainStep
    from oracle.step import OracleTrainStep
    sc = gsx.scenes.config(cfg, n)
    if cfg == 3:
        # reduced instance: fewer, larger Gaussians and a smaller image so that the CPU side takes seconds
        sc.scaling_raw += 1.2
        sc.target_scene.scaling_raw += 1.2
        sc.cameras = [gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)]
    cam = sc.cameras[0]
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    if cfg == 1:
        gt = sc.target
    else:
        tg = OracleTrainStep(sc.target_scene)
        gt = np.ascontiguousarray(np.clip(tg.forward(cam.viewmat, cam.K, W, H)[0], 0, 1).transpose(2, 0, 1))
    # reg: the MCMC defaults of the scale / opacity L1 terms (trainer.cpp:136-174)
    ts = TrainStep(sc, cuda, use_ssim=use_ssim, scale_reg=reg, opacity_reg=reg)
    ref = OracleTrainStep(sc, lambda_dssim=0.2 if use_ssim else 0.0, scale_reg=reg, opacity_reg=reg)
    gt_d = torch.from_numpy(gt[None].copy()).to(cuda)

    from oracle.checks import step_with_truth
    for it in range(2):
        ts.step(vm, Km, W, H, gt_d)
        truth = step_with_truth(ref, cam.viewmat, cam.K, W, H, gt)
        torch.cuda.synchronize()
        if it == 0:
            check_forward_bit_exact(ts, ref)
            check_loss(ts, ref)
            check_first_step(ts, ref, truth, tag=f"step cfg{cfg} n={n} reg={reg}: ")
            if reg:
                # loss values of the two terms on the updated parameters (which agree to the Adam tolerance)
                got = [float(x) for x in ts.regularization_losses().cpu()]
                want = [orc.l1_regularization("exp", ref.params["scaling"], None, reg),
                        orc.l1_regularization("sigmoid", ref.params["opacity"], None, reg)]
                assert np.allclose(got, want, rtol=1e-4, atol=0), (got, want)
        else:
            # the second iteration starts from parameters that already differ in the last bits (Adam state is only
            # toleranced), so a few alpha-threshold decisions may differ: loss and parameters are compared, the
            # element-wise gradient bars apply to the first iteration
            loss = [float(x) for x in ts.loss_out.cpu()]
            assert abs(loss[0] - ref.loss[0]) <= 1e-5 and abs(loss[2] - ref.loss[2]) <= 1e-5, (loss, ref.loss)
            check_params_close(ts, ref, 2, 5e-3)


@pytest.mark.parametrize("cfg,n,freeze,reg", [(1, 10_000, False, 0.0), (3, 30_000, False, 0.0),
                                              (3, 30_001, True, 0.0), (3, 20_003, False, 0.01),
                                              (3, 37, True, 0.0), (3, 130, False, 0.01)])
def test_fused_update_equals_separate_kernels(gsx, cuda, cfg, n, freeze, reg):
    """epilogue + SH backward + activation VJPs + Adam in one pass (gsx_backward_update_fused) leaves parameters and
    both moments bit-identical to the separate kernels, over three iterations (K = 1 and K = 16 paths, with and
    without the frozen shN group, Gaussian counts that are not a multiple of the block size or of a wave - down to
    less than one wave -, with the scale / opacity regularisation gradients folded in)"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(cfg, n)
    if cfg == 3:
        sc.scaling_raw += 1.2
        sc.cameras = [gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)]
    cam = sc.cameras[0]
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(3)).to(cuda)
    a = TrainStep(sc, cuda, use_ssim=cfg != 1, fused_update=False, scale_reg=reg, opacity_reg=reg)
    b = TrainStep(sc, cuda, use_ssim=cfg != 1, fused_update=True, scale_reg=reg, opacity_reg=reg)
    a.freeze_shN_early = b.freeze_shN_early = freeze
    for it in range(3):
        a.step(vm, Km, W, H, gt)
        b.step(vm, Km, W, H, gt)
        torch.cuda.synchronize()
        # the backward accumulators are summed with atomics, so two runs agree to rounding, not bitwise: feed the
        # fused tail the SAME accumulators to compare the tails themselves
        if it == 0:
            for k in a.params:
                d = (a.params[k] - b.params[k]).abs().max().item()
                assert d <= 2.1 * max(a.lrs.values()), k
    # exact comparison of the two tails on identical inputs
    a2 = TrainStep(sc, cuda, use_ssim=cfg != 1, fused_update=False, scale_reg=reg, opacity_reg=reg)
    b2 = TrainStep(sc, cuda, use_ssim=cfg != 1, fused_update=True, scale_reg=reg, opacity_reg=reg)
    a2.freeze_shN_early = b2.freeze_shN_early = freeze
    for it in range(2):
        for ts in (a2, b2):
            ts.iteration += 1
            ts.forward(vm, Km, W, H)
            ts.loss_forward(gt)
        a2.fused_update = True   # stop the separate path after the accumulation as well
        a2.backward()
        a2.fused_update = False
        b2.backward()
        b2.ws_bwd.copy_(a2.ws_bwd)  # identical accumulators
        # separate tail on a2
        lb, s, N_ = a2.lib, a2._stream(), a2.N
        import ctypes
        from lichtfeld_studio_amd.trainer import _p
        from lichtfeld_studio_amd._lib import c_i, c_sz, c_u32, check
        P, A, J, G, V = a2.params, a2.act, a2.proj, a2.grads, a2.v_act
        ws, wsn = _p(a2.ws_bwd), c_sz(a2.ws_bwd.numel())
        check(lb.gsx_rasterize_bwd_finish(c_u32(N_), _p(P["means"]), _p(A["quats"]), _p(A["scales"]), _p(a2.viewmat),
                                          ws, wsn, c_i(1), c_u32(3), _p(G["means"]), _p(V["quats"]),
                                          _p(V["scales"]), _p(a2.v_colors), _p(V["opacities"]), s))
        check(lb.gsx_sh_colors_from_world_bwd(c_u32(N_), c_u32(a2.K), c_u32(a2.sh_degree), _p(P["means"]),
                                              _p(J["radii"]), _p(a2.viewmat), _p(a2.colors), _p(a2.v_colors),
                                              _p(G["shs"]), s))
        check(lb.gsx_activate_params_bwd(c_u32(N_), _p(P["opacity"]), _p(P["scaling"]), _p(P["rotation"]),
                                         _p(V["opacities"]), _p(V["scales"]), _p(V["quats"]), _p(G["opacity"]),
                                         _p(G["scaling"]), _p(G["rotation"]), s))
        a2.regularization_losses(with_grads=True)
        a2.adam()
        b2.adam()
        torch.cuda.synchronize()
        for k in a2.params:
            for name, x, y in (("param", a2.params[k], b2.params[k]), ("exp_avg", a2.exp_avg[k], b2.exp_avg[k]),
                               ("exp_avg_sq", a2.exp_avg_sq[k], b2.exp_avg_sq[k])):
                assert torch.equal(x.view(torch.int32), y.view(torch.int32)), f"{name} {k} iteration {it}"
        assert float(b2.ws_bwd.view(torch.float32).abs().max()) == 0.0  # accumulators left cleared
        # keep the two states identical for the next iteration (they are, bit for bit)


@pytest.mark.parametrize("W,H", [(309, 205), (64, 48), (9, 7)])
def test_fused_loss_equals_separate_kernels(gsx, cuda, W, H):
    """gsx_photometric_loss_forward / _backward against image_from_render + fusedssim + partials + fusedssim_backward
    + render_grad_from_loss: same d loss / d render per pixel, same loss up to summation order (ragged image sizes,
    an image smaller than the SSIM window: no valid crop)"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(3, 20_000)
    sc.scaling_raw += 1.2
    cam = gsx.scenes.orbit_camera(0.7, 4.0, W, H, 0.93 * W)
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(5)).to(cuda)
    a = TrainStep(sc, cuda, fused_loss=False)
    b = TrainStep(sc, cuda, fused_loss=True)
    for ts in (a, b):
        ts.forward(vm, Km, W, H)
        # push part of the render outside [0, 1] so that the clamp and its VJP matter
        ts.render.mul_(1.6).sub_(0.1)
        ts.loss_forward(gt)
        ts.backward()
    torch.cuda.synchronize()
    la, lb = a.loss_out.cpu().numpy(), b.loss_out.cpu().numpy()
    assert np.abs(la - lb).max() <= 2e-6, (la, lb)
    va, vb = a.v_render.cpu().numpy(), b.v_render.cpu().numpy()
    assert (va != 0).mean() > 0.3
    assert np.abs(va - vb).max() <= 1e-6 * np.abs(va).max()
    assert np.array_equal(va == 0, vb == 0)  # the clamp mask


@pytest.mark.parametrize("W,H,tw,th", [(309, 205, 401, 10), (64, 48, 4, 3), (9, 7, 1, 1), (1237, 822, 78, 52)])
def test_loss_backward_that_also_orders_the_tiles(gsx, cuda, W, H, tw, th):
    """gsx_photometric_loss_backward_order = gsx_photometric_loss_backward_finish (d loss / d render and the loss
    value bit for bit) + gsx_tile_order by cost (a permutation of the tiles, cost classes falling), in one launch;
    tile grids of every size beside images of every size (the extra workgroup does not depend on the image)"""
    from lichtfeld_studio_amd._lib import c_f, c_p, c_u32, check, lib
    L = lib()
    g = torch.Generator().manual_seed(W * 7 + tw)
    render = (torch.rand((H, W, 3), generator=g) * 1.6 - 0.3).to(cuda)
    gt = torch.rand((3, H, W), generator=g).to(cuda)
    dm = [torch.empty((3, H, W), dtype=torch.float32, device=cuda) for _ in range(3)]
    n_part = L.gsx_photometric_partials(c_u32(H), c_u32(W))
    l1p, ssp = (torch.empty(n_part, dtype=torch.float32, device=cuda) for _ in range(2))
    s = c_p(torch.cuda.current_stream(cuda).cuda_stream)
    P = lambda t: c_p(t.data_ptr())
    check(L.gsx_photometric_loss_forward(c_u32(H), c_u32(W), c_f(1e-4), c_f(9e-4), P(render), P(gt), P(dm[0]),
                                         P(dm[1]), P(dm[2]), P(l1p), P(ssp), s))
    rng = np.random.default_rng(tw * 31 + th)
    T = tw * th
    cost = np.concatenate([np.zeros(T // 10, np.int64), rng.integers(0, 40, T - T // 10 - T // 5),
                           rng.integers(0, 1 << 21, T // 5)])[:T]
    cost = np.resize(cost, T)
    rng.shuffle(cost)
    cost_d = torch.from_numpy(cost.astype(np.int32)).to(cuda)
    out = {}
    for name in ("finish", "order"):
        v = torch.full((H, W, 3), 7.0, dtype=torch.float32, device=cuda)
        loss = torch.full((3,), -1.0, dtype=torch.float32, device=cuda)
        order = torch.full((T,), -1, dtype=torch.int32, device=cuda)
        common = (c_u32(H), c_u32(W), c_f(0.2), P(render), P(gt), P(dm[0]), P(dm[1]), P(dm[2]), P(l1p), P(ssp),
                  P(loss), P(v))
        if name == "finish":
            check(L.gsx_photometric_loss_backward_finish(*common, s))
        else:
            check(L.gsx_photometric_loss_backward_order(*common, c_u32(tw), c_u32(th), P(cost_d), P(order), s))
        torch.cuda.synchronize()
        out[name] = (v.cpu().numpy(), loss.cpu().numpy(), order.cpu().numpy().astype(np.int64))
    assert np.array_equal(out["finish"][0].view(np.int32), out["order"][0].view(np.int32))
    assert np.array_equal(out["finish"][1].view(np.int32), out["order"][1].view(np.int32))
    assert (out["finish"][0] != 0).any() and np.all(out["finish"][2] == -1)
    o = out["order"][2]
    assert np.array_equal(np.sort(o), np.arange(T))

    def klass(n):  # 16 classes per octave
        if n == 0:
            return 0
        e = int(n).bit_length() - 1
        m = (n >> (e - 4)) & 15 if e >= 4 else (n << (4 - e)) & 15
        return e * 16 + m + 1
    assert np.all(np.diff(np.array([klass(int(n)) for n in cost[o]])) <= 0)
    # the same order (up to the order inside a class) as the kernel of its own
    ref = torch.full((T,), -1, dtype=torch.int32, device=cuda)
    from lichtfeld_studio_amd._lib import c_i64
    check(L.gsx_tile_order(c_i64(-1), c_p(None), P(cost_d), c_u32(tw), c_u32(th), P(ref), s))
    r = ref.cpu().numpy().astype(np.int64)
    assert np.array_equal(np.array([klass(int(n)) for n in cost[o]]), np.array([klass(int(n)) for n in cost[r]]))
    # null tile tensors are refused
    with pytest.raises(gsx._lib.GsxError):
        check(L.gsx_photometric_loss_backward_order(*common, c_u32(tw), c_u32(th), c_p(None), P(order), s))


@pytest.mark.parametrize("n", [1, 255, 300_001, 3_000_000])
def test_l1_regularization_kernels(gsx, orc, cuda, n):
    """gsx_exp_l1_regularization / gsx_sigmoid_l1_regularization: gradients added onto existing ones bit for bit as
    the checker adds them, loss = weight * mean to 2e-6 relative (summation order differs); without a gradient
    tensor only the loss is produced; weight 0 touches nothing"""
    from lichtfeld_studio_amd._lib import c_f, c_i64, c_p, check, lib
    L = lib()
    rng = np.random.default_rng(n)
    x = rng.normal(-2.0, 2.0, n).astype(np.float32)
    g0 = rng.normal(0, 1e-3, n).astype(np.float32)
    xd = torch.from_numpy(x).to(cuda)
    partials = torch.empty(L.gsx_l1_regularization_partials(), dtype=torch.float32, device=cuda)
    s = c_p(torch.cuda.current_stream(cuda).cuda_stream)
    for mode, fn in (("exp", L.gsx_exp_l1_regularization), ("sigmoid", L.gsx_sigmoid_l1_regularization)):
        want_g = g0.copy()
        want_loss = orc.l1_regularization(mode, x, want_g, 0.01)
        gd = torch.from_numpy(g0).to(cuda)
        out = torch.full((2,), -7.0, dtype=torch.float32, device=cuda)
        check(fn(c_p(xd.data_ptr()), c_p(gd.data_ptr()), c_i64(n), c_f(0.01), c_p(partials.data_ptr()),
                 c_p(out.data_ptr()), s))
        check(fn(c_p(xd.data_ptr()), c_p(None), c_i64(n), c_f(0.01), c_p(partials.data_ptr()),
                 c_p(out.data_ptr() + 4), s))
        torch.cuda.synchronize()
        assert np.array_equal(gd.cpu().numpy().view(np.int32), want_g.view(np.int32)), mode
        got = out.cpu().numpy()
        assert got[0] == got[1]
        assert abs(got[0] - want_loss) <= 2e-6 * abs(want_loss), (mode, got, want_loss)
        before = gd.clone()
        out.fill_(-7.0)
        check(fn(c_p(xd.data_ptr()), c_p(gd.data_ptr()), c_i64(n), c_f(0.0), c_p(partials.data_ptr()),
                 c_p(out.data_ptr()), s))
        torch.cuda.synchronize()
        assert torch.equal(before, gd) and float(out[0]) == -7.0


def test_speculative_emission_and_overlap_change_nothing(gsx, cuda):
    """the step with the second stream and the early, capacity-bounded tile emission produces the same image and
    parameters bit for bit as the single-stream step; when the buffers turn out too small (capacity forced down)
    only their first `capacity` entries are written early and the emission is repeated after they have grown"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(3, 20_000)
    sc.scaling_raw += 1.2
    cam = gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(3)).to(cuda)
    a = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=False)
    b = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=True)
    for it in range(3):
        if it == 2:
            b.cap = 1000  # far below the ~1e5 intersections: the early emission must stop at 1000 entries
            b.keys[0][1000:].fill_(-1)
        a.forward(vm, Km, W, H)
        b.forward(vm, Km, W, H)
        torch.cuda.synchronize()
        assert a.n_isects == b.n_isects and a.n_isects > 50_000
        assert torch.equal(a.isect_ids[:a.n_isects], b.isect_ids[:b.n_isects])
        assert torch.equal(a.flatten_ids[:a.n_isects], b.flatten_ids[:b.n_isects])
        assert torch.equal(a.render, b.render)
        for ts in (a, b):
            ts.iteration += 1
            ts.loss_forward(gt)
            ts.backward()
        b.ws_bwd.copy_(a.ws_bwd)  # the accumulators are atomic sums: give both tails the same ones
        a.adam()
        b.adam()
        if b.loss_pending:
            torch.cuda.current_stream(cuda).wait_event(b.ev_loss_join)
            b.loss_pending = False
        torch.cuda.synchronize()
        assert torch.equal(a.loss_out, b.loss_out)
        for k in a.params:
            assert torch.equal(a.params[k], b.params[k]), k


def test_pair_count_on_the_device_changes_nothing(gsx, cuda):
    """the step whose tile lists come from gsx_tile_lists (count on the device, no host wait) against the step that
    fetches the count: keys, order, ranges, image and loss bit for bit in every iteration; parameters bit for bit
    when both tails are given the same accumulators"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(3, 20_000)
    sc.scaling_raw += 1.2
    cam = gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(3)).to(cuda)
    a = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=False)
    b = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=True, device_count=True)
    for it in range(4):
        a.forward(vm, Km, W, H)
        b._check_capacity()
        b.forward(vm, Km, W, H)
        torch.cuda.synchronize()
        assert b._lists_active == (it > 0), "the first iteration sizes the buffers with the count on the host"
        assert a.n_isects == b.n_isects and a.n_isects > 50_000
        assert torch.equal(a.isect_ids[:a.n_isects], b.isect_ids[:b.n_isects])
        assert torch.equal(a.flatten_ids[:a.n_isects], b.flatten_ids[:b.n_isects])
        assert torch.equal(a.offsets, b.offsets) and int(b.offsets_full[-1]) == a.n_isects or it == 0
        assert torch.equal(a.render, b.render) and torch.equal(a.last_ids, b.last_ids)
        for ts in (a, b):
            ts.iteration += 1
            ts.loss_forward(gt)
            ts.backward()
        b.ws_bwd.copy_(a.ws_bwd)  # the accumulators are atomic sums: give both tails the same ones
        a.adam()
        b.adam()
        if b.loss_pending:
            torch.cuda.current_stream(cuda).wait_event(b.ev_loss_join)
            b.loss_pending = False
        torch.cuda.synchronize()
        assert torch.equal(a.loss_out, b.loss_out)
        for k in a.params:
            assert torch.equal(a.params[k], b.params[k]), k
    assert b.lists_error() == (0, 0)


def test_loss_value_from_the_backward_loss_kernel(gsx, cuda):
    """a whole step leaves the loss reduction to the backward loss kernel (its first workgroup adds up the partial
    sums): loss, L1 and SSIM terms, d loss / d render and the parameters equal, bit for bit, those of the path with
    the separate reduction launch"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(3, 20_000)
    sc.scaling_raw += 1.2
    cam = gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(5)).to(cuda)
    for overlap in (False, True):
        a = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=overlap)
        b = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=overlap)
        for it in range(2):
            a.iteration += 1
            a.forward(vm, Km, W, H)
            a.loss_forward(gt)  # with its own reduction launch
            a.backward()
            b.iteration += 1
            b.forward(vm, Km, W, H)
            b.loss_out.fill_(-1.0)
            b.loss_forward(gt, finish=False)
            b.backward()
            torch.cuda.synchronize()
            assert torch.equal(a.loss_out, b.loss_out) and float(b.loss_out[0]) > 0, (overlap, it)
            assert torch.equal(a.v_render, b.v_render)
            b.ws_bwd.copy_(a.ws_bwd)
            for ts in (a, b):
                ts.adam()
                if ts.loss_pending:
                    torch.cuda.current_stream(cuda).wait_event(ts.ev_loss_join)
                    ts.loss_pending = False
        torch.cuda.synchronize()
        for k in a.params:
            assert torch.equal(a.params[k], b.params[k]), k


def test_pairs_outgrowing_the_buffers_hold_the_step_back(gsx, cuda):
    """count on the device, and a camera that suddenly sees several times the pairs the buffers hold: that step
    renders nothing, the optimiser leaves parameters and moments untouched, and the next step starts with larger
    buffers and with the held step counted back out - after which the state equals the one of a run whose buffers
    were large enough from the start"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(3, 20_000)
    sc.scaling_raw += 1.2
    far = gsx.scenes.orbit_camera(0.7, 9.0, 309, 205, 287.0)
    near = gsx.scenes.orbit_camera(0.7, 3.0, 309, 205, 287.0)
    W, H = far.width, far.height
    t = lambda a: torch.from_numpy(a[None].copy()).to(cuda)
    cams = [(t(far.viewmat), t(far.K)), (t(near.viewmat), t(near.K))]
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(3)).to(cuda)
    a = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=True, device_count=True)
    b = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=True)
    a.step(*cams[0], W, H, gt)
    b.step(*cams[0], W, H, gt)
    torch.cuda.synchronize()
    n_far, cap_far = a.n_isects, a.cap
    before = {k: v.clone() for k, v in a.params.items()}
    m_before = {k: v.clone() for k, v in a.exp_avg.items()}
    a.step(*cams[1], W, H, gt)  # does not fit
    torch.cuda.synchronize()
    assert a.n_isects > cap_far > n_far, (a.n_isects, cap_far, n_far)
    assert a.lists_error() == (1, 1)
    assert float(a.alpha.max()) == 0.0, "a step that does not fit renders nothing"
    for k in before:
        assert torch.equal(a.params[k], before[k]) and torch.equal(a.exp_avg[k], m_before[k]), k
    assert a.step_count == 2
    a.step(*cams[1], W, H, gt)  # grows the buffers, forgets the held step, runs it again
    b.step(*cams[1], W, H, gt)
    torch.cuda.synchronize()
    assert a.steps_held == 1 and a.step_count == b.step_count == 2 and a.iteration == b.iteration == 2
    assert a.cap >= a.n_isects == b.n_isects and a.lists_error() == (0, 0)
    # the two runs add up the first step's gradients in different (atomic) orders: the parameters the second step
    # renders agree to rounding, not to the bit
    diff = (a.render - b.render).abs()
    assert float(diff.max()) <= 2e-3 and float((diff > 2e-6).float().mean()) < 1e-2, float(diff.max())
    for k in a.params:
        assert torch.allclose(a.params[k], b.params[k], rtol=0, atol=2.2 * a.lrs["opacity"]), k
        close = (a.params[k] - b.params[k]).abs() <= 1e-6 + 1e-3 * a.lrs["opacity"]
        assert close.float().mean() > 0.999, k


@pytest.mark.parametrize("n,degree,cfg", [(1, 3, 3), (300, 0, 3), (70_001, 3, 3), (40_000, 2, 3), (5_000, 0, 1)])
def test_one_front_pass(gsx, cuda, n, degree, cfg):
    """activations + projection + SH colours + records as one launch: every output equals, bit for bit, what the
    separate launches write (records and projection outputs of Gaussians that touch no tile are never written by
    either and are not compared).  Configuration 1 has one SH coefficient per Gaussian: the entry point then runs the
    two launches itself."""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(cfg, n)
    sc.scaling_raw += 0.8
    cam = gsx.scenes.orbit_camera(1.1, 4.0, 413, 277, 380.0)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    a = TrainStep(sc, cuda, fused_update=True, fused_loss=True, sh_degree=degree, one_front_pass=False)
    b = TrainStep(sc, cuda, fused_update=True, fused_loss=True, sh_degree=degree, one_front_pass=True)
    for ts in (a, b):
        ts.records.zero_()
        for t in ts.proj.values():
            t.zero_()
        ts.forward(vm, Km, W, H)
    torch.cuda.synchronize()
    assert a.n_isects == b.n_isects
    for k in ("opacities", "scales", "quats"):
        assert torch.equal(a.act[k], b.act[k]), k
    for k in a.proj:
        assert torch.equal(a.proj[k], b.proj[k]), k
    assert torch.equal(a.colors, b.colors)
    assert torch.equal(a.records, b.records)
    assert torch.equal(a.render, b.render) and torch.equal(a.last_ids, b.last_ids)
    if n > 1000 and cfg == 3:
        live = (a.proj["radii"].reshape(-1, 2) > 0).all(-1)
        assert 0.05 < float(live.float().mean()) < 0.95  # both kinds of Gaussian are present


def test_tile_visiting_order(gsx, cuda):
    """gsx_tile_order returns a permutation of the tiles with the list lengths falling from class to class (16 classes
    per octave); rasterizing in that order changes nothing: forward outputs bit for bit, backward accumulators to
    atomic-order rounding"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(3, 30_000)
    sc.scaling_raw += 1.0
    cam = gsx.scenes.orbit_camera(0.4, 4.0, 413, 277, 380.0)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(5)).to(cuda)
    a = TrainStep(sc, cuda, fused_update=True, fused_loss=True)
    b = TrainStep(sc, cuda, fused_update=True, fused_loss=True)
    a.order_tiles, b.order_tiles = False, True
    for ts in (a, b):
        ts.forward(vm, Km, W, H)
        ts.iteration += 1
        ts.loss_forward(gt)
        ts.backward()
    torch.cuda.synchronize()
    T = a.tw * a.th
    order = b.tile_order.cpu().numpy().astype(np.int64)
    assert np.array_equal(np.sort(order), np.arange(T))
    # after the forward pass the order is by what the pass reported per tile: entries up to the last contributor
    off = b.offsets.cpu().numpy().reshape(-1).astype(np.int64)
    last = b.last_ids.cpu().numpy()[0].astype(np.int64)
    alpha = b.alpha.cpu().numpy()[0, :, :, 0]
    walk = np.zeros(T, np.int64)
    for ty in range(b.th):
        for tx in range(b.tw):
            blk = (slice(ty * 16, (ty + 1) * 16), slice(tx * 16, (tx + 1) * 16))
            hit = alpha[blk] > 0
            if hit.any():
                walk[ty * b.tw + tx] = last[blk][hit].max() - off[ty * b.tw + tx] + 1
    assert np.array_equal(b.tile_walk.cpu().numpy().astype(np.int64), walk)
    assert walk.max() > 2 * max(1, int(np.median(walk)))  # uneven costs
    visited = walk[order]

    def klass(n):  # 16 classes per octave
        if n == 0:
            return 0
        e = int(n).bit_length() - 1
        m = (n >> (e - 4)) & 15 if e >= 4 else (n << (4 - e)) & 15
        return e * 16 + m + 1
    classes = np.array([klass(int(n)) for n in visited])
    assert np.all(np.diff(classes) <= 0)
    # lists of every size class, empty ones and a few very long ones, through the C ABI alone
    import ctypes
    from lichtfeld_studio_amd._lib import c_i64, c_p, c_u32, check, lib
    rng = np.random.default_rng(1)
    lens2 = np.concatenate([np.zeros(300, np.int64), rng.integers(0, 40, 3000), rng.integers(0, 5000, 700),
                            [1, 15, 16, 17, 31, 32, 33, 1 << 20, (1 << 20) + 1, 3 << 19]])
    rng.shuffle(lens2)
    tw2, th2 = 401, 10
    assert lens2.size == tw2 * th2
    off2 = torch.from_numpy(np.concatenate([[0], np.cumsum(lens2)[:-1]]).astype(np.int32)).to(cuda)
    out2 = torch.full((lens2.size,), -1, dtype=torch.int32, device=cuda)
    stream = c_p(torch.cuda.current_stream(cuda).cuda_stream)
    cost2 = torch.from_numpy(lens2.astype(np.int32)).to(cuda)
    for offsets_arg, cost_arg in ((c_p(off2.data_ptr()), c_p(None)), (c_p(None), c_p(cost2.data_ptr()))):
        out2.fill_(-1)
        check(lib().gsx_tile_order(c_i64(int(lens2.sum())), offsets_arg, cost_arg, c_u32(tw2), c_u32(th2),
                                   c_p(out2.data_ptr()), stream))
        o2 = out2.cpu().numpy().astype(np.int64)
        assert np.array_equal(np.sort(o2), np.arange(lens2.size))
        assert np.all(np.diff(np.array([klass(int(n)) for n in lens2[o2]])) <= 0)
        assert klass(int(lens2[o2[0]])) == klass(3 << 19)
    assert torch.equal(a.render, b.render) and torch.equal(a.alpha, b.alpha) and torch.equal(a.last_ids, b.last_ids)
    ga = a.ws_bwd.view(torch.float32).cpu().numpy().astype(np.float64)
    gb = b.ws_bwd.view(torch.float32).cpu().numpy().astype(np.float64)
    assert np.abs(ga).max() > 0 and np.abs(ga - gb).max() <= 1e-4 * np.abs(ga).max()
