"""The two C++ drivers of a training iteration (csrc/host/train_step.cpp: gsx::TrainStep over the fused entry points;
csrc/host/ops_path.cpp: the step issued operator by operator through the gsplat/Ops.h mirror, with autograd and ATen
glue, as LichtFeld's trainer issues it) against the Python step driver and the CPU checker."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")

from step_checks import N  # noqa: E402

LR_NAMES = ("means", "sh0", "shN", "scaling", "rotation", "opacity")


def _reduced_cfg3(gsx, n):
    sc = gsx.scenes.config(3, n)
    sc.scaling_raw += 1.2  # fewer, larger Gaussians and a smaller image: the CPU side takes seconds
    sc.target_scene.scaling_raw += 1.2
    cam = gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)
    return sc, cam


def _cpp_step(cpp, sc, cuda, **kw):
    from lichtfeld_studio_amd.trainer import DEFAULT_LRS
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(cuda)
    return cpp.TrainStep(t(sc.means), t(np.concatenate([sc.sh0, sc.shN], 1)), t(sc.scaling_raw), t(sc.rotation_raw),
                         t(sc.opacity_raw.reshape(-1)), [DEFAULT_LRS[k] for k in LR_NAMES], sh_degree=sc.sh_degree,
                         **kw)


def _cpp_state(cs, lrs):
    names = ("means", "shs", "scaling", "rotation", "opacity")
    params = dict(means=N(cs.means), shs=N(cs.shs), scaling=N(cs.scaling_raw), rotation=N(cs.rotation_raw),
                  opacity=N(cs.opacity_raw))
    return dict(params=params, exp_avg={k: N(v) for k, v in zip(names, cs.exp_avg)},
                exp_avg_sq={k: N(v) for k, v in zip(names, cs.exp_avg_sq)}, lrs=lrs, grads=None)


def test_cpp_train_step_equals_python_step_and_checker(gsx, orc, cpp, cuda):
    """gsx::TrainStep against TrainStep on the configuration bench.py times (fused update, fused loss, two streams,
    pair count on the device) and against the CPU checker: forward outputs and loss bit for bit, moments and
    parameters to the bars of oracle/checks.py (the backward rasterizer adds with atomics)"""
    from lichtfeld_studio_amd.trainer import TrainStep
    from oracle.checks import step_with_truth
    from oracle.step import OracleTrainStep
    sc, cam = _reduced_cfg3(gsx, 30_000)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    tg = OracleTrainStep(sc.target_scene)
    gt = np.ascontiguousarray(np.clip(tg.forward(cam.viewmat, cam.K, W, H)[0], 0, 1).transpose(2, 0, 1))
    gt_d = torch.from_numpy(gt[None].copy()).to(cuda)
    py = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=True, device_count=True)
    cs = _cpp_step(cpp, sc, cuda)
    ref = OracleTrainStep(sc, lambda_dssim=0.2)
    py.step(vm, Km, W, H, gt_d)
    cs.step(vm, Km, W, H, gt_d)
    truth = step_with_truth(ref, cam.viewmat, cam.K, W, H, gt)
    torch.cuda.synchronize()
    assert cs.n_isects() == py.n_isects == ref.fwd[7].shape[0] > 10_000
    assert cs.pair_capacity() >= cs.n_isects() and cs.lists_error() == (0, 0)
    for name, a, b, r in (("image", cs.render, py.render, ref.fwd[0]), ("alpha", cs.alpha, py.alpha, ref.fwd[1]),
                          ("last ids", cs.last_ids, py.last_ids, ref.fwd[8])):
        assert torch.equal(a, b), name
        assert np.array_equal(N(a).view(np.uint32), np.asarray(r).view(np.uint32)), name + " vs checker"
    assert torch.equal(cs.loss_out, py.loss_out)
    loss = [float(x) for x in cs.loss_out.cpu()]
    assert max(abs(a - b) for a, b in zip(loss, ref.loss)) <= 1e-5, (loss, ref.loss)
    from oracle import checks
    checks.check_update_from_identical_state("c++ step: ", _cpp_state(cs, py.lrs), ref, truth, None)
    names = ("means", "shs", "scaling", "rotation", "opacity")
    params = dict(zip(names, (cs.means, cs.shs, cs.scaling_raw, cs.rotation_raw, cs.opacity_raw)))
    for k in names:  # the two GPU runs differ by the order of the atomic additions only
        moved = (params[k] - py.params[k]).abs()
        assert float(moved.max()) <= 2.2 * py.lrs["opacity"], k
        assert float((moved <= 1e-6 + 1e-3 * py.lrs["opacity"]).float().mean()) > 0.999, k
    # further iterations (the forward pass now orders its tiles by the previous step's costs; the second camera
    # tensor switches that off again): losses track each other, nothing is held back
    vm2 = vm.clone()
    for it, v in enumerate((vm, vm2, vm2, vm)):
        py.step(v, Km, W, H, gt_d)
        cs.step(v, Km, W, H, gt_d)
        torch.cuda.synchronize()
        a, b = float(cs.loss_out[0]), float(py.loss_out[0])
        assert abs(a - b) <= 1e-5, (it, a, b)
    assert cs.iteration == py.iteration == 5 and cs.step_count == py.step_count == 5
    assert cs.lists_error() == (0, 0) and py.lists_error() == (0, 0) and cs.steps_held == 0


def test_cpp_train_step_grows_its_buffers(gsx, cpp, cuda):
    """a camera that suddenly sees several times the pairs the buffers hold: that step renders nothing and is held
    back from the optimiser; the next one starts with larger buffers and with the held step counted back out"""
    sc, _ = _reduced_cfg3(gsx, 20_000)
    far = gsx.scenes.orbit_camera(0.7, 9.0, 309, 205, 287.0)
    near = gsx.scenes.orbit_camera(0.7, 3.0, 309, 205, 287.0)
    W, H = far.width, far.height
    t = lambda a: torch.from_numpy(a[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(3)).to(cuda)
    cs = _cpp_step(cpp, sc, cuda, initial_pair_capacity=4096)  # the first pass sizes the buffers by its own count
    cs.step(t(far.viewmat), t(far.K), W, H, gt)
    torch.cuda.synchronize()
    cap0 = cs.pair_capacity()
    assert cap0 >= cs.n_isects() > 4096 and cs.lists_error() == (0, 0) and float(cs.alpha.max()) > 0.0
    before = [x.clone() for x in (cs.means, cs.shs, cs.opacity_raw)]
    cs.step(t(near.viewmat), t(near.K), W, H, gt)
    torch.cuda.synchronize()
    assert cs.n_isects() > cap0, (cs.n_isects(), cap0)
    assert cs.lists_error() == (1, 1) and float(cs.alpha.max()) == 0.0
    for a, b in zip(before, (cs.means, cs.shs, cs.opacity_raw)):
        assert torch.equal(a, b)
    cs.step(t(near.viewmat), t(near.K), W, H, gt)
    torch.cuda.synchronize()
    assert cs.steps_held == 1 and cs.step_count == 2 and cs.iteration == 2
    assert cs.pair_capacity() >= cs.n_isects() and cs.lists_error() == (0, 0) and float(cs.alpha.max()) > 0.0


@pytest.mark.parametrize("which", ["python", "cpp"])
def test_failed_look_back_is_raised_by_the_next_step(gsx, cpp, cuda, which):
    """Bit 1 of the tile lists' sticky error word (a chained pass gave up waiting for its predecessor) holds the
    optimiser; the update kernel reports the word to pinned host memory, and the step after that raises instead of
    training on in silence.  The bit is set from the host here: no kernel is made to wait."""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc, cam = _reduced_cfg3(gsx, 5_000)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(3)).to(cuda)
    if which == "python":
        ts = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=True, device_count=True)
        step = lambda: ts.step(vm, Km, W, H, gt)
        means = lambda: ts.params["means"]

        def set_bits(bits):
            torch.cuda.synchronize()
            ts.lists_ws[ts._lists_error_at:ts._lists_error_at + 4].copy_(
                torch.tensor([bits, 0, 0, 0], dtype=torch.uint8, device=cuda))
        error = gsx._lib.GsxError
    else:
        ts = _cpp_step(cpp, sc, cuda)
        step = lambda: ts.step(vm, Km, W, H, gt)
        means = lambda: ts.means
        set_bits = ts.debug_set_lists_error
        error = RuntimeError
    step()
    step()
    torch.cuda.synchronize()
    set_bits(2)
    before = means().clone()
    step()  # held back by the update kernel, which reports the word
    torch.cuda.synchronize()
    assert torch.equal(before, means()) and ts.lists_error() == (2, 1)
    with pytest.raises(error, match="look-back"):
        step()
    ts.clear_lists_error()
    assert ts.lists_error() == (0, 0) and ts.steps_held == 1
    step()
    torch.cuda.synchronize()
    assert not torch.equal(before, means()) and ts.step_count == 3


def test_ops_path_trainer_tracks_the_fused_step(gsx, cpp, cuda):
    """The step issued as LichtFeld's trainer issues it (autograd around rasterize_from_world_with_sh_fwd / _bwd,
    ATen activations / cat / clamp / l1_loss, fused_ssim, one Adam launch per group) against the step driver: ATen's
    sigmoid / exp / normalize differ from the library's in the last bit, so nothing is bit-exact across the two;
    losses agree to 1e-5 and the parameters to a small fraction of their learning rates over three iterations."""
    from lichtfeld_studio_amd.trainer import DEFAULT_LRS, TrainStep
    sc, cam = _reduced_cfg3(gsx, 30_000)
    W, H = cam.width, cam.height
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, H, W), generator=torch.Generator().manual_seed(7)).to(cuda)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(cuda)
    op = cpp.OpsPathTrainer(t(sc.means), t(sc.sh0), t(sc.shN), t(sc.scaling_raw), t(sc.rotation_raw),
                            t(sc.opacity_raw.reshape(-1, 1)), int(sc.sh_degree), [DEFAULT_LRS[k] for k in LR_NAMES],
                            0.2, False)
    ts = TrainStep(sc, cuda)
    for it in range(3):
        loss = op.train_step(it + 1, vm, Km, W, H, gt[0])
        ts.step(vm, Km, W, H, gt)
        torch.cuda.synchronize()
        assert abs(float(loss) - float(ts.loss_out[0])) <= 1e-5, it
    means, sh0, shN, scaling, rotation, opacity = op.parameters()
    got = dict(means=means, shs=torch.cat([sh0, shN], 1), scaling=scaling, rotation=rotation,
               opacity=opacity.reshape(-1))
    lr_of = dict(means="means", shs="sh0", scaling="scaling", rotation="rotation", opacity="opacity")
    for k, a in got.items():
        moved = (a.detach() - ts.params[k]).abs()
        lr = ts.lrs[lr_of[k]]
        assert float(moved.max()) <= 3 * 2.2 * lr, k
        assert float(torch.quantile(moved.reshape(-1)[:4_000_000], 0.999)) <= 0.02 * 3 * lr + 1e-7, k
    # the operator pair itself: a second forward pass with other tensors in between leaves the first pass's records
    # in place behind its `colors` output, and a backward pass without them (cloned colours) gives the same gradients
    # up to the order of the atomic additions
    means, quats, scales, opac, shs = (t(x) for x in gsx.scenes.activate(sc))
    ut = cpp.UnscentedTransformParameters()
    args = (3, None, None, W, H, 16, vm, None, Km, cpp.CameraModelType.PINHOLE, 0.3, 0.01, 1e4, 0.0, 1.0, False, 0, ut,
            cpp.ShutterType.GLOBAL, None, None, None)
    f1 = cpp.rasterize_from_world_with_sh_fwd(means, quats, scales, opac, shs, *args)
    f2 = cpp.rasterize_from_world_with_sh_fwd(means.clone(), quats, scales * 1.01, opac, shs, *args)
    assert not torch.equal(f1[0], f2[0])
    v_r = torch.randn_like(f1[0])
    v_a = torch.zeros_like(f1[1])
    empty = torch.empty(0, device=cuda)
    bwd = lambda colors: cpp.rasterize_from_world_with_sh_bwd(
        means, quats, scales, opac, shs, *args, f1[1], f1[8], f1[6], f1[7], colors, f1[2], f1[3], f1[4], empty, v_r, v_a)
    fast, general = bwd(f1[5]), bwd(f1[5].clone())
    for name, a, b in zip(("v_means", "v_quats", "v_scales", "v_opacities", "v_sh"), fast, general):
        assert float((a - b).abs().max()) <= 1e-4 * float(b.abs().max()) + 1e-12, name
    # ... and the general composition (RGB + depth renders through it) composites the same colours
    args_d = args[:16] + (3,) + args[17:]
    f3 = cpp.rasterize_from_world_with_sh_fwd(means, quats, scales, opac, shs, *args_d)
    assert torch.equal(f3[0][..., :3], f1[0]) and torch.equal(f3[7], f1[7]) and torch.equal(f3[6], f1[6])
