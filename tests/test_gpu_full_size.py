"""The measured configurations at their FULL sizes on the GPU, against the CPU restatement run on the same inputs in
the same test (the box's host cores finish one 1M-Gaussian iteration in about two seconds), plus size-independent
properties of the stage outputs.  Configuration 1 (the plumbing case) is in test_gpu_step.py."""
import time

import numpy as np
import pytest

from oracle.checks import step_with_truth
from step_checks import N, check_first_step, check_forward_bit_exact, check_loss
from test_golden import binoms

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]
torch = pytest.importorskip("torch")


def T(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def stage_properties(ts):
    """what must hold for any input: keys sorted, ranges partition the list, tile counts add up, ids in range"""
    n = ts.n_isects
    ids = N(ts.isect_ids[:n])
    flat = N(ts.flatten_ids[:n])
    off = N(ts.offsets).reshape(-1)
    # with the pair count on the device no per-Gaussian tile counts exist: how often the lists name each Gaussian
    tiles_per_gauss = np.bincount(flat, minlength=ts.N) if ts._lists_active else N(ts.tiles_per_gauss)
    radii = N(ts.proj["radii"])[0]
    assert int(tiles_per_gauss.sum(dtype=np.int64)) == n, "sum of tile counts = number of intersections"
    assert (tiles_per_gauss[(radii <= 0).any(-1)] == 0).all(), "culled Gaussians touch no tile"
    assert (np.diff(ids) >= 0).all(), "keys ascending"
    tile_of = ids >> 32
    assert tile_of.min() >= 0 and tile_of.max() < off.size
    np.testing.assert_array_equal(np.searchsorted(tile_of, np.arange(off.size)), off)
    assert flat.min() >= 0 and flat.max() < ts.N
    assert np.array_equal(np.bincount(flat, minlength=ts.N), tiles_per_gauss), "every Gaussian once per tile it touches"
    depth_bits = N(ts.proj["depths"])[0].view(np.uint32)[flat]
    assert np.array_equal((ids & 0xFFFFFFFF).astype(np.uint32), depth_bits), "low key word = depth bits"
    alpha = N(ts.alpha)
    assert alpha.min() >= 0.0 and alpha.max() <= 1.0
    last = N(ts.last_ids).reshape(-1, 1)
    return n


def target_image(gsx, sc, cam, cuda):
    """the independent target scene rendered by the same forward, clamped, CHW"""
    from lichtfeld_studio_amd.trainer import TrainStep
    tg = TrainStep(sc.target_scene, cuda)
    vm, Km = T(cam.viewmat[None], cuda), T(cam.K[None], cuda)
    r = tg.forward(vm, Km, cam.width, cam.height)
    gt = r[0].clamp(0, 1).permute(2, 0, 1).contiguous()[None]
    del tg
    return gt


def test_config2_eight_cameras_forward(gsx, orc, cuda):
    """500k Gaussians, SH degree 3, 8 cameras at 1237x822, forward only: images bit-exact"""
    ops = gsx.ops
    sc = gsx.scenes.config(2)
    means, quats, scales, op, shs = gsx.scenes.activate(sc)
    d = [T(x, cuda) for x in (means, quats, scales, op, shs)]
    bg = np.zeros((1, 3), np.float32)
    ut = ops.UnscentedTransformParameters()
    for cam in sc.cameras:
        W, H = cam.width, cam.height
        got = ops.rasterize_from_world_with_sh_fwd(*d, 3, T(bg, cuda), None, W, H, 16, T(cam.viewmat[None], cuda), None,
                                                   T(cam.K[None], cuda), 0, 0.3, 0.01, 1e4, 0.0, 1.0, False, 0, ut, 4,
                                                   return_isect_ids=True)
        ref = orc.rasterize_from_world_with_sh_fwd(means, quats, scales, op, shs, 3, bg, W, H, 16, cam.viewmat[None],
                                                   cam.K[None])
        assert np.array_equal(N(got[10]), ref[10]), "tile keys"
        assert np.array_equal(N(got[7]), ref[7]), "sort order"
        assert np.array_equal(N(got[6]), ref[6]), "per-tile ranges"
        assert np.array_equal(N(got[0]).view(np.uint32), ref[0].view(np.uint32)), "image bit-exact"
        assert np.array_equal(N(got[8]), ref[8]), "last ids"
        assert ref[10].shape[0] > 500_000


def _full_step(gsx, cuda, cfg):
    from lichtfeld_studio_amd.trainer import TrainStep
    from oracle.step import OracleTrainStep
    t0 = time.time()
    sc = gsx.scenes.config(cfg)
    cam = sc.cameras[0]
    gt_d = target_image(gsx, sc, cam, cuda)
    gt = N(gt_d)[0]
    ts = TrainStep(sc, cuda)
    ref = OracleTrainStep(sc)
    vm, Km = T(cam.viewmat[None], cuda), T(cam.K[None], cuda)
    t1 = time.time()
    ts.step(vm, Km, cam.width, cam.height, gt_d)
    torch.cuda.synchronize()
    t2 = time.time()
    truth = step_with_truth(ref, cam.viewmat, cam.K, cam.width, cam.height, gt)
    t3 = time.time()
    print(f"cfg{cfg}: setup {t1 - t0:.1f}s gpu step {t2 - t1:.2f}s cpu step + float64 backward {t3 - t2:.1f}s "
          f"n_isects {ts.n_isects}", flush=True)
    n = stage_properties(ts)
    check_forward_bit_exact(ts, ref, min_isects=1_000_000)
    check_loss(ts, ref)
    check_first_step(ts, ref, truth, tag=f"cfg{cfg} full size: ")
    return sc, cam, ts, ref, n


def test_config3_full_step(gsx, orc, cuda):
    """1M Gaussians, 1237x822: forward + 0.8 L1 + 0.2 (1 - SSIM) + backward + Adam"""
    _full_step(gsx, cuda, 3)


def test_config3_full_size_on_the_benchmarked_path(gsx, orc, cuda):
    """Configuration 3 at full size through exactly the code path bench.py times: one-pass backward + update
    (fused_update), two-kernel loss (fused_loss), second stream (overlap), tile visiting order on.  Two iterations
    from the same camera tensors, so the second forward pass reuses the tile order formed from the first one's costs
    and both side-stream joins are exercised.  Before the second iteration the GPU state is set to the checker's, so
    that it, too, starts from identical parameters and moments: keys / order / ranges / image bit-exact, loss <= 1e-5,
    parameters and both moments by the element-wise bars, in both iterations."""
    from lichtfeld_studio_amd.trainer import TrainStep
    from oracle.step import OracleTrainStep
    sc = gsx.scenes.config(3)
    cam = sc.cameras[0]
    gt_d = target_image(gsx, sc, cam, cuda)
    gt = N(gt_d)[0]
    ts = TrainStep(sc, cuda, fused_update=True, fused_loss=True, overlap=True, device_count=True)
    assert ts.order_tiles and ts.fused_loss and ts.side is not None and ts.device_count
    ref = OracleTrainStep(sc)
    vm, Km = T(cam.viewmat[None], cuda), T(cam.K[None], cuda)
    prev = None
    for it in range(2):
        reused = getattr(ts, "have_walk", False) and ts._walk_cam == (vm.data_ptr(), Km.data_ptr(), cam.width, cam.height)
        assert reused == (it == 1), "the second forward pass must run with the order left by the first"
        ts.step(vm, Km, cam.width, cam.height, gt_d)
        torch.cuda.synchronize()
        truth = step_with_truth(ref, cam.viewmat, cam.K, cam.width, cam.height, gt)
        assert ts._lists_active == (it == 1), "from the second iteration on the pair count stays on the device"
        stage_properties(ts)
        check_forward_bit_exact(ts, ref, min_isects=1_000_000)
        check_loss(ts, ref)
        check_first_step(ts, ref, truth, tag=f"cfg3 bench path, iteration {it + 1}: ", prev=prev)
        prev = ({k: v.copy() for k, v in ref.exp_avg.items()}, {k: v.copy() for k, v in ref.exp_avg_sq.items()})
        for k in ts.params:  # identical state for the next iteration
            ts.params[k].copy_(T(ref.params[k], cuda))
            ts.exp_avg[k].copy_(T(ref.exp_avg[k], cuda))
            ts.exp_avg_sq[k].copy_(T(ref.exp_avg_sq[k], cuda))
    assert ts.lists_error() == (0, 0)


def test_config4_step_relocation_noise(gsx, orc, cuda):
    """3M Gaussians, 1920x1080: one iteration, then MCMC relocation of the 5 % lowest-opacity Gaussians (multinomial
    draw over the alive ones' opacities made on the host and given to both sides) and noise injection"""
    sc, cam, ts, ref, _ = _full_step(gsx, cuda, 4)
    n_total = ts.N
    op = 1.0 / (1.0 + np.exp(-ref.params["opacity"].astype(np.float64)))
    order = np.argsort(op, kind="stable")
    n_dead = n_total // 20
    dead = np.sort(order[:n_dead]).astype(np.int64)
    alive = np.sort(order[n_dead:]).astype(np.int64)
    rng = np.random.default_rng(44)
    p = op[alive] / op[alive].sum()
    sampled = alive[rng.choice(alive.size, size=n_dead, replace=True, p=p)].astype(np.int64)
    assert np.unique(sampled).size < sampled.size  # ratios above 2 occur
    b = binoms(51)
    ts.relocate(T(sampled, cuda), T(dead, cuda), T(b, cuda))
    ref.relocate(sampled, dead, b)
    torch.cuda.synchronize()
    for k in ("scaling", "opacity", "shs", "rotation"):
        # rows that the relocation rewrote or copied: bit-identical; all other rows are covered by the step checks
        a, r = N(ts.params[k]), ref.params[k]
        touched = np.concatenate([sampled, dead])
        if k in ("scaling", "opacity"):
            a0, r0 = a[touched], r[touched]
            close = np.abs(a0 - r0) <= 1e-3 * np.abs(r0) + 5e-3 * 1e-3
            assert close.mean() > 0.999, k  # inputs differ by the Adam tolerance of the step before
        assert np.array_equal(a[dead], a[sampled]), f"{k}: dead rows are copies of the sampled rows"
    for k in ts.params:
        assert float(ts.exp_avg[k][T(sampled, cuda)].abs().max()) == 0.0
        assert float(ts.exp_avg_sq[k][T(sampled, cuda)].abs().max()) == 0.0
    # noise: the same N(0,1) draws on both sides
    noise = rng.standard_normal((n_total, 3)).astype(np.float32)
    before = N(ts.params["means"]).copy()
    ts.inject_noise(T(noise, cuda))
    ref.inject_noise(noise)
    torch.cuda.synchronize()
    moved = N(ts.params["means"]) - before
    assert np.abs(moved).max() > 0
    d = np.abs(N(ts.params["means"]) - ref.params["means"])
    lr = ts.lrs["means"]
    assert np.quantile(d, 0.999) <= 1e-3 * lr + 1e-3 * np.quantile(np.abs(moved), 0.999)


def test_mcmc_relocate_bit_exact_from_identical_state(gsx, orc, cuda):
    """relocation + noise from IDENTICAL parameters on both sides (no training step before): every tensor bit-exact"""
    from lichtfeld_studio_amd.trainer import TrainStep
    from oracle.step import OracleTrainStep
    sc = gsx.scenes.config(3, 200_000)
    ts, ref = TrainStep(sc, cuda), OracleTrainStep(sc)
    rng = np.random.default_rng(7)
    for k in ts.params:  # non-zero moments, so that clearing them is visible
        m = rng.standard_normal(ref.exp_avg[k].shape).astype(np.float32)
        ref.exp_avg[k][...] = m
        ref.exp_avg_sq[k][...] = m * m
        ts.exp_avg[k].copy_(T(m, cuda))
        ts.exp_avg_sq[k].copy_(T(m * m, cuda))
    perm = rng.permutation(ts.N)
    dead, alive = np.sort(perm[:10_000]).astype(np.int64), perm[10_000:]
    sampled = alive[rng.integers(0, 3000, 10_000)].astype(np.int64)  # few distinct sources: ratios up to the clamp
    b = binoms(51)
    ts.relocate(T(sampled, cuda), T(dead, cuda), T(b, cuda))
    ref.relocate(sampled, dead, b)
    noise = rng.standard_normal((ts.N, 3)).astype(np.float32)
    ts.inject_noise(T(noise, cuda))
    ref.inject_noise(noise)
    torch.cuda.synchronize()
    for k in ts.params:
        assert np.array_equal(N(ts.params[k]).view(np.uint32), ref.params[k].view(np.uint32)), k
        assert np.array_equal(N(ts.exp_avg[k]).view(np.uint32), ref.exp_avg[k].view(np.uint32)), k
        assert np.array_equal(N(ts.exp_avg_sq[k]).view(np.uint32), ref.exp_avg_sq[k].view(np.uint32)), k
    counts = np.bincount(sampled, minlength=ts.N)
    assert counts.max() + 1 > 3


def test_config5_stress_step(gsx, orc, cuda):
    """6M Gaussians, 3840x2160, broad scale distribution, 70 % of the means in a small ball (long tile lists)"""
    sc, cam, ts, ref, n = _full_step(gsx, cuda, 5)
    off = N(ts.offsets).reshape(-1)
    lengths = np.diff(np.concatenate([off, [n]]))
    print(f"cfg5: n_isects {n}, max tile list {int(lengths.max())}, mean {lengths.mean():.0f}", flush=True)
    assert n > 10_000_000


def test_config5_literal_scales_overflow_is_reported(gsx, cuda):
    """the stress configuration with the log-scale mean as stated (-3.5) has 2.7e9 intersections: more than the int32
    ids of flatten_ids can index (in the reference as well); the count pass must say so instead of launching"""
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config5_literal()
    cam = sc.cameras[0]
    ts = TrainStep(sc, cuda)
    with pytest.raises(gsx._lib.GsxError, match="do not fit int32") as e:
        ts.forward(T(cam.viewmat[None], cuda), T(cam.K[None], cuda), cam.width, cam.height)
    assert e.value.status == -5


def test_mcmc_add_new_gs_bit_exact(gsx, orc, cuda):
    """MCMC::add_new_gs: 5 % growth from identical parameters on both sides (sampled sources given to both): the grown
    parameter and moment tensors are bit-identical, and a training step runs on the grown state"""
    from lichtfeld_studio_amd.trainer import TrainStep
    from oracle.step import OracleTrainStep
    sc = gsx.scenes.config(3, 100_000)
    sc.scaling_raw += 0.8
    cam = gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)
    ts, ref = TrainStep(sc, cuda), OracleTrainStep(sc)
    rng = np.random.default_rng(17)
    for k in ts.params:
        m = rng.standard_normal(ref.exp_avg[k].shape).astype(np.float32)
        ref.exp_avg[k][...] = m
        ref.exp_avg_sq[k][...] = m * m
        ts.exp_avg[k].copy_(T(m, cuda))
        ts.exp_avg_sq[k].copy_(T(m * m, cuda))
    n_new = ts.N // 20
    sampled = rng.integers(0, 2000, n_new).astype(np.int64)  # few sources: ratios up to the clamp
    b = binoms(51)
    ts.add_new_gs(T(sampled, cuda), T(b, cuda))
    ref.add_new_gs(sampled, b)
    torch.cuda.synchronize()
    assert ts.N == 105_000
    for k in ts.params:
        assert np.array_equal(N(ts.params[k]).view(np.uint32), ref.params[k].view(np.uint32)), k
        assert np.array_equal(N(ts.exp_avg[k]).view(np.uint32), ref.exp_avg[k].view(np.uint32)), k
        assert np.array_equal(N(ts.exp_avg_sq[k]).view(np.uint32), ref.exp_avg_sq[k].view(np.uint32)), k
    vm, Km = T(cam.viewmat[None], cuda), T(cam.K[None], cuda)
    gt = torch.rand((1, 3, cam.height, cam.width), generator=torch.Generator().manual_seed(1)).to(cuda)
    ts.step(vm, Km, cam.width, cam.height, gt)
    ref.step(cam.viewmat, cam.K, cam.width, cam.height, N(gt)[0])
    torch.cuda.synchronize()
    check_forward_bit_exact(ts, ref, min_isects=10_000)


def test_config5_tile_lists_in_one_call(gsx, cuda):
    """gsx_tile_lists at the stress configuration (1.7e8 pairs, tile lists up to 1e5 entries, 20 000 workgroups per
    chained pass): flatten_ids and tile_offsets element for element those of the separate operators, which the step
    test above holds against the CPU checker"""
    from lichtfeld_studio_amd.trainer import TrainStep
    from test_gpu_tile_lists import Lists
    sc = gsx.scenes.config(5)
    cam = sc.cameras[0]
    ts = TrainStep(sc, cuda)
    ts.forward(T(cam.viewmat[None], cuda), T(cam.K[None], cuda), cam.width, cam.height)
    torch.cuda.synchronize()
    n = ts.n_isects
    assert n > 100_000_000
    want_flat, want_off = ts.flatten_ids[:n].clone(), ts.offsets.reshape(-1).clone()
    J = ts.proj
    lists = Lists(gsx, cuda, ts.N, ts.tw, ts.th, cap=n + 4096, side=True)
    for rep in range(2):
        counts, err = lists.run(J["means2d"], J["radii"], J["depths"])
        assert err == 0 and counts[0] == n and counts[1] == n, (rep, counts, err)
        assert torch.equal(lists.flat[:n], want_flat), f"flatten_ids, call {rep}"
        assert torch.equal(lists.off[:-1], want_off), f"tile_offsets, call {rep}"
        assert int(lists.off[-1]) == n
