"""The C++ host layer (gsplat/Ops.h names over at::Tensor, csrc/host/gsplat_ops.cpp) on the GPU: same results as the
CPU checker and as the ctypes binding, through the functions a LichtFeld build would link."""
import numpy as np
import pytest

from test_gpu_parity import N, T, _fused_inputs, binoms, bits_equal

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _ut(cpp):
    return cpp.UnscentedTransformParameters()


def test_cpp_fused_forward_backward(gsx, orc, cpp, cuda):
    sc, cam, h, d = _fused_inputs(gsx, cuda, 8000)
    args = (3, d["bg"], None, cam.width, cam.height, 16, d["vm"], None, d["K"], cpp.CameraModelType.PINHOLE, 0.3, 0.01,
            1e4, 0.0, 1.0, False, 0, _ut(cpp), cpp.ShutterType.GLOBAL, None, None, None)
    got = cpp.rasterize_from_world_with_sh_fwd(d["means"], d["quats"], d["scales"], d["op"], d["shs"], *args)
    renders, alphas, radii, means2d, depths, colors, offsets, flat, last_ids, comp = got
    ref = orc.rasterize_from_world_with_sh_fwd(h["means"], h["quats"], h["scales"], h["op"], h["shs"], 3, h["bg"],
                                               cam.width, cam.height, 16, h["vm"], h["K"])
    r_renders, r_alphas, r_radii, r_means2d, r_depths, r_colors, r_offsets, r_flat, r_last, r_comp, r_ids = ref
    bits_equal(N(radii), r_radii, "radii")
    bits_equal(N(flat), r_flat, "sort order")
    bits_equal(N(offsets), r_offsets, "per-tile ranges")
    bits_equal(N(last_ids), r_last, "last ids")
    bits_equal(N(renders), r_renders, "image")
    bits_equal(N(alphas), r_alphas, "alpha")
    assert comp is None or comp.numel() == 0  # calc_compensations == false: undefined tensor

    rng = np.random.default_rng(5)
    v_img = rng.standard_normal(r_renders.shape).astype(np.float32)
    v_alpha = rng.standard_normal(r_alphas.shape).astype(np.float32)
    g = cpp.rasterize_from_world_with_sh_bwd(d["means"], d["quats"], d["scales"], d["op"], d["shs"], *args, alphas,
                                             last_ids, offsets, flat, colors, radii, means2d, depths,
                                             torch.empty(0, device=cuda), T(v_img, cuda), T(v_alpha, cuda))
    v_means, v_quats, v_scales, v_op, v_sh = [N(x) for x in g]
    o = orc.rasterize_from_world_with_sh_bwd(h["means"], h["quats"], h["scales"], h["op"], h["shs"], 3, h["bg"],
                                             cam.width, cam.height, 16, h["vm"], h["K"], 1.0, False, r_alphas, r_last,
                                             r_offsets, r_flat, r_colors, r_radii, None, v_img, v_alpha)
    o_means, o_quats, o_scales, o_op, o_sh = o
    for name, a, b in (("v_means", v_means, o_means), ("v_opacities", v_op.reshape(-1), o_op.reshape(-1)),
                       ("v_sh", v_sh, o_sh)):
        scale = float(np.abs(b).max())
        assert np.abs(a - b).max() <= 1e-3 * scale, name
    # the same gradients through the ctypes binding (atomic order differs between runs: compare with a tolerance)
    ops = gsx.ops
    g2 = ops.rasterize_from_world_with_sh_bwd(d["means"], d["quats"], d["scales"], d["op"], d["shs"], 3, d["bg"], None,
                                              cam.width, cam.height, 16, d["vm"], None, d["K"], 0, 0.3, 0.01, 1e4, 0.0,
                                              1.0, False, 0, ops.UnscentedTransformParameters(), 4, None, None, None,
                                              alphas, last_ids, offsets, flat, colors, radii, means2d, depths, None,
                                              T(v_img, cuda), T(v_alpha, cuda))
    for name, a, b in zip(("v_means", "v_quats", "v_scales", "v_opacities", "v_sh"), g, g2):
        a, b = N(a), N(b)
        assert np.abs(a - b).max() <= 1e-4 * np.abs(b).max() + 1e-12, name


def test_cpp_stage_functions_match_checker(gsx, orc, cpp, cuda):
    sc, cam, h, d = _fused_inputs(gsx, cuda, 5000)
    ut = _ut(cpp)
    radii, means2d, depths, conics, comp = cpp.projection_ut_3dgs_fused(
        d["means"], d["quats"], d["scales"], d["op"], d["vm"], None, d["K"], cam.width, cam.height, 0.3, 0.01, 1e4,
        0.0, True, cpp.CameraModelType.PINHOLE, ut, cpp.ShutterType.GLOBAL, None, None, None)
    r = orc.projection_ut_3dgs_fused(h["means"], h["quats"], h["scales"], h["op"], h["vm"], h["K"], cam.width,
                                     cam.height, 0.3, 0.01, 1e4, 0.0, True)
    bits_equal(N(radii), r[0], "radii")
    vis = r[0][0, :, 0] > 0
    bits_equal(N(means2d)[0][vis], r[1][0][vis], "means2d")
    bits_equal(N(depths)[0][vis], r[2][0][vis], "depths")
    bits_equal(N(conics)[0][vis], r[3][0][vis], "conics")
    bits_equal(N(comp)[0][vis], r[4][0][vis], "compensations")

    tw, th = (cam.width + 15) // 16, (cam.height + 15) // 16
    tiles, ids, flat = cpp.intersect_tile(means2d, radii, depths, None, None, 1, 16, tw, th, True)
    o_tiles, o_ids, o_flat = orc.intersect_tile(r[1], r[0], r[2], 1, 16, tw, th, True)
    bits_equal(N(tiles), o_tiles, "tiles_per_gauss")
    bits_equal(N(ids), o_ids, "sorted keys")
    bits_equal(N(flat), o_flat, "sorted values")
    offsets = cpp.intersect_offset(ids, 1, tw, th)
    bits_equal(N(offsets), orc.intersect_offset(o_ids, 1, tw, th), "offsets")
    # unsorted: same multiset of keys, emission order = Gaussian order
    _, ids_u, flat_u = cpp.intersect_tile(means2d, radii, depths, None, None, 1, 16, tw, th, False)
    _, o_ids_u, o_flat_u = orc.intersect_tile(r[1], r[0], r[2], 1, 16, tw, th, False)
    bits_equal(N(ids_u), o_ids_u, "unsorted keys")
    bits_equal(N(flat_u), o_flat_u, "unsorted values")

    rng = np.random.default_rng(2)
    dirs = rng.standard_normal((4000, 3)).astype(np.float32)
    coeffs = rng.standard_normal((4000, 16, 3)).astype(np.float32)
    mask = rng.random(4000) > 0.2
    v_col = rng.standard_normal((4000, 3)).astype(np.float32)
    col = cpp.spherical_harmonics_fwd(3, T(dirs, cuda), T(coeffs, cuda), T(mask, cuda))
    bits_equal(N(col)[mask], orc.spherical_harmonics_fwd(3, dirs, coeffs, mask)[mask], "sh fwd")
    v_coeffs, v_dirs = cpp.spherical_harmonics_bwd(16, 3, T(dirs, cuda), T(coeffs, cuda), T(mask, cuda),
                                                   T(v_col, cuda), True)
    o_vc, o_vd = orc.spherical_harmonics_bwd(16, 3, dirs, coeffs, mask, v_col, True)
    bits_equal(N(v_coeffs), o_vc, "sh bwd coeffs")
    bits_equal(N(v_dirs), o_vd, "sh bwd dirs")

    q = rng.standard_normal((1000, 4)).astype(np.float32)
    bits_equal(N(cpp.quats_to_rotmats(T(q, cuda))), orc.quats_to_rotmats(q), "rotmats")


def test_cpp_relocation_noise_ssim_adam(gsx, orc, cpp, cuda):
    rng = np.random.default_rng(9)
    M = 5000
    op = rng.uniform(0.01, 0.99, M).astype(np.float32)
    sc = np.exp(rng.normal(-3, 1, (M, 3))).astype(np.float32)
    ratios = rng.integers(1, 52, M).astype(np.int32)
    b = binoms(51)
    no, ns = cpp.relocation(T(op, cuda), T(sc, cuda), T(ratios, cuda), T(b, cuda), 51)
    ro, rs = orc.relocation(op, sc, ratios, b, 51)
    bits_equal(N(no), ro, "new opacities")
    bits_equal(N(ns), rs, "new scales")

    raw_o = rng.normal(0, 2, M).astype(np.float32)
    raw_s = rng.normal(-3, 1, (M, 3)).astype(np.float32)
    raw_q = rng.standard_normal((M, 4)).astype(np.float32)
    noise = rng.standard_normal((M, 3)).astype(np.float32)
    means = rng.standard_normal((M, 3)).astype(np.float32)
    dm = T(means, cuda)
    cpp.add_noise(T(raw_o, cuda), T(raw_s, cuda), T(raw_q, cuda), T(noise, cuda), dm, 1.6e-4)
    orc.add_noise(raw_o, raw_s, raw_q, noise, means, 1.6e-4)
    bits_equal(N(dm), means, "noised means")

    a = rng.random((1, 3, 45, 61)).astype(np.float32)
    g = rng.random((1, 3, 45, 61)).astype(np.float32)
    m, d1, d2, d3 = cpp.fusedssim(1e-4, 9e-4, T(a, cuda), T(g, cuda), True)
    om, o1, o2, o3 = orc.fusedssim(1e-4, 9e-4, a, g, True)
    assert np.abs(N(m) - om).max() <= 1e-5
    dmap = rng.standard_normal(a.shape).astype(np.float32)
    di = cpp.fusedssim_backward(1e-4, 9e-4, T(a, cuda), T(g, cuda), T(dmap, cuda), d1, d2, d3)
    oi = orc.fusedssim_backward(1e-4, 9e-4, a, g, dmap, o1, o2, o3)
    assert np.abs(N(di) - oi).max() <= 1e-5 * max(1.0, float(np.abs(oi).max()))
    val = float(cpp.fused_ssim_value(T(a[0], cuda), T(g[0], cuda), "valid"))
    assert abs(val - float(om[:, :, 5:-5, 5:-5].mean(dtype=np.float64))) <= 1e-5
    val = float(cpp.fused_ssim_value(T(a, cuda), T(g, cuda), "same"))
    assert abs(val - float(om.mean(dtype=np.float64))) <= 1e-5
    with pytest.raises(RuntimeError, match="padding"):
        cpp.fused_ssim_value(T(a, cuda), T(g, cuda), "reflect")

    n = 70_001
    p = rng.standard_normal(n).astype(np.float32)
    m1 = (rng.standard_normal(n) * 0.1).astype(np.float32)
    m2 = (rng.random(n) * 0.01).astype(np.float32)
    gr = rng.standard_normal(n).astype(np.float32)
    dp, dm1, dm2 = T(p, cuda), T(m1, cuda), T(m2, cuda)
    bc1, bc2 = 1.0 / (1 - 0.9 ** 3), 1.0 / np.sqrt(1 - 0.999 ** 3)
    cpp.adam_step_wrapper(dp, dm1, dm2, T(gr, cuda), 1e-3, 0.9, 0.999, 1e-15, bc1, bc2)
    orc.adam_step(p, m1, m2, gr, 1e-3, 0.9, 0.999, 1e-15, bc1, bc2)
    bits_equal(N(dm1), m1, "exp_avg")
    bits_equal(N(dm2), m2, "exp_avg_sq")
    bits_equal(N(dp), p, "param")



def test_cpp_errors_on_device(gsx, cpp, cuda):
    sc, cam, h, d = _fused_inputs(gsx, cuda, 500)
    ut = _ut(cpp)
    with pytest.raises(RuntimeError, match="gsx"):  # two cameras: not built
        vm2 = torch.cat([d["vm"], d["vm"]])
        K2 = torch.cat([d["K"], d["K"]])
        cpp.projection_ut_3dgs_fused(d["means"], d["quats"], d["scales"], d["op"], vm2, None, K2, cam.width,
                                     cam.height, 0.3, 0.01, 1e4, 0.0, False, cpp.CameraModelType.PINHOLE, ut,
                                     cpp.ShutterType.GLOBAL, None, None, None)
    with pytest.raises(RuntimeError, match="gsx"):
        cpp.projection_ut_3dgs_fused(d["means"], d["quats"], d["scales"], d["op"], d["vm"], None, d["K"], cam.width,
                                     cam.height, 0.3, 0.01, 1e4, 0.0, False, cpp.CameraModelType.ORTHO, ut,
                                     cpp.ShutterType.GLOBAL, None, None, None)
    with pytest.raises(RuntimeError, match="contiguous"):
        cpp.quats_to_rotmats(d["quats"].t().contiguous().t())
    with pytest.raises(RuntimeError, match="radial_coeffs must be"):  # the pinhole model reads six per camera
        cpp.projection_ut_3dgs_fused(d["means"], d["quats"], d["scales"], d["op"], d["vm"], None, d["K"], cam.width,
                                     cam.height, 0.3, 0.01, 1e4, 0.0, False, cpp.CameraModelType.PINHOLE, ut,
                                     cpp.ShutterType.GLOBAL, torch.zeros((1, 4), device=cuda), None, None)
    with pytest.raises(RuntimeError, match="scales must be"):
        cpp.projection_ut_3dgs_fused(d["means"], d["quats"], d["scales"][:100].contiguous(), d["op"], d["vm"], None,
                                     d["K"], cam.width, cam.height, 0.3, 0.01, 1e4, 0.0, False,
                                     cpp.CameraModelType.PINHOLE, ut, cpp.ShutterType.GLOBAL, None, None, None)


def test_cpp_camera_models_and_rolling_shutter(gsx, cpp, cuda):
    """the C++ layer hands camera model, coefficient rows, shutter type and the end-of-frame pose to the same kernels
    as the ctypes binding: forward outputs identical bit for bit (fisheye with a rolling shutter, render mode RGB+D)"""
    from scipy.spatial.transform import Rotation
    sc, cam, h, d = _fused_inputs(gsx, cuda, 6000)
    step = np.eye(4)
    step[:3, :3] = Rotation.from_rotvec([0.01, -0.015, 0.02]).as_matrix()
    step[:3, 3] = [0.05, -0.03, 0.08]
    vm1 = T((step @ h["vm"][0].astype(np.float64)).astype(np.float32)[None], cuda)
    radial = T(np.asarray([[0.03, -0.004, 0.0006, 0.0]], np.float32), cuda)
    got = cpp.rasterize_from_world_with_sh_fwd(
        d["means"], d["quats"], d["scales"], d["op"], d["shs"], 3, d["bg"], None, cam.width, cam.height, 16, d["vm"],
        vm1, d["K"], cpp.CameraModelType.FISHEYE, 0.3, 0.01, 1e4, 0.0, 1.0, False, 3, _ut(cpp),
        cpp.ShutterType.ROLLING_LEFT_TO_RIGHT, radial, None, None)
    ops = gsx.ops
    want = ops.rasterize_from_world_with_sh_fwd(
        d["means"], d["quats"], d["scales"], d["op"], d["shs"], 3, d["bg"], None, cam.width, cam.height, 16, d["vm"],
        vm1, d["K"], 2, 0.3, 0.01, 1e4, 0.0, 1.0, False, 3, ops.UnscentedTransformParameters(), 1, radial, None, None)
    assert tuple(got[0].shape) == (1, cam.height, cam.width, 4) and float(got[1].mean()) > 0.01
    for k, name in ((0, "renders"), (1, "alphas"), (2, "radii"), (6, "offsets"), (7, "flatten_ids"), (8, "last_ids")):
        assert torch.equal(got[k], want[k]), name
    plain = ops.rasterize_from_world_with_sh_fwd(
        d["means"], d["quats"], d["scales"], d["op"], d["shs"], 3, d["bg"], None, cam.width, cam.height, 16, d["vm"],
        None, d["K"], 2, 0.3, 0.01, 1e4, 0.0, 1.0, False, 3, ops.UnscentedTransformParameters(), 4, radial, None, None)
    assert float((plain[0] - want[0]).abs().max()) > 0.05  # the shutter matters
