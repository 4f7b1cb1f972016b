"""The committed fixtures of tests/golden/ (written by tests/golden/make_fixtures.py) against the CPU checker (here)
and against the GPU kernels (-m gpu).  sort32 / ssim40 / relocation51 hold expected values computed WITHOUT the checker
(Python's stable sort, the float64 SSIM definition, Eq. 9 in float64); scene200 freezes the checker's stage outputs."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLD, name), allow_pickle=False))


def same_bits(a, b, name):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    assert a.shape == b.shape and a.dtype == b.dtype, f"{name}: {a.shape} {a.dtype} vs {b.shape} {b.dtype}"
    assert a.tobytes() == b.tobytes(), f"{name}: {(a != b).sum()} elements differ"


def binoms(n_max=51):
    b = np.zeros((n_max, n_max), np.float32)
    for n in range(n_max):
        for k in range(n + 1):
            x = np.float32(1.0)
            for i in range(k):
                x = np.float32(x * (np.float32(n - i) / np.float32(i + 1)))
            b[n, k] = x
    return b


def relocation_inputs(g):
    """every (n, opacity) combination of the table as one flat call; scales = 1 so that new_scales = the factor"""
    op64, ratios = g["opacities"], g["ratios"]
    op = np.tile(op64.astype(np.float32), ratios.size)
    rat = np.repeat(ratios, op64.size).astype(np.int32)
    return op, np.ones((op.size, 3), np.float32), rat


def check_relocation(g, new_op, new_sc):
    n_op = g["opacities"].size
    new_op = new_op.reshape(-1, n_op)
    factor = new_sc.reshape(-1, n_op, 3)
    assert np.abs(factor - factor[..., :1]).max() == 0.0  # one factor for the three axes
    np.testing.assert_allclose(new_op, g["new_opacities_f64"], rtol=3e-5, atol=1e-7)
    # the fp32 alternating binomial sum is stable while C(n-1, k) * o'^k stays small: n <= 12 for every opacity of the
    # table; beyond that the reference's own fp32 arithmetic loses digits (checker and kernel agree bit for bit there,
    # test_gpu_parity.test_relocation), so only positivity and finiteness are fixed
    np.testing.assert_allclose(factor[:12, :, 0], g["scale_factor_f64"][:12], rtol=2e-3)
    assert np.isfinite(factor).all()


def sorted_fixture_checks(g, keys, vals):
    same_bits(keys, g["sorted_keys"], "sorted keys")
    same_bits(vals, g["sorted_vals"], "sorted values (tie order)")


SCENE_FWD = ("radii", "isect_ids", "flatten_ids", "tile_offsets", "last_ids", "render_colors", "render_alphas")


# ------------------------------------------------------------------------------------------------------------
# CPU: the checker against the fixtures
# ------------------------------------------------------------------------------------------------------------
def test_checker_sort32(orc):
    g = load("sort32.npz")
    k, v = orc.radix_sort_pairs(g["keys"], g["vals"], int(g["end_bit"]))
    sorted_fixture_checks(g, k, v)
    same_bits(orc.intersect_offset(g["clean_sorted_keys"], 1, 8, 4), g["offsets"], "offsets with empty tiles")


def test_checker_ssim40(orc):
    g = load("ssim40.npz")
    m = orc.fusedssim(0.01 ** 2, 0.03 ** 2, g["img1"], g["img2"], False)[0]
    assert np.abs(m - g["ssim_map_f64"]).max() <= 1e-5
    assert abs(m[:, :, 5:-5, 5:-5].mean(dtype=np.float64) - float(g["mean_valid"])) <= 1e-5


def test_checker_relocation51(orc):
    g = load("relocation51.npz")
    op, sc, rat = relocation_inputs(g)
    check_relocation(g, *orc.relocation(op, sc, rat, binoms(), 51))


def test_checker_scene200(orc):
    g = load("scene200.npz")
    W, H = int(g["width"]), int(g["height"])
    f = orc.rasterize_from_world_with_sh_fwd(g["means"], g["quats"], g["scales"], g["opacities"], g["sh_coeffs"], 3,
                                             g["background"], W, H, 16, g["viewmat"], g["K"])
    got = dict(zip(("render_colors", "render_alphas", "radii", "means2d", "depths", "colors", "tile_offsets",
                    "flatten_ids", "last_ids", "compensations", "isect_ids"), f))
    for name in SCENE_FWD + ("means2d", "depths", "colors"):
        same_bits(got[name], g[name], name)
    b = orc.rasterize_from_world_with_sh_bwd(g["means"], g["quats"], g["scales"], g["opacities"], g["sh_coeffs"], 3,
                                             g["background"], W, H, 16, g["viewmat"], g["K"], 1.0, False,
                                             g["render_alphas"], g["last_ids"], g["tile_offsets"], g["flatten_ids"],
                                             g["colors"], g["radii"], None, g["v_render_colors"], g["v_render_alphas"])
    for name, a in zip(("v_means", "v_quats", "v_scales", "v_opacities", "v_sh_coeffs"), b):
        same_bits(a, g[name], name)
    # structure of the frozen data itself: keys sorted, ranges partition the list, last id inside the tile's range
    ids = g["isect_ids"]
    assert (np.diff(ids) >= 0).all()
    off = g["tile_offsets"].reshape(-1)
    assert (np.diff(off) >= 0).all() and off[0] == 0 and off[-1] <= ids.size
    tiles = (ids >> 32).astype(np.int64)
    np.testing.assert_array_equal(np.searchsorted(tiles, np.arange(off.size)), off)


# ------------------------------------------------------------------------------------------------------------
# GPU: the kernels (through the C ABI) against the same fixtures
# ------------------------------------------------------------------------------------------------------------
def _T(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


@pytest.mark.gpu
def test_gpu_sort32(gsx, cuda):
    g = load("sort32.npz")
    ops = gsx.ops
    k, v = ops.radix_sort_double_buffer(32, 5, 0, _T(g["keys"], cuda), _T(g["vals"], cuda))
    sorted_fixture_checks(g, k.cpu().numpy(), v.cpu().numpy())
    off = ops.intersect_offset(_T(g["clean_sorted_keys"], cuda), 1, 8, 4)
    same_bits(off.cpu().numpy(), g["offsets"], "offsets with empty tiles")


@pytest.mark.gpu
def test_gpu_ssim40(gsx, cuda):
    g = load("ssim40.npz")
    m = gsx.ops.fusedssim(0.01 ** 2, 0.03 ** 2, _T(g["img1"], cuda), _T(g["img2"], cuda), False)[0].cpu().numpy()
    assert np.abs(m - g["ssim_map_f64"]).max() <= 1e-5


@pytest.mark.gpu
def test_gpu_relocation51(gsx, cuda):
    g = load("relocation51.npz")
    op, sc, rat = relocation_inputs(g)
    o, s = gsx.ops.relocation(_T(op, cuda), _T(sc, cuda), _T(rat, cuda), _T(binoms(), cuda), 51)
    check_relocation(g, o.cpu().numpy(), s.cpu().numpy())


@pytest.mark.gpu
def test_gpu_scene200(gsx, cuda):
    g = load("scene200.npz")
    ops = gsx.ops
    W, H = int(g["width"]), int(g["height"])
    d = {k: _T(g[k], cuda) for k in ("means", "quats", "scales", "opacities", "sh_coeffs", "background", "viewmat", "K",
                                     "v_render_colors", "v_render_alphas")}
    ut = ops.UnscentedTransformParameters()
    f = ops.rasterize_from_world_with_sh_fwd(d["means"], d["quats"], d["scales"], d["opacities"], d["sh_coeffs"], 3,
                                             d["background"], None, W, H, 16, d["viewmat"], None, d["K"], 0, 0.3, 0.01,
                                             1e4, 0.0, 1.0, False, 0, ut, 4, return_isect_ids=True)
    names = ("render_colors", "render_alphas", "radii", "means2d", "depths", "colors", "tile_offsets", "flatten_ids",
             "last_ids", "compensations", "isect_ids")
    got = dict(zip(names, f))
    for name in SCENE_FWD:
        same_bits(got[name].cpu().numpy(), g[name], name)
    vis = g["radii"][0, :, 0] > 0
    for name in ("means2d", "depths", "colors"):
        same_bits(got[name].cpu().numpy()[0][vis], g[name][0][vis], name)
    b = ops.rasterize_from_world_with_sh_bwd(d["means"], d["quats"], d["scales"], d["opacities"], d["sh_coeffs"], 3,
                                             d["background"], None, W, H, 16, d["viewmat"], None, d["K"], 0, 0.3, 0.01,
                                             1e4, 0.0, 1.0, False, 0, ut, 4, None, None, None, got["render_alphas"],
                                             got["last_ids"], got["tile_offsets"], got["flatten_ids"], got["colors"],
                                             got["radii"], got["means2d"], got["depths"], None, d["v_render_colors"],
                                             d["v_render_alphas"])
    for name, a in zip(("v_means", "v_quats", "v_scales", "v_opacities", "v_sh_coeffs"), b):
        a, ref = a.cpu().numpy().reshape(g[name].shape), g[name]
        err = np.abs(a - ref).max()
        assert err <= 1e-3 * np.abs(ref).max(), f"{name}: {err} vs scale {np.abs(ref).max()}"
