"""Pins the checker's rasterizer (forward and backward) against an independent float64 numpy model written from the
mathematics of ray / 3D-Gaussian compositing (3DGUT, arXiv 2412.12507), and against central finite differences of
that model.  The model evaluates the peak response of a Gaussian along a ray as
|a|^2 - (a.b)^2 / |b|^2 (a = M (o - mu), b = M d) rather than through the cross product the reference uses, so a
wrong operand order or a dropped term in the restatement shows up."""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation

TILE = 16


def scene(n=120, W=48, H=32, seed=0, opac_lo=0.3):
    rng = np.random.default_rng(seed)
    means = np.stack([rng.uniform(-0.5, 0.5, n), rng.uniform(-0.33, 0.33, n), rng.uniform(-0.4, 0.4, n)], 1)
    quats = rng.normal(0, 1, (n, 4))
    scales = np.exp(rng.uniform(np.log(0.04), np.log(0.15), (n, 3)))
    opac = rng.uniform(opac_lo, 0.99, n)
    colors = rng.uniform(0, 1, (n, 3))
    V = np.eye(4)
    V[:3, :3] = Rotation.from_euler("xyz", [0.1, -0.15, 0.05]).as_matrix()
    V[:3, 3] = [0.02, -0.03, 2.0]
    K = np.array([[60.0, 0, W / 2], [0, 58.0, H / 2], [0, 0, 1]])
    f32 = lambda a: np.ascontiguousarray(a, dtype=np.float32)
    return dict(means=f32(means), quats=f32(quats), scales=f32(scales), opac=f32(opac), colors=f32(colors), V=f32(V),
                K=f32(K), W=W, H=H, bg=f32([[0.2, 0.1, 0.3]]))


def lists(orc, s):
    radii, m2, depths, conics, _ = orc.projection_ut_3dgs_fused(s["means"], s["quats"], s["scales"], s["opac"],
                                                                s["V"][None], s["K"][None], s["W"], s["H"])
    tw, th = (s["W"] + TILE - 1) // TILE, (s["H"] + TILE - 1) // TILE
    _, ids, flat = orc.intersect_tile(m2, radii, depths, 1, TILE, tw, th)
    off = orc.intersect_offset(ids, 1, tw, th)
    return off, flat, tw, th


def model_render(p, s, off, flat, tw, th, return_last=False):
    """float64 model.  p: dict of float64 arrays means, quats, scales, opac, colors."""
    W, H = s["W"], s["H"]
    V, K = s["V"].astype(np.float64), s["K"].astype(np.float64)
    Rc, t = V[:3, :3], V[:3, 3]
    cam_o = -Rc.T @ t
    n = p["means"].shape[0]
    M = np.zeros((n, 3, 3))
    for g in range(n):
        q = p["quats"][g] / np.linalg.norm(p["quats"][g])
        Rg = Rotation.from_quat([q[1], q[2], q[3], q[0]]).as_matrix()
        M[g] = np.diag(1.0 / p["scales"][g]) @ Rg.T
    img = np.zeros((H, W, 3))
    alpha_img = np.zeros((H, W))
    last = np.zeros((H, W), np.int64)
    offs = off.ravel()
    n_is = flat.shape[0]
    for i in range(H):
        for j in range(W):
            tile = (i // TILE) * tw + (j // TILE)
            lo = offs[tile]
            hi = n_is if tile == tw * th - 1 else offs[tile + 1]
            dc = np.array([(j + 0.5 - K[0, 2]) / K[0, 0], (i + 0.5 - K[1, 2]) / K[1, 1], 1.0])
            d = Rc.T @ (dc / np.linalg.norm(dc))
            T, pix, cur = 1.0, np.zeros(3), 0
            for idx in range(lo, hi):
                g = flat[idx]
                a = M[g] @ (cam_o - p["means"][g])
                b = M[g] @ d
                dist2 = a @ a - (a @ b) ** 2 / (b @ b)
                al = min(0.999, p["opac"][g] * np.exp(-0.5 * dist2))
                if al < 1.0 / 255.0:
                    continue
                nT = T * (1 - al)
                if nT <= 1e-4:
                    break
                pix += p["colors"][g] * al * T
                T, cur = nT, idx
            img[i, j] = pix + T * s["bg"][0].astype(np.float64)
            alpha_img[i, j] = 1 - T
            last[i, j] = cur
    if return_last:
        return img, alpha_img, last
    return img, alpha_img


def as_f64(s):
    return {k: s[k].astype(np.float64) for k in ("means", "quats", "scales", "opac", "colors")}


def test_forward_matches_float64_model(orc):
    s = scene()
    off, flat, tw, th = lists(orc, s)
    assert flat.shape[0] > 60
    r, a, last = orc.rasterize_to_pixels_from_world_3dgs_fwd(s["means"], s["quats"], s["scales"], s["colors"][None],
                                                             s["opac"][None], s["bg"], None, s["W"], s["H"], TILE,
                                                             s["V"][None], s["K"][None], off, flat)
    img, al, mlast = model_render(as_f64(s), s, off, flat, tw, th, True)
    assert al.mean() > 0.3 and (al > 0.9998).any()  # covered, and some pixels saturate (early termination exercised)
    np.testing.assert_allclose(r[0], img, atol=2e-5)
    np.testing.assert_allclose(a[0, :, :, 0], al, atol=2e-5)
    assert np.array_equal(last[0], mlast)
    # alphas = 1 - T and render = sum c alpha T + T bg: a constant-colour scene renders colour * alpha + T bg
    ones = np.full_like(s["colors"], 0.7)
    r1, a1, _ = orc.rasterize_to_pixels_from_world_3dgs_fwd(s["means"], s["quats"], s["scales"], ones[None],
                                                            s["opac"][None], s["bg"], None, s["W"], s["H"], TILE,
                                                            s["V"][None], s["K"][None], off, flat)
    np.testing.assert_allclose(r1[0], 0.7 * a1[0] + (1 - a1[0]) * s["bg"][0], atol=1e-6)
    # no background: plain sum
    r2, _, _ = orc.rasterize_to_pixels_from_world_3dgs_fwd(s["means"], s["quats"], s["scales"], s["colors"][None],
                                                           s["opac"][None], None, None, s["W"], s["H"], TILE,
                                                           s["V"][None], s["K"][None], off, flat)
    np.testing.assert_allclose(r2[0], r[0] - (1 - a[0]) * s["bg"][0], atol=1e-6)


def test_forward_single_gaussian_analytic(orc):
    """one isotropic Gaussian on the optical axis: alpha(pixel) = o exp(-|mu x d|^2 / (2 s^2)), d the unit pixel ray"""
    W = H = 32
    s0, o, z = 0.2, 0.8, 3.0
    V = np.eye(4, dtype=np.float32)
    V[2, 3] = z
    K = np.array([[40, 0, 16], [0, 40, 16], [0, 0, 1]], np.float32)
    sc = dict(means=np.zeros((1, 3), np.float32), quats=np.array([[1, 0, 0, 0]], np.float32),
              scales=np.full((1, 3), s0, np.float32), opac=np.array([o], np.float32),
              colors=np.array([[0.2, 0.5, 0.9]], np.float32), V=V, K=K, W=W, H=H)
    off, flat, tw, th = lists(orc, sc)
    r, a, _ = orc.rasterize_to_pixels_from_world_3dgs_fwd(sc["means"], sc["quats"], sc["scales"], sc["colors"][None],
                                                          sc["opac"][None], None, None, W, H, TILE, V[None], K[None],
                                                          off, flat)
    jj, ii = np.meshgrid(np.arange(W) + 0.5, np.arange(H) + 0.5)
    d = np.stack([(jj - 16) / 40, (ii - 16) / 40, np.ones_like(jj)], -1)
    d /= np.linalg.norm(d, axis=-1, keepdims=True)
    mu = np.array([0, 0, z])
    perp2 = (np.cross(np.broadcast_to(mu, d.shape), d) ** 2).sum(-1)
    al = o * np.exp(-0.5 * perp2 / s0 ** 2)
    al[al < 1 / 255] = 0
    np.testing.assert_allclose(a[0, :, :, 0], al, atol=2e-6)
    np.testing.assert_allclose(r[0], al[..., None] * sc["colors"][0], atol=2e-6)


def test_forward_is_invariant_to_storage_order(orc):
    s = scene(seed=3)
    perm = np.random.default_rng(1).permutation(s["means"].shape[0])
    outs = []
    for order in (np.arange(len(perm)), perm):
        t = dict(s, **{k: np.ascontiguousarray(s[k][order]) for k in ("means", "quats", "scales", "opac", "colors")})
        off, flat, tw, th = lists(orc, t)
        outs.append(orc.rasterize_to_pixels_from_world_3dgs_fwd(t["means"], t["quats"], t["scales"],
                                                                t["colors"][None], t["opac"][None], t["bg"], None,
                                                                t["W"], t["H"], TILE, t["V"][None], t["K"][None], off,
                                                                flat))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])


def test_backward_matches_finite_differences_of_the_model(orc):
    s = scene(n=24, seed=5)
    off, flat, tw, th = lists(orc, s)
    rng = np.random.default_rng(7)
    W, H = s["W"], s["H"]
    w_img = rng.normal(0, 1, (H, W, 3))
    w_al = rng.normal(0, 1, (H, W))
    r, a, last = orc.rasterize_to_pixels_from_world_3dgs_fwd(s["means"], s["quats"], s["scales"], s["colors"][None],
                                                             s["opac"][None], s["bg"], None, W, H, TILE, s["V"][None],
                                                             s["K"][None], off, flat)
    args = (s["means"], s["quats"], s["scales"], s["colors"][None], s["opac"][None], s["bg"])
    g32 = orc.rasterize_to_pixels_from_world_3dgs_bwd(*args, None, W, H, TILE, s["V"][None], s["K"][None], off, flat, a,
                                                      last, w_img[None].astype(np.float32),
                                                      w_al[None, :, :, None].astype(np.float32))
    g64, b64 = orc.rasterize_bwd_f64(*args, W, H, TILE, s["V"][None], s["K"][None], off, flat, a, last,
                                     w_img[None].astype(np.float32), w_al[None, :, :, None].astype(np.float32))
    # the absolute-value chain: never below the value, zero only where the value is, and u * bound is the scale of the
    # fp32 evaluation's own error (it would not be if a term were missing from the chain or the chain were inflated)
    assert (b64 >= np.abs(g64) * (1 - 1e-12)).all() and ((b64 == 0) == (g64 == 0)).all()
    c32 = np.concatenate([g32[0], g32[1], g32[2], g32[3][0], g32[4].reshape(-1, 1)], 1).astype(np.float64)
    need = (np.abs(c32 - g64) - 1e-3 * np.abs(g64)) / np.maximum(2.0 ** -24 * b64, 1e-300)
    assert need.max() < 64, need.max()
    assert np.quantile(np.abs(c32 - g64)[b64 > 0] / (2.0 ** -24 * b64[b64 > 0]), 0.99) > 0.05
    w32i, w32a = w_img.astype(np.float32).astype(np.float64), w_al.astype(np.float32).astype(np.float64)

    def loss(p):
        img, al = model_render(p, s, off, flat, tw, th)
        return (img * w32i).sum() + (al * w32a).sum()

    base = as_f64(s)
    cols = dict(means=(0, 3), quats=(3, 7), scales=(7, 10), colors=(10, 13), opac=(13, 14))
    cat32 = np.concatenate([g32[0], g32[1], g32[2], g32[3][0], g32[4].reshape(-1, 1)], 1)
    scale_of = {k: np.abs(g64[:, lo:hi]).max() for k, (lo, hi) in cols.items()}
    checked = 0
    for g in (0, 3, 7, 11, 16, 21):
        for name, (lo, hi) in cols.items():
            for c in range(hi - lo):
                h = 1e-6
                pp, pm = {k: v.copy() for k, v in base.items()}, {k: v.copy() for k, v in base.items()}
                if name == "opac":
                    pp[name][g] += h
                    pm[name][g] -= h
                else:
                    pp[name][g, c] += h
                    pm[name][g, c] -= h
                num = (loss(pp) - loss(pm)) / (2 * h)
                tol = 2e-4 * scale_of[name] + 1e-3 * abs(num)
                assert abs(g64[g, lo + c] - num) <= tol, (g, name, c, g64[g, lo + c], num)
                assert abs(cat32[g, lo + c] - num) <= 5 * tol, (g, name, c, cat32[g, lo + c], num)
                checked += 1
    assert checked == 6 * 14
    # colour gradient closed form: v_colors[g] = sum_pixels alpha T v_render; zero for Gaussians that reach no pixel
    assert np.all(np.abs(g64[:, 10:13]).sum(1)[np.bincount(flat, minlength=24) == 0] == 0)


@pytest.mark.parametrize("trial", range(10))
def test_record_pixel_bounds_are_conservative(gsx, orc, trial):
    """The per-Gaussian pixel bounds the GPU rasterizers skip by (csrc/gsx_record.h, compiled here for the host) must
    contain every pixel that reaches alpha >= 1/255 in the checker's per-pair arithmetic: brute force over all pixels
    for Gaussians from sub-pixel to screen-filling, anisotropy up to ~1e3, opacities from below the threshold to 1,
    cameras inside the cloud, long focal lengths and an off-centre crop of a large image.  Trials 7 and 8: larger
    draws of the most anisotropic case - among them needles that reach towards the camera plane, whose silhouette is
    an ellipse hundreds of image widths long (nearly a parabola: the region must give up on those).  Trial 9: thin
    needles far from the camera at a long focal length (axis ratios up to ~150 at every angle, where the region's
    quadratic form is a small sum of large terms); most of them must still get a proper region."""
    seed, base = 100 + trial, trial
    if trial in (7, 8):
        seed, base = [2005, 3105][trial - 7], 5
    needles = trial == 9
    if needles:
        base = 7
    rng = np.random.default_rng(seed)
    n, W, H = (1200 if trial < 7 else 6000), 160, 120
    trial = base
    f = [150.0, 400.0, 80.0, 1000.0, 150.0, 150.0, 3200.0, 3200.0][trial]
    radius = [4.0, 4.0, 2.0, 6.0, 1.0, 4.0, 4.0, 4.0][trial]
    cam = gsx.scenes.orbit_camera(0.3 + trial, radius, W, H, f)
    if trial == 6:  # a 160x120 window far from the principal point of a 3840x2160 image
        cam.K = gsx.scenes.intrinsics(W, H, f, f, 1900.0, -950.0)
    spread = [0.6, 0.6, 0.6, 0.3, 0.8, 0.6, 0.5, 0.05][trial]
    means = rng.normal(0, spread, (n, 3)).astype(np.float32)
    if trial == 6:
        means += np.linalg.inv(cam.viewmat)[:3, :3] @ np.array([-2.2, 1.3, 0.0], np.float32)  # into the window
    aniso = [0.3, 1.0, 1.5, 0.5, 1.0, 2.0, 1.0, 1.0][trial]
    log_s = rng.uniform(np.log(1e-4), np.log(0.5), (n, 1)) + rng.normal(0, aniso, (n, 3))
    if needles:
        log_s = rng.normal(-5.0, 1.0, (n, 3))
        log_s[:, 0] += rng.uniform(0.0, 5.0, n)
    scales = np.exp(log_s).astype(np.float32)
    quats = rng.normal(0, 1, (n, 4)).astype(np.float32)
    op = np.exp(rng.uniform(np.log(1 / 300), 0, n)).astype(np.float32)
    bounds, count, outside, blocks_true, blocks_hit = orc.record_bounds_check(means, quats, scales, op, cam.viewmat,
                                                                              cam.K, W, H)
    assert outside.sum() == 0, f"{(outside > 0).sum()} Gaussians have contributing pixels outside their region"
    assert (count > 0).sum() > 100  # the case is not vacuous
    box = np.maximum(bounds[:, 2] - bounds[:, 0] + 1, 0) * np.maximum(bounds[:, 3] - bounds[:, 1] + 1, 0)
    proper = box < W * H
    assert box[proper].sum() < 3.0 * max(count[proper].sum(), 1) + 16 * proper.sum()  # and they are tight
    assert (box[op < 1 / 256] == 0).all()  # below the alpha threshold: empty
    assert (blocks_hit >= blocks_true).all()
    if needles:
        print('blocks hit / true over all needles', blocks_hit.sum(), blocks_true.sum())
        assert blocks_hit.sum() < 1.5 * blocks_true.sum()  # few needles lose their region to the conditioning guard
    assert blocks_hit[proper].sum() < 2.5 * blocks_true[proper].sum() + 6 * proper.sum()  # 8x8 block test is tight
