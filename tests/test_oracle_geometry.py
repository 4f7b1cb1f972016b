"""Pins the checker's projection, spherical harmonics, tile intersection, sort and offsets against independent
statements of the mathematics (float64 numpy models, closed forms, brute force), since the reference holds no
golden vectors for this path (its only test, tests/test_render_modes.cpp, checks tensor shapes)."""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation


def look_cam(W=640, H=480, f=500.0, z=4.0):
    V = np.eye(4, dtype=np.float32)
    V[2, 3] = z
    K = np.array([[f, 0, W / 2], [0, f, H / 2], [0, 0, 1]], np.float32)
    return V, K, W, H


# ---------------------------------------------------------------------------------------------
# unscented-transform projection
# ---------------------------------------------------------------------------------------------
def ut_project_f64(mean, quat_wxyz, scale, V, K, alpha=0.1, beta=2.0, kappa=0.0, eps2d=0.3):
    """Unscented transform of N(mean, R diag(s^2) R^T) through the pinhole camera, written from the definition
    (Wan & van der Merwe 2000 weights; sigma points along the principal axes) in float64."""
    q = np.asarray(quat_wxyz, np.float64)
    q = q / np.linalg.norm(q)
    Rg = Rotation.from_quat([q[1], q[2], q[3], q[0]]).as_matrix()
    lam = float(np.float32(np.float32(alpha) * np.float32(alpha) * np.float32(3.0 + kappa)) - np.float32(3.0))
    n = 3.0
    pts = [np.asarray(mean, np.float64)]
    for sgn in (+1, -1):
        for i in range(3):
            pts.append(mean + sgn * np.sqrt(n + lam) * scale[i] * Rg[:, i])
    wm = np.array([lam / (n + lam)] + [1 / (2 * (n + lam))] * 6)
    wc = wm.copy()
    wc[0] += 1 - alpha * alpha + beta
    Rc, t = V[:3, :3].astype(np.float64), V[:3, 3].astype(np.float64)
    uv = []
    for p in pts:
        c = Rc @ p + t
        uv.append(np.array([K[0, 0] * c[0] / c[2] + K[0, 2], K[1, 1] * c[1] / c[2] + K[1, 2]]))
    uv = np.array(uv)
    m = (wm[:, None] * uv).sum(0)
    d = uv - m
    cov = (wc[:, None, None] * d[:, :, None] * d[:, None, :]).sum(0)
    det0 = np.linalg.det(cov)
    cov = cov + eps2d * np.eye(2)
    comp = np.sqrt(max(0.0, det0 / np.linalg.det(cov)))
    return m, cov, comp, (Rc @ mean + t)[2]


def ewa_cov_f64(mean, quat_wxyz, scale, V, K):
    """Jacobian (EWA) projection of the same Gaussian: J W Sigma W^T J^T (Zwicker et al. 2001)."""
    q = np.asarray(quat_wxyz, np.float64)
    q = q / np.linalg.norm(q)
    Rg = Rotation.from_quat([q[1], q[2], q[3], q[0]]).as_matrix()
    Sigma = Rg @ np.diag(np.asarray(scale, np.float64) ** 2) @ Rg.T
    Wm, t = V[:3, :3].astype(np.float64), V[:3, 3].astype(np.float64)
    x, y, z = Wm @ mean + t
    J = np.array([[K[0, 0] / z, 0, -K[0, 0] * x / z ** 2], [0, K[1, 1] / z, -K[1, 1] * y / z ** 2]])
    return J @ Wm @ Sigma @ Wm.T @ J.T


def test_projection_isotropic_on_axis_closed_form(orc):
    V, K, W, H = look_cam()
    s, f, z, o = 0.05, 500.0, 4.0, 0.8
    r = orc.projection_ut_3dgs_fused(np.zeros((1, 3)), [[1, 0, 0, 0]], [[s, s, s]], [o], V[None], K[None], W, H,
                                     calc_compensations=True)
    radii, m2, depth, conic, comp = r
    np.testing.assert_allclose(m2[0, 0], [W / 2, H / 2], atol=2e-2)
    var = (f * s / z) ** 2  # up to O(s^2/z^2) relative
    cov = var + 0.3
    np.testing.assert_allclose(conic[0, 0], [1 / cov, 0, 1 / cov], rtol=2e-3, atol=1e-5)
    assert depth[0, 0] == np.float32(z)
    ext = min(3.33, np.sqrt(2 * np.log(o * np.sqrt(var * var / (cov * cov)) * 255)))
    assert abs(int(radii[0, 0, 0]) - np.ceil(ext * np.sqrt(cov))) <= 1 and radii[0, 0, 0] == radii[0, 0, 1]
    np.testing.assert_allclose(comp[0, 0], var / cov, rtol=2e-3)


def test_projection_matches_float64_unscented_transform_and_ewa_limit(orc):
    rng = np.random.default_rng(0)
    V = np.eye(4, dtype=np.float32)
    V[:3, :3] = Rotation.from_euler("xyz", [0.2, -0.3, 0.1]).as_matrix()
    V[:3, 3] = [0.1, -0.2, 5.0]
    K = np.array([[600, 0, 330], [0, 580, 250], [0, 0, 1]], np.float32)
    W, H = 640, 480
    n = 300
    means = rng.uniform(-1, 1, (n, 3)).astype(np.float32)
    quats = rng.normal(0, 1, (n, 4)).astype(np.float32)
    scales = np.exp(rng.uniform(np.log(0.05), np.log(0.3), (n, 3))).astype(np.float32)
    radii, m2, depth, conic, comp = orc.projection_ut_3dgs_fused(means, quats, scales, None, V[None], K[None], W, H,
                                                                 calc_compensations=True)
    checked = 0
    for i in range(n):
        if radii[0, i, 0] == 0:
            continue
        m, cov, c, z = ut_project_f64(means[i].astype(np.float64), quats[i], scales[i].astype(np.float64), V, K)
        # -99 p0 + 16.7 sum(p_i): the weights amplify fp32 rounding of pixel coordinates (~600) about 100x
        np.testing.assert_allclose(m2[0, i], m, atol=3e-2)
        np.testing.assert_allclose(conic[0, i], [np.linalg.inv(cov)[0, 0], np.linalg.inv(cov)[0, 1],
                                                 np.linalg.inv(cov)[1, 1]], rtol=3e-2, atol=2e-5)
        np.testing.assert_allclose(depth[0, i], z, rtol=1e-6)
        np.testing.assert_allclose(comp[0, i], c, rtol=2e-2)
        ext = 3.33
        b = 0.5 * (cov[0, 0] + cov[1, 1])
        v1 = b + np.sqrt(max(0.01, b * b - np.linalg.det(cov)))
        rx = np.ceil(min(ext * np.sqrt(cov[0, 0]), ext * np.sqrt(v1)))
        ry = np.ceil(min(ext * np.sqrt(cov[1, 1]), ext * np.sqrt(v1)))
        assert abs(radii[0, i, 0] - rx) <= 1 and abs(radii[0, i, 1] - ry) <= 1
        checked += 1
    assert checked > 100
    # the float64 model itself: for small Gaussians the unscented transform tends to the Jacobian (EWA) projection
    for i in range(20):
        s = scales[i].astype(np.float64) * 0.02
        _, cov, _, _ = ut_project_f64(means[i].astype(np.float64), quats[i], s, V, K, eps2d=0.0)
        np.testing.assert_allclose(cov, ewa_cov_f64(means[i].astype(np.float64), quats[i], s, V, K), rtol=2e-3,
                                   atol=1e-9)


def test_projection_plain_route_equals_the_general_route_to_rounding(orc):
    """the trainer's camera takes the sigma points through the pose as a matrix and projects with one reciprocal per
    point; with all-zero distortion coefficients the same camera takes the general route (quaternion rotation, a
    division per coordinate).  Same function, other rounding: radii within one unit on a handful of Gaussians, image
    points within what the unscented weights (-99, +16.7) make of a few ulp, depths within 4 ulp - and the plain
    route is no further from the float64 model than the general one"""
    rng = np.random.default_rng(3)
    V = np.eye(4, dtype=np.float32)
    V[:3, :3] = Rotation.from_euler("xyz", [0.2, -0.3, 0.1]).as_matrix()
    V[:3, 3] = [0.1, -0.2, 5.0]
    K = np.array([[600, 0, 330], [0, 580, 250], [0, 0, 1]], np.float32)
    W, H = 640, 480
    n = 4000
    means = rng.uniform(-1.5, 1.5, (n, 3)).astype(np.float32)
    quats = rng.normal(0, 1, (n, 4)).astype(np.float32)
    scales = np.exp(rng.uniform(np.log(0.01), np.log(0.3), (n, 3))).astype(np.float32)
    plain = orc.projection_ut_3dgs_fused(means, quats, scales, None, V[None], K[None], W, H)
    with orc.distortion(radial=[0.0] * 6, tangential=[0.0] * 2, thin_prism=[0.0] * 4):
        general = orc.projection_ut_3dgs_fused(means, quats, scales, None, V[None], K[None], W, H)
    ra, rb = plain[0][0].astype(np.int64), general[0][0].astype(np.int64)
    assert np.abs(ra - rb).max() <= 1 and (ra != rb).any(axis=1).mean() < 2e-3
    vis = (ra[:, 0] > 0) & (rb[:, 0] > 0)
    assert vis.sum() > 3000
    assert np.abs(plain[1][0][vis] - general[1][0][vis]).max() < 0.03
    assert (np.abs(plain[2][0][vis] - general[2][0][vis]) <= 4 * np.spacing(np.abs(general[2][0][vis]))).all()
    assert not np.array_equal(plain[1][0][vis], general[1][0][vis])  # they ARE two evaluations
    err_p, err_g = [], []
    for i in np.flatnonzero(vis)[:200]:
        m, _, _, _ = ut_project_f64(means[i].astype(np.float64), quats[i], scales[i].astype(np.float64), V, K)
        err_p.append(np.abs(plain[1][0, i] - m).max())
        err_g.append(np.abs(general[1][0, i] - m).max())
    assert np.mean(err_p) <= 1.5 * np.mean(err_g) + 1e-5, (np.mean(err_p), np.mean(err_g))


def test_projection_culling_cases(orc):
    V, K, W, H = look_cam()
    one = lambda mean, s=0.05, o=0.9, **kw: orc.projection_ut_3dgs_fused(
        [mean], [[1, 0, 0, 0]], [[s, s, s]], None if o is None else [o], V[None], K[None], W, H, **kw)[0][0, 0]
    assert one([0, 0, 0])[0] > 0
    assert tuple(one([0, 0, -3.995])) == (0, 0)            # z = 0.005 < near 0.01
    assert tuple(one([0, 0, 0], far_plane=3.0)) == (0, 0)  # z = 4 > far
    # a sigma point behind the camera plane: z_c = 0.1, sigma points at z_c -/+ 0.173 * 1.0 along the view axis
    behind = orc.projection_ut_3dgs_fused([[0, 0, -3.9]], [[1, 0, 0, 0]], [[1e-3, 1e-3, 1.0]], [0.9], V[None], K[None],
                                          W, H)[0][0, 0]
    assert tuple(behind) == (0, 0)
    ahead = orc.projection_ut_3dgs_fused([[0, 0, -3.9]], [[1, 0, 0, 0]], [[1e-3, 1e-3, 0.5]], [0.9], V[None], K[None],
                                         W, H)[0][0, 0]
    assert ahead[0] > 0
    assert tuple(one([2.9, 0, 0])) == (0, 0)               # u = 320 + 500*2.9/4 = 682 >= 1.1 W... outside the margin
    assert one([2.7, 0, 0])[0] > 0                         # u = 657.5 inside the 10 % margin and bbox touches the image
    assert tuple(one([0, 0, 0], o=0.003)) == (0, 0)        # opacity * compensation < 1/255
    assert one([0, 0, 0], o=0.01)[0] > 0
    assert tuple(one([0, 0, 0], s=1e-4, radius_clip=3.0)) == (0, 0)  # radius <= radius_clip
    # opacity-aware extent shrinks the radius (Section B.2 of arXiv 2402.00525)
    assert one([0, 0, 0], o=0.01)[0] < one([0, 0, 0], o=0.9)[0] <= one([0, 0, 0], o=None)[0]
    # require_all_sigma_points_valid = False keeps a Gaussian with one invalid sigma point
    ut = dict(require_all_sigma_points_valid=False)
    assert orc.projection_ut_3dgs_fused([[2.88, 0, 0]], [[1, 0, 0, 0]], [[0.3, 0.3, 0.3]], None, V[None], K[None], W,
                                        H, ut=ut)[0][0, 0, 0] > 0


# ---------------------------------------------------------------------------------------------
# spherical harmonics
# ---------------------------------------------------------------------------------------------
def sh_basis_polynomials(d):
    """Real SH basis in the explicit polynomial form of the original 3DGS / tiny-cuda-nn code (an algebraically
    different statement from the Sloan recurrences the reference's gsplat kernel uses), degrees 0-3."""
    x, y, z = d[..., 0], d[..., 1], d[..., 2]
    xx, yy, zz, xy, yz, xz = x * x, y * y, z * z, x * y, y * z, x * z
    return np.stack([
        0.28209479177387814 * np.ones_like(x),
        -0.4886025119029199 * y, 0.4886025119029199 * z, -0.4886025119029199 * x,
        1.0925484305920792 * xy, -1.0925484305920792 * yz, 0.31539156525252005 * (2 * zz - xx - yy),
        -1.0925484305920792 * xz, 0.5462742152960396 * (xx - yy),
        -0.5900435899266435 * y * (3 * xx - yy), 2.890611442640554 * xy * z,
        -0.4570457994644658 * y * (4 * zz - xx - yy), 0.3731763325901154 * z * (2 * zz - 3 * xx - 3 * yy),
        -0.4570457994644658 * x * (4 * zz - xx - yy), 1.445305721320277 * z * (xx - yy),
        -0.5900435899266435 * x * (xx - 3 * yy)], -1)


def sh_band4_scipy(d):
    """The nine real spherical harmonics of degree 4 in float64 from scipy's complex ones (an independent statement
    of the band: sqrt(2) Im / Re parts, m = -4 .. 4), without the reference's sign convention - callers fix the nine
    signs against the checker's forward basis, which test_sh_basis_* pin."""
    from scipy import special
    x, y, z = d[..., 0], d[..., 1], d[..., 2]
    theta, phi = np.arccos(np.clip(z, -1, 1)), np.arctan2(y, x)
    out = []
    for m in range(-4, 5):
        Y = special.sph_harm_y(4, abs(m), theta, phi)
        out.append(Y.real if m == 0 else np.sqrt(2) * (Y.imag if m < 0 else Y.real))
    return np.stack(out, -1)


def sh_basis_25(orc, d):
    """float64 basis of degrees 0-4: the polynomial form for 0-3, scipy's band for 4 with the signs of the checker"""
    dn = d / np.linalg.norm(d, axis=-1, keepdims=True)
    probe = np.random.default_rng(5).normal(0, 1, (64, 3))
    probe /= np.linalg.norm(probe, axis=1, keepdims=True)
    got = checker_basis(orc, probe.astype(np.float32), 4)[:, 16:25]
    raw = sh_band4_scipy(probe)
    sign = np.sign((got * raw).sum(0))
    np.testing.assert_allclose(got, raw * sign, atol=5e-6)  # the band itself, up to the nine signs
    return np.concatenate([sh_basis_polynomials(dn), sh_band4_scipy(dn) * sign], -1)


def checker_basis(orc, dirs, degree, K=25):
    """basis values through the checker: colour of a one-hot coefficient vector"""
    n = dirs.shape[0]
    B = np.zeros((n, K))
    for k in range((degree + 1) ** 2):
        co = np.zeros((n, K, 3), np.float32)
        co[:, k, 0] = 1.0
        B[:, k] = orc.spherical_harmonics_fwd(degree, dirs, co)[:, 0]
    return B


def test_sh_basis_matches_polynomial_form(orc):
    rng = np.random.default_rng(0)
    d = rng.normal(0, 1, (2000, 3))
    dn = d / np.linalg.norm(d, axis=1, keepdims=True)
    scale = rng.uniform(0.1, 10, (2000, 1))  # the kernel normalises the direction itself
    B = checker_basis(orc, (dn * scale).astype(np.float32), 3)
    np.testing.assert_allclose(B[:, :16], sh_basis_polynomials(dn), atol=3e-6)
    # lower degrees use the leading bases only
    for deg in (0, 1, 2):
        Bd = checker_basis(orc, dn.astype(np.float32), deg)
        nb = (deg + 1) ** 2
        np.testing.assert_allclose(Bd[:, :nb], sh_basis_polynomials(dn)[:, :nb], atol=3e-6)
        assert np.all(Bd[:, nb:] == 0)


def test_sh_basis_degree4_orthonormal_and_harmonic(orc):
    # Gauss-Legendre x uniform-phi product quadrature integrates polynomials of degree <= 8 on the sphere exactly
    nt, nphi = 12, 24
    ct, wt = np.polynomial.legendre.leggauss(nt)
    phi = (np.arange(nphi) + 0.5) * 2 * np.pi / nphi
    CT, PH = np.meshgrid(ct, phi, indexing="ij")
    st = np.sqrt(1 - CT ** 2)
    d = np.stack([st * np.cos(PH), st * np.sin(PH), CT], -1).reshape(-1, 3)
    w = (wt[:, None] * np.ones(nphi)[None] * 2 * np.pi / nphi).reshape(-1)
    B = checker_basis(orc, d.astype(np.float32), 4)
    G = (B * w[:, None]).T @ B
    np.testing.assert_allclose(G, np.eye(25), atol=2e-5)
    # parity (-1)^l under d -> -d pins the degree of each band
    Bm = checker_basis(orc, (-d).astype(np.float32), 4)
    deg = np.concatenate([[l] * (2 * l + 1) for l in range(5)])
    np.testing.assert_allclose(Bm, B * ((-1.0) ** deg)[None], atol=2e-6)
    # the m = 0 members are the Legendre polynomials in z, with positive sign at the pole
    pole = checker_basis(orc, np.array([[0, 0, 1.0]], np.float32), 4)[0]
    for l in range(5):
        assert abs(pole[l * l + l] - np.sqrt((2 * l + 1) / (4 * np.pi))) < 2e-6


def test_sh_colour_and_adjoint(orc):
    rng = np.random.default_rng(1)
    n, K = 500, 25
    dirs = rng.normal(0, 1, (n, 3)).astype(np.float32)
    co = rng.normal(0, 1, (n, K, 3)).astype(np.float32)
    masks = rng.uniform(0, 1, n) < 0.7
    dn = dirs / np.linalg.norm(dirs, axis=1, keepdims=True)
    for deg in range(5):
        col = orc.spherical_harmonics_fwd(deg, dirs, co, masks)
        nb = (deg + 1) ** 2
        want = np.einsum("nk,nkc->nc", sh_basis_25(orc, dn.astype(np.float64))[:, :nb], co[:, :nb].astype(np.float64))
        np.testing.assert_allclose(col[masks], want[masks], atol=2e-5)
        assert np.all(col[~masks] == 0)
        # backward = transpose of forward:  <v, fwd(c)> == <bwd(v), c>
        v = rng.normal(0, 1, (n, 3)).astype(np.float32)
        vc, vd = orc.spherical_harmonics_bwd(K, deg, dirs, co, masks, v, True)
        lhs = (v[masks].astype(np.float64) * col[masks]).sum()
        rhs = (vc.astype(np.float64) * co).sum()
        assert abs(lhs - rhs) < 1e-3 * max(1.0, abs(lhs))
        assert np.all(vc[~masks] == 0) and np.all(vc[:, nb:] == 0)
        # direction gradient against central differences of the float64 polynomial form
        h = 1e-6
        for j in range(3):
            dp, dm = dirs.astype(np.float64).copy(), dirs.astype(np.float64).copy()
            dp[:, j] += h
            dm[:, j] -= h
            fp = np.einsum("nk,nkc->nc", sh_basis_25(orc, dp)[:, :nb], co[:, :nb].astype(np.float64))
            fm = np.einsum("nk,nkc->nc", sh_basis_25(orc, dm)[:, :nb], co[:, :nb].astype(np.float64))
            num = ((fp - fm) / (2 * h) * v).sum(1)
            np.testing.assert_allclose(vd[masks, j], num[masks], rtol=2e-3, atol=2e-4)


def test_sh_colors_from_world_glue(orc):
    """dirs = means - campos with campos = -R^T t, radii mask, +0.5 and clamp at 0 (Rasterization.cpp:356-378)"""
    rng = np.random.default_rng(2)
    n, K = 300, 16
    V = np.eye(4, dtype=np.float32)
    V[:3, :3] = Rotation.from_euler("xyz", [0.3, 0.5, -0.2]).as_matrix()
    V[:3, 3] = [0.3, -0.1, 4.0]
    campos = np.linalg.inv(V.astype(np.float64))[:3, 3]
    means = rng.normal(0, 1, (n, 3)).astype(np.float32)
    co = rng.normal(0, 0.6, (n, K, 3)).astype(np.float32)
    radii = rng.integers(0, 3, (n, 2)).astype(np.int32)
    col = orc.sh_colors_from_world(3, means, co, radii, V)
    d = means.astype(np.float64) - campos
    want = np.maximum(np.einsum("nk,nkc->nc", sh_basis_polynomials(d / np.linalg.norm(d, axis=1, keepdims=True)),
                                co.astype(np.float64)) + 0.5, 0)
    vis = (radii > 0).all(1)
    np.testing.assert_allclose(col[vis], want[vis], atol=3e-5)
    assert np.all(col[~vis] == 0) and (col[vis] == 0).any() and (col[vis] > 0).any()
    v = rng.normal(0, 1, (n, 3)).astype(np.float32)
    vsh = orc.sh_colors_from_world_bwd(3, means, K, radii, V, col, v)
    Bm = sh_basis_polynomials(d / np.linalg.norm(d, axis=1, keepdims=True))
    want_v = Bm[:, :, None] * np.where(col > 0, v, 0)[:, None, :] * vis[:, None, None]
    np.testing.assert_allclose(vsh, want_v, atol=3e-5)


# ---------------------------------------------------------------------------------------------
# tile intersection, sort, offsets
# ---------------------------------------------------------------------------------------------
def brute_force_tiles(means2d, radii, tile, tw, th):
    out = []
    for g in range(means2d.shape[0]):
        rx, ry = radii[g]
        if rx <= 0 or ry <= 0:
            out.append([])
            continue
        x0 = min(max(0, int(np.floor(np.float32(means2d[g, 0] / tile) - np.float32(rx / tile)))), tw)
        x1 = min(max(0, int(np.ceil(np.float32(means2d[g, 0] / tile) + np.float32(rx / tile)))), tw)
        y0 = min(max(0, int(np.floor(np.float32(means2d[g, 1] / tile) - np.float32(ry / tile)))), th)
        y1 = min(max(0, int(np.ceil(np.float32(means2d[g, 1] / tile) + np.float32(ry / tile)))), th)
        out.append([i * tw + j for i in range(y0, y1) for j in range(x0, x1)])
    return out


def test_intersect_brute_force_and_invariants(orc):
    rng = np.random.default_rng(0)
    n, W, H, tile = 400, 200, 120, 16
    tw, th = (W + 15) // 16, (H + 15) // 16
    means2d = rng.uniform(-60, 260, (1, n, 2)).astype(np.float32)  # includes centres left of / above the image
    radii = rng.integers(0, 40, (1, n, 2)).astype(np.int32)
    radii[0, ::9] = 0
    depths = np.exp(rng.normal(1, 0.5, (1, n))).astype(np.float32)
    tpg, ids, flat = orc.intersect_tile(means2d, radii, depths, 1, tile, tw, th, sort=False)
    want = brute_force_tiles(means2d[0], radii[0], tile, tw, th)
    assert [len(t) for t in want] == list(tpg[0])
    assert tpg.sum() == ids.shape[0] == flat.shape[0] > 0
    exp_ids = np.array([(t << 32) | int(depths[0, g].view(np.uint32)) for g, ts in enumerate(want) for t in ts],
                       np.int64)
    exp_flat = np.array([g for g, ts in enumerate(want) for _ in ts], np.int32)
    assert np.array_equal(ids, exp_ids) and np.array_equal(flat, exp_flat)
    # sorted: stable ascending on (tile, depth bits); ties keep emission order
    _, sid, sflat = orc.intersect_tile(means2d, radii, depths, 1, tile, tw, th, sort=True)
    order = np.argsort(exp_ids, kind="stable")
    assert np.array_equal(sid, exp_ids[order]) and np.array_equal(sflat, exp_flat[order])
    off = orc.intersect_offset(sid, 1, tw, th)
    tiles = (sid >> 32)
    cnt = np.bincount(tiles, minlength=tw * th)
    assert np.array_equal(off.ravel(), np.concatenate([[0], np.cumsum(cnt)[:-1]]))
    assert np.all(np.diff(off.ravel()) >= 0)
    assert np.all(orc.intersect_offset(np.zeros(0, np.int64), 1, tw, th) == 0)


def test_intersect_packed_rows_brute_force(orc):
    """packed rows (Intersect.cpp:32-39): the rows of a [C, N] problem that have a footprint, in any order, each naming
    its camera - keys are (camera << (32 + tile bits)) | tile << 32 | depth bits by brute force, values the packed row
    index; sorted, the camera / tile / depth part of the keys equals that of the unpacked problem"""
    rng = np.random.default_rng(5)
    C, n, W, H, tile = 3, 300, 200, 120, 16
    tw, th = (W + 15) // 16, (H + 15) // 16
    means2d = rng.uniform(-60, 260, (C, n, 2)).astype(np.float32)
    radii = rng.integers(0, 40, (C, n, 2)).astype(np.int32)
    radii[:, ::7] = 0
    depths = np.exp(rng.normal(1, 0.5, (C, n))).astype(np.float32)
    keep = np.argwhere((radii > 0).all(-1))
    keep = keep[rng.permutation(len(keep))]  # packed rows come in no particular order
    cam_ids, gauss_ids = keep[:, 0].astype(np.int64), keep[:, 1].astype(np.int64)
    pm, pr, pd = means2d[cam_ids, gauss_ids], radii[cam_ids, gauss_ids], depths[cam_ids, gauss_ids]
    tpg, ids, flat = orc.intersect_tile_packed(pm, pr, pd, cam_ids, C, tile, tw, th, sort=False)
    want = brute_force_tiles(pm, pr, tile, tw, th)
    assert [len(t) for t in want] == list(tpg) and tpg.sum() == ids.shape[0] > 1000
    tile_bits = orc.tile_n_bits(tw * th)
    exp_ids = np.array([(int(cam_ids[r]) << (32 + tile_bits)) | (t << 32) | int(pd[r].view(np.uint32))
                        for r, ts in enumerate(want) for t in ts], np.int64)
    exp_flat = np.array([r for r, ts in enumerate(want) for _ in ts], np.int32)
    assert np.array_equal(ids, exp_ids) and np.array_equal(flat, exp_flat)
    _, sid, sflat = orc.intersect_tile_packed(pm, pr, pd, cam_ids, C, tile, tw, th, sort=True)
    order = np.argsort(exp_ids, kind="stable")
    assert np.array_equal(sid, exp_ids[order]) and np.array_equal(sflat, exp_flat[order])
    # against the unpacked problem: same multiset of keys; per key the same (camera, Gaussian) set
    _, uid, uflat = orc.intersect_tile(means2d, radii, depths, C, tile, tw, th, sort=True)
    assert np.array_equal(sid, uid)
    packed_pairs = sorted(zip(sid.tolist(), (cam_ids[sflat] * n + gauss_ids[sflat]).tolist()))
    assert packed_pairs == sorted(zip(uid.tolist(), uflat.tolist()))


def test_intersect_key_layout_and_bits(orc):
    assert [orc.tile_n_bits(t) for t in (1, 2, 255, 256, 4056, 8160, 32400)] == [1, 2, 8, 9, 12, 13, 15]
    # one Gaussian covering a 2x3 block of tiles: row-major emission, depth bits in the low word
    m2 = np.array([[[40.0, 24.0]]], np.float32)
    rad = np.array([[[20, 10]]], np.int32)
    dep = np.array([[2.5]], np.float32)
    tpg, ids, flat = orc.intersect_tile(m2, rad, dep, 1, 16, 10, 10, sort=False)
    # x tiles floor(2.5 - 1.25) = 1 .. ceil(2.5 + 1.25) = 4 -> 1, 2, 3 ; y tiles floor(1.5 - 0.625) = 0 .. ceil(2.125) = 3
    tiles = [(i * 10 + j) for i in range(0, 3) for j in range(1, 4)]
    assert tpg[0, 0] == 9 and list(ids >> 32) == tiles and np.all(flat == 0)
    assert np.all((ids & 0xffffffff) == int(dep.view(np.uint32)[0, 0]))


def test_radix_sort_is_stable_on_bit_range(orc):
    rng = np.random.default_rng(1)
    n = 20000
    keys = rng.integers(0, 1 << 50, n, dtype=np.int64)
    keys[::3] = keys[0]  # many ties
    vals = np.arange(n, dtype=np.int32)
    for end_bit in (1, 7, 33, 45, 64):
        mask = (1 << end_bit) - 1 if end_bit < 64 else -1
        k, v = orc.radix_sort_pairs(keys, vals, end_bit)
        order = np.argsort((keys & mask).astype(np.uint64), kind="stable")
        assert np.array_equal(k, keys[order]) and np.array_equal(v, vals[order])


# ---------------------------------------------------------------------------------------------------------------
# OpenCV pinhole distortion (Cameras.cuh:473-815)
# ---------------------------------------------------------------------------------------------------------------
_RADIAL = [-0.12, 0.03, -0.004, 0.02, -0.005, 0.001]
_TANGENTIAL = [8e-4, -6e-4]
_THIN_PRISM = [3e-4, -1e-4, -2e-4, 1e-4]


def _rays(n, seed, half_fov=0.6):
    r = np.random.default_rng(seed)
    uv = r.uniform(-np.tan(half_fov), np.tan(half_fov), (n, 2))
    z = r.uniform(0.5, 6.0, (n, 1))
    return np.concatenate([uv * z, z], 1).astype(np.float32)


def test_distortion_off_is_the_pinhole_model(orc):
    """all coefficients zero: image points, rays and the whole UT projection equal the perfect pinhole's bit for bit"""
    pts = _rays(2000, 0)
    a, va = orc.camera_project(pts, 300.0, 310.0, 200.0, 150.0, 400, 300)
    with orc.distortion([0] * 6, [0] * 2, [0] * 4):
        b, vb = orc.camera_project(pts, 300.0, 310.0, 200.0, 150.0, 400, 300)
        rb, okb = orc.camera_unproject(a, 300.0, 310.0, 200.0, 150.0)
    ra, oka = orc.camera_unproject(a, 300.0, 310.0, 200.0, 150.0)
    assert np.array_equal(a.view(np.int32), b.view(np.int32)) and np.array_equal(va, vb)
    assert okb.all() and oka.all() and np.abs(ra - rb).max() <= 1.2e-7  # one Newton step of size 0 later


def test_distortion_special_cases(orc):
    """radial-only: the image radius is f r (1 + k1 r^2 + k2 r^4 + k3 r^6) / (1 + k4 r^2 + ...) along the ray's own
    direction; tangential / thin-prism terms on the axes; validity: icD <= 0.8 and z <= 0 are invalid"""
    f, c = 250.0, 160.0
    pts = _rays(500, 1)
    u, v = pts[:, 0] / pts[:, 2], pts[:, 1] / pts[:, 2]
    r2 = (u.astype(np.float64) ** 2 + v.astype(np.float64) ** 2)
    k = np.array(_RADIAL, np.float64)
    with orc.distortion(radial=_RADIAL):
        ip, _ = orc.camera_project(pts, f, f, c, c, 320, 320, margin=10.0)
    scale = (1 + r2 * (k[0] + r2 * (k[1] + r2 * k[2]))) / (1 + r2 * (k[3] + r2 * (k[4] + r2 * k[5])))
    assert np.abs(ip[:, 0] - (f * u * scale + c)).max() < 2e-4 and np.abs(ip[:, 1] - (f * v * scale + c)).max() < 2e-4
    x = np.linspace(-0.5, 0.5, 11).astype(np.float32)
    on_x = np.stack([x, np.zeros_like(x), np.ones_like(x)], 1)
    with orc.distortion(tangential=[2e-3, -3e-3], thin_prism=[1e-3, 2e-3, -1e-3, 5e-4]):
        ip, _ = orc.camera_project(on_x, 1.0, 1.0, 0.0, 0.0, 4, 4, margin=10.0)
    xx = x.astype(np.float64) ** 2
    assert np.allclose(ip[:, 0], x + (-3e-3) * 3 * xx + xx * (1e-3 + xx * 2e-3), atol=1e-7)
    assert np.allclose(ip[:, 1], 2e-3 * xx + xx * (-1e-3 + xx * 5e-4), atol=1e-7)
    with orc.distortion(radial=[-0.5, 0, 0, 0, 0, 0]):  # icD = 1 - 0.5 r^2 <= 0.8 beyond r^2 = 0.4
        p = np.array([[0.5, 0, 1], [0.7, 0, 1], [0.1, 0, -1]], np.float32)
        _, ok = orc.camera_project(p, 100.0, 100.0, 100.0, 100.0, 200, 200)
    assert list(ok) == [True, False, False]


def test_undistortion_inverts_the_projection(orc):
    """Newton undistortion of projected rays returns the rays (a wrong Jacobian entry stalls the 5 iterations), and
    agrees with an independent solve of the float64 forward model by scipy"""
    from scipy.optimize import fsolve
    f, c = 400.0, 320.0
    pts = _rays(3000, 2)
    with orc.distortion(_RADIAL, _TANGENTIAL, _THIN_PRISM):
        ip, ok = orc.camera_project(pts, f, 1.1 * f, c, c - 40, 640, 560, margin=0.5)
        rays, conv = orc.camera_unproject(ip, f, 1.1 * f, c, c - 40)
    assert ok.sum() > 2500 and conv[ok].all()
    want = pts / np.linalg.norm(pts, axis=1, keepdims=True)
    assert np.abs(rays[ok] - want[ok]).max() < 3e-6
    k, p, s = (np.array(a, np.float64) for a in (_RADIAL, _TANGENTIAL, _THIN_PRISM))

    def forward(uv):
        u, v = uv
        r2 = u * u + v * v
        icd = (1 + r2 * (k[0] + r2 * (k[1] + r2 * k[2]))) / (1 + r2 * (k[3] + r2 * (k[4] + r2 * k[5])))
        return np.array([icd * u + 2 * p[0] * u * v + p[1] * (r2 + 2 * u * u) + r2 * (s[0] + r2 * s[1]),
                         icd * v + p[0] * (r2 + 2 * v * v) + 2 * p[1] * u * v + r2 * (s[2] + r2 * s[3])])

    for i in np.nonzero(ok)[0][:40]:
        target = np.array([(ip[i, 0] - c) / f, (ip[i, 1] - (c - 40)) / (1.1 * f)], np.float64)
        sol = fsolve(lambda uv: forward(uv) - target, target, xtol=1e-12)
        ray = np.array([sol[0], sol[1], 1.0]) / np.linalg.norm([sol[0], sol[1], 1.0])
        assert np.abs(rays[i] - ray).max() < 3e-6


# ---------------------------------------------------------------------------------------------------------------
# OpenCV fisheye and equirectangular models (Cameras.cuh:757-1037; gsx_camera.h)
# ---------------------------------------------------------------------------------------------------------------
def test_camera_primitives(orc):
    """atan2 on the whole plane, cbrt, asin, cos against numpy in float64 (<= 2e-7 absolute / 3e-7 relative)"""
    r = np.random.default_rng(0)
    y, x = r.normal(0, 1, 20000).astype(np.float32), r.normal(0, 1, 20000).astype(np.float32)
    y[:100], x[100:200] = 0.0, 0.0
    y[200:300] *= 1e-6
    x[300:400] *= 1e6
    assert np.abs(orc.math_camera("atan2", y, x) - np.arctan2(y.astype(np.float64), x)).max() < 3e-7
    assert orc.math_camera("atan2", [0.0], [0.0])[0] == 0.0
    v = np.concatenate([r.normal(0, 100, 5000), r.normal(0, 1e-3, 5000), [0.0, 8.0, -27.0]]).astype(np.float32)
    got = orc.math_camera("cbrt", v)
    assert np.abs(got - np.cbrt(v.astype(np.float64))).max() <= 3e-7 * np.abs(np.cbrt(v)).max()
    assert np.all(np.abs(got - np.cbrt(v.astype(np.float64))) <= 3e-7 * np.abs(np.cbrt(v.astype(np.float64))) + 1e-30)
    s = r.uniform(-1, 1, 20000).astype(np.float32)
    assert np.abs(orc.math_camera("asin", s) - np.arcsin(s.astype(np.float64))).max() < 4e-7
    a = r.uniform(-np.pi, np.pi, 20000).astype(np.float32)
    assert np.abs(orc.math_camera("cos", a) - np.cos(a.astype(np.float64))).max() < 2.5e-7


def test_fisheye_field_of_view_limit(orc):
    """the limit is the smallest positive root of the derivative 1 + 3 k1 t^2 + 5 k2 t^4 + 7 k3 t^6 (+ 9 k4 t^8) of
    the forward polynomial (beyond it the mapping folds back): numpy's roots of the same polynomial"""
    cases = [(-0.05, 0.0, 0.0), (0.1, -0.02, 0.0), (-0.02, 0.003, -0.0004), (0.05, 0.01, 0.001), (0.2, -0.05, 0.004),
             (-0.3, 0.05, -0.01), (0.0, -0.01, 0.0), (0.0, 0.0, -1e-3)]
    for k1, k2, k3 in cases:
        a, b, c = 3 * k1, 5 * k2, 7 * k3
        got = float(orc.math_camera("max_angle_sq", [a], [b], [c])[0])
        roots = np.roots([c, b, a, 1.0])  # in x = t^2
        pos = sorted(float(z.real) for z in roots if abs(z.imag) < 1e-9 and z.real > 0)
        if pos:
            assert abs(got - pos[0]) <= 2e-5 * pos[0], (k1, k2, k3, got, pos)
        else:
            assert got > 1e38, (k1, k2, k3, got)


def _fisheye_rays(n, seed, max_theta):
    r = np.random.default_rng(seed)
    theta = r.uniform(0.0, max_theta, n)
    phi = r.uniform(-np.pi, np.pi, n)
    d = r.uniform(0.5, 5.0, n)
    return (d[:, None] * np.stack([np.sin(theta) * np.cos(phi), np.sin(theta) * np.sin(phi), np.cos(theta)], 1)), theta


@pytest.mark.parametrize("k", [None, [0.03, -0.004, 0.0006, 0.0], [-0.02, 0.003, -0.0004, 0.00003]])
def test_fisheye_projection_closed_form_and_round_trip(orc, k):
    """image radius = f (theta + k1 theta^3 + k2 theta^5 + k3 theta^7 + k4 theta^9) along the ray's azimuth (the
    equidistant model when k = 0), in float64; the Newton inverse returns the unit ray; rays beyond the field of
    view / behind the camera are invalid or clamped onto the rim"""
    W, H, f = 640, 480, 200.0
    pts, theta = _fisheye_rays(4000, 3, 1.3)
    with orc.camera_model(2, W, H, radial=k):
        ip, ok = orc.camera_project(pts.astype(np.float32), f, f, W / 2, H / 2, W, H, margin=0.1)
        rays, conv = orc.camera_unproject(ip, f, f, W / 2, H / 2)
        behind, okb = orc.camera_project(np.array([[0.1, 0.2, -1.0]], np.float32), f, f, W / 2, H / 2, W, H)
    kk = np.zeros(4) if k is None else np.array(k, np.float64)
    rad = theta + kk[0] * theta ** 3 + kk[1] * theta ** 5 + kk[2] * theta ** 7 + kk[3] * theta ** 9
    az = np.arctan2(pts[:, 1], pts[:, 0])
    want = np.stack([f * rad * np.cos(az) + W / 2, f * rad * np.sin(az) + H / 2], 1)
    assert np.abs(ip - want).max() < 2e-3  # pixels; float32 at a few hundred pixels
    inside = (want[:, 0] >= -0.1 * W) & (want[:, 0] < 1.1 * W) & (want[:, 1] >= -0.1 * H) & (want[:, 1] < 1.1 * H)
    edge = np.minimum(np.abs(want[:, 0] + 0.1 * W), np.abs(want[:, 0] - 1.1 * W)) < 1e-2
    assert np.array_equal(ok[~edge], inside[~edge]) and ok.sum() > 1000
    assert not okb[0]
    unit = pts / np.linalg.norm(pts, axis=1, keepdims=True)
    assert conv[ok].all() and np.abs(rays[ok] - unit[ok]).max() < 5e-6


def test_equirectangular_closed_form_and_round_trip(orc):
    """pixel = ((azimuth / 2 pi + 1/2) W, (elevation / pi + 1/2) H) with azimuth = atan2(x, z), elevation =
    asin(y / |p|): every direction is valid, including behind the camera; the unprojection returns the unit ray"""
    W, H = 1024, 512
    r = np.random.default_rng(5)
    pts = r.normal(0, 1, (5000, 3))
    pts *= r.uniform(0.5, 4.0, (5000, 1)) / np.linalg.norm(pts, axis=1, keepdims=True)
    with orc.camera_model(3, W, H):
        ip, ok = orc.camera_project(pts.astype(np.float32), 1.0, 1.0, 0.0, 0.0, W, H)
        rays, conv = orc.camera_unproject(ip, 1.0, 1.0, 0.0, 0.0)
    az, el = np.arctan2(pts[:, 0], pts[:, 2]), np.arcsin(pts[:, 1] / np.linalg.norm(pts, axis=1))
    want = np.stack([(az / (2 * np.pi) + 0.5) * W, (el / np.pi + 0.5) * H], 1)
    assert ok.all() and conv.all() and np.abs(ip[:, 0] - want[:, 0]).max() < 1.5e-4
    # asin is ill-conditioned at the poles: one float32 rounding of y / |p| moves the elevation by 6e-8 / cos(el)
    assert np.all(np.abs(ip[:, 1] - want[:, 1]) < 1.5e-4 + H / np.pi * 1.2e-7 / np.cos(el))
    unit = pts / np.linalg.norm(pts, axis=1, keepdims=True)
    assert np.abs(rays - unit).max() < 3e-6


# ---------------------------------------------------------------------------------------------------------------
# rolling shutter (Cameras.cuh:268-414)
# ---------------------------------------------------------------------------------------------------------------
def _pose(rotvec, t):
    from scipy.spatial.transform import Rotation
    vm = np.eye(4)
    vm[:3, :3] = Rotation.from_rotvec(rotvec).as_matrix()
    vm[:3, 3] = t
    return vm


def _pose_at(vm0, vm1, rel):
    """float64 model of the pose at a relative frame time: translation lerp, rotation slerp as the geodesic
    R1 (R1^T R0)^(1 - rel) ... written through the rotation vector so that times outside [0, 1] (image points in the
    margin around the image) extrapolate, as the quaternion formula does"""
    from scipy.spatial.transform import Rotation
    R0, R1 = Rotation.from_matrix(vm0[:3, :3]), Rotation.from_matrix(vm1[:3, :3])
    # quaternion slerp q0 (q0^-1 q1)^rel; the view rotation is that quaternion's matrix
    R = (R0 * Rotation.from_rotvec(rel * (R0.inv() * R1).as_rotvec())).as_matrix()
    return R, (1 - rel) * vm0[:3, 3] + rel * vm1[:3, 3]


def _rel_time(rs_type, x, y, W, H):
    return [np.floor(y) / (H - 1), np.floor(x) / (W - 1), (H - np.ceil(y)) / (H - 1), (W - np.ceil(x)) / (W - 1)][rs_type]


@pytest.mark.parametrize("rs_type", [0, 1, 2, 3])
def test_rolling_shutter_pixel_rays(orc, rs_type):
    """a pixel's world ray is the global-shutter ray under the pose interpolated to the pixel's exposure time (row or
    column over H - 1 / W - 1, in the shutter's direction): numpy / scipy Slerp in float64"""
    W, H, f = 320, 240, 300.0
    vm0, vm1 = _pose([0.02, -0.01, 0.03], [0.1, -0.2, 4.0]), _pose([-0.05, 0.06, -0.02], [0.4, 0.1, 3.7])
    r = np.random.default_rng(rs_type)
    ip = np.stack([r.integers(0, W, 400) + 0.5, r.integers(0, H, 400) + 0.5], 1)
    with orc.rolling_shutter(rs_type, vm1, W, H):
        o, d, ok = orc.pixel_world_rays(ip, vm0, f, f, W / 2, H / 2)
    assert ok.all()
    for k in range(ip.shape[0]):
        R, t = _pose_at(vm0, vm1, _rel_time(rs_type, ip[k, 0], ip[k, 1], W, H))
        cam = np.array([(ip[k, 0] - W / 2) / f, (ip[k, 1] - H / 2) / f, 1.0])
        assert np.abs(o[k] - (-R.T @ t)).max() < 3e-6
        assert np.abs(d[k] - R.T @ (cam / np.linalg.norm(cam))).max() < 1e-6
    # first / last row (column) are exposed under the start / end pose exactly
    ends = {0: ([[5.5, 0.5]], [[5.5, H - 0.5]]), 1: ([[0.5, 7.5]], [[W - 0.5, 7.5]]),
            2: ([[5.5, H - 0.5]], [[5.5, 0.5]]), 3: ([[W - 0.5, 7.5]], [[0.5, 7.5]])}[rs_type]
    with orc.rolling_shutter(rs_type, vm1, W, H):
        o0 = orc.pixel_world_rays(ends[0], vm0, f, f, W / 2, H / 2)[0][0]
        o1 = orc.pixel_world_rays(ends[1], vm0, f, f, W / 2, H / 2)[0][0]
    if rs_type in (0, 1):
        assert np.abs(o0 - (-vm0[:3, :3].T @ vm0[:3, 3])).max() < 3e-6
        assert np.abs(o1 - (-vm1[:3, :3].T @ vm1[:3, 3])).max() < 3e-6
    else:  # (H - ceil(y)) / (H - 1): the last row is at time 0, the first at 1 + 1 / (H - 1) of the frame
        assert np.abs(o0 - (-vm0[:3, :3].T @ vm0[:3, 3])).max() < 3e-6


@pytest.mark.parametrize("rs_type", [0, 1, 2, 3])
def test_rolling_shutter_projection_is_a_fixed_point(orc, rs_type):
    """the image point of a world point satisfies p = project(pose(time(p)) X) (float64 model): the iteration of
    Cameras.cuh:346-414 converges for a moderate motion; with the end pose = the start pose, and for GLOBAL, the
    plain projection comes back bit for bit"""
    W, H, f = 320, 240, 300.0
    vm0, vm1 = _pose([0.02, -0.01, 0.03], [0.1, -0.2, 4.0]), _pose([0.01, 0.01, 0.02], [0.15, -0.15, 3.9])
    r = np.random.default_rng(10 + rs_type)
    X = r.normal(0, 0.6, (500, 3))
    with orc.rolling_shutter(rs_type, vm1, W, H):
        ip, ok = orc.world_project(X.astype(np.float32), vm0, f, f, W / 2, H / 2, W, H)
    with orc.rolling_shutter(rs_type, vm0, W, H):
        same, ok_same = orc.world_project(X.astype(np.float32), vm0, f, f, W / 2, H / 2, W, H)
    with orc.rolling_shutter(4, vm1, W, H):
        glob, ok_glob = orc.world_project(X.astype(np.float32), vm0, f, f, W / 2, H / 2, W, H)
    plain, ok_plain = orc.world_project(X.astype(np.float32), vm0, f, f, W / 2, H / 2, W, H)
    assert np.array_equal(glob, plain) and np.array_equal(ok_glob, ok_plain)
    assert np.array_equal(ok_same, ok_plain)
    assert np.abs(same[ok_plain] - plain[ok_plain]).max() < 2e-4  # slerp(q, q, t) and the lerp round differently
    assert ok.sum() > 300
    moved = 0
    for k in np.flatnonzero(ok):
        R, t = _pose_at(vm0, vm1, _rel_time(rs_type, ip[k, 0], ip[k, 1], W, H))
        c = R @ X[k].astype(np.float32).astype(np.float64) + t
        want = np.array([f * c[0] / c[2] + W / 2, f * c[1] / c[2] + H / 2])
        # the time is a step function of the pixel: at a row / column boundary the iteration may alternate between two
        # neighbouring times; the fixed point is then met to one row's worth of motion
        assert np.abs(ip[k] - want).max() < 0.05, (k, ip[k], want)
        moved += np.abs(ip[k] - plain[k]).max() > 0.5
    assert moved > 100  # the motion matters
