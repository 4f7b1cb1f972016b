"""Pins the checker's SSIM, Adam, relocation, noise, activations and photometric loss against the definitions
(Wang et al. 2004 SSIM in float64, torch.optim.Adam, the closed forms of MCMC Eq. 9, torch autograd)."""
import math

import numpy as np
import pytest

torch = pytest.importorskip("torch")

C1, C2 = 0.01 ** 2, 0.03 ** 2


def gauss_window():
    g = np.exp(-((np.arange(11) - 5.0) ** 2) / (2 * 1.5 ** 2))
    return g / g.sum()


def ssim_direct_f64(x, y):
    """non-separable 11x11 Gaussian-window SSIM with zero padding, float64 (Wang et al. 2004)"""
    g = gauss_window()
    w2 = np.outer(g, g)
    H, W = x.shape
    xp, yp = np.pad(x, 5), np.pad(y, 5)
    out = np.zeros((H, W))
    for i in range(H):
        for j in range(W):
            a, b = xp[i:i + 11, j:j + 11], yp[i:i + 11, j:j + 11]
            mu1, mu2 = (w2 * a).sum(), (w2 * b).sum()
            s1 = (w2 * a * a).sum() - mu1 ** 2
            s2 = (w2 * b * b).sum() - mu2 ** 2
            s12 = (w2 * a * b).sum() - mu1 * mu2
            out[i, j] = ((2 * mu1 * mu2 + C1) * (2 * s12 + C2)) / ((mu1 ** 2 + mu2 ** 2 + C1) * (s1 + s2 + C2))
    return out


def test_ssim_window_and_map(orc):
    assert abs(gauss_window()[5] - 0.26601171493530273) < 1e-7  # src/training/kernels/ssim.cu:16-27
    rng = np.random.default_rng(0)
    H, W = 23, 40
    x = rng.uniform(0, 1, (1, 2, H, W)).astype(np.float32)
    y = np.clip(x + rng.normal(0, 0.15, x.shape), 0, 1).astype(np.float32)
    m, d1, d2, d3 = orc.fusedssim(C1, C2, x, y, True)
    for c in range(2):
        np.testing.assert_allclose(m[0, c], ssim_direct_f64(x[0, c].astype(np.float64), y[0, c].astype(np.float64)),
                                   atol=2e-5)
    assert np.all(orc.fusedssim(C1, C2, x, x, False)[0] > 1 - 1e-5)  # SSIM(x, x) = 1
    assert orc.fusedssim(C1, C2, x, y, False)[1] is None


def test_ssim_backward_against_autograd_of_the_definition(orc):
    rng = np.random.default_rng(1)
    H, W = 19, 27
    x = rng.uniform(0, 1, (1, 3, H, W)).astype(np.float32)
    y = np.clip(x + rng.normal(0, 0.2, x.shape), 0, 1).astype(np.float32)
    dL = rng.normal(0, 1, x.shape).astype(np.float32)
    m, d1, d2, d3 = orc.fusedssim(C1, C2, x, y, True)
    got = orc.fusedssim_backward(C1, C2, x, y, dL, d1, d2, d3)
    # the definition, differentiated by torch in float64 (depth-wise conv2d with the outer-product window)
    g = torch.tensor(gauss_window(), dtype=torch.float64)
    w = (g[:, None] * g[None, :]).expand(3, 1, 11, 11).contiguous()
    X = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    Y = torch.tensor(y, dtype=torch.float64)
    conv = lambda t: torch.nn.functional.conv2d(t, w, padding=5, groups=3)
    mu1, mu2 = conv(X), conv(Y)
    s1, s2, s12 = conv(X * X) - mu1 ** 2, conv(Y * Y) - mu2 ** 2, conv(X * Y) - mu1 * mu2
    mp = ((2 * mu1 * mu2 + C1) * (2 * s12 + C2)) / ((mu1 ** 2 + mu2 ** 2 + C1) * (s1 + s2 + C2))
    np.testing.assert_allclose(m, mp.detach().numpy(), atol=2e-5)
    (mp * torch.tensor(dL, dtype=torch.float64)).sum().backward()
    ref = X.grad.numpy()
    np.testing.assert_allclose(got, ref, atol=2e-4 * np.abs(ref).max())


def test_adam_matches_torch_optim(orc):
    rng = np.random.default_rng(2)
    n = 5000
    p0 = rng.normal(0, 1, n).astype(np.float32)
    p = p0.copy()
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    tp = torch.tensor(p0.copy(), requires_grad=True)
    opt = torch.optim.Adam([tp], lr=1.6e-4, betas=(0.9, 0.999), eps=1e-15)
    for t in range(1, 4):
        g = rng.normal(0, 1, n).astype(np.float32)
        bc1 = 1.0 / (1.0 - math.pow(0.9, t))
        bc2 = 1.0 / math.sqrt(1.0 - math.pow(0.999, t))
        orc.adam_step(p, m, v, g, 1.6e-4, 0.9, 0.999, 1e-15, bc1, bc2)
        tp.grad = torch.tensor(g)
        opt.step()
        np.testing.assert_allclose(p - p0, tp.detach().numpy() - p0, rtol=2e-3, atol=2.5e-7)
        st = opt.state[tp]
        np.testing.assert_allclose(m, st["exp_avg"].numpy(), rtol=1e-5, atol=5e-8)
        # the kernel forms (1 - beta2) in fp32 (adam_kernels.cuh:30): 1.0f - 0.999f is 1.3e-5 below 1e-3
        np.testing.assert_allclose(v, st["exp_avg_sq"].numpy(), rtol=5e-5, atol=1e-12)
    # textbook float64 single step
    g = np.array([0.5, -2.0, 0.0], np.float32)
    p, m, v = np.ones(3, np.float32), np.zeros(3, np.float32), np.zeros(3, np.float32)
    orc.adam_step(p, m, v, g, 0.1, 0.9, 0.999, 1e-15, 1 / (1 - 0.9), 1 / math.sqrt(1 - 0.999))
    np.testing.assert_allclose(p, [0.9, 1.1, 1.0], rtol=1e-6)  # first step moves by lr * sign(g)


def binoms(n_max=51):
    b = np.zeros((n_max, n_max), np.float32)
    for n in range(n_max):
        for k in range(n + 1):
            x = np.float32(1.0)
            for i in range(k):
                x = np.float32(x * (np.float32(n - i) / np.float32(i + 1)))
            b[n, k] = x
    return b


def test_relocation_closed_forms(orc):
    b = binoms()
    assert b[4, 2] == 6 and abs(b[10, 5] - 252) < 1e-3 and abs(b[50, 25] / math.comb(50, 25) - 1) < 1e-5
    rng = np.random.default_rng(3)
    M = 400
    op = rng.uniform(0.01, 0.95, M).astype(np.float32)
    sc = np.exp(rng.normal(-4, 1, (M, 3))).astype(np.float32)
    # n = 1: identity
    o1, s1 = orc.relocation(op, sc, np.ones(M, np.int32), b, 51)
    np.testing.assert_allclose(o1, op, rtol=1e-5)
    np.testing.assert_allclose(s1, sc, rtol=1e-5)
    # n = 2: o' = 1 - sqrt(1 - o); denominator = o' + (o' - o'^2 / sqrt(2))
    o2, s2 = orc.relocation(op, sc, np.full(M, 2, np.int32), b, 51)
    o64 = op.astype(np.float64)
    no = 1 - np.sqrt(1 - o64)
    np.testing.assert_allclose(o2, no, rtol=2e-5)
    np.testing.assert_allclose(s2, sc * (o64 / (2 * no - no ** 2 / np.sqrt(2)))[:, None], rtol=1e-4)
    # general n (Eq. 9 of "3D Gaussian Splatting as Markov Chain Monte Carlo") in float64, where fp32 is still stable
    for n in (3, 5, 8, 12):
        on, sn = orc.relocation(op, sc, np.full(M, n, np.int32), b, 51)
        no = 1 - (1 - o64) ** (1.0 / n)
        den = sum(math.comb(i - 1, k) * (-1) ** k / math.sqrt(k + 1) * no ** (k + 1) for i in range(1, n + 1)
                  for k in range(i))
        np.testing.assert_allclose(on, no, rtol=5e-5)
        np.testing.assert_allclose(sn, sc * (o64 / den)[:, None], rtol=2e-3)


def test_add_noise_closed_forms(orc):
    n = 64
    rng = np.random.default_rng(4)
    noise = rng.normal(0, 1, (n, 3)).astype(np.float32)
    raw_o = rng.normal(-6, 1, n).astype(np.float32)  # low opacity: the gate is open
    s = np.float32(-3.0)
    means = np.zeros((n, 3), np.float32)
    # identity rotation + equal scales: covariance = e^{2s} I
    orc.add_noise(raw_o, np.full((n, 3), s, np.float32), np.tile([[2.0, 0, 0, 0]], (n, 1)).astype(np.float32), noise,
                  means, 10.0)
    o = 1 / (1 + np.exp(-raw_o.astype(np.float64)))
    gate = 1 / (1 + np.exp(100 * o - 0.5))
    np.testing.assert_allclose(means, (10.0 * gate * np.exp(2 * float(s)))[:, None] * noise, rtol=2e-5)
    # general rotation: R diag(e^{2 s}) R^T, un-normalised quaternion
    from scipy.spatial.transform import Rotation
    q = rng.normal(0, 1, (n, 4)).astype(np.float32)
    rs = rng.normal(-3, 0.5, (n, 3)).astype(np.float32)
    means = np.zeros((n, 3), np.float32)
    orc.add_noise(raw_o, rs, q, noise, means, 1.0)
    for i in range(n):
        qq = q[i].astype(np.float64) / np.linalg.norm(q[i])
        R = Rotation.from_quat([qq[1], qq[2], qq[3], qq[0]]).as_matrix()
        cov = R @ np.diag(np.exp(2 * rs[i].astype(np.float64))) @ R.T
        np.testing.assert_allclose(means[i], gate[i] * cov @ noise[i], rtol=1e-4, atol=1e-9)
    # opaque Gaussians get (almost) no noise: gate = sigmoid(-100 (o - 0.005))
    means = np.zeros((4, 3), np.float32)
    orc.add_noise(np.full(4, 3.0, np.float32), rs[:4], q[:4], noise[:4], means, 1.0)
    assert np.abs(means).max() < 1e-30


def test_activations_and_vjps_against_torch(orc):
    rng = np.random.default_rng(5)
    n = 1000
    ro, rs, rq = rng.normal(0, 2, n), rng.normal(-4, 1, (n, 3)), rng.normal(0, 1, (n, 4))
    op, sc, qt = orc.activate_params(ro, rs, rq)
    t = lambda a: torch.tensor(np.asarray(a, np.float32), dtype=torch.float64, requires_grad=True)
    to, ts_, tq = t(ro), t(rs), t(rq)
    o_ref, s_ref = torch.sigmoid(to), torch.exp(ts_)
    q_ref = torch.nn.functional.normalize(tq, dim=-1)
    np.testing.assert_allclose(op, o_ref.detach().numpy(), rtol=3e-7)
    np.testing.assert_allclose(sc, s_ref.detach().numpy(), rtol=3e-7)
    np.testing.assert_allclose(qt, q_ref.detach().numpy(), rtol=0, atol=2e-7)
    vo, vs, vq = rng.normal(0, 1, n), rng.normal(0, 1, (n, 3)), rng.normal(0, 1, (n, 4))
    ((o_ref * torch.tensor(vo)).sum() + (s_ref * torch.tensor(vs)).sum() + (q_ref * torch.tensor(vq)).sum()).backward()
    go, gs, gq = orc.activate_params_bwd(ro, rs, rq, vo, vs, vq)
    np.testing.assert_allclose(go, to.grad.numpy(), rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(gs, ts_.grad.numpy(), rtol=2e-5, atol=1e-9)
    np.testing.assert_allclose(gq, tq.grad.numpy(), rtol=2e-4, atol=2e-6)


def test_photometric_loss_against_torch(orc):
    """loss = 0.8 L1 + 0.2 (1 - mean(SSIM[5:-5, 5:-5])) on clamp(render): value and d loss / d render"""
    rng = np.random.default_rng(6)
    H, W = 31, 45
    render = rng.uniform(-0.2, 1.2, (H, W, 3)).astype(np.float32)  # some values outside [0, 1]: the clamp masks them
    gt = rng.uniform(0, 1, (3, H, W)).astype(np.float32)
    loss, l1, ss, image, v = orc.photometric_loss(render, gt, 0.2, True)
    R = torch.tensor(render, dtype=torch.float64, requires_grad=True)
    img = torch.clamp(R.permute(2, 0, 1), 0.0, 1.0)[None]
    G = torch.tensor(gt, dtype=torch.float64)[None]
    g = torch.tensor(gauss_window(), dtype=torch.float64)
    w = (g[:, None] * g[None, :]).expand(3, 1, 11, 11).contiguous()
    conv = lambda t: torch.nn.functional.conv2d(t, w, padding=5, groups=3)
    mu1, mu2 = conv(img), conv(G)
    s1, s2, s12 = conv(img * img) - mu1 ** 2, conv(G * G) - mu2 ** 2, conv(img * G) - mu1 * mu2
    mp = ((2 * mu1 * mu2 + C1) * (2 * s12 + C2)) / ((mu1 ** 2 + mu2 ** 2 + C1) * (s1 + s2 + C2))
    ssim = mp[:, :, 5:H - 5, 5:W - 5].mean()
    L = 0.8 * torch.nn.functional.l1_loss(img, G) + 0.2 * (1 - ssim)
    L.backward()
    assert abs(loss - L.item()) < 2e-6 and abs(ss - ssim.item()) < 1e-5 and abs(l1 - (img - G).abs().mean().item()) < 1e-6
    np.testing.assert_allclose(image, img[0].detach().numpy(), atol=1e-7)
    ref = R.grad.numpy()
    np.testing.assert_allclose(v, ref, atol=3e-4 * np.abs(ref).max())
    assert np.all(v[(render < 0) | (render > 1)] == 0)
    # lambda = 0 (configuration 1): pure L1
    loss0, l10, _, _, v0 = orc.photometric_loss(render, gt, 0.0, True)
    assert abs(loss0 - l10) < 1e-9
    inside = (render >= 0) & (render <= 1)
    np.testing.assert_allclose(v0[inside], (np.sign(np.clip(render, 0, 1) - gt.transpose(1, 2, 0)) / (3 * H * W))[inside],
                               rtol=1e-6)


def test_l1_regularization_matches_autograd(orc):
    """regularization.cu:20-90 pinned by autograd of the definition: loss = w mean(exp(x)) resp. w mean(sigmoid(x)),
    gradients ADDED onto what the tensor already holds (a dropped 1/n, a missing chain-rule factor or an overwrite
    instead of an accumulation fails)"""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(5)
    x = rng.normal(-1.0, 1.5, (4001, 3)).astype(np.float32)
    g0 = rng.normal(0, 1e-4, x.shape).astype(np.float32)
    for mode, f in (("exp", torch.exp), ("sigmoid", torch.sigmoid)):
        t = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
        loss = 0.013 * f(t).mean()
        loss.backward()
        g = g0.copy()
        got = orc.l1_regularization(mode, x, g, 0.013)
        assert abs(got - loss.item()) <= 1e-6 * loss.item()
        want = g0.astype(np.float64) + t.grad.numpy()
        assert np.abs(g - want).max() <= 2e-6 * np.abs(want).max()
        assert orc.l1_regularization(mode, x, None, 0.013) == got
        g2 = g0.copy()
        assert orc.l1_regularization(mode, x, g2, 0.0) == 0.0 and np.array_equal(g2, g0)


def test_philox_known_answers_and_normal_draws(orc):
    """Philox4x32-10 against the known-answer vectors of the Random123 distribution (kat_vectors: zero, all-ones and
    pi-digit inputs); the Box-Muller rows: moments, independence of the three columns, Kolmogorov-Smirnov against
    N(0,1), different (seed, offset) give different rows, the same give the same"""
    from scipy import stats
    kat = [([0, 0, 0, 0], [0, 0], "6627e8d5 e169c58d bc57ac4c 9b00dbd8"),
           ([0xffffffff] * 4, [0xffffffff] * 2, "408f276d 41c83b0e a20bc7c6 6d5451fd"),
           ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
            "d16cfe09 94fdcceb 5001e420 24126ea1")]
    for ctr, key, want in kat:
        assert " ".join("%08x" % v for v in orc.philox4x32_10(ctr, key)) == want
    z = orc.philox_randn3(400_000, 11, 5)
    assert np.isfinite(z).all() and np.abs(z).max() < 6.0  # |z| <= sqrt(2 * 24 ln 2) = 5.77
    assert np.abs(z.mean(0)).max() < 6e-3 and np.abs(z.std(0) - 1).max() < 4e-3
    c = np.corrcoef(z.T)
    assert np.abs(c - np.eye(3)).max() < 6e-3
    for k in range(3):
        assert stats.kstest(z[:100_000, k].astype(np.float64), "norm").pvalue > 1e-3
    assert np.array_equal(z, orc.philox_randn3(400_000, 11, 5))
    assert not np.array_equal(z[:100], orc.philox_randn3(100, 11, 6))
    assert not np.array_equal(z[:100], orc.philox_randn3(100, 12, 5))
