"""Synthetic scenes and cameras for the measured configurations.

Every array comes from numpy's PCG64 ``default_rng(seed)`` so that the GPU path, the CPU checker and
the committed fixtures see identical inputs.  Parameters are the *raw* trainable tensors of
LichtFeld's SplatData (include/core/splat_data.hpp:68-79): means [N,3], sh0 [N,1,3], shN [N,K-1,3],
scaling_raw [N,3] (log), rotation_raw [N,4] (w,x,y,z), opacity_raw [N,1] (logit).
"""
from dataclasses import dataclass, field

import numpy as np

SH_C0 = 0.2820947917738781


@dataclass
class Camera:
    width: int
    height: int
    viewmat: np.ndarray  # [4,4] row-major world->camera
    K: np.ndarray  # [3,3]


@dataclass
class Scene:
    name: str
    means: np.ndarray
    sh0: np.ndarray
    shN: np.ndarray
    scaling_raw: np.ndarray
    rotation_raw: np.ndarray
    opacity_raw: np.ndarray
    sh_degree: int
    cameras: list = field(default_factory=list)

    @property
    def n(self):
        return self.means.shape[0]

    def params(self):
        return dict(means=self.means, sh0=self.sh0, shN=self.shN, scaling_raw=self.scaling_raw,
                    rotation_raw=self.rotation_raw, opacity_raw=self.opacity_raw)


def intrinsics(width, height, fx, fy=None, cx=None, cy=None):
    fy = fx if fy is None else fy
    cx = width / 2.0 if cx is None else cx
    cy = height / 2.0 if cy is None else cy
    return np.array([[fx, 0, cx], [0, fy, cy], [0, 0, 1]], np.float32)


def look_at(eye, target=(0.0, 0.0, 0.0), up=(0.0, 1.0, 0.0)):
    """Row-major world->camera [R|t] with +z looking from eye to target (OpenCV convention, y down)."""
    eye = np.asarray(eye, np.float64)
    f = np.asarray(target, np.float64) - eye
    f /= np.linalg.norm(f)
    upv = np.asarray(up, np.float64)
    r = np.cross(f, upv)
    if np.linalg.norm(r) < 1e-6:
        r = np.cross(f, np.array([1.0, 0.0, 0.0]))
    r /= np.linalg.norm(r)
    d = np.cross(f, r)  # camera y (down)
    R = np.stack([r, d, f], 0)
    t = -R @ eye
    V = np.eye(4)
    V[:3, :3] = R
    V[:3, 3] = t
    return V.astype(np.float32)


def fibonacci_cameras(n, radius, width, height, f):
    cams = []
    ga = np.pi * (3.0 - np.sqrt(5.0))
    for i in range(n):
        y = 1.0 - 2.0 * (i + 0.5) / n
        r = np.sqrt(max(0.0, 1.0 - y * y))
        th = ga * i
        eye = radius * np.array([np.cos(th) * r, y, np.sin(th) * r])
        cams.append(Camera(width, height, look_at(eye), intrinsics(width, height, f)))
    return cams


def orbit_camera(angle, radius, width, height, f, elevation=0.3):
    eye = radius * np.array([np.cos(angle) * np.cos(elevation), np.sin(elevation), np.sin(angle) * np.cos(elevation)])
    return Camera(width, height, look_at(eye), intrinsics(width, height, f))


def _normalize(q):
    return (q / np.linalg.norm(q, axis=-1, keepdims=True)).astype(np.float32)


def _sh(rng, n, degree, dc_is_colour):
    K = (degree + 1) ** 2
    dc = rng.uniform(0.0, 1.0, (n, 1, 3))
    if dc_is_colour:
        dc = (dc - 0.5) / SH_C0
    rest = rng.normal(0.0, 0.05, (n, K - 1, 3))
    return dc.astype(np.float32), rest.astype(np.float32)


def plumbing_scene(n=10_000, seed=0, width=256, height=256, f=280.0):
    """BASELINE configuration 1: SH degree 0, one pinhole camera at distance 4 looking at the origin."""
    rng = np.random.default_rng(seed)
    means = rng.normal(0.0, 0.5, (n, 3)).astype(np.float32)
    scaling_raw = rng.normal(-4.0, 0.5, (n, 3)).astype(np.float32)
    rotation_raw = _normalize(rng.normal(0.0, 1.0, (n, 4)))
    opacity_raw = rng.normal(0.0, 1.0, (n, 1)).astype(np.float32)
    sh0, shN = _sh(rng, n, 0, dc_is_colour=True)
    V = np.eye(4, dtype=np.float32)
    V[2, 3] = 4.0
    cam = Camera(width, height, V, intrinsics(width, height, f, f, width / 2.0, height / 2.0))
    target = rng.uniform(0.0, 1.0, (3, height, width)).astype(np.float32)
    sc = Scene("cfg1", means, sh0, shN, scaling_raw, rotation_raw, opacity_raw, 0, [cam])
    sc.target = target
    return sc


def cluster_scene(n, seed, name, sh_degree=3, n_clusters=32, cluster_sigma=0.3, logscale_mu=-4.5, logscale_sigma=0.7,
                  opacity_sigma=1.5, ball_fraction=0.0, ball_radius=0.5, geometry_only=False):
    """BASELINE configurations 2-5: mixture of isotropic clusters inside [-2,2]^3 (optionally with a
    fraction of the means concentrated in a ball at the origin), SH degree 3.  geometry_only: the SH coefficients
    (drawn last, most of the generator's time) are left out - means, scales, rotations, opacities are the same."""
    rng = np.random.default_rng(seed)
    centres = rng.uniform(-2.0, 2.0, (n_clusters, 3))
    cid = rng.integers(0, n_clusters, n)
    means = centres[cid] + rng.normal(0.0, cluster_sigma, (n, 3))
    if ball_fraction > 0.0:
        in_ball = rng.uniform(0.0, 1.0, n) < ball_fraction
        d = rng.normal(0.0, 1.0, (n, 3))
        d /= np.linalg.norm(d, axis=-1, keepdims=True)
        rad = ball_radius * rng.uniform(0.0, 1.0, (n, 1)) ** (1.0 / 3.0)
        means = np.where(in_ball[:, None], d * rad, means)
    means = means.astype(np.float32)
    scaling_raw = rng.normal(logscale_mu, logscale_sigma, (n, 3)).astype(np.float32)
    rotation_raw = _normalize(rng.normal(0.0, 1.0, (n, 4)))
    opacity_raw = rng.normal(0.0, opacity_sigma, (n, 1)).astype(np.float32)
    if geometry_only:
        sh0, shN = np.zeros((n, 1, 3), np.float32), np.zeros((n, 0, 3), np.float32)
        return Scene(name, means, sh0, shN, scaling_raw, rotation_raw, opacity_raw, 0, [])
    sh0, shN = _sh(rng, n, sh_degree, dc_is_colour=False)
    return Scene(name, means, sh0, shN, scaling_raw, rotation_raw, opacity_raw, sh_degree, [])


CFG5_LOGSCALE_MU = -5.0


def config5_literal(n=6_000_000, geometry_only=False):
    """Configuration 5 with the log-scale mean exactly as stated (-3.5): more intersections than int32 can index."""
    sc = cluster_scene(n, 5, "cfg5-literal", logscale_mu=-3.5, logscale_sigma=1.0, ball_fraction=0.7,
                       geometry_only=geometry_only)
    sc.cameras = [orbit_camera(2.6, 4.0, 3840, 2160, 3200.0)]
    return sc


def config(idx, n_override=None):
    """The five BASELINE configurations (1-based).  n_override shrinks N for parity tests."""
    if idx == 1:
        return plumbing_scene(n_override or 10_000, 0)
    if idx == 2:
        sc = cluster_scene(n_override or 500_000, 1, "cfg2")
        sc.cameras = fibonacci_cameras(8, 4.0, 1237, 822, 1150.0)
        return sc
    if idx == 3:
        sc = cluster_scene(n_override or 1_000_000, 2, "cfg3")
        sc.cameras = [orbit_camera(0.7, 4.0, 1237, 822, 1150.0)]
        sc.target_scene = cluster_scene(n_override or 1_000_000, 3, "cfg3-target")
        return sc
    if idx == 4:
        sc = cluster_scene(n_override or 3_000_000, 4, "cfg4")
        sc.cameras = [orbit_camera(1.9, 4.0, 1920, 1080, 1600.0)]
        sc.target_scene = cluster_scene(n_override or 3_000_000, 40, "cfg4-target")
        return sc
    if idx == 5:
        # BASELINE states log-scales ~N(-3.5, 1): at 3840x2160 / f = 3200 that is 2.7e9 tile intersections, beyond
        # the int32 index space of flatten_ids (the reference's too).  CFG5_LOGSCALE_MU = -5.0 keeps the unit
        # variance (the heavy tail) and gives 1.7e8 keys with tile lists up to 1e5 entries - the "100M+ keys, long
        # tail" that the configuration is described by.  config5_literal() is the stated distribution.
        sc = cluster_scene(n_override or 6_000_000, 5, "cfg5", logscale_mu=CFG5_LOGSCALE_MU, logscale_sigma=1.0,
                           ball_fraction=0.7)
        sc.cameras = [orbit_camera(2.6, 4.0, 3840, 2160, 3200.0)]
        sc.target_scene = cluster_scene(n_override or 6_000_000, 50, "cfg5-target", logscale_mu=CFG5_LOGSCALE_MU,
                                        logscale_sigma=1.0, ball_fraction=0.7)
        return sc
    raise ValueError(idx)


def activate(sc):
    """SplatData getters (src/core/splat_data.cpp:271-286) in numpy float32, for feeding the activated-
    parameter entry points: opacity = sigmoid, scales = exp, quats = normalize, shs = cat(sh0, shN)."""
    op = (1.0 / (1.0 + np.exp(-sc.opacity_raw.astype(np.float64)))).astype(np.float32).reshape(-1)
    scales = np.exp(sc.scaling_raw.astype(np.float64)).astype(np.float32)
    nrm = np.maximum(np.linalg.norm(sc.rotation_raw.astype(np.float64), axis=-1, keepdims=True), 1e-12)
    quats = (sc.rotation_raw / nrm).astype(np.float32)
    shs = np.concatenate([sc.sh0, sc.shN], 1).astype(np.float32)
    return sc.means, quats, scales, op, shs
