"""gs::training::rasterize mirror (rasterizer.py): the reference's own hot-path test (tests/test_render_modes.cpp:
50 random Gaussians, 128x128, fx = fy = 100, SH degree 3, five render modes, shapes / definedness) plus what that
test does not check - the values, against the CPU checker."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


def _fixture(cuda):
    """setupTestData of test_render_modes.cpp:22-69 (same distributions; numpy generator, seed 42)"""
    r = np.random.default_rng(42)
    n = 50
    means = r.normal(0, 1, (n, 3)).astype(np.float32)
    means[:, 2] = np.abs(means[:, 2]) + 2.0
    scales = np.abs(r.normal(0, 1, (n, 3)) * 0.1 + 0.3).astype(np.float32)
    q = r.normal(0, 1, (n, 4))
    q = (q / np.linalg.norm(q, axis=1, keepdims=True)).astype(np.float32)
    op = (r.uniform(0, 1, (n, 1)) * 0.8 + 0.2).astype(np.float32)
    sh = (r.normal(0, 1, (n, 16, 3)) * 0.1).astype(np.float32)
    V = np.eye(4, dtype=np.float32)
    V[2, 3] = 3.0
    K = np.array([[100, 0, 64], [0, 100, 64], [0, 0, 1]], np.float32)
    host = dict(means=means, scales=scales, q=q, op=op, sh=sh, V=V[None], K=K[None], bg=np.full(3, 0.5, np.float32))
    return host, {k: torch.from_numpy(v).to(cuda) for k, v in host.items()}


@pytest.mark.parametrize("mode,has_image,has_depth", [(0, True, False), (1, False, True), (2, False, True),
                                                      (3, True, True), (4, True, True)])
def test_render_modes(gsx, orc, cuda, mode, has_image, has_depth):
    from lichtfeld_studio_amd.rasterizer import RenderMode, rasterize
    h, d = _fixture(cuda)
    out = rasterize(d["V"], d["K"], 128, 128, d["means"], d["op"], d["scales"], d["q"], d["sh"], 3, d["bg"],
                    render_mode=RenderMode(mode))
    # the reference's assertions (test_render_modes.cpp:107-210)
    assert (out.image is not None) == has_image and (out.depth is not None) == has_depth
    if has_image:
        assert tuple(out.image.shape) == (3, 128, 128)
    if has_depth:
        assert tuple(out.depth.shape) == (1, 128, 128)
    assert tuple(out.alpha.shape) == (1, 128, 128) and out.width == 128 and out.height == 128
    assert tuple(out.radii.shape) == (50,) and out.visibility.dtype == torch.bool and int(out.visibility.sum()) > 10
    # values: the checker's fused forward in the same mode, then the reference's post-processing
    ref = orc.rasterize_from_world_with_sh_fwd(h["means"], h["q"], h["scales"], h["op"].reshape(-1), h["sh"], 3,
                                               h["bg"][None], 128, 128, 16, h["V"], h["K"], render_mode=mode)
    rendered, alpha = ref[0][0], ref[1][0]
    if has_image:
        img = rendered if mode == 0 else rendered[..., :3]
        want = np.clip(img, 0, 1).transpose(2, 0, 1)
        assert np.abs(out.image.cpu().numpy() - want).max() <= 1e-5
    if has_depth:
        dep = rendered[..., -1:]
        if mode in (2, 4):
            dep = dep / np.maximum(alpha, 1e-10)
        assert np.abs(out.depth.cpu().numpy() - dep.transpose(2, 0, 1)).max() <= 1e-4 * np.abs(dep).max()
    assert np.abs(out.alpha.cpu().numpy() - alpha.transpose(2, 0, 1)).max() <= 1e-5


def test_rasterize_checks_and_options(gsx, cuda):
    """TORCH_CHECK cases of rasterizer.cpp:24-87; opacity [N,1] accepted; antialiased lowers alpha (compensation);
    undefined background = black; zero distortion vectors (what a pinhole gs::Camera carries) change nothing"""
    from lichtfeld_studio_amd.rasterizer import rasterize
    h, d = _fixture(cuda)
    args = (d["V"], d["K"], 128, 128, d["means"], d["op"], d["scales"], d["q"], d["sh"], 3)
    with pytest.raises(RuntimeError, match="Packed mode"):
        rasterize(*args, d["bg"], packed=True)
    with pytest.raises(RuntimeError, match="viewmat must be"):
        rasterize(d["V"][0], *args[1:], d["bg"])
    with pytest.raises(RuntimeError, match="Not enough SH coefficients"):
        rasterize(*args[:8], d["sh"][:, :4].contiguous(), 3, d["bg"])
    with pytest.raises(RuntimeError, match="means3D must be on CUDA"):
        rasterize(*args[:4], d["means"].cpu(), *args[5:], d["bg"])
    with pytest.raises(RuntimeError, match="bg_color must be reshapeable"):
        rasterize(*args, torch.zeros(4, device=cuda))
    base = rasterize(*args, d["bg"])
    black = rasterize(*args, None)
    assert float((base.image - black.image).max()) > 0.01 and torch.equal(base.alpha, black.alpha)
    aa = rasterize(*args, d["bg"], antialiased=True)
    assert float(aa.alpha.sum()) < float(base.alpha.sum())
    zero = rasterize(*args, d["bg"], radial_distortion=torch.zeros(4, device=cuda),
                     tangential_distortion=torch.zeros(2, device=cuda))
    assert float((zero.image - base.image).abs().max()) <= 1e-6
    bent = rasterize(*args, d["bg"], radial_distortion=torch.tensor([-0.2, 0.05], device=cuda))
    assert float((bent.image - base.image).abs().max()) > 0.005
    # gs::Camera::camera_model_type() reaches the kernels (rasterizer.cpp:135): the fisheye image is another one, and
    # the mirror's output is the operator's
    fish = rasterize(*args, d["bg"], camera_model=2, radial_distortion=torch.tensor([0.02, -0.003], device=cuda))
    assert float((fish.image - base.image).abs().max()) > 0.005 and float(fish.alpha.mean()) > 0.01
    pano = rasterize(*args, d["bg"], camera_model=3)
    assert float((pano.image - base.image).abs().max()) > 0.005 and float(pano.alpha.sum()) > 0
    with pytest.raises(RuntimeError, match="PINHOLE, FISHEYE and EQUIRECTANGULAR"):
        rasterize(*args, d["bg"], camera_model=1)
