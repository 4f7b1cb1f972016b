"""Host-side mirror of gs::training::rasterize (src/training/rasterization/rasterizer.cpp:14-243): the caller of the
fused `--gut` rasterization that the trainer's eval renders and the viewer use.  Validation, constants and the
per-render-mode post-processing follow the reference; the rendering itself is ops.rasterize_from_world_with_sh_fwd."""
from dataclasses import dataclass
from enum import IntEnum
from typing import Optional

import torch

from . import ops


class RenderMode(IntEnum):
    """rasterizer.hpp render modes in the order Rasterization.cpp:374-393 switches on"""
    RGB = 0
    D = 1
    ED = 2
    RGB_D = 3
    RGB_ED = 4


@dataclass
class RenderOutput:
    image: Optional[torch.Tensor]   # [3,H,W] clamped to [0,1], None in the depth-only modes
    alpha: torch.Tensor             # [1,H,W]
    depth: Optional[torch.Tensor]   # [1,H,W], None in RGB mode
    means2d: torch.Tensor           # [1,N,2]
    depths: torch.Tensor            # [N]
    radii: torch.Tensor             # [N] max over the two axes
    visibility: torch.Tensor        # [N] bool
    width: int
    height: int


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)  # TORCH_CHECK


def _pad(t, n, dev):
    """rasterizer.cpp:97-120 pads the coefficient vectors with zeros; the pinhole kernel reads 6 radial / 2 tangential
    values (ProjectionUT3DGSFused.cu:101-106), the fisheye one 4 radial (:124), so the radial vector is padded to 6
    or 4 here (the reference always pads to 4)"""
    if t is None or t.numel() == 0:
        return None
    _check(t.dim() == 1, f"distortion coefficients must be 1D, got {tuple(t.shape)}")
    t = t.to(dev, torch.float32)
    if t.numel() < n:
        t = torch.cat([t, torch.zeros(n - t.numel(), dtype=torch.float32, device=dev)])
    return t[:n].reshape(1, n).contiguous()


def rasterize(viewmat, K, image_width, image_height, means3D, opacities, scales, rotations, sh_coeffs, sh_degree,
              bg_color=None, scaling_modifier=1.0, packed=False, antialiased=False, render_mode=RenderMode.RGB,
              radial_distortion=None, tangential_distortion=None, camera_model=0):
    """viewmat [1,4,4], K [1,3,3]; the Gaussian tensors are the model's getters (activated opacity [N] or [N,1],
    activated scales [N,3], normalised rotations [N,4], sh_coeffs [N,K,3]); bg_color [3] or None."""
    _check(not packed, "Packed mode is not supported in this implementation")
    _check(viewmat.dim() == 3 and tuple(viewmat.shape) == (1, 4, 4),
           f"viewmat must be [1, 4, 4] after transpose and unsqueeze, got {tuple(viewmat.shape)}")
    _check(viewmat.is_cuda, "viewmat must be on CUDA")
    _check(K.is_cuda, "K must be on CUDA")
    if opacities.dim() == 2 and opacities.shape[1] == 1:
        opacities = opacities.squeeze(-1)
    N = means3D.shape[0]
    _check(means3D.dim() == 2 and means3D.shape[1] == 3, f"means3D must be [N, 3], got {tuple(means3D.shape)}")
    _check(opacities.dim() == 1 and opacities.shape[0] == N, f"opacities must be [N], got {tuple(opacities.shape)}")
    _check(scales.dim() == 2 and tuple(scales.shape) == (N, 3), f"scales must be [N, 3], got {tuple(scales.shape)}")
    _check(rotations.dim() == 2 and tuple(rotations.shape) == (N, 4),
           f"rotations must be [N, 4], got {tuple(rotations.shape)}")
    _check(sh_coeffs.dim() == 3 and sh_coeffs.shape[0] == N and sh_coeffs.shape[2] == 3,
           f"sh_coeffs must be [N, K, 3], got {tuple(sh_coeffs.shape)}")
    need = (sh_degree + 1) * (sh_degree + 1)
    _check(sh_coeffs.shape[1] >= need,
           f"Not enough SH coefficients. Expected at least {need} but got {sh_coeffs.shape[1]}")
    for t, name in ((means3D, "means3D"), (opacities, "opacities"), (scales, "scales"), (rotations, "rotations"),
                    (sh_coeffs, "sh_coeffs")):
        _check(t.is_cuda, f"{name} must be on CUDA")
    dev = means3D.device
    if bg_color is None or bg_color.numel() == 0:
        bg = torch.zeros((1, 3), dtype=torch.float32, device=dev)  # rasterizer.cpp:149
    else:
        bg = bg_color.reshape(1, -1).to(dev, torch.float32)
        _check(tuple(bg.shape) == (1, 3), f"bg_color must be reshapeable to [1, 3], got {tuple(bg.shape)}")
    mode = RenderMode(int(render_mode))
    # rasterizer.cpp:90-95: eps2d 0.3, near 0.01, far 1e4, radius_clip 0, tile 16, compensations iff antialiased
    out = ops.rasterize_from_world_with_sh_fwd(
        means3D.contiguous(), rotations.contiguous(), scales.contiguous(), opacities.contiguous(),
        sh_coeffs.contiguous(), sh_degree, bg, None, image_width, image_height, 16, viewmat.contiguous(), None,
        K.contiguous(), int(camera_model), 0.3, 0.01, 10000.0, 0.0, float(scaling_modifier), bool(antialiased),
        int(mode), ops.UnscentedTransformParameters(), 4,
        _pad(radial_distortion, 4 if int(camera_model) == ops.CameraModelType.FISHEYE else 6, dev),
        _pad(tangential_distortion, 2, dev), None)
    rendered, alpha, radii, means2d, depths = out[0], out[1], out[2], out[3], out[4]
    image = depth = None
    if mode == RenderMode.RGB:
        image = rendered
    elif mode == RenderMode.D:
        depth = rendered
    elif mode == RenderMode.ED:
        depth = rendered / alpha.clamp_min(1e-10)
    elif mode == RenderMode.RGB_D:
        image, depth = rendered[..., :-1], rendered[..., -1:]
    else:
        image, depth = rendered[..., :-1], rendered[..., -1:] / alpha.clamp_min(1e-10)
    chw = lambda t: t.squeeze(0).permute(2, 0, 1)
    r = radii.squeeze(0).max(-1).values
    return RenderOutput(image=None if image is None else torch.clamp(chw(image), 0.0, 1.0), alpha=chw(alpha),
                        depth=None if depth is None else chw(depth), means2d=means2d.contiguous(),
                        depths=depths.squeeze(0), radii=r, visibility=r > 0, width=image_width, height=image_height)
