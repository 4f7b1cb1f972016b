"""gsx - MI355X (gfx950) implementation of the 3D-Gaussian-splatting training step behind LichtFeld-Studio's
gsplat/Ops.h: projection, SH colour, tile intersection + radix sort + ranges, rasterize forward / backward,
fused SSIM, fused Adam, MCMC relocation / noise.  Kernels live in csrc/*.hip behind the C ABI of include/gsx.h;
the modules here mirror the reference's host interface over torch tensors.

The directory name is not a Python identifier; load it with

    spec = importlib.util.spec_from_file_location("lichtfeld_studio_amd", ".../lichtfeld-studio_amd/__init__.py",
                                                  submodule_search_locations=[".../lichtfeld-studio_amd"])
"""
from . import _lib, scenes  # noqa: F401

__all__ = ["_lib", "ops", "scenes", "build"]


def __getattr__(name):
    # these import torch (or drive a compiler): loaded on first use
    if name in ("ops", "build", "build_ext", "trainer", "rasterizer", "fastgs", "ply"):
        import importlib
        return importlib.import_module(f"{__name__}.{name}")
    raise AttributeError(name)
