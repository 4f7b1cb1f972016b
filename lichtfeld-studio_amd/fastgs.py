"""Host-side mirror of the reference's default rasterization backend: fast_gs::rasterization::forward_wrapper /
backward_wrapper (src/training/fastgs/rasterization/include/rasterization_api.h:25-75) and the caller
gs::training::fast_rasterize (src/training/rasterization/fast_rasterizer.cpp:12-66), over the C ABI of
include/gsx_fastgs.h.  Tensors are torch CUDA tensors (device memory and streams only); every kernel is the library's.
"""
import ctypes

import numpy as np
import torch

from . import _lib as L
from ._lib import c_i, c_i64, c_p, c_sz, c_u32, check, lib


class Settings(ctypes.Structure):
    """gsx_fastgs_settings"""
    _fields_ = [("active_sh_bases", ctypes.c_uint32), ("total_bases_sh_rest", ctypes.c_uint32),
                ("width", ctypes.c_uint32), ("height", ctypes.c_uint32), ("fx", ctypes.c_float),
                ("fy", ctypes.c_float), ("cx", ctypes.c_float), ("cy", ctypes.c_float),
                ("near_plane", ctypes.c_float), ("far_plane", ctypes.c_float)]


def _p(t):
    return c_p(None) if t is None else c_p(t.data_ptr())


def _stream(dev):
    return c_p(torch.cuda.current_stream(dev).cuda_stream)


def _check_input(t, name):
    """CHECK_INPUT of the reference's wrapper (rasterization_api.cu:35-40): contiguous CUDA float tensors"""
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
        raise ValueError(f"{name} must be a contiguous CUDA float tensor")


def _host16(w2c, cam_position):
    """w2c [4,4] (or [1,4,4]) and cam_position [3] as host float32 arrays (a device tensor costs a synchronising copy)"""
    to_np = lambda a: (a.detach().cpu().numpy() if isinstance(a, torch.Tensor) else np.asarray(a))
    w = np.ascontiguousarray(to_np(w2c), dtype=np.float32).reshape(-1)[-16:].copy()
    c = np.ascontiguousarray(to_np(cam_position), dtype=np.float32).reshape(-1)[:3].copy()
    return w, c


_functions_typed = False


def _typed():
    global _functions_typed
    lb = lib()
    if not _functions_typed:
        for name in ("gsx_fastgs_primitive_state_bytes", "gsx_fastgs_instance_state_bytes",
                     "gsx_fastgs_pixel_state_bytes", "gsx_fastgs_accum_bytes"):
            getattr(lb, name).restype = c_sz
        _functions_typed = True
    return lb


_accum = {}  # (device index, N) -> zeroed accumulator the backward leaves zeroed


def _accumulator(dev, N):
    lb = _typed()
    key = (dev.index, N)
    if key not in _accum:
        _accum.clear()  # one size at a time: the count changes when the model grows
        _accum[key] = torch.zeros(lb.gsx_fastgs_accum_bytes(c_u32(N)), dtype=torch.uint8, device=dev)
    return _accum[key]


def forward_wrapper(means, scales_raw, rotations_raw, opacities_raw, sh_coefficients_0, sh_coefficients_rest, w2c,
                    cam_position, active_sh_bases, width, height, focal_x, focal_y, center_x, center_y, near_plane,
                    far_plane, background=None):
    """rasterization_api.h:25-43.  Returns the reference's 11-tuple (image [3,H,W], alpha [1,H,W], per_primitive,
    per_tile, per_instance, per_bucket buffers, n_visible_primitives, n_instances, n_buckets, two selectors): the
    buffers are this library's state blobs (per_tile holds the per-pixel state, per_bucket is empty: no checkpoints
    are stored), n_visible_primitives is -1 (never needed on the host here), n_buckets and the selectors are 0.
    background (optional, [3] CUDA tensor): blended in the kernel as fast_rasterizer.cpp:63 does afterwards."""
    lb = _typed()
    for t, name in ((means, "means"), (scales_raw, "scales_raw"), (rotations_raw, "rotations_raw"),
                    (opacities_raw, "opacities_raw"), (sh_coefficients_0, "sh_coefficients_0"),
                    (sh_coefficients_rest, "sh_coefficients_rest")):
        _check_input(t, name)
    dev = means.device
    N, B = means.shape[0], sh_coefficients_rest.shape[1]
    S = Settings(active_sh_bases, B, width, height, focal_x, focal_y, center_x, center_y, near_plane, far_plane)
    w, c = _host16(w2c, cam_position)
    e = lambda *s, dt=torch.float32: torch.empty(s, dtype=dt, device=dev)
    prim = e(lb.gsx_fastgs_primitive_state_bytes(c_u32(N)), dt=torch.uint8)
    n_host = torch.zeros(1, dtype=torch.int64, pin_memory=True)
    s = _stream(dev)
    with torch.cuda.device(dev):
        check(lb.gsx_fastgs_preprocess(c_u32(N), _p(means), _p(scales_raw), _p(rotations_raw), _p(opacities_raw),
                                       _p(sh_coefficients_0), _p(sh_coefficients_rest), c_p(w.ctypes.data),
                                       c_p(c.ctypes.data), ctypes.byref(S), _p(prim), c_sz(prim.numel()),
                                       c_p(n_host.data_ptr()), c_i(1), s))
        n_instances = int(n_host[0])
        inst = e(lb.gsx_fastgs_instance_state_bytes(c_i64(n_instances), c_u32(width), c_u32(height)), dt=torch.uint8)
        pix = e(lb.gsx_fastgs_pixel_state_bytes(c_u32(width), c_u32(height)), dt=torch.uint8)
        image, alpha = e(3, height, width), e(1, height, width)
        check(lb.gsx_fastgs_render(c_u32(N), ctypes.byref(S), _p(prim), c_sz(prim.numel()), c_i64(n_instances),
                                   _p(inst), c_sz(inst.numel()), _p(background), _p(image), _p(alpha), _p(pix),
                                   c_sz(pix.numel()), s))
    return (image, alpha, prim, pix, inst, e(0, dt=torch.uint8), -1, n_instances, 0, 0, 0)


def backward_wrapper(densification_info, grad_image, grad_alpha, image, alpha, means, scales_raw, rotations_raw,
                     sh_coefficients_rest, per_primitive_buffers, per_tile_buffers, per_instance_buffers,
                     per_bucket_buffers, w2c, cam_position, active_sh_bases, width, height, focal_x, focal_y,
                     center_x, center_y, near_plane, far_plane, n_visible_primitives, n_instances, n_buckets,
                     primitive_primitive_indices_selector, instance_primitive_indices_selector,
                     w2c_requires_grad=False, background=None):
    """rasterization_api.h:45-75 -> (grad_means, grad_scales_raw, grad_rotations_raw, grad_opacities_raw [N,1],
    grad_sh_coefficients_0 [N,1,3], grad_sh_coefficients_rest [N,B,3], grad_w2c [4,4] or None).
    densification_info: [2,N] CUDA tensor updated in place, or an empty tensor / None (rasterization_api.cu:130)."""
    lb = _typed()
    dev = means.device
    N, B = means.shape[0], sh_coefficients_rest.shape[1]
    S = Settings(active_sh_bases, B, width, height, focal_x, focal_y, center_x, center_y, near_plane, far_plane)
    w, c = _host16(w2c, cam_position)
    z = lambda *s: torch.empty(s, dtype=torch.float32, device=dev)
    g_means, g_scales, g_rot, g_op = z(N, 3), z(N, 3), z(N, 4), z(N, 1)
    g_sh0, g_shN = z(N, 1, 3), z(N, B, 3)
    g_w2c = z(4, 4) if w2c_requires_grad else None
    info = densification_info if densification_info is not None and densification_info.numel() > 0 else None
    if info is not None and tuple(info.shape) != (2, N):
        raise ValueError("densification_info must be [2, N]")
    acc = _accumulator(dev, N)
    for t, name, shape in ((grad_image, "grad_image", (3, height, width)), (grad_alpha, "grad_alpha", (1, height, width))):
        if not (t.is_cuda and t.dtype == torch.float32 and tuple(t.shape) == shape):
            raise ValueError(f"{name} must be a CUDA float tensor of shape {shape}")
    for t, name in ((per_primitive_buffers, "per_primitive_buffers"), (per_tile_buffers, "per_tile_buffers"),
                    (per_instance_buffers, "per_instance_buffers")):
        if not (t.is_cuda and t.dtype == torch.uint8 and t.is_contiguous()):
            raise ValueError(f"{name} must be the byte tensor forward_wrapper returned")
    gi, ga = grad_image.contiguous(), grad_alpha.contiguous()
    with torch.cuda.device(dev):
        check(lb.gsx_fastgs_backward(c_u32(N), _p(means), _p(scales_raw), _p(rotations_raw), _p(sh_coefficients_rest),
                                     c_p(w.ctypes.data), c_p(c.ctypes.data), ctypes.byref(S),
                                     _p(per_primitive_buffers), c_sz(per_primitive_buffers.numel()),
                                     c_i64(n_instances), _p(per_instance_buffers),
                                     c_sz(per_instance_buffers.numel()), _p(per_tile_buffers),
                                     c_sz(per_tile_buffers.numel()), _p(background), _p(gi), _p(ga), _p(acc),
                                     c_sz(acc.numel()),
                                     _p(g_means), _p(g_scales), _p(g_rot), _p(g_op), _p(g_sh0), _p(g_shN), _p(g_w2c),
                                     _p(info), _stream(dev)))
    return g_means, g_scales, g_rot, g_op, g_sh0, g_shN, g_w2c


def instance_list(per_instance_buffers, n_instances, width, height):
    """the sorted instance list (primitive index per instance) and the first instance of every tile, as tensors
    copied out of the instance state (tests / inspection)"""
    lb = _typed()
    S = Settings(1, 0, width, height, 1.0, 1.0, 0.0, 0.0, 0.0, 1.0)
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    check(lb.gsx_fastgs_instance_list(ctypes.byref(S), c_i64(n_instances), _p(per_instance_buffers), ctypes.byref(a),
                                      ctypes.byref(b)))
    base = per_instance_buffers.data_ptr()
    n_tiles = ((width + 15) // 16) * ((height + 15) // 16)
    as_i32 = per_instance_buffers.view(torch.int32)
    inst = as_i32[(a.value - base) // 4:(a.value - base) // 4 + n_instances].clone()
    offs = as_i32[(b.value - base) // 4:(b.value - base) // 4 + n_tiles].clone()
    return inst, offs


def primitive_records(per_primitive_buffers, N):
    """-> (records [N,12] float32: mean2d, conic, opacity, colour, box half-widths, depth; n_touched [N] int32)"""
    lb = _typed()
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    check(lb.gsx_fastgs_primitive_records(c_u32(N), _p(per_primitive_buffers), ctypes.byref(a), ctypes.byref(b)))
    base = per_primitive_buffers.data_ptr()
    rec = per_primitive_buffers.view(torch.float32)[(a.value - base) // 4:(a.value - base) // 4 + 12 * N]
    cnt = per_primitive_buffers.view(torch.int32)[(b.value - base) // 4:(b.value - base) // 4 + N]
    return rec.reshape(N, 12).clone(), cnt.clone()


def fast_rasterize(means, scales_raw, rotations_raw, opacities_raw, sh0, shN, w2c, cam_position, sh_degree, width,
                   height, fx, fy, cx, cy, bg_color):
    """gs::training::fast_rasterize (fast_rasterizer.cpp:12-66): near 0.01, far 1e10, image + (1 - alpha) * bg.
    -> (image [3,H,W], alpha [1,H,W], saved) with `saved` the argument pack fast_rasterize_backward needs."""
    bases = (sh_degree + 1) * (sh_degree + 1)
    out = forward_wrapper(means, scales_raw, rotations_raw, opacities_raw, sh0, shN, w2c, cam_position, bases, width,
                          height, fx, fy, cx, cy, 0.01, 1e10, background=bg_color)
    saved = dict(out=out, args=(means, scales_raw, rotations_raw, shN), cam=(w2c, cam_position),
                 scalars=(bases, width, height, fx, fy, cx, cy, 0.01, 1e10), bg=bg_color)
    return out[0], out[1], saved


def fast_rasterize_backward(saved, grad_image, grad_alpha, densification_info=None, w2c_requires_grad=False):
    """FastGSRasterize::backward (fast_rasterizer_autograd.cpp:93-163) including the background blend's gradient"""
    image, alpha, prim, pix, inst, bucket, nv, ni, nb, s1, s2 = saved["out"]
    means, scales_raw, rotations_raw, shN = saved["args"]
    return backward_wrapper(densification_info, grad_image, grad_alpha, image, alpha, means, scales_raw, rotations_raw,
                            shN, prim, pix, inst, bucket, *saved["cam"], *saved["scalars"], nv, ni, nb, s1, s2,
                            w2c_requires_grad=w2c_requires_grad, background=saved["bg"])
