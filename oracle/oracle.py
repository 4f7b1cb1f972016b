"""numpy front-end of the CPU checker (oracle/libgsx_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline
leg of bench.py.  The shipped package never imports it.

Function names and argument order follow the reference's gsplat/Ops.h (see each docstring); arrays
are numpy, C-contiguous, float32 / int32 / int64 / uint8 as the reference's tensors are.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgsx_oracle.so")
_lib = None

c_f = ctypes.c_float
c_i = ctypes.c_int
c_u32 = ctypes.c_uint32
c_i64 = ctypes.c_int64
c_p = ctypes.c_void_p


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import build as _b  # noqa: F401  (package import)
            _b.build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_tile_n_bits.restype = c_u32
        _lib.orc_num_threads.restype = c_i
        _lib.orc_get_image_size.restype = c_u32
    return _lib


def _p(a):
    if a is None:
        return c_p(None)
    assert a.flags["C_CONTIGUOUS"], "array must be contiguous"
    return c_p(a.ctypes.data)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _chk(rc, name):
    if rc != 0:
        raise RuntimeError(f"oracle {name} failed with code {rc}")


UT_DEFAULT = dict(alpha=0.1, beta=2.0, kappa=0.0, in_image_margin_factor=0.1, require_all_sigma_points_valid=True)


class distortion:
    """Context manager: OpenCV pinhole distortion coefficients (radial [6], tangential [2], thin_prism [4], each
    optional) for every projection / pixel-ray inside the block, as the reference dispatches on "any coefficient
    tensor given" (ProjectionUT3DGSFused.cu:86-113)."""

    def __init__(self, radial=None, tangential=None, thin_prism=None):
        f = lambda a, n: None if a is None else np.ascontiguousarray(np.asarray(a, np.float32).reshape(-1)[:n])
        self.args = (f(radial, 6), f(tangential, 2), f(thin_prism, 4))

    def __enter__(self):
        lib().orc_set_distortion(*[_p(a) for a in self.args])
        return self

    def __exit__(self, *exc):
        lib().orc_set_distortion(None, None, None)
        return False


class camera_model:
    """Context manager: the OpenCV fisheye (model 2, radial [4] optional) or the equirectangular model (3) for every
    projection / pixel ray inside the block; W, H = the image size."""

    def __init__(self, model, W, H, radial=None):
        self.model, self.W, self.H = int(model), int(W), int(H)
        self.radial = None if radial is None else np.ascontiguousarray(np.asarray(radial, np.float32).reshape(-1)[:4])

    def __enter__(self):
        lib().orc_set_camera_model(c_i(self.model), _p(self.radial), None, None, c_u32(self.W), c_u32(self.H))
        return self

    def __exit__(self, *exc):
        lib().orc_set_camera_model(c_i(0), None, None, None, c_u32(0), c_u32(0))
        return False


class rolling_shutter:
    """Context manager: shutter type (gsplat/Cameras.h:16-22: 0 top-to-bottom, 1 left-to-right, 2 bottom-to-top,
    3 right-to-left, 4 global) and end-of-frame pose viewmat1 [4,4] for every projection / pixel ray inside the block;
    W, H = the image size (the exposure time of a pixel is its row / column over H - 1 / W - 1)."""

    def __init__(self, rs_type, viewmat1, W, H):
        self.rs_type, self.W, self.H = int(rs_type), int(W), int(H)
        self.vm1 = None if viewmat1 is None else np.ascontiguousarray(np.asarray(viewmat1, np.float32).reshape(4, 4))

    def __enter__(self):
        L = lib()
        self.prev = (L.orc_get_image_size(0), L.orc_get_image_size(1))
        L.orc_set_image_size(c_u32(self.W), c_u32(self.H))
        L.orc_set_rolling_shutter(c_i(self.rs_type), _p(self.vm1))
        return self

    def __exit__(self, *exc):
        lib().orc_set_rolling_shutter(c_i(4), None)
        lib().orc_set_image_size(c_u32(self.prev[0]), c_u32(self.prev[1]))
        return False


def world_project(points, viewmat, fx, fy, cx, cy, W, H, margin=0.1):
    """world points [n,3] -> (image points [n,2], valid [n]) under the current camera model and shutter"""
    pts, vm = _f32(points).reshape(-1, 3), _f32(viewmat).reshape(4, 4)
    out = np.zeros((pts.shape[0], 2), np.float32)
    valid = np.zeros(pts.shape[0], np.uint8)
    lib().orc_world_project(c_i64(pts.shape[0]), _p(pts), _p(vm), c_f(fx), c_f(fy), c_f(cx), c_f(cy), c_u32(W),
                            c_u32(H), c_f(margin), _p(out), _p(valid))
    return out, valid.astype(bool)


def pixel_world_rays(image_points, viewmat, fx, fy, cx, cy):
    """pixel positions [n,2] -> (origins [n,3], directions [n,3], valid [n]) under the current model and shutter"""
    ip, vm = _f32(image_points).reshape(-1, 2), _f32(viewmat).reshape(4, 4)
    o, d = np.zeros((ip.shape[0], 3), np.float32), np.zeros((ip.shape[0], 3), np.float32)
    valid = np.zeros(ip.shape[0], np.uint8)
    lib().orc_pixel_world_rays(c_i64(ip.shape[0]), _p(ip), _p(vm), c_f(fx), c_f(fy), c_f(cx), c_f(cy), _p(o), _p(d),
                               _p(valid))
    return o, d, valid.astype(bool)


def math_camera(which, x, x2=None, x3=None):
    """probes of gsx_camera.h's primitives: "atan2" (x, x2), "cbrt", "asin", "cos", "max_angle_sq" (x, x2, x3)"""
    idx = {"atan2": 0, "cbrt": 1, "asin": 2, "cos": 3, "max_angle_sq": 4}[which]
    x = _f32(x).reshape(-1)
    x2 = x if x2 is None else _f32(x2).reshape(-1)
    x3 = x if x3 is None else _f32(x3).reshape(-1)
    y = np.zeros_like(x)
    lib().orc_math_camera(c_i(idx), c_i64(x.size), _p(x), _p(x2), _p(x3), _p(y))
    return y


def camera_project(points, fx, fy, cx, cy, W, H, margin=0.1):
    """camera-space points [n,3] -> (image points [n,2], valid [n]) under the current camera model"""
    pts = _f32(points)
    n = pts.shape[0]
    out, valid = np.zeros((n, 2), np.float32), np.zeros(n, np.uint8)
    lib().orc_camera_project(c_i64(n), _p(pts), c_f(fx), c_f(fy), c_f(cx), c_f(cy), c_u32(W), c_u32(H), c_f(margin),
                             _p(out), _p(valid))
    return out, valid.astype(bool)


def camera_unproject(image_points, fx, fy, cx, cy):
    """image points [n,2] -> (unit camera rays [n,3], valid [n]) under the current camera model"""
    ip = _f32(image_points)
    n = ip.shape[0]
    rays, valid = np.zeros((n, 3), np.float32), np.zeros(n, np.uint8)
    lib().orc_camera_unproject(c_i64(n), _p(ip), c_f(fx), c_f(fy), c_f(cx), c_f(cy), _p(rays), _p(valid))
    return rays, valid.astype(bool)


def philox4x32_10(ctr, key):
    c, k = np.asarray(ctr, np.uint32).copy(), np.asarray(key, np.uint32).copy()
    out = np.zeros(4, np.uint32)
    lib().orc_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def philox_randn3(n, seed, offset):
    """[n,3] N(0,1) rows, row i a function of (seed, offset, i): the draws gsx_add_noise_philox consumes"""
    out = np.zeros((n, 3), np.float32)
    lib().orc_philox_randn3(c_u32(n), ctypes.c_uint64(seed), ctypes.c_uint64(offset), _p(out))
    return out


def num_threads():
    return lib().orc_num_threads()


def set_num_threads(n):
    lib().orc_set_num_threads(c_i(int(n)))


def tile_n_bits(n_tiles):
    return int(lib().orc_tile_n_bits(c_u32(n_tiles)))


def projection_ut_3dgs_fused(means, quats, scales, opacities, viewmats0, Ks, image_width, image_height, eps2d=0.3,
                             near_plane=0.01, far_plane=1e4, radius_clip=0.0, calc_compensations=False, ut=None):
    """gsplat/Ops.h:69-98 (perfect pinhole, global shutter).  Returns radii, means2d, depths, conics, compensations.
    Outputs of culled Gaussians (radii == 0) are zero here (uninitialised in the reference)."""
    ut = dict(UT_DEFAULT, **(ut or {}))
    means, quats, scales = _f32(means), _f32(quats), _f32(scales)
    opacities, viewmats0, Ks = _f32(opacities), _f32(viewmats0), _f32(Ks)
    C, N = viewmats0.shape[0], means.shape[0]
    radii = np.zeros((C, N, 2), np.int32)
    means2d = np.zeros((C, N, 2), np.float32)
    depths = np.zeros((C, N), np.float32)
    conics = np.zeros((C, N, 3), np.float32)
    comp = np.zeros((C, N), np.float32) if calc_compensations else None
    rc = lib().orc_projection_ut_3dgs_fused(
        c_u32(C), c_u32(N), _p(means), _p(quats), _p(scales), _p(opacities), _p(viewmats0), _p(Ks),
        c_u32(image_width), c_u32(image_height), c_f(eps2d), c_f(near_plane), c_f(far_plane), c_f(radius_clip),
        c_f(ut["alpha"]), c_f(ut["beta"]), c_f(ut["kappa"]), c_f(ut["in_image_margin_factor"]),
        c_i(1 if ut["require_all_sigma_points_valid"] else 0), _p(radii), _p(means2d), _p(depths), _p(conics),
        _p(comp))
    _chk(rc, "projection_ut_3dgs_fused")
    return radii, means2d, depths, conics, comp


def spherical_harmonics_fwd(degrees_to_use, dirs, coeffs, masks=None):
    """gsplat/Ops.h:12-17.  dirs [N,3], coeffs [N,K,3], masks bool [N] -> colors [N,3] (masked-out rows 0)."""
    dirs, coeffs = _f32(dirs), _f32(coeffs)
    N, K = coeffs.shape[0], coeffs.shape[1]
    m = None if masks is None else np.ascontiguousarray(masks, dtype=np.uint8)
    colors = np.zeros((N, 3), np.float32)
    _chk(lib().orc_spherical_harmonics_fwd(c_u32(N), c_u32(K), c_u32(degrees_to_use), _p(dirs), _p(coeffs), _p(m),
                                           _p(colors)), "spherical_harmonics_fwd")
    return colors


def spherical_harmonics_bwd(K, degrees_to_use, dirs, coeffs, masks, v_colors, compute_v_dirs=False):
    """gsplat/Ops.h:18-25 -> (v_coeffs [N,K,3], v_dirs [N,3] or None)."""
    dirs, coeffs, v_colors = _f32(dirs), _f32(coeffs), _f32(v_colors)
    N = coeffs.shape[0]
    m = None if masks is None else np.ascontiguousarray(masks, dtype=np.uint8)
    v_coeffs = np.zeros((N, K, 3), np.float32)
    v_dirs = np.zeros((N, 3), np.float32) if compute_v_dirs else None
    _chk(lib().orc_spherical_harmonics_bwd(c_u32(N), c_u32(K), c_u32(degrees_to_use), _p(dirs), _p(coeffs), _p(m),
                                           _p(v_colors), _p(v_coeffs), _p(v_dirs)), "spherical_harmonics_bwd")
    return v_coeffs, v_dirs


def intersect_tile_count(means2d, radii, C, tile_size, tile_width, tile_height):
    """The first launch of intersect_tile alone (IntersectTile.cu:46-114 with null outputs, Intersect.cpp:58-76):
    -> tiles_per_gauss [C,N] i32 and the number of intersections (an int64: it may exceed what int32 indexes)."""
    means2d = _f32(means2d)
    radii = np.ascontiguousarray(radii, dtype=np.int32)
    N = means2d.shape[1]
    tpg = np.zeros((C, N), np.int32)
    cum = np.zeros((C, N), np.int64)
    n_isects = c_i64(0)
    _chk(lib().orc_intersect_tile_count(c_u32(C), c_u32(N), _p(means2d), _p(radii), c_u32(tile_size),
                                        c_u32(tile_width), c_u32(tile_height), _p(tpg), _p(cum),
                                        ctypes.byref(n_isects)), "intersect_tile_count")
    return tpg, int(n_isects.value)


def intersect_tile(means2d, radii, depths, C, tile_size, tile_width, tile_height, sort=True):
    """gsplat/Ops.h:28-38 (unpacked).  -> tiles_per_gauss [C,N] i32, isect_ids [I] i64, flatten_ids [I] i32."""
    means2d, depths = _f32(means2d), _f32(depths)
    radii = np.ascontiguousarray(radii, dtype=np.int32)
    N = means2d.shape[1]
    tpg = np.zeros((C, N), np.int32)
    cum = np.zeros((C, N), np.int64)
    n_isects = c_i64(0)
    _chk(lib().orc_intersect_tile_count(c_u32(C), c_u32(N), _p(means2d), _p(radii), c_u32(tile_size),
                                        c_u32(tile_width), c_u32(tile_height), _p(tpg), _p(cum),
                                        ctypes.byref(n_isects)), "intersect_tile_count")
    n = n_isects.value
    ids = np.zeros((n,), np.int64)
    flat = np.zeros((n,), np.int32)
    if n:
        _chk(lib().orc_intersect_tile_emit(c_u32(C), c_u32(N), _p(means2d), _p(radii), _p(depths), _p(cum),
                                           c_u32(tile_size), c_u32(tile_width), c_u32(tile_height), _p(ids), _p(flat)),
             "intersect_tile_emit")
    if n and sort:
        end_bit = 32 + tile_n_bits(tile_width * tile_height) + tile_n_bits(C)
        ids, flat = radix_sort_pairs(ids, flat, end_bit)
    return tpg, ids, flat


def intersect_tile_packed(means2d, radii, depths, camera_ids, C, tile_size, tile_width, tile_height, sort=True):
    """gsplat/Ops.h:28-38 with packed rows (means2d [nnz,2], camera_ids [nnz]; Intersect.cpp:32-39,
    IntersectTile.cu:50, 86-94).  -> tiles_per_gauss [nnz] i32, isect_ids [I] i64, flatten_ids [I] i32 (packed row
    indices)."""
    means2d, depths = _f32(means2d), _f32(depths)
    radii = np.ascontiguousarray(radii, dtype=np.int32)
    camera_ids = np.ascontiguousarray(camera_ids, dtype=np.int64)
    nnz = means2d.shape[0]
    tpg = np.zeros((nnz,), np.int32)
    cum = np.zeros((nnz,), np.int64)
    n_isects = c_i64(0)
    _chk(lib().orc_intersect_tile_count(c_u32(1), c_u32(nnz), _p(means2d), _p(radii), c_u32(tile_size),
                                        c_u32(tile_width), c_u32(tile_height), _p(tpg), _p(cum),
                                        ctypes.byref(n_isects)), "intersect_tile_count")
    n = n_isects.value
    ids = np.zeros((n,), np.int64)
    flat = np.zeros((n,), np.int32)
    if n:
        _chk(lib().orc_intersect_tile_emit_packed(c_u32(nnz), _p(means2d), _p(radii), _p(depths), _p(camera_ids),
                                                  _p(cum), c_u32(tile_size), c_u32(tile_width), c_u32(tile_height),
                                                  _p(ids), _p(flat)), "intersect_tile_emit_packed")
    if n and sort:
        end_bit = 32 + tile_n_bits(tile_width * tile_height) + tile_n_bits(C)
        ids, flat = radix_sort_pairs(ids, flat, end_bit)
    return tpg, ids, flat


def radix_sort_pairs(keys, vals, end_bit):
    """gsplat/Intersect.h:39-46: stable ascending sort on bits [0, end_bit)."""
    keys = np.ascontiguousarray(keys, dtype=np.int64)
    vals = np.ascontiguousarray(vals, dtype=np.int32)
    ko, vo = np.empty_like(keys), np.empty_like(vals)
    _chk(lib().orc_radix_sort_pairs(c_i64(keys.shape[0]), _p(keys), _p(vals), c_u32(end_bit), _p(ko), _p(vo)),
         "radix_sort_pairs")
    return ko, vo


def intersect_offset(isect_ids, C, tile_width, tile_height):
    """gsplat/Ops.h:39-43 -> offsets [C, tile_height, tile_width] i32."""
    isect_ids = np.ascontiguousarray(isect_ids, dtype=np.int64)
    off = np.zeros((C, tile_height, tile_width), np.int32)
    _chk(lib().orc_intersect_offset(c_i64(isect_ids.shape[0]), _p(isect_ids), c_u32(C), c_u32(tile_width),
                                    c_u32(tile_height), _p(off)), "intersect_offset")
    return off


def rasterize_to_pixels_from_world_3dgs_fwd(means, quats, scales, colors, opacities, backgrounds, masks, image_width,
                                            image_height, tile_size, viewmats0, Ks, tile_offsets, flatten_ids,
                                            return_pairs=False):
    """gsplat/Ops.h:100-129 (C == 1).  colors [1,N,CDIM], opacities [1,N] ->
    renders [1,H,W,CDIM], alphas [1,H,W,1], last_ids [1,H,W]."""
    means, quats, scales = _f32(means), _f32(quats), _f32(scales)
    colors, opacities = _f32(colors), _f32(opacities)
    backgrounds, viewmats0, Ks = _f32(backgrounds), _f32(viewmats0), _f32(Ks)
    tile_offsets = np.ascontiguousarray(tile_offsets, dtype=np.int32)
    flatten_ids = np.ascontiguousarray(flatten_ids, dtype=np.int32)
    m = None if masks is None else np.ascontiguousarray(masks, dtype=np.uint8)
    C, N, CDIM = 1, means.shape[0], colors.shape[-1]
    H, W = image_height, image_width
    renders = np.zeros((C, H, W, CDIM), np.float32)
    alphas = np.zeros((C, H, W, 1), np.float32)
    last_ids = np.zeros((C, H, W), np.int32)
    pairs = c_i64(0)
    _chk(lib().orc_rasterize_to_pixels_from_world_3dgs_fwd(
        c_u32(C), c_u32(N), c_i64(flatten_ids.shape[0]), _p(means), _p(quats), _p(scales), _p(colors), c_u32(CDIM),
        _p(opacities), _p(backgrounds), _p(m), c_u32(W), c_u32(H), c_u32(tile_size), _p(viewmats0), _p(Ks),
        _p(tile_offsets), _p(flatten_ids), _p(renders), _p(alphas), _p(last_ids), ctypes.byref(pairs)),
        "rasterize_fwd")
    if return_pairs:
        return renders, alphas, last_ids, pairs.value
    return renders, alphas, last_ids


def rasterize_to_pixels_from_world_3dgs_bwd(means, quats, scales, colors, opacities, backgrounds, masks, image_width,
                                            image_height, tile_size, viewmats0, Ks, tile_offsets, flatten_ids,
                                            render_alphas, last_ids, v_render_colors, v_render_alphas):
    """gsplat/Ops.h:131-166 (C == 1, 1 to 4 channels) -> v_means, v_quats, v_scales, v_colors [1,N,CDIM],
    v_opacities [1,N]."""
    means, quats, scales = _f32(means), _f32(quats), _f32(scales)
    colors, opacities = _f32(colors), _f32(opacities)
    backgrounds, viewmats0, Ks = _f32(backgrounds), _f32(viewmats0), _f32(Ks)
    render_alphas, v_render_colors, v_render_alphas = _f32(render_alphas), _f32(v_render_colors), _f32(v_render_alphas)
    tile_offsets = np.ascontiguousarray(tile_offsets, dtype=np.int32)
    flatten_ids = np.ascontiguousarray(flatten_ids, dtype=np.int32)
    last_ids = np.ascontiguousarray(last_ids, dtype=np.int32)
    m = None if masks is None else np.ascontiguousarray(masks, dtype=np.uint8)
    N = means.shape[0]
    cdim = colors.shape[-1]
    v_means = np.zeros((N, 3), np.float32)
    v_quats = np.zeros((N, 4), np.float32)
    v_scales = np.zeros((N, 3), np.float32)
    v_colors = np.zeros((1, N, cdim), np.float32)
    v_opac = np.zeros((1, N), np.float32)
    _chk(lib().orc_rasterize_to_pixels_from_world_3dgs_bwd(
        c_u32(1), c_u32(N), c_i64(flatten_ids.shape[0]), _p(means), _p(quats), _p(scales), _p(colors), c_u32(cdim),
        _p(opacities),
        _p(backgrounds), _p(m), c_u32(image_width), c_u32(image_height), c_u32(tile_size), _p(viewmats0), _p(Ks),
        _p(tile_offsets), _p(flatten_ids), _p(render_alphas), _p(last_ids), _p(v_render_colors), _p(v_render_alphas),
        _p(v_means), _p(v_quats), _p(v_scales), _p(v_colors), _p(v_opac)), "rasterize_bwd")
    return v_means, v_quats, v_scales, v_colors, v_opac


def rasterize_bwd_f64(means, quats, scales, colors, opacities, backgrounds, image_width, image_height, tile_size,
                      viewmats0, Ks, tile_offsets, flatten_ids, render_alphas, last_ids, v_render_colors,
                      v_render_alphas):
    """float64 evaluation of the rasterizer backward (same pair selection as the fp32 pass) and a running
    error-bound scale.  -> (grads [N,14], bound [N,14]) float64; columns: mean 3, quat 4, scale 3, colour 3,
    opacity 1."""
    means, quats, scales = _f32(means), _f32(quats), _f32(scales)
    colors, opacities = _f32(colors), _f32(opacities)
    backgrounds, viewmats0, Ks = _f32(backgrounds), _f32(viewmats0), _f32(Ks)
    render_alphas, v_render_colors, v_render_alphas = _f32(render_alphas), _f32(v_render_colors), _f32(v_render_alphas)
    tile_offsets = np.ascontiguousarray(tile_offsets, dtype=np.int32)
    flatten_ids = np.ascontiguousarray(flatten_ids, dtype=np.int32)
    last_ids = np.ascontiguousarray(last_ids, dtype=np.int32)
    N = means.shape[0]
    grads = np.zeros((N, 14), np.float64)
    bound = np.zeros((N, 14), np.float64)
    _chk(lib().orc_rasterize_bwd_f64(
        c_u32(N), c_i64(flatten_ids.shape[0]), _p(means), _p(quats), _p(scales), _p(colors), _p(opacities),
        _p(backgrounds), c_u32(image_width), c_u32(image_height), c_u32(tile_size), _p(viewmats0), _p(Ks),
        _p(tile_offsets), _p(flatten_ids), _p(render_alphas), _p(last_ids), _p(v_render_colors), _p(v_render_alphas),
        _p(grads), _p(bound)), "rasterize_bwd_f64")
    return grads, bound


def fusedssim(C1, C2, img1, img2, train=True):
    """include/kernels/ssim.cuh:11-19.  img [B,CH,H,W] -> (map, dm_dmu1, dm_dsigma1_sq, dm_dsigma12)."""
    img1, img2 = _f32(img1), _f32(img2)
    B, CH, H, W = img1.shape
    ssim_map = np.zeros_like(img1)
    d1 = np.zeros_like(img1) if train else None
    d2 = np.zeros_like(img1) if train else None
    d3 = np.zeros_like(img1) if train else None
    _chk(lib().orc_fusedssim(c_i(B), c_i(CH), c_i(H), c_i(W), c_f(C1), c_f(C2), _p(img1), _p(img2), _p(ssim_map),
                             _p(d1), _p(d2), _p(d3)), "fusedssim")
    return ssim_map, d1, d2, d3


def fusedssim_backward(C1, C2, img1, img2, dL_dmap, dm_dmu1, dm_dsigma1_sq, dm_dsigma12):
    """include/kernels/ssim.cuh:21-28 -> dL/dimg1."""
    img1, img2, dL_dmap = _f32(img1), _f32(img2), _f32(dL_dmap)
    d1, d2, d3 = _f32(dm_dmu1), _f32(dm_dsigma1_sq), _f32(dm_dsigma12)  # keep the converted arrays alive
    B, CH, H, W = img1.shape
    out = np.zeros_like(img1)
    _chk(lib().orc_fusedssim_backward(c_i(B), c_i(CH), c_i(H), c_i(W), c_f(C1), c_f(C2), _p(img1), _p(img2),
                                      _p(dL_dmap), _p(d1), _p(d2), _p(d3), _p(out)), "fusedssim_backward")
    return out


def adam_step(param, exp_avg, exp_avg_sq, grad, lr, beta1, beta2, eps, bias_correction1_rcp,
              bias_correction2_sqrt_rcp):
    """fastgs/optimizer adam_step (adam_kernels.cuh:13-36); param / exp_avg / exp_avg_sq are updated in place."""
    for a in (param, exp_avg, exp_avg_sq):
        assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    grad = _f32(grad)
    _chk(lib().orc_adam_step(_p(param), _p(exp_avg), _p(exp_avg_sq), _p(grad), c_i64(param.size), c_f(lr), c_f(beta1),
                             c_f(beta2), c_f(eps), c_f(bias_correction1_rcp), c_f(bias_correction2_sqrt_rcp)),
         "adam_step")


def relocation(opacities, scales, ratios, binoms, n_max):
    """gsplat/Ops.h:52-57 -> (new_opacities [M], new_scales [M,3])."""
    opacities, scales, binoms = _f32(opacities), _f32(scales), _f32(binoms)
    ratios = np.ascontiguousarray(ratios, dtype=np.int32)
    M = opacities.shape[0]
    no = np.zeros((M,), np.float32)
    ns = np.zeros((M, 3), np.float32)
    _chk(lib().orc_relocation(c_i(M), _p(opacities), _p(scales), _p(ratios), _p(binoms), c_i(n_max), _p(no), _p(ns)),
         "relocation")
    return no, ns


def add_noise(raw_opacities, raw_scales, raw_quats, noise, means, current_lr):
    """gsplat/Ops.h:59-65; means is updated in place."""
    assert means.dtype == np.float32 and means.flags["C_CONTIGUOUS"]
    ro, rs, rq, nz = _f32(raw_opacities), _f32(raw_scales), _f32(raw_quats), _f32(noise)
    _chk(lib().orc_add_noise(c_i(means.shape[0]), _p(ro), _p(rs), _p(rq), _p(nz), _p(means), c_f(current_lr)),
         "add_noise")


def quats_to_rotmats(quats):
    """gsplat/Ops.h:46-48 -> [N,3,3] row-major."""
    quats = _f32(quats)
    out = np.zeros((quats.shape[0], 3, 3), np.float32)
    _chk(lib().orc_quats_to_rotmats(c_i(quats.shape[0]), _p(quats), _p(out)), "quats_to_rotmats")
    return out


def sh_colors_from_world(sh_degree, means, sh_coeffs, radii, viewmat):
    """Rasterization.cpp:356-378: colours [N,3] = max(SH(means - campos) + 0.5, 0), 0 where radii == 0."""
    means, sh_coeffs, viewmat = _f32(means), _f32(sh_coeffs), _f32(viewmat)
    radii = np.ascontiguousarray(radii, dtype=np.int32)
    N, K = sh_coeffs.shape[0], sh_coeffs.shape[1]
    colors = np.zeros((N, 3), np.float32)
    _chk(lib().orc_sh_colors_from_world(c_u32(N), c_u32(K), c_u32(sh_degree), _p(means), _p(sh_coeffs), _p(radii),
                                        _p(viewmat), _p(colors)), "sh_colors_from_world")
    return colors


def sh_colors_from_world_bwd(sh_degree, means, K, radii, viewmat, colors, v_colors):
    """Rasterization.cpp:608-624 -> v_sh_coeffs [N,K,3]."""
    means, viewmat, colors, v_colors = _f32(means), _f32(viewmat), _f32(colors), _f32(v_colors)
    radii = np.ascontiguousarray(radii, dtype=np.int32)
    N = means.shape[0]
    out = np.zeros((N, K, 3), np.float32)
    _chk(lib().orc_sh_colors_from_world_bwd(c_u32(N), c_u32(K), c_u32(sh_degree), _p(means), _p(radii), _p(viewmat),
                                            _p(colors), _p(v_colors), _p(out)), "sh_colors_from_world_bwd")
    return out


def _fit_backgrounds(backgrounds, channels):
    """[C,3] background under a render with another channel count: zeros for missing channels, surplus ones dropped
    (Rasterization.cpp:401-407 passes it on as it is, and its kernel then reads past each row's end)"""
    if backgrounds is None:
        return None
    b = _f32(backgrounds)
    if b.shape[-1] > channels:
        return np.ascontiguousarray(b[..., :channels])
    if b.shape[-1] < channels:
        return np.ascontiguousarray(np.concatenate([b, np.zeros(b.shape[:-1] + (channels - b.shape[-1],), np.float32)], -1))
    return b


def rasterize_from_world_with_sh_fwd(means, quats, scales, opacities, sh_coeffs, sh_degree, backgrounds, image_width,
                                     image_height, tile_size, viewmats0, Ks, eps2d=0.3, near_plane=0.01, far_plane=1e4,
                                     radius_clip=0.0, scaling_modifier=1.0, calc_compensations=False, ut=None,
                                     render_mode=0):
    """gsplat/Ops.h:174-220 (C == 1, no masks; render_mode 0 RGB, 1 / 2 depth, 3 / 4 RGB + depth,
    Rasterization.cpp:372-393).  Returns the reference's 10-tuple plus the sorted isect_ids (for key parity checks)
    as an 11th element."""
    scaled = _f32(scales) * np.float32(scaling_modifier) if scaling_modifier != 1.0 else _f32(scales)
    radii, means2d, depths, conics, comp = projection_ut_3dgs_fused(
        means, quats, scaled, opacities, viewmats0, Ks, image_width, image_height, eps2d, near_plane, far_plane,
        radius_clip, calc_compensations, ut)
    if render_mode in (0, 3, 4):
        colors = sh_colors_from_world(sh_degree, means, sh_coeffs, radii[0], viewmats0[0])[None]
        if render_mode != 0:
            colors = np.ascontiguousarray(np.concatenate([colors, depths[..., None]], -1))  # :385-387
    else:
        colors = np.ascontiguousarray(depths[..., None])  # :389-392
    final_op = _f32(opacities).reshape(1, -1)
    if calc_compensations:
        final_op = final_op * comp
    tw = (image_width + tile_size - 1) // tile_size
    th = (image_height + tile_size - 1) // tile_size
    _, isect_ids, flatten_ids = intersect_tile(means2d, radii, depths, 1, tile_size, tw, th, True)
    offsets = intersect_offset(isect_ids, 1, tw, th)
    renders, alphas, last_ids = rasterize_to_pixels_from_world_3dgs_fwd(
        means, quats, scaled, colors, final_op, _fit_backgrounds(backgrounds, colors.shape[-1]), None, image_width,
        image_height, tile_size, viewmats0, Ks, offsets, flatten_ids)
    return renders, alphas, radii, means2d, depths, colors, offsets, flatten_ids, last_ids, comp, isect_ids


def rasterize_from_world_with_sh_bwd(means, quats, scales, opacities, sh_coeffs, sh_degree, backgrounds, image_width,
                                     image_height, tile_size, viewmats0, Ks, scaling_modifier, calc_compensations,
                                     render_alphas, last_ids, tile_offsets, flatten_ids, colors, radii, compensations,
                                     v_render_colors, v_render_alphas, render_mode=0):
    """gsplat/Ops.h:222-270 -> v_means, v_quats, v_scales, v_opacities [1,N], v_sh_coeffs [N,K,3]."""
    scaled = _f32(scales) * np.float32(scaling_modifier) if scaling_modifier != 1.0 else _f32(scales)
    final_op = _f32(opacities).reshape(1, -1)
    if calc_compensations:
        final_op = final_op * compensations
    v_means, v_quats, v_scales, v_colors, v_opac = rasterize_to_pixels_from_world_3dgs_bwd(
        means, quats, scaled, colors, final_op, _fit_backgrounds(backgrounds, np.shape(colors)[-1]), None, image_width,
        image_height, tile_size, viewmats0, Ks,
        tile_offsets, flatten_ids, render_alphas, last_ids, v_render_colors, v_render_alphas)
    K = sh_coeffs.shape[1]
    if render_mode in (0, 3, 4):  # Rasterization.cpp:581-624: the depth channel's gradient is dropped
        v_sh = sh_colors_from_world_bwd(sh_degree, means, K, radii[0], viewmats0[0],
                                        np.ascontiguousarray(colors[0][:, :3]), np.ascontiguousarray(v_colors[0][:, :3]))
    else:
        v_sh = np.zeros((means.shape[0], K, 3), np.float32)  # :625-629
    if scaling_modifier != 1.0:
        v_scales = v_scales * np.float32(scaling_modifier)
    return v_means, v_quats, v_scales, v_opac, v_sh


def activate_params(opacity_raw, scaling_raw, rotation_raw):
    """src/core/splat_data.cpp:271-286 -> (opacities [N], scales [N,3], quats [N,4])"""
    o, sc, r = _f32(opacity_raw).reshape(-1), _f32(scaling_raw), _f32(rotation_raw)
    N = o.shape[0]
    op, scales, quats = np.zeros(N, np.float32), np.zeros((N, 3), np.float32), np.zeros((N, 4), np.float32)
    _chk(lib().orc_activate_params(c_u32(N), _p(o), _p(sc), _p(r), _p(op), _p(scales), _p(quats)), "activate_params")
    return op, scales, quats


def activate_params_bwd(opacity_raw, scaling_raw, rotation_raw, v_opacities, v_scales, v_quats):
    o, sc, r = _f32(opacity_raw).reshape(-1), _f32(scaling_raw), _f32(rotation_raw)
    N = o.shape[0]
    vo, vs, vr = np.zeros(N, np.float32), np.zeros((N, 3), np.float32), np.zeros((N, 4), np.float32)
    g_o, g_s, g_q = _f32(v_opacities).reshape(-1), _f32(v_scales), _f32(v_quats)
    _chk(lib().orc_activate_params_bwd(c_u32(N), _p(o), _p(sc), _p(r), _p(g_o), _p(g_s), _p(g_q), _p(vo), _p(vs),
                                       _p(vr)),
         "activate_params_bwd")
    return vo, vs, vr


def l1_regularization(mode, params, grads, weight):
    """regularization.cu:20-90: mode "exp" (scaling_raw) or "sigmoid" (opacity_raw); grads (float32 array of the same
    size, or None) is updated in place; returns the loss value weight * mean(f(params))."""
    x = _f32(params).reshape(-1)
    if grads is not None:
        assert grads.dtype == np.float32 and grads.flags.c_contiguous and grads.size == x.size
    f = lib().orc_l1_regularization
    f.restype = ctypes.c_double
    return float(f(c_i(0 if mode == "exp" else 1), _p(x), _p(grads) if grads is not None else None,
                   ctypes.c_int64(x.size), ctypes.c_float(weight)))


def photometric_loss(render_hwc, gt_chw, lambda_dssim, with_grad=True):
    """trainer.cpp:126-129 on clamp(render) -> (loss, l1, ssim, image [3,H,W], v_render [H,W,3] or None)"""
    render_hwc, gt_chw = _f32(render_hwc), _f32(gt_chw)
    H, W = render_hwc.shape[0], render_hwc.shape[1]
    image = np.zeros((3, H, W), np.float32)
    out = np.zeros(3, np.float64)
    v = np.zeros((H, W, 3), np.float32) if with_grad else None
    _chk(lib().orc_photometric_loss(c_u32(H), c_u32(W), c_f(lambda_dssim), _p(render_hwc), _p(gt_chw), _p(image),
                                    _p(out), _p(v)), "photometric_loss")
    return float(out[0]), float(out[1]), float(out[2]), image, v


def math_unary(which, x):
    names = {"exp": 0, "log": 1, "rsqrt": 2, "sin": 3, "acos": 4, "sigmoid": 5, "sat_u32": 6}
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_math_unary(c_i(names[which]), c_i64(x.size), _p(x), _p(y))
    return y


def math_pow(x, e):
    x, e = _f32(x), _f32(e)
    y = np.empty_like(x)
    lib().orc_math_pow(c_i64(x.size), _p(x), _p(e), _p(y))
    return y


def math_binary(which, x, x2):
    names = {"pow": 7, "div": 8, "sqrt": 9, "fma": 10, "min_limit": 15}
    x, x2 = _f32(x), _f32(x2)
    y = np.empty_like(x)
    lib().orc_math_binary(c_i(names[which]), c_i64(x.size), _p(x), _p(x2), _p(y))
    return y


def math_quat(which, inp, n_out):
    names = {"quat_cast": 0, "mat3_cast": 1, "quat_to_rotmat": 2, "quat_rotate": 3, "slerp": 4}
    inp = _f32(inp).ravel()
    out = np.zeros((n_out,), np.float32)
    lib().orc_math_quat(c_i(names[which]), _p(inp), _p(out))
    return out


def record_bounds_check(means, quats, scales, opacities, viewmat, K, W, H):
    """Per-Gaussian contribution region of the rasterizers (csrc/gsx_record.h: pixel bounds, power cut-off, ellipse
    test per 8x8 block) against a brute-force pass over every pixel of the image -> (bounds [N,4] = jmin, imin, jmax,
    imax; true_count [N] pixels with alpha >= 1/255; violations [N] = contributing pixels outside the bounds or below
    the cut-off + contributing blocks the block test rejects; blocks_true [N]; blocks_hit [N])."""
    means, quats, scales, opacities = _f32(means), _f32(quats), _f32(scales), _f32(opacities)
    viewmat, K = _f32(viewmat), _f32(K)
    N = means.shape[0]
    bounds = np.zeros((N, 4), np.int32)
    cnt, bad, bt, bh = (np.zeros(N, np.int64) for _ in range(4))
    _chk(lib().orc_record_bounds_check(c_u32(N), _p(means), _p(quats), _p(scales), _p(opacities), _p(viewmat), _p(K),
                                       c_u32(W), c_u32(H), _p(bounds), _p(cnt), _p(bad), _p(bt), _p(bh)),
         "record_bounds_check")
    return bounds, cnt, bad, bt, bh
