"""Host-side mirror of the reference's operator interface (gsplat/Ops.h:9-272, include/kernels/ssim.cuh,
fastgs/optimizer adam_step) over torch tensors: same function names, argument order and meaning, same error
behaviour (non-device or non-contiguous tensors raise, zero-size inputs return without launching), outputs
freshly allocated like the reference's at::empty / at::zeros.  Every function calls the C ABI of libgsx.so on
torch's current stream; torch is only used for device memory and streams.
"""
import ctypes

import torch

from . import _lib as L
from ._lib import UTParams, c_f, c_i, c_i64, c_p, c_sz, c_u32, check, lib

CameraModelType = type("CameraModelType", (), dict(PINHOLE=0, ORTHO=1, FISHEYE=2, EQUIRECTANGULAR=3))
ShutterType = type("ShutterType", (), dict(ROLLING_TOP_TO_BOTTOM=0, ROLLING_LEFT_TO_RIGHT=1, ROLLING_BOTTOM_TO_TOP=2,
                                           ROLLING_RIGHT_TO_LEFT=3, GLOBAL=4))
UnscentedTransformParameters = UTParams
ALPHA_THRESHOLD = 1.0 / 255.0


def _check_input(x, name):
    """CHECK_INPUT of gsplat/Common.h:12-17"""
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _ptr(x):
    return c_p(None) if x is None else c_p(x.data_ptr())


def _stream(dev):
    return c_p(torch.cuda.current_stream(dev).cuda_stream)


def _workspace(nbytes, dev):
    return torch.empty((max(int(nbytes), 256),), dtype=torch.uint8, device=dev)


def _f32(x, name):
    _check_input(x, name)
    if x.dtype != torch.float32:
        raise RuntimeError(f"{name} must be float32")
    return x


def _sized(x, name, *shape):
    """The kernels index by these extents: a tensor of another shape would be read or written out of bounds.  None
    in `shape` leaves that extent free; a None tensor passes."""
    if x is None:
        return
    if x.dim() != len(shape) or any(s is not None and int(d) != int(s) for d, s in zip(x.shape, shape)):
        want = ", ".join("*" if s is None else str(int(s)) for s in shape)
        raise RuntimeError(f"{name} must be [{want}], got {tuple(x.shape)}")


def _check_camera_tensors(C, camera_model, viewmats0, viewmats1, Ks, radial_coeffs, tangential_coeffs,
                          thin_prism_coeffs):
    """[C,4,4] poses, [C,3,3] intrinsics; coefficient rows as the kernels read them (ProjectionUT3DGSFused.cu:101-
    126): radial [C,6] (pinhole) or [C,4] (fisheye), tangential [C,2], thin prism [C,4]"""
    _sized(viewmats0, "viewmats0", C, 4, 4), _sized(viewmats1, "viewmats1", C, 4, 4), _sized(Ks, "Ks", C, 3, 3)
    _sized(radial_coeffs, "radial_coeffs", C, 4 if camera_model == CameraModelType.FISHEYE else 6)
    _sized(tangential_coeffs, "tangential_coeffs", C, 2), _sized(thin_prism_coeffs, "thin_prism_coeffs", C, 4)


# ------------------------------------------------------------------------------------------------
def spherical_harmonics_fwd(degrees_to_use, dirs, coeffs, masks=None):
    """Ops.h:12-17"""
    _f32(dirs, "dirs"), _f32(coeffs, "coeffs")
    if masks is not None:
        _check_input(masks, "masks")
    if coeffs.size(-1) != 3:
        raise RuntimeError("coeffs must have last dimension 3")  # SphericalHarmonics.cpp:27
    if dirs.size(-1) != 3:
        raise RuntimeError("dirs must have last dimension 3")
    K = coeffs.size(-2)
    N = dirs.numel() // 3
    if coeffs.numel() != N * K * 3 or (masks is not None and masks.numel() != N):
        raise RuntimeError(f"coeffs must be [..., K, 3] and masks [...] over the {N} directions, got "
                           f"{tuple(coeffs.shape)}" + ("" if masks is None else f" / {tuple(masks.shape)}"))
    colors = torch.empty_like(dirs)
    m8 = None if masks is None else masks.view(torch.uint8) if masks.dtype == torch.bool else masks
    with torch.cuda.device(dirs.device):
        check(lib().gsx_spherical_harmonics_fwd(c_u32(N), c_u32(K), c_u32(degrees_to_use), _ptr(dirs), _ptr(coeffs),
                                                _ptr(m8), _ptr(colors), _stream(dirs.device)))
    return colors


def spherical_harmonics_bwd(K, degrees_to_use, dirs, coeffs, masks, v_colors, compute_v_dirs):
    """Ops.h:18-25 -> (v_coeffs, v_dirs or None)"""
    _f32(dirs, "dirs"), _f32(coeffs, "coeffs"), _f32(v_colors, "v_colors")
    if masks is not None:
        _check_input(masks, "masks")
    if v_colors.size(-1) != 3 or coeffs.size(-1) != 3 or dirs.size(-1) != 3:
        raise RuntimeError("last dimension must be 3")
    N = dirs.numel() // 3
    if coeffs.size(-2) != K or coeffs.numel() != N * K * 3 or v_colors.numel() != N * 3 or \
            (masks is not None and masks.numel() != N):
        raise RuntimeError(f"coeffs must be [..., {K}, 3], v_colors [..., 3] and masks [...] over the {N} directions")
    v_coeffs = torch.empty_like(coeffs)
    v_dirs = torch.empty_like(dirs) if compute_v_dirs else None
    m8 = None if masks is None else masks.view(torch.uint8) if masks.dtype == torch.bool else masks
    with torch.cuda.device(dirs.device):
        check(lib().gsx_spherical_harmonics_bwd(c_u32(N), c_u32(K), c_u32(degrees_to_use), _ptr(dirs), _ptr(coeffs),
                                                _ptr(m8), _ptr(v_colors), _ptr(v_coeffs), _ptr(v_dirs),
                                                _stream(dirs.device)))
    return v_coeffs, v_dirs


def intersect_tile(means2d, radii, depths, camera_ids, gaussian_ids, C, tile_size, tile_width, tile_height,
                   sort=True):
    """Ops.h:28-38 -> (tiles_per_gauss [C,N] i32, isect_ids [I] i64, flatten_ids [I] i32)"""
    _f32(means2d, "means2d"), _check_input(radii, "radii"), _f32(depths, "depths")
    if radii.dtype != torch.int32:
        raise RuntimeError("radii must be int32")
    if means2d.dim() == 2:
        if camera_ids is None or gaussian_ids is None:  # Intersect.cpp:34-36
            raise RuntimeError("When packed is set, camera_ids and gaussian_ids must be provided.")
        return _intersect_tile_packed(means2d, radii, depths, camera_ids, gaussian_ids, C, tile_size, tile_width,
                                      tile_height, sort)
    dev = means2d.device
    N = means2d.size(1)
    _sized(means2d, "means2d", C, N, 2), _sized(radii, "radii", C, N, 2), _sized(depths, "depths", C, N)
    tiles_per_gauss = torch.empty_like(depths, dtype=torch.int32)
    n_isects = c_i64(0)
    # sort == True with one camera: depth order first, then a sort on the tile bits only (same result as the
    # reference's single sort on every bit, Intersect.cpp:104-113; see gsx.h)
    two_level = bool(sort) and C == 1
    with torch.cuda.device(dev):
        order = None
        cum = torch.empty((C * N,), dtype=torch.int64, device=dev)
        if two_level:
            order = torch.empty((N,), dtype=torch.int32, device=dev)
            ws = _workspace(lib().gsx_intersect_tile_count_ordered_workspace_bytes(c_u32(N)), dev)
            check(lib().gsx_intersect_tile_count_ordered(
                c_u32(N), _ptr(means2d), _ptr(radii), _ptr(depths), c_u32(tile_size), c_u32(tile_width),
                c_u32(tile_height), _ptr(order), _ptr(tiles_per_gauss), _ptr(cum), _ptr(ws), c_sz(ws.numel()),
                ctypes.byref(n_isects), c_i(1), _stream(dev)))
        else:
            ws = _workspace(lib().gsx_intersect_tile_count_workspace_bytes(c_u32(C), c_u32(N)), dev)
            check(lib().gsx_intersect_tile_count(c_u32(C), c_u32(N), _ptr(means2d), _ptr(radii), c_u32(tile_size),
                                                 c_u32(tile_width), c_u32(tile_height), _ptr(tiles_per_gauss),
                                                 _ptr(cum), _ptr(ws), c_sz(ws.numel()), ctypes.byref(n_isects),
                                                 _stream(dev)))
        n = n_isects.value
        isect_ids = torch.empty((n,), dtype=torch.int64, device=dev)
        flatten_ids = torch.empty((n,), dtype=torch.int32, device=dev)
        if n and two_level:  # ws still holds the sorted depth keys (with the tile rectangles) the emission reads
            check(lib().gsx_intersect_tile_emit_ordered(
                c_u32(N), _ptr(means2d), _ptr(radii), _ptr(depths), _ptr(cum), _ptr(order), _ptr(ws),
                c_u32(tile_size), c_u32(tile_width), c_u32(tile_height), c_i64((1 << 63) - 1), _ptr(isect_ids),
                _ptr(flatten_ids), _stream(dev)))
        elif n:
            check(lib().gsx_intersect_tile_emit(c_u32(C), c_u32(N), _ptr(means2d), _ptr(radii), _ptr(depths),
                                                _ptr(cum), _ptr(order), c_u32(tile_size), c_u32(tile_width),
                                                c_u32(tile_height), _ptr(isect_ids), _ptr(flatten_ids),
                                                _stream(dev)))
        if n and sort:
            tile_n_bits = lib().gsx_n_bits(c_u32(tile_width * tile_height))
            cam_n_bits = lib().gsx_n_bits(c_u32(C))
            isect_ids, flatten_ids = radix_sort_double_buffer(n, tile_n_bits, cam_n_bits, isect_ids, flatten_ids,
                                                              begin_bit=32 if two_level else 0)
    return tiles_per_gauss, isect_ids, flatten_ids


def _intersect_tile_packed(means2d, radii, depths, camera_ids, gaussian_ids, C, tile_size, tile_width, tile_height,
                           sort):
    """packed rows [nnz] (Intersect.cpp:32-39): the count of one camera with nnz rows, the emission with each row's
    camera from camera_ids (IntersectTile.cu:86-94), the reference's one sort over all bits"""
    _check_input(camera_ids, "camera_ids"), _check_input(gaussian_ids, "gaussian_ids")
    if camera_ids.dtype != torch.int64 or gaussian_ids.dtype != torch.int64:
        raise RuntimeError("camera_ids and gaussian_ids must be int64")
    dev = means2d.device
    nnz = means2d.size(0)
    _sized(means2d, "means2d", nnz, 2), _sized(radii, "radii", nnz, 2), _sized(depths, "depths", nnz)
    _sized(camera_ids, "camera_ids", nnz), _sized(gaussian_ids, "gaussian_ids", nnz)
    tiles_per_gauss = torch.empty_like(depths, dtype=torch.int32)
    n_isects = c_i64(0)
    with torch.cuda.device(dev):
        cum = torch.empty((nnz,), dtype=torch.int64, device=dev)
        ws = _workspace(lib().gsx_intersect_tile_count_workspace_bytes(c_u32(1), c_u32(nnz)), dev)
        check(lib().gsx_intersect_tile_count(c_u32(1), c_u32(nnz), _ptr(means2d), _ptr(radii), c_u32(tile_size),
                                             c_u32(tile_width), c_u32(tile_height), _ptr(tiles_per_gauss), _ptr(cum),
                                             _ptr(ws), c_sz(ws.numel()), ctypes.byref(n_isects), _stream(dev)))
        n = n_isects.value
        isect_ids = torch.empty((n,), dtype=torch.int64, device=dev)
        flatten_ids = torch.empty((n,), dtype=torch.int32, device=dev)
        if n:
            check(lib().gsx_intersect_tile_emit_packed(
                c_u32(C), c_u32(nnz), _ptr(means2d), _ptr(radii), _ptr(depths), _ptr(camera_ids), _ptr(cum),
                c_u32(tile_size), c_u32(tile_width), c_u32(tile_height), _ptr(isect_ids), _ptr(flatten_ids),
                _stream(dev)))
        if n and sort:
            tile_n_bits = lib().gsx_n_bits(c_u32(tile_width * tile_height))
            cam_n_bits = lib().gsx_n_bits(c_u32(C))
            isect_ids, flatten_ids = radix_sort_double_buffer(n, tile_n_bits, cam_n_bits, isect_ids, flatten_ids)
    return tiles_per_gauss, isect_ids, flatten_ids


def _tile_lists(means2d, radii, depths, tile_size, tile_width, tile_height):
    """(flatten_ids [I] i32, offsets [1,Th,Tw] i32) of one camera, as intersect_tile(sort=True) + intersect_offset
    return them, without forming the 64-bit keys: pairs in depth order with their 16-bit tile index as the sort key
    (for a caller that keeps no isect_ids: Rasterization.cpp:413-424).  None where the grid needs the 64-bit keys."""
    if means2d.size(0) != 1 or not lib().gsx_intersect_tile_pairs_fit(c_u32(tile_width), c_u32(tile_height)):
        return None
    dev = means2d.device
    N = means2d.size(1)
    _sized(means2d, "means2d", 1, N, 2), _sized(radii, "radii", 1, N, 2), _sized(depths, "depths", 1, N)
    if radii.dtype != torch.int32:
        raise RuntimeError("radii must be int32")
    offsets = torch.empty((1, tile_height, tile_width), dtype=torch.int32, device=dev)
    n_isects = c_i64(0)
    with torch.cuda.device(dev):
        st = _stream(dev)
        order = torch.empty((N,), dtype=torch.int32, device=dev)
        tiles_per_gauss = torch.empty((N,), dtype=torch.int32, device=dev)
        cum = torch.empty((N,), dtype=torch.int64, device=dev)
        ws = _workspace(lib().gsx_intersect_tile_count_ordered_workspace_bytes(c_u32(N)), dev)
        check(lib().gsx_intersect_tile_count_ordered(
            c_u32(N), _ptr(means2d), _ptr(radii), _ptr(depths), c_u32(tile_size), c_u32(tile_width),
            c_u32(tile_height), _ptr(order), _ptr(tiles_per_gauss), _ptr(cum), _ptr(ws), c_sz(ws.numel()),
            ctypes.byref(n_isects), c_i(1), st))
        n = n_isects.value if N else 0
        keys = [torch.empty((n,), dtype=torch.int16, device=dev) for _ in range(2)]
        vals = [torch.empty((n,), dtype=torch.int32, device=dev) for _ in range(2)]
        sel = c_i(0)
        if n:
            check(lib().gsx_intersect_tile_emit_pairs(
                c_u32(N), _ptr(cum), _ptr(order), _ptr(ws), c_u32(tile_size), c_u32(tile_width), c_u32(tile_height),
                c_i64(n), _ptr(keys[0]), _ptr(vals[0]), st))
            ws2 = _workspace(lib().gsx_radix_sort_pairs_workspace_bytes(c_i64(n)), dev)
            check(lib().gsx_radix_sort_tile_pairs(
                c_i64(n), _ptr(keys[0]), _ptr(vals[0]), _ptr(keys[1]), _ptr(vals[1]),
                c_u32(lib().gsx_n_bits(c_u32(tile_width * tile_height))), _ptr(ws2), c_sz(ws2.numel()),
                ctypes.byref(sel), st))
        check(lib().gsx_intersect_tile_pairs_offset(c_i64(n), _ptr(keys[sel.value]), c_u32(tile_width),
                                                    c_u32(tile_height), _ptr(offsets), st))
    return vals[sel.value], offsets


def radix_sort_double_buffer(n_isects, tile_n_bits, cam_n_bits, isect_ids, flatten_ids, begin_bit=0):
    """Intersect.h:39-46.  Returns the sorted (isect_ids, flatten_ids); like the reference's DoubleBuffer the
    result may live in either the input tensors or the internally allocated pair.  begin_bit > 0 sorts on the
    key bits from there up only (stable)."""
    _check_input(isect_ids, "isect_ids"), _check_input(flatten_ids, "flatten_ids")
    if n_isects <= 0:
        return isect_ids, flatten_ids
    if isect_ids.dtype != torch.int64 or flatten_ids.dtype != torch.int32 or isect_ids.numel() < n_isects or \
            flatten_ids.numel() < n_isects:
        raise RuntimeError(f"isect_ids (int64) and flatten_ids (int32) must hold {n_isects} entries")
    dev = isect_ids.device
    with torch.cuda.device(dev):
        k1, v1 = torch.empty_like(isect_ids), torch.empty_like(flatten_ids)
        ws = _workspace(lib().gsx_radix_sort_pairs_workspace_bytes(c_i64(n_isects)), dev)
        sel = c_i(0)
        check(lib().gsx_radix_sort_pairs(c_i64(n_isects), _ptr(isect_ids), _ptr(flatten_ids), _ptr(k1), _ptr(v1),
                                         c_u32(begin_bit), c_u32(32 + tile_n_bits + cam_n_bits), _ptr(ws),
                                         c_sz(ws.numel()),
                                         ctypes.byref(sel), _stream(dev)))
    return (k1, v1) if sel.value else (isect_ids, flatten_ids)


def intersect_offset(isect_ids, C, tile_width, tile_height):
    """Ops.h:39-43 -> offsets [C, tile_height, tile_width] i32"""
    _check_input(isect_ids, "isect_ids")
    if isect_ids.dtype != torch.int64:
        raise RuntimeError("isect_ids must be int64")
    dev = isect_ids.device
    offsets = torch.empty((C, tile_height, tile_width), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        check(lib().gsx_intersect_offset(c_i64(isect_ids.numel()), _ptr(isect_ids), c_u32(C), c_u32(tile_width),
                                         c_u32(tile_height), _ptr(offsets), _stream(dev)))
    return offsets


def quats_to_rotmats(quats):
    """Ops.h:46-48"""
    _f32(quats, "quats")
    N = quats.size(0)
    _sized(quats, "quats", N, 4)
    out = torch.empty((N, 3, 3), dtype=quats.dtype, device=quats.device)
    with torch.cuda.device(quats.device):
        check(lib().gsx_quats_to_rotmats(c_i(N), _ptr(quats), _ptr(out), _stream(quats.device)))
    return out


def relocation(opacities, scales, ratios, binoms, n_max):
    """Ops.h:52-57 -> (new_opacities, new_scales)"""
    _f32(opacities, "opacities"), _f32(scales, "scales"), _check_input(ratios, "ratios"), _f32(binoms, "binoms")
    if ratios.dtype != torch.int32:
        raise RuntimeError("ratios must be int32")
    n = opacities.size(0)
    _sized(opacities, "opacities", n), _sized(scales, "scales", n, 3), _sized(ratios, "ratios", n)
    _sized(binoms, "binoms", n_max, n_max)
    new_opacities, new_scales = torch.empty_like(opacities), torch.empty_like(scales)
    with torch.cuda.device(opacities.device):
        check(lib().gsx_relocation(c_i(opacities.size(0)), _ptr(opacities), _ptr(scales), _ptr(ratios), _ptr(binoms),
                                   c_i(n_max), _ptr(new_opacities), _ptr(new_scales), _stream(opacities.device)))
    return new_opacities, new_scales


def add_noise(raw_opacities, raw_scales, raw_quats, noise, means, current_lr):
    """Ops.h:59-65; means is modified in place"""
    for t, n in ((raw_opacities, "raw_opacities"), (raw_scales, "raw_scales"), (raw_quats, "raw_quats"),
                 (noise, "noise"), (means, "means")):
        _f32(t, n)
    n = means.size(0)
    _sized(means, "means", n, 3), _sized(noise, "noise", n, 3), _sized(raw_quats, "raw_quats", n, 4)
    _sized(raw_scales, "raw_scales", n, 3)
    if raw_opacities.numel() != n:
        raise RuntimeError(f"raw_opacities must hold {n} values, got {tuple(raw_opacities.shape)}")
    with torch.cuda.device(means.device):
        check(lib().gsx_add_noise(c_i(means.size(0)), _ptr(raw_opacities), _ptr(raw_scales), _ptr(raw_quats),
                                  _ptr(noise), _ptr(means), c_f(current_lr), _stream(means.device)))


def projection_ut_3dgs_fused(means, quats, scales, opacities, viewmats0, viewmats1, Ks, image_width, image_height,
                             eps2d, near_plane, far_plane, radius_clip, calc_compensations, camera_model, ut_params,
                             rs_type, radial_coeffs=None, tangential_coeffs=None, thin_prism_coeffs=None):
    """Ops.h:69-98 -> (radii [C,N,2] i32, means2d [C,N,2], depths [C,N], conics [C,N,3], compensations [C,N] or
    None).  Rows of culled Gaussians hold unspecified values except radii == 0 (Projection.cpp:70-73 at::empty)."""
    _f32(means, "means"), _f32(quats, "quats"), _f32(scales, "scales")
    if opacities is not None:
        _f32(opacities, "opacities")
    _f32(viewmats0, "viewmats0"), _f32(Ks, "Ks")
    for t, n in ((viewmats1, "viewmats1"), (radial_coeffs, "radial_coeffs"), (tangential_coeffs, "tangential_coeffs"),
                 (thin_prism_coeffs, "thin_prism_coeffs")):
        if t is not None:
            _f32(t, n)
    dev = means.device
    N, C = means.size(0), viewmats0.size(0)
    _sized(means, "means", N, 3), _sized(quats, "quats", N, 4), _sized(scales, "scales", N, 3)
    _sized(opacities, "opacities", N)
    _check_camera_tensors(C, camera_model, viewmats0, viewmats1, Ks, radial_coeffs, tangential_coeffs,
                          thin_prism_coeffs)
    radii = torch.empty((C, N, 2), dtype=torch.int32, device=dev)
    means2d = torch.empty((C, N, 2), dtype=torch.float32, device=dev)
    depths = torch.empty((C, N), dtype=torch.float32, device=dev)
    conics = torch.empty((C, N, 3), dtype=torch.float32, device=dev)
    comp = torch.zeros((C, N), dtype=torch.float32, device=dev) if calc_compensations else None
    with torch.cuda.device(dev):
        check(lib().gsx_projection_ut_3dgs_fused(
            c_u32(C), c_u32(N), _ptr(means), _ptr(quats), _ptr(scales), _ptr(opacities), _ptr(viewmats0),
            _ptr(viewmats1), _ptr(Ks), c_u32(image_width), c_u32(image_height), c_f(eps2d), c_f(near_plane),
            c_f(far_plane), c_f(radius_clip), c_i(camera_model), ut_params, c_i(rs_type), _ptr(radial_coeffs),
            _ptr(tangential_coeffs), _ptr(thin_prism_coeffs), _ptr(radii), _ptr(means2d), _ptr(depths), _ptr(conics),
            _ptr(comp), _stream(dev)))
    return radii, means2d, depths, conics, comp


# colour channel counts the rasterizers are built for (gsplat/Rasterization.cpp:106-128 lists up to 513)
RASTER_CHANNELS = (1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 64, 65, 128, 129, 256, 257, 512, 513)


def _fit_backgrounds(backgrounds, channels):
    """The fused operators hand the caller's background ([C,3] from gs::training::rasterize, rasterizer.cpp:84-87,
    147) to a kernel that blends `channels` values per pixel (Rasterization.cpp:401-407): with RGB + depth it would
    read one float past each row.  Here the missing channels' background is 0 and surplus ones are dropped (for one
    camera the values the reference's kernel reads)."""
    if backgrounds is None or backgrounds.numel() == 0:
        return None
    have = backgrounds.size(-1)
    if have > channels:
        return backgrounds[..., :channels].contiguous()
    if have < channels:
        pad = torch.zeros(backgrounds.shape[:-1] + (channels - have,), dtype=backgrounds.dtype,
                          device=backgrounds.device)
        return torch.cat([backgrounds, pad], -1).contiguous()
    return backgrounds


def _check_backgrounds(backgrounds, C, channels):
    if backgrounds is not None and tuple(backgrounds.shape) != (C, channels):
        raise RuntimeError(f"backgrounds must be [C, channels] = [{C}, {channels}], got {tuple(backgrounds.shape)}")


def rasterize_to_pixels_from_world_3dgs_fwd(means, quats, scales, colors, opacities, backgrounds, masks, image_width,
                                            image_height, tile_size, viewmats0, viewmats1, Ks, camera_model,
                                            ut_params, rs_type, radial_coeffs, tangential_coeffs, thin_prism_coeffs,
                                            tile_offsets, flatten_ids):
    """Ops.h:100-129 -> (renders [C,H,W,channels], alphas [C,H,W,1], last_ids [C,H,W] i32)"""
    for t, n in ((means, "means"), (quats, "quats"), (scales, "scales"), (colors, "colors"),
                 (opacities, "opacities"), (viewmats0, "viewmats0"), (Ks, "Ks")):
        _f32(t, n)
    _check_input(tile_offsets, "tile_offsets"), _check_input(flatten_ids, "flatten_ids")
    if backgrounds is not None and backgrounds.numel() == 0:
        backgrounds = None
    if backgrounds is not None:
        _f32(backgrounds, "backgrounds")
    if masks is not None:
        _check_input(masks, "masks")
    dev = means.device
    C, N = tile_offsets.size(0), means.size(0)
    channels = colors.size(-1)
    _check_backgrounds(backgrounds, C, channels)
    th, tw = (image_height + tile_size - 1) // tile_size, (image_width + tile_size - 1) // tile_size
    _sized(means, "means", N, 3), _sized(quats, "quats", N, 4), _sized(scales, "scales", N, 3)
    _sized(colors, "colors", C, N, channels), _sized(opacities, "opacities", C, N)
    _sized(tile_offsets, "tile_offsets", C, th, tw), _sized(masks, "masks", C, th, tw)
    _check_camera_tensors(C, camera_model, viewmats0, viewmats1, Ks, radial_coeffs, tangential_coeffs,
                          thin_prism_coeffs)
    if tile_offsets.dtype != torch.int32 or flatten_ids.dtype != torch.int32:
        raise RuntimeError("tile_offsets and flatten_ids must be int32")
    renders = torch.empty((C, image_height, image_width, channels), dtype=torch.float32, device=dev)
    alphas = torch.empty((C, image_height, image_width, 1), dtype=torch.float32, device=dev)
    last_ids = torch.empty((C, image_height, image_width), dtype=torch.int32, device=dev)
    m8 = None if masks is None else masks.view(torch.uint8) if masks.dtype == torch.bool else masks
    with torch.cuda.device(dev):
        ws = _workspace(lib().gsx_raster_records_bytes(c_u32(N)) + lib().gsx_tile_order_bytes(c_u32(tw), c_u32(th)),
                        dev)  # records + room for the tile visiting order
        check(lib().gsx_rasterize_to_pixels_from_world_3dgs_fwd(
            c_u32(C), c_u32(N), c_i64(flatten_ids.numel()), _ptr(means), _ptr(quats), _ptr(scales), _ptr(colors),
            c_u32(channels), _ptr(opacities), _ptr(backgrounds), _ptr(m8), c_u32(image_width), c_u32(image_height),
            c_u32(tile_size), _ptr(viewmats0), _ptr(viewmats1), _ptr(Ks), c_i(camera_model), ut_params, c_i(rs_type),
            _ptr(radial_coeffs), _ptr(tangential_coeffs), _ptr(thin_prism_coeffs), _ptr(tile_offsets),
            _ptr(flatten_ids), _ptr(renders), _ptr(alphas), _ptr(last_ids), _ptr(ws), c_sz(ws.numel()),
            _stream(dev)))
    return renders, alphas, last_ids


def rasterize_to_pixels_from_world_3dgs_bwd(means, quats, scales, colors, opacities, backgrounds, masks, image_width,
                                            image_height, tile_size, viewmats0, viewmats1, Ks, camera_model,
                                            ut_params, rs_type, radial_coeffs, tangential_coeffs, thin_prism_coeffs,
                                            tile_offsets, flatten_ids, render_alphas, last_ids, v_render_colors,
                                            v_render_alphas):
    """Ops.h:131-166 -> (v_means [N,3], v_quats [N,4], v_scales [N,3], v_colors [C,N,3], v_opacities [C,N])"""
    for t, n in ((means, "means"), (quats, "quats"), (scales, "scales"), (colors, "colors"),
                 (opacities, "opacities"), (viewmats0, "viewmats0"), (Ks, "Ks"), (render_alphas, "render_alphas"),
                 (v_render_colors, "v_render_colors"), (v_render_alphas, "v_render_alphas")):
        _f32(t, n)
    _check_input(tile_offsets, "tile_offsets"), _check_input(flatten_ids, "flatten_ids")
    _check_input(last_ids, "last_ids")
    if colors.size(-1) not in RASTER_CHANNELS:
        raise RuntimeError("Unsupported number of channels: %d (built: %s)" % (colors.size(-1), RASTER_CHANNELS))
    if backgrounds is not None and backgrounds.numel() == 0:
        backgrounds = None
    dev = means.device
    C, N = tile_offsets.size(0), means.size(0)
    channels = colors.size(-1)
    _check_backgrounds(backgrounds, C, channels)
    th, tw = (image_height + tile_size - 1) // tile_size, (image_width + tile_size - 1) // tile_size
    _sized(means, "means", N, 3), _sized(quats, "quats", N, 4), _sized(scales, "scales", N, 3)
    _sized(colors, "colors", C, N, channels), _sized(opacities, "opacities", C, N)
    _sized(tile_offsets, "tile_offsets", C, th, tw), _sized(masks, "masks", C, th, tw)
    _sized(render_alphas, "render_alphas", C, image_height, image_width, 1)
    _sized(last_ids, "last_ids", C, image_height, image_width)
    _sized(v_render_colors, "v_render_colors", C, image_height, image_width, channels)
    _sized(v_render_alphas, "v_render_alphas", C, image_height, image_width, 1)
    _check_camera_tensors(C, camera_model, viewmats0, viewmats1, Ks, radial_coeffs, tangential_coeffs,
                          thin_prism_coeffs)
    if tile_offsets.dtype != torch.int32 or flatten_ids.dtype != torch.int32 or last_ids.dtype != torch.int32:
        raise RuntimeError("tile_offsets, flatten_ids and last_ids must be int32")
    v_means, v_quats, v_scales = torch.empty_like(means), torch.empty_like(quats), torch.empty_like(scales)
    v_colors, v_opacities = torch.empty_like(colors), torch.empty_like(opacities)
    m8 = None if masks is None else masks.view(torch.uint8) if masks.dtype == torch.bool else masks
    with torch.cuda.device(dev):
        ws = _workspace(lib().gsx_rasterize_bwd_workspace_bytes_for(c_u32(N), c_u32(channels)) +
                        lib().gsx_tile_order_bytes(c_u32(tw), c_u32(th)), dev)  # + room for the tile visiting order
        check(lib().gsx_rasterize_to_pixels_from_world_3dgs_bwd(
            c_u32(C), c_u32(N), c_i64(flatten_ids.numel()), _ptr(means), _ptr(quats), _ptr(scales), _ptr(colors),
            c_u32(colors.size(-1)), _ptr(opacities), _ptr(backgrounds), _ptr(m8), c_u32(image_width),
            c_u32(image_height), c_u32(tile_size),
            _ptr(viewmats0), _ptr(viewmats1), _ptr(Ks), c_i(camera_model), ut_params, c_i(rs_type),
            _ptr(radial_coeffs), _ptr(tangential_coeffs), _ptr(thin_prism_coeffs), _ptr(tile_offsets),
            _ptr(flatten_ids), _ptr(render_alphas), _ptr(last_ids), _ptr(v_render_colors), _ptr(v_render_alphas),
            _ptr(v_means), _ptr(v_quats), _ptr(v_scales), _ptr(v_colors), _ptr(v_opacities), _ptr(ws),
            c_sz(ws.numel()), _stream(dev)))
    return v_means, v_quats, v_scales, v_colors, v_opacities


def rasterize_from_world_with_sh_fwd(means, quats, scales, opacities, sh_coeffs, sh_degree, backgrounds, masks,
                                     image_width, image_height, tile_size, viewmats0, viewmats1, Ks, camera_model,
                                     eps2d, near_plane, far_plane, radius_clip, scaling_modifier, calc_compensations,
                                     render_mode, ut_params, rs_type, radial_coeffs=None, tangential_coeffs=None,
                                     thin_prism_coeffs=None, return_isect_ids=False):
    """Ops.h:174-220 (Rasterization.cpp:279-467).  -> (render_colors, render_alphas, radii, means2d, depths, colors,
    tile_offsets, flatten_ids, last_ids, compensations).  render_mode: 0 RGB, 1 / 2 depth (one channel), 3 / 4
    RGB + depth (four channels), as Rasterization.cpp:372-393."""
    for t, n in ((means, "means"), (quats, "quats"), (scales, "scales"), (opacities, "opacities"),
                 (sh_coeffs, "sh_coeffs"), (viewmats0, "viewmats0"), (Ks, "Ks")):
        _f32(t, n)
    if render_mode not in (0, 1, 2, 3, 4):
        raise RuntimeError("render_mode %d: must be 0 (RGB), 1 (D), 2 (ED), 3 (RGB_D) or 4 (RGB_ED)" % render_mode)
    dev = means.device
    N, C = means.size(0), viewmats0.size(0)
    opacities = opacities.reshape(-1)
    scaled_scales = scales if scaling_modifier == 1.0 else scales * scaling_modifier  # Rasterization.cpp:327
    radii, means2d, depths, conics, comp = projection_ut_3dgs_fused(
        means, quats, scaled_scales, opacities, viewmats0, viewmats1, Ks, image_width, image_height, eps2d,
        near_plane, far_plane, radius_clip, calc_compensations, camera_model, ut_params, rs_type, radial_coeffs,
        tangential_coeffs, thin_prism_coeffs)
    _sized(sh_coeffs, "sh_coeffs", N, None, 3)
    K = sh_coeffs.size(1)
    if render_mode in (0, 3, 4):
        colors = torch.empty((C, N, 3), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            check(lib().gsx_sh_colors_from_world(c_u32(N), c_u32(K), c_u32(sh_degree), _ptr(means), _ptr(sh_coeffs),
                                                 _ptr(radii), _ptr(viewmats0), _ptr(colors), _stream(dev)))
        if render_mode != 0:  # RGB + depth (Rasterization.cpp:385-387)
            colors = torch.cat([colors, depths.unsqueeze(-1)], -1).contiguous()
    else:  # depth only (:389-392)
        colors = depths.unsqueeze(-1).contiguous()
    final_opacities = opacities.unsqueeze(0)
    if calc_compensations and comp is not None:
        final_opacities = (final_opacities * comp).contiguous()
    tile_width = (image_width + tile_size - 1) // tile_size
    tile_height = (image_height + tile_size - 1) // tile_size
    lists = None if return_isect_ids else _tile_lists(means2d, radii, depths, tile_size, tile_width, tile_height)
    if lists is not None:
        isect_ids = None
        flatten_ids, offsets = lists
    else:
        _, isect_ids, flatten_ids = intersect_tile(means2d, radii, depths, None, None, C, tile_size, tile_width,
                                                   tile_height, True)
        offsets = intersect_offset(isect_ids, C, tile_width, tile_height)
    renders, alphas, last_ids = rasterize_to_pixels_from_world_3dgs_fwd(
        means, quats, scaled_scales, colors, final_opacities, _fit_backgrounds(backgrounds, colors.size(-1)), masks,
        image_width, image_height, tile_size, viewmats0, viewmats1, Ks, camera_model, ut_params, rs_type, radial_coeffs, tangential_coeffs,
        thin_prism_coeffs, offsets, flatten_ids)
    out = (renders, alphas, radii, means2d, depths, colors, offsets, flatten_ids, last_ids, comp)
    return out + (isect_ids,) if return_isect_ids else out


def rasterize_from_world_with_sh_bwd(means, quats, scales, opacities, sh_coeffs, sh_degree, backgrounds, masks,
                                     image_width, image_height, tile_size, viewmats0, viewmats1, Ks, camera_model,
                                     eps2d, near_plane, far_plane, radius_clip, scaling_modifier, calc_compensations,
                                     render_mode, ut_params, rs_type, radial_coeffs, tangential_coeffs,
                                     thin_prism_coeffs, render_alphas, last_ids, tile_offsets, flatten_ids, colors,
                                     radii, means2d, depths, compensations, v_render_colors, v_render_alphas):
    """Ops.h:222-270 (Rasterization.cpp:469-642) -> (v_means, v_quats, v_scales, v_opacities [C,N], v_sh_coeffs)"""
    for t, n in ((means, "means"), (quats, "quats"), (scales, "scales"), (opacities, "opacities"),
                 (sh_coeffs, "sh_coeffs"), (v_render_colors, "v_render_colors"),
                 (v_render_alphas, "v_render_alphas")):
        _f32(t, n)
    if render_mode not in (0, 1, 2, 3, 4):
        raise RuntimeError("render_mode %d: must be 0 (RGB), 1 (D), 2 (ED), 3 (RGB_D) or 4 (RGB_ED)" % render_mode)
    dev = means.device
    N = means.size(0)
    final_opacities = opacities.reshape(1, -1)
    if calc_compensations and compensations is not None and compensations.numel() > 0:
        final_opacities = (final_opacities * compensations).contiguous()
    scaled_scales = scales if scaling_modifier == 1.0 else scales * scaling_modifier
    v_means, v_quats, v_scales, v_colors, v_opacities = rasterize_to_pixels_from_world_3dgs_bwd(
        means, quats, scaled_scales, colors, final_opacities, _fit_backgrounds(backgrounds, colors.size(-1)), masks,
        image_width, image_height, tile_size, viewmats0, viewmats1, Ks, camera_model, ut_params, rs_type, radial_coeffs, tangential_coeffs,
        thin_prism_coeffs, tile_offsets, flatten_ids, render_alphas, last_ids, v_render_colors, v_render_alphas)
    _sized(sh_coeffs, "sh_coeffs", N, None, 3), _sized(radii, "radii", 1, N, 2)
    K = sh_coeffs.size(1)
    if render_mode in (0, 3, 4):
        rgb, v_rgb = colors, v_colors
        if render_mode != 0:  # the depth channel's gradient is dropped (Rasterization.cpp:587-606)
            rgb, v_rgb = colors[..., :3].contiguous(), v_colors[..., :3].contiguous()
        v_sh = torch.empty_like(sh_coeffs)
        with torch.cuda.device(dev):
            check(lib().gsx_sh_colors_from_world_bwd(c_u32(N), c_u32(K), c_u32(sh_degree), _ptr(means), _ptr(radii),
                                                     _ptr(viewmats0), _ptr(rgb), _ptr(v_rgb), _ptr(v_sh),
                                                     _stream(dev)))
    else:
        v_sh = torch.zeros_like(sh_coeffs)  # :625-629
    if scaling_modifier != 1.0:
        v_scales = v_scales * scaling_modifier  # Rasterization.cpp:633
    return v_means, v_quats, v_scales, v_opacities, v_sh


# ------------------------------------------------------------------------------------------------
def fusedssim(C1, C2, img1, img2, train):
    """include/kernels/ssim.cuh:11-19 -> (ssim_map, dm_dmu1, dm_dsigma1_sq, dm_dsigma12)"""
    _f32(img1, "img1"), _f32(img2, "img2")
    if img1.dim() != 4 or img1.shape != img2.shape:
        raise RuntimeError(f"img1 and img2 must be [B, C, H, W] of one shape, got {tuple(img1.shape)} / "
                           f"{tuple(img2.shape)}")
    B, CH, H, W = img1.shape
    ssim_map = torch.empty_like(img1)
    if train:
        d1, d2, d3 = torch.empty_like(img1), torch.empty_like(img1), torch.empty_like(img1)
    else:
        d1 = d2 = d3 = None
    with torch.cuda.device(img1.device):
        check(lib().gsx_fusedssim(c_i(B), c_i(CH), c_i(H), c_i(W), c_f(C1), c_f(C2), _ptr(img1), _ptr(img2),
                                  _ptr(ssim_map), _ptr(d1), _ptr(d2), _ptr(d3), _stream(img1.device)))
    empty = torch.empty((0,), dtype=img1.dtype, device=img1.device)
    return ssim_map, (d1 if train else empty), (d2 if train else empty), (d3 if train else empty)


def fusedssim_backward(C1, C2, img1, img2, dL_dmap, dm_dmu1, dm_dsigma1_sq, dm_dsigma12):
    """include/kernels/ssim.cuh:21-28 -> dL_dimg1"""
    for t, n in ((img1, "img1"), (img2, "img2"), (dL_dmap, "dL_dmap"), (dm_dmu1, "dm_dmu1"),
                 (dm_dsigma1_sq, "dm_dsigma1_sq"), (dm_dsigma12, "dm_dsigma12")):
        _f32(t, n)
        if t.shape != img1.shape or t.dim() != 4:
            raise RuntimeError(f"{n} must be [B, C, H, W] like img1 {tuple(img1.shape)}, got {tuple(t.shape)}")
    B, CH, H, W = img1.shape
    out = torch.empty_like(img1)
    with torch.cuda.device(img1.device):
        check(lib().gsx_fusedssim_backward(c_i(B), c_i(CH), c_i(H), c_i(W), c_f(C1), c_f(C2), _ptr(img1), _ptr(img2),
                                           _ptr(dL_dmap), _ptr(dm_dmu1), _ptr(dm_dsigma1_sq), _ptr(dm_dsigma12),
                                           _ptr(out), _stream(img1.device)))
    return out


def adam_step(param, exp_avg, exp_avg_sq, param_grad, lr, beta1, beta2, eps, bias_correction1_rcp,
              bias_correction2_sqrt_rcp):
    """fast_gs::optimizer::adam_step_wrapper (fastgs/optimizer/src/adam_api.cu:8-33); in place"""
    for t, n in ((param, "param"), (exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq"), (param_grad, "param_grad")):
        _f32(t, n)
        if t.numel() != param.numel():
            raise RuntimeError(f"{n} must hold {param.numel()} elements like param, got {t.numel()}")
    with torch.cuda.device(param.device):
        check(lib().gsx_adam_step(_ptr(param), _ptr(exp_avg), _ptr(exp_avg_sq), _ptr(param_grad),
                                  c_i64(param.numel()), c_f(lr), c_f(beta1), c_f(beta2), c_f(eps),
                                  c_f(bias_correction1_rcp), c_f(bias_correction2_sqrt_rcp), _stream(param.device)))


def adam_step_multi(groups):
    """All parameter groups of one optimiser step in a single launch.  groups: list of dicts with the keyword
    arguments of adam_step (tensors may be None / grad None to skip)."""
    if not groups:
        return
    arr = (L.AdamGroup * len(groups))()
    dev = None
    for i, g in enumerate(groups):
        p = g["param"]
        dev = p.device
        for n in ("param", "exp_avg", "exp_avg_sq"):
            _f32(g[n], n)
        grad = g.get("param_grad")
        if grad is not None:
            _f32(grad, "param_grad")
        for n, t in (("exp_avg", g["exp_avg"]), ("exp_avg_sq", g["exp_avg_sq"]), ("param_grad", grad)):
            if t is not None and t.numel() != p.numel():
                raise RuntimeError(f"group {i}: {n} must hold {p.numel()} elements like param, got {t.numel()}")
        arr[i] = L.AdamGroup(p.data_ptr(), g["exp_avg"].data_ptr(), g["exp_avg_sq"].data_ptr(),
                             None if grad is None else grad.data_ptr(), p.numel(), g["lr"], g["beta1"], g["beta2"],
                             g["eps"], g["bias_correction1_rcp"], g["bias_correction2_sqrt_rcp"])
    with torch.cuda.device(dev):
        check(lib().gsx_adam_step_multi(arr, c_i(len(groups)), _stream(dev)))
