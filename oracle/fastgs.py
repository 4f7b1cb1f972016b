"""numpy front-end of the fastgs part of the CPU checker (oracle/fastgs_oracle.cpp).

TEST INFRASTRUCTURE ONLY (tests/).  Names follow fast_gs::rasterization::forward_wrapper / backward_wrapper
(src/training/fastgs/rasterization/include/rasterization_api.h:25-75) and the caller fast_rasterize
(src/training/rasterization/fast_rasterizer.cpp:12-66).
"""
import ctypes

import numpy as np

from .oracle import _chk, _f32, _p, c_i, c_u32, lib


class Settings(ctypes.Structure):
    """FastGSSettings (rasterization_api.h:12-23) without the tensors"""
    _fields_ = [("active_sh_bases", ctypes.c_uint32), ("total_bases_sh_rest", ctypes.c_uint32),
                ("width", ctypes.c_uint32), ("height", ctypes.c_uint32), ("fx", ctypes.c_float),
                ("fy", ctypes.c_float), ("cx", ctypes.c_float), ("cy", ctypes.c_float),
                ("near_plane", ctypes.c_float), ("far_plane", ctypes.c_float)]


def settings(active_sh_bases, total_bases_sh_rest, width, height, fx, fy, cx, cy, near_plane=0.01, far_plane=1e10):
    return Settings(active_sh_bases, total_bases_sh_rest, width, height, fx, fy, cx, cy, near_plane, far_plane)


def grid(S):
    return (S.width + 15) // 16, (S.height + 15) // 16


def preprocess(means, scales_raw, rotations_raw, opacities_raw, sh0, shN, w2c, cam_position, S):
    """preprocess_cu per primitive -> dict(n_touched u32 [N], bounds u16 [N,4], mean2d, conic_opacity, color, depth)"""
    means, scales_raw, rotations_raw = _f32(means), _f32(scales_raw), _f32(rotations_raw)
    opacities_raw, sh0, shN = _f32(opacities_raw).reshape(-1), _f32(sh0).reshape(-1, 3), _f32(shN)
    w2c, cam_position = _f32(w2c).reshape(4, 4), _f32(cam_position).reshape(3)
    N = means.shape[0]
    assert shN.reshape(N, -1, 3).shape[1] == S.total_bases_sh_rest
    out = dict(n_touched=np.zeros(N, np.uint32), bounds=np.zeros((N, 4), np.uint16), mean2d=np.zeros((N, 2), np.float32),
               conic_opacity=np.zeros((N, 4), np.float32), color=np.zeros((N, 3), np.float32),
               depth=np.zeros(N, np.float32))
    _chk(lib().orc_fgs_preprocess(c_u32(N), _p(means), _p(scales_raw), _p(rotations_raw), _p(opacities_raw), _p(sh0),
                                  _p(shN), _p(w2c), _p(cam_position), ctypes.byref(S), _p(out["n_touched"]),
                                  _p(out["bounds"]), _p(out["mean2d"]), _p(out["conic_opacity"]), _p(out["color"]),
                                  _p(out["depth"])), "fgs_preprocess")
    return out


def instances(pre, S):
    """-> (instance_primitive u32 [n_instances], tile_ranges u32 [T,2])"""
    gw, gh = grid(S)
    n = int(pre["n_touched"].sum())
    inst = np.zeros(max(n, 1), np.uint32)
    ranges = np.zeros((gw * gh, 2), np.uint32)
    _chk(lib().orc_fgs_instances(c_u32(pre["n_touched"].shape[0]), _p(pre["n_touched"]), _p(pre["bounds"]),
                                 _p(pre["mean2d"]), _p(pre["conic_opacity"]), _p(pre["depth"]), c_u32(gw), c_u32(gh),
                                 c_u32(n), _p(inst), _p(ranges)), "fgs_instances")
    return inst[:n], ranges


def blend(pre, inst, ranges, S, extents=None):
    W, H = S.width, S.height
    image, alpha = np.zeros((3, H, W), np.float32), np.zeros((1, H, W), np.float32)
    trans, ncon = np.zeros((H, W), np.float32), np.zeros((H, W), np.uint32)
    viol = ctypes.c_int64(0)
    inst_c = np.ascontiguousarray(inst if inst.size else np.zeros(1, np.uint32))
    ext = _f32(extents)  # kept alive across the call
    _chk(lib().orc_fgs_blend(c_u32(W), c_u32(H), _p(inst_c), _p(ranges), _p(pre["mean2d"]), _p(pre["conic_opacity"]),
                             _p(pre["color"]), _p(image), _p(alpha), _p(trans), _p(ncon), _p(ext),
                             ctypes.byref(viol)), "fgs_blend")
    return image, alpha, trans, ncon, viol.value


def forward(means, scales_raw, rotations_raw, opacities_raw, sh0, shN, w2c, cam_position, S):
    """forward_wrapper -> dict(image [3,H,W], alpha [1,H,W], + everything the backward needs)"""
    pre = preprocess(means, scales_raw, rotations_raw, opacities_raw, sh0, shN, w2c, cam_position, S)
    inst, ranges = instances(pre, S)
    image, alpha, trans, ncon, _ = blend(pre, inst, ranges, S)
    return dict(pre, image=image, alpha=alpha, transmittance=trans, n_contributions=ncon, instance_primitive=inst,
                tile_ranges=ranges)


def blend_bwd(fwd, S, grad_image, grad_alpha):
    N = fwd["n_touched"].shape[0]
    g = dict(mean2d=np.zeros((N, 2)), conic=np.zeros((N, 3)), raw_opacity=np.zeros(N), color=np.zeros((N, 3)))
    inst = fwd["instance_primitive"]
    inst_c = np.ascontiguousarray(inst if inst.size else np.zeros(1, np.uint32))
    gi, ga = _f32(grad_image), _f32(grad_alpha)  # kept alive across the call
    _chk(lib().orc_fgs_blend_bwd(c_u32(N), c_u32(S.width), c_u32(S.height), _p(inst_c), _p(fwd["tile_ranges"]),
                                 _p(fwd["mean2d"]), _p(fwd["conic_opacity"]), _p(fwd["color"]),
                                 _p(fwd["transmittance"]), _p(fwd["n_contributions"]), _p(gi), _p(ga), _p(g["mean2d"]),
                                 _p(g["conic"]), _p(g["raw_opacity"]), _p(g["color"])), "fgs_blend_bwd")
    return g


def preprocess_bwd(means, scales_raw, rotations_raw, shN, w2c, cam_position, S, n_touched, grad_mean2d, grad_conic,
                   grad_color, want_w2c=False, densification_info=None):
    means, scales_raw, rotations_raw, shN = _f32(means), _f32(scales_raw), _f32(rotations_raw), _f32(shN)
    N, B = means.shape[0], S.total_bases_sh_rest
    out = dict(means=np.zeros((N, 3), np.float32), scales_raw=np.zeros((N, 3), np.float32),
               rotations_raw=np.zeros((N, 4), np.float32), sh0=np.zeros((N, 1, 3), np.float32),
               shN=np.zeros((N, B, 3), np.float32))
    gw = np.zeros((4, 4), np.float64) if want_w2c else None
    if densification_info is not None:
        assert densification_info.dtype == np.float32 and densification_info.shape == (2, N)
    w, cp = _f32(w2c).reshape(4, 4), _f32(cam_position).reshape(3)  # temporaries kept alive across the call
    gm, gc, gcol = _f32(grad_mean2d), _f32(grad_conic), _f32(grad_color)
    _chk(lib().orc_fgs_preprocess_bwd(c_u32(N), _p(means), _p(scales_raw), _p(rotations_raw), _p(shN), _p(w), _p(cp),
                                      ctypes.byref(S), _p(n_touched), _p(gm), _p(gc), _p(gcol), _p(out["means"]),
                                      _p(out["scales_raw"]), _p(out["rotations_raw"]), _p(out["sh0"]), _p(out["shN"]),
                                      _p(gw), _p(densification_info)), "fgs_preprocess_bwd")
    out["w2c"] = gw
    return out


def backward(fwd, means, scales_raw, rotations_raw, shN, w2c, cam_position, S, grad_image, grad_alpha, want_w2c=False,
             densification_info=None):
    """backward_wrapper -> dict(means, scales_raw, rotations_raw, opacities_raw [N,1], sh0, shN, w2c)"""
    g = blend_bwd(fwd, S, grad_image, grad_alpha)
    out = preprocess_bwd(means, scales_raw, rotations_raw, shN, w2c, cam_position, S, fwd["n_touched"], g["mean2d"],
                         g["conic"], g["color"], want_w2c, densification_info)
    out["opacities_raw"] = g["raw_opacity"].astype(np.float32).reshape(-1, 1)
    out["blend"] = g
    return out


def loss_f64(P, w2c, cam_position, S, inst, ranges, weight_image, weight_alpha, decisions, max_list, record):
    """the double model's scalar loss; P: dict of float64 arrays means, scales_raw, rotations_raw, opacities_raw, sh0,
    shN; w2c / cam_position float64"""
    d = lambda a: np.ascontiguousarray(a, np.float64)
    f = lib().orc_fgs_loss_f64
    f.restype = ctypes.c_double
    inst_c = np.ascontiguousarray(inst if inst.size else np.zeros(1, np.uint32))
    arrs = [d(P[k]) for k in ("means", "scales_raw", "rotations_raw", "opacities_raw", "sh0", "shN")]
    w, cp, wi, wa = d(w2c), d(cam_position), _f32(weight_image), _f32(weight_alpha)  # kept alive across the call
    return float(f(c_u32(arrs[0].shape[0]), *[_p(a) for a in arrs], _p(w), _p(cp), ctypes.byref(S), _p(inst_c),
                   _p(ranges), _p(wi), _p(wa), _p(decisions), c_u32(max_list), c_i(1 if record else 0)))
