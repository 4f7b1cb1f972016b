"""Trained model <-> binary PLY (SplatData::save_ply, src/core/splat_data.cpp:446-475 / load_ply,
src/loader/formats/ply.cpp:500-637).  The interleaved row image is built and taken apart by GPU kernels; the host
moves it between pinned memory and the file."""
import ctypes
import math
import os

import torch

from . import _lib as L
from ._lib import c_p, c_u32, check, lib


def _p(t):
    return c_p(t.data_ptr())


def _stream(dev):
    return c_p(torch.cuda.current_stream(dev).cuda_stream)


def save_ply(params, path):
    """params: dict of float32 device tensors means [N,3], shs [N,K,3], opacity [N], scaling [N,3], rotation [N,4]
    (raw, as the trainer holds them).  Writes `path` (parent directories are created, splat_data.cpp:117)."""
    lb = lib()
    means, shs = params["means"], params["shs"]
    dev = means.device
    if dev.type != "cuda":
        raise ValueError("save_ply: parameters must live on the GPU")
    N, K = shs.shape[0], shs.shape[1]
    row = lb.gsx_ply_row_floats(c_u32(K))
    rows = torch.empty((N, row), dtype=torch.float32, device=dev)
    check(lb.gsx_ply_pack_rows(ctypes.c_uint64(N), c_u32(K), _p(means.contiguous()), _p(shs.contiguous()),
                               _p(params["opacity"].contiguous()), _p(params["scaling"].contiguous()),
                               _p(params["rotation"].contiguous()), _p(rows), _stream(dev)))
    host = torch.empty((N, row), dtype=torch.float32, pin_memory=True)
    host.copy_(rows)  # synchronous device -> pinned host copy
    d = os.path.dirname(os.path.abspath(path))
    os.makedirs(d, exist_ok=True)
    check(lb.gsx_ply_write_file(os.fsencode(path), ctypes.c_uint64(N), c_u32(K), c_p(host.data_ptr())))
    return path


def load_ply(path, device="cuda:0"):
    """-> dict(means, shs [N,K,3], opacity [N], scaling, rotation, sh_degree) of float32 tensors on `device`."""
    lb = lib()
    dev = torch.device(device)
    layout = L.PlyLayout()
    check(lb.gsx_ply_read_file_header(os.fsencode(path), ctypes.byref(layout)))
    N, stride = int(layout.vertex_count), int(layout.stride_floats)
    K = lb.gsx_ply_layout_sh_coeffs(ctypes.byref(layout))
    host = torch.empty((N, max(stride, 1)), dtype=torch.float32, pin_memory=True)
    if N:
        check(lb.gsx_ply_read_file_rows(os.fsencode(path), ctypes.byref(layout), c_p(host.data_ptr())))
    rows = host.to(dev)
    e = lambda *s: torch.empty(s, dtype=torch.float32, device=dev)
    out = dict(means=e(N, 3), shs=e(N, K, 3), opacity=e(N), scaling=e(N, 3), rotation=e(N, 4))
    check(lb.gsx_ply_unpack_rows(ctypes.byref(layout), _p(rows), _p(out["means"]), _p(out["shs"]), _p(out["opacity"]),
                                 _p(out["scaling"]), _p(out["rotation"]), _stream(dev)))
    torch.cuda.synchronize(dev)
    bn = K - (layout.dc_count // 3 if layout.dc_count > 0 and layout.dc_count % 3 == 0 and layout.dc_start >= 0 else 1)
    out["sh_degree"] = int(math.sqrt(bn + 1)) - 1  # ply.cpp:620
    return out
