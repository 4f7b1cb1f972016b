"""Model file format (binary PLY): the numpy restatement of the reference's writer and reader, the host-side header
code of the library against it, and (GPU) the pack / unpack kernels against it bit for bit."""
import ctypes
import os

import numpy as np
import pytest

from oracle import ply as oply


def _params(n, K, seed=0):
    r = np.random.default_rng(seed)
    return dict(means=r.normal(0, 1, (n, 3)).astype(np.float32), shs=r.normal(0, 0.3, (n, K, 3)).astype(np.float32),
                opacity=r.normal(0, 1, n).astype(np.float32), scaling=r.normal(-4, 0.5, (n, 3)).astype(np.float32),
                rotation=r.normal(0, 1, (n, 4)).astype(np.float32))


def _write_custom(path, names, rows, newline="\n", extra_header=()):
    lines = ["ply", "format binary_little_endian 1.0", *extra_header, f"element vertex {rows.shape[0]}"]
    lines += [f"property float {a}" for a in names] + ["end_header"]
    with open(path, "wb") as f:
        f.write((newline.join(lines) + newline).encode("ascii"))
        f.write(np.ascontiguousarray(rows, "<f4").tobytes())


def test_writer_row_layout_by_hand(tmp_path):
    """pins the restated writer: attribute order of splat_data.cpp:402-418 and the channel-major coefficient order
    that sh.transpose(1, 2).flatten(1) produces, on values that name their own (Gaussian, coefficient, channel)"""
    N, K = 2, 3
    shs = np.zeros((N, K, 3), np.float32)
    for v in range(N):
        for k in range(K):
            for c in range(3):
                shs[v, k, c] = 100 * v + 10 * k + c
    P = dict(means=np.array([[1, 2, 3], [4, 5, 6]], np.float32), shs=shs, opacity=np.array([0.5, -0.5], np.float32),
             scaling=np.array([[-1, -2, -3], [-4, -5, -6]], np.float32),
             rotation=np.array([[2, 0, 0, 0], [0, 3, 0, 4]], np.float32))
    rows = oply.rows_from_params(P["means"], shs, P["opacity"], P["scaling"], P["rotation"])
    want0 = [1, 2, 3, 0, 0, 0, 0, 1, 2,          # xyz, normals, f_dc = coefficient 0 in channel order
             10, 20, 11, 21, 12, 22,             # f_rest: R of coefficients 1, 2; then G; then B
             0.5, -1, -2, -3, 1, 0, 0, 0]        # opacity, scales, normalised rotation
    want1 = [4, 5, 6, 0, 0, 0, 100, 101, 102, 110, 120, 111, 121, 112, 122, -0.5, -4, -5, -6, 0, 0.6, 0, 0.8]
    assert np.allclose(rows[0], want0, atol=0) and np.allclose(rows[1], want1, rtol=1e-7)
    assert oply.attribute_names(K) == ["x", "y", "z", "nx", "ny", "nz", "f_dc_0", "f_dc_1", "f_dc_2", "f_rest_0",
                                       "f_rest_1", "f_rest_2", "f_rest_3", "f_rest_4", "f_rest_5", "opacity",
                                       "scale_0", "scale_1", "scale_2", "rot_0", "rot_1", "rot_2", "rot_3"]
    path = tmp_path / "m.ply"
    oply.write_ply(path, P["means"], shs, P["opacity"], P["scaling"], P["rotation"])
    got = oply.read_ply(path)
    assert np.array_equal(got["shs"], shs) and np.array_equal(got["means"], P["means"])
    assert np.array_equal(got["opacity"], P["opacity"]) and np.array_equal(got["scaling"], P["scaling"])
    assert np.allclose(got["rotation"], [[1, 0, 0, 0], [0, 0.6, 0, 0.8]]) and got["sh_degree"] == 0  # int(sqrt(2 + 1)) - 1


@pytest.mark.parametrize("K,deg", [(1, 3), (4, 1), (9, 2), (16, 3)])
def test_reader_round_trip_and_degree(tmp_path, K, deg):
    """writer -> reader returns the tensors (rotation normalised); K = 1 has no f_rest block and reads back with
    the reference's 15 zero coefficients (ply.cpp:554), hence degree 3"""
    P = _params(257, K, K)
    path = tmp_path / "m.ply"
    oply.write_ply(path, P["means"], P["shs"], P["opacity"], P["scaling"], P["rotation"])
    got = oply.read_ply(path)
    assert got["sh_degree"] == deg
    if K == 1:
        assert got["shs"].shape == (257, 16, 3) and not got["shs"][:, 1:].any()
        assert np.array_equal(got["shs"][:, :1], P["shs"])
    else:
        assert np.array_equal(got["shs"], P["shs"])
    n = np.linalg.norm(P["rotation"].astype(np.float64), axis=1, keepdims=True)
    assert np.abs(got["rotation"] - P["rotation"] / n).max() < 2e-7
    for k in ("means", "opacity", "scaling"):
        assert np.array_equal(got[k], P[k])


def _layout_tuple(layout):
    g = lambda o: None if o < 0 else 4 * o
    return dict(vertex_count=layout.vertex_count, vertex_stride=4 * layout.stride_floats,
                pos=[g(o) for o in layout.pos], opacity=g(layout.opacity), scale=[g(o) for o in layout.scale],
                rot=[g(o) for o in layout.rot], dc_start=g(layout.dc_start), rest_start=g(layout.rest_start),
                dc_count=layout.dc_count, rest_count=layout.rest_count)


def _odd_names():
    return ["scale_2", "x", "confidence", "rot_1", "z", "f_rest_0", "f_rest_1", "f_rest_2", "f_rest_3", "f_rest_4",
            "f_rest_5", "f_rest_6", "f_rest_7", "f_rest_8", "opacity", "y", "rot_0", "f_dc_0", "f_dc_1", "f_dc_2",
            "scale_0", "rot_3"]  # scale_1 and rot_2 missing, one unknown property, shuffled order


def test_library_header_code_matches_restatement(gsx, tmp_path):
    """gsx_ply_format_header writes the restated writer's header byte for byte; gsx_ply_parse_header finds what the
    restated parse_header finds on LF / CRLF files, shuffled and missing properties, comment lines; and reports
    the reference's error cases"""
    from lichtfeld_studio_amd._lib import PlyLayout, lib
    L = lib()
    for N, K in ((0, 1), (12345, 4), (10**9, 16)):
        n = L.gsx_ply_format_header(ctypes.c_uint64(N), ctypes.c_uint32(K), None, ctypes.c_size_t(0))
        buf = ctypes.create_string_buffer(n + 1)
        assert L.gsx_ply_format_header(ctypes.c_uint64(N), ctypes.c_uint32(K), buf, ctypes.c_size_t(n + 1)) == n
        assert buf.raw[:n] == oply.header_bytes(N, K)
        assert L.gsx_ply_row_floats(ctypes.c_uint32(K)) == len(oply.attribute_names(K))
        small = ctypes.create_string_buffer(16)
        assert L.gsx_ply_format_header(ctypes.c_uint64(N), ctypes.c_uint32(K), small, ctypes.c_size_t(16)) < 0
    rows = np.zeros((3, len(_odd_names())), np.float32)
    cases = []
    for nl in ("\n", "\r\n"):
        p = tmp_path / f"odd{len(nl)}.ply"
        _write_custom(p, _odd_names(), rows, nl, extra_header=("# a comment line", "comment made by a test", ""))
        cases.append(open(p, "rb").read())
    cases.append(oply.header_bytes(7, 16) + b"\0" * (7 * 62 * 4))
    for data in cases:
        layout = PlyLayout()
        assert L.gsx_ply_parse_header(data, ctypes.c_size_t(len(data)), ctypes.byref(layout)) == 0
        off, want = oply.parse_header(data)
        assert layout.data_offset == off and _layout_tuple(layout) == want
    bad = {b"plx\nformat binary_little_endian 1.0\nelement vertex 1\nproperty float x\nend_header\n": "missing PLY",
           b"ply\nformat ascii 1.0\nelement vertex 1\nproperty float x\nend_header\n": "only binary",
           b"ply\nformat binary_little_endian 1.0\nproperty float x\nend_header\n": "only binary",
           b"ply\nformat binary_little_endian 1.0\nelement vertex 1\nproperty float x\n": "no end_header",
           b"ply\nformat binary_little_endian 1.0\nelement vertex 1\nproperty uchar red\nend_header\n": "not float32",
           b"ply\n": "too small"}
    for data, word in bad.items():
        layout = PlyLayout()
        assert L.gsx_ply_parse_header(data, ctypes.c_size_t(len(data)), ctypes.byref(layout)) < 0
        assert word.lower() in L.gsx_last_error().decode().lower(), (word, L.gsx_last_error())
        if word not in ("not float32",):
            with pytest.raises(RuntimeError):
                oply.parse_header(data)
    layout = PlyLayout()
    assert L.gsx_ply_read_file_header(os.fsencode(tmp_path / "absent.ply"), ctypes.byref(layout)) < 0
    assert "does not exist" in L.gsx_last_error().decode()


# ---------------------------------------------------------------- GPU
@pytest.mark.gpu
@pytest.mark.parametrize("n,K", [(1, 1), (1000, 4), (50_001, 16)])
def test_save_ply_writes_the_restated_file(gsx, cuda, tmp_path, n, K):
    import torch
    from lichtfeld_studio_amd.ply import load_ply, save_ply
    P = _params(n, K, n)
    P["rotation"][0] = 0.0  # zero quaternion: x / max(|x|, 1e-12) = 0
    dev = {k: torch.from_numpy(v).to(cuda) for k, v in P.items()}
    save_ply(dev, str(tmp_path / "sub" / "gpu.ply"))
    oply.write_ply(tmp_path / "cpu.ply", P["means"], P["shs"], P["opacity"], P["scaling"], P["rotation"])
    a, b = open(tmp_path / "sub" / "gpu.ply", "rb").read(), open(tmp_path / "cpu.ply", "rb").read()
    assert a == b
    got, want = load_ply(str(tmp_path / "cpu.ply"), cuda), oply.read_ply(tmp_path / "cpu.ply")
    assert got["sh_degree"] == want["sh_degree"]
    for k in ("means", "shs", "opacity", "scaling", "rotation"):
        assert np.array_equal(got[k].cpu().numpy().view(np.int32), want[k].view(np.int32)), k


@pytest.mark.gpu
@pytest.mark.parametrize("newline", ["\n", "\r\n"])
def test_load_ply_foreign_layouts(gsx, cuda, tmp_path, newline):
    """shuffled property order with an unknown property and missing components; a positions-only file (defaults:
    zero SH with 16 coefficients, opacity 0, log-scale -5, identity rotation); an empty file"""
    from lichtfeld_studio_amd.ply import load_ply
    r = np.random.default_rng(3)
    files = []
    rows = r.normal(0, 1, (777, len(_odd_names()))).astype(np.float32)
    _write_custom(tmp_path / "odd.ply", _odd_names(), rows, newline, extra_header=("comment x",))
    files.append("odd.ply")
    _write_custom(tmp_path / "pos.ply", ["x", "y", "z"], r.normal(0, 1, (100, 3)).astype(np.float32), newline)
    files.append("pos.ply")
    _write_custom(tmp_path / "noxyz.ply", ["y", "z", "opacity", "f_dc_0", "f_dc_1"],
                  r.normal(0, 1, (10, 5)).astype(np.float32), newline)  # no x: positions stay 0; f_dc count 2: zeros
    files.append("noxyz.ply")
    _write_custom(tmp_path / "empty.ply", oply.attribute_names(16), np.zeros((0, 62), np.float32), newline)
    files.append("empty.ply")
    for name in files:
        got, want = load_ply(str(tmp_path / name), cuda), oply.read_ply(tmp_path / name)
        assert got["sh_degree"] == want["sh_degree"], name
        for k in ("means", "shs", "opacity", "scaling", "rotation"):
            assert got[k].shape == want[k].shape, (name, k)
            assert np.array_equal(got[k].cpu().numpy().view(np.int32), want[k].view(np.int32)), (name, k)


@pytest.mark.gpu
def test_trained_state_round_trips_through_ply(gsx, cuda, tmp_path):
    """a training step's parameters -> file -> parameters: everything but the rotation comes back bit for bit, the
    rotation normalised, and the reloaded model renders the same image"""
    import torch
    from lichtfeld_studio_amd.ply import load_ply, save_ply
    from lichtfeld_studio_amd.trainer import TrainStep
    sc = gsx.scenes.config(3, 20_000)
    sc.scaling_raw += 1.2
    cam = gsx.scenes.orbit_camera(0.7, 4.0, 309, 205, 287.0)
    vm = torch.from_numpy(cam.viewmat[None].copy()).to(cuda)
    Km = torch.from_numpy(cam.K[None].copy()).to(cuda)
    gt = torch.rand((1, 3, 205, 309), generator=torch.Generator().manual_seed(3)).to(cuda)
    ts = TrainStep(sc, cuda, fused_update=True, fused_loss=True)
    ts.step(vm, Km, 309, 205, gt)
    save_ply(ts.params, str(tmp_path / "m.ply"))
    back = load_ply(str(tmp_path / "m.ply"), cuda)
    assert back["sh_degree"] == 3
    for k in ("means", "shs", "opacity", "scaling"):
        assert torch.equal(back[k], ts.params[k]), k
    q = ts.params["rotation"]
    assert (back["rotation"] - q / q.norm(dim=1, keepdim=True)).abs().max().item() < 3e-7
    img0 = ts.forward(vm, Km, 309, 205).clone()
    ts.params["rotation"].copy_(back["rotation"])
    img1 = ts.forward(vm, Km, 309, 205)
    assert (img0 - img1).abs().max().item() < 1e-4
