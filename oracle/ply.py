"""CPU restatement of the model file format (numpy): writer SplatData::save_ply (src/core/splat_data.cpp:113-169,
402-418, 484-506) and reader load_ply (src/loader/formats/ply.cpp:185-323, 446-496, 500-637).

TEST INFRASTRUCTURE ONLY (tests/).

The writer goes through tinyply (vcpkg dependency, absent from the reference tree): its binary writer emits
"ply / format binary_little_endian 1.0 / element vertex N / property float <name> ... / end_header" and then the
properties of each vertex interleaved in declaration order.  The exact header bytes are "parity unpinned" (no file
written by the reference exists in its tree); what pins them is the reference's own reader, restated below, which
must read the file back.
"""
import numpy as np


def attribute_names(K):
    """SplatData::get_attribute_names (splat_data.cpp:402-418) for sh0 [N,1,3] and shN [N,K-1,3]"""
    a = ["x", "y", "z", "nx", "ny", "nz"]
    a += [f"f_dc_{i}" for i in range(3)]
    a += [f"f_rest_{i}" for i in range(3 * (K - 1))]
    a += ["opacity"] + [f"scale_{i}" for i in range(3)] + [f"rot_{i}" for i in range(4)]
    return a


def rows_from_params(means, shs, opacity_raw, scaling_raw, rotation_raw):
    """to_point_cloud (splat_data.cpp:484-506) + the interleave of write_ply_impl: [N, 14 + 3K] float32"""
    means = np.asarray(means, np.float32)
    shs = np.asarray(shs, np.float32)
    N, K = shs.shape[0], shs.shape[1]
    sh0 = shs[:, :1].transpose(0, 2, 1).reshape(N, -1)   # _sh0.transpose(1, 2).flatten(1)
    shN = shs[:, 1:].transpose(0, 2, 1).reshape(N, -1)   # _shN.transpose(1, 2).flatten(1)
    q = np.asarray(rotation_raw, np.float32)
    # F.normalize: x / max(||x||_2, 1e-12); fp32 sum of squares in index order, IEEE sqrt and division
    n = np.sqrt(((q[:, 0] * q[:, 0] + q[:, 1] * q[:, 1]) + q[:, 2] * q[:, 2]) + q[:, 3] * q[:, 3], dtype=np.float32)
    qn = q / np.maximum(n, np.float32(1e-12))[:, None]
    return np.concatenate([means, np.zeros_like(means), sh0, shN, np.asarray(opacity_raw, np.float32).reshape(N, 1),
                           np.asarray(scaling_raw, np.float32), qn.astype(np.float32)], axis=1).astype(np.float32)


def header_bytes(N, K):
    lines = ["ply", "format binary_little_endian 1.0", f"element vertex {N}"]
    lines += [f"property float {a}" for a in attribute_names(K)] + ["end_header"]
    return ("\n".join(lines) + "\n").encode("ascii")


def write_ply(path, means, shs, opacity_raw, scaling_raw, rotation_raw):
    rows = rows_from_params(means, shs, opacity_raw, scaling_raw, rotation_raw)
    with open(path, "wb") as f:
        f.write(header_bytes(rows.shape[0], np.asarray(shs).shape[1]))
        f.write(rows.astype("<f4").tobytes())
    return rows


def parse_header(data):
    """parse_header (ply.cpp:185-323) -> (data_offset, layout dict with BYTE offsets as the reference keeps them)"""
    if len(data) < 10:
        raise RuntimeError("File too small to be valid PLY")
    if data[:5] == b"ply\r\n":
        pos = 5
    elif data[:4] == b"ply\n":
        pos = 4
    else:
        raise RuntimeError("Invalid PLY file - missing PLY header")
    L = dict(vertex_count=0, vertex_stride=0, pos=[None] * 3, opacity=None, scale=[None] * 3, rot=[None] * 4,
             dc_start=None, rest_start=None, dc_count=0, rest_count=0)
    binary = found_vertex = False
    lines = 0
    while pos < len(data) and lines < 10000:
        nl = data.find(b"\n", pos)
        if nl < 0:
            break
        line = data[pos:nl]
        pos = nl + 1
        if line.endswith(b"\r"):
            line = line[:-1]
        lines += 1
        if len(line) == 0 or line[:1] == b"#":
            continue
        if line.startswith(b"format binary_little_endian"):
            binary = True
        elif line.startswith(b"element vertex "):
            L["vertex_count"] = int(line[15:].split()[0])
            L["vertex_stride"] = 0
            found_vertex = True
        elif line.startswith(b"property float ") and found_vertex:
            name = line[15:].rstrip(b" \t\r").decode("ascii")
            at = L["vertex_stride"]
            if len(name) == 1:
                if name in "xyz":
                    L["pos"]["xyz".index(name)] = at
            elif name == "opacity":
                L["opacity"] = at
            elif name.startswith("f_dc_"):
                idx = int(name[5:])
                if idx == 0:
                    L["dc_start"] = at
                L["dc_count"] = max(L["dc_count"], idx + 1)
            elif name.startswith("f_rest_"):
                idx = int(name[7:])
                if idx == 0:
                    L["rest_start"] = at
                L["rest_count"] = max(L["rest_count"], idx + 1)
            elif len(name) == 7 and name.startswith("scale_"):
                idx = ord(name[6]) - ord("0")
                if 0 <= idx < 3:
                    L["scale"][idx] = at
            elif len(name) == 5 and name.startswith("rot_"):
                idx = ord(name[4]) - ord("0")
                if 0 <= idx < 4:
                    L["rot"][idx] = at
            L["vertex_stride"] += 4
        elif line.startswith(b"end_header"):
            if not binary or not found_vertex:
                raise RuntimeError("Only binary PLY with position supported")
            return pos, L
    if lines >= 10000:
        raise RuntimeError("Header too large - exceeded 10000 lines")
    raise RuntimeError("No end_header found in PLY file")


def read_ply(path):
    """load_ply (ply.cpp:500-637) -> dict(means [N,3], shs [N,K,3] (sh0 and shN concatenated), opacity [N],
    scaling [N,3], rotation [N,4], sh_degree)"""
    data = open(path, "rb").read()
    off, L = parse_header(data)
    N, stride = L["vertex_count"], L["vertex_stride"]
    raw = np.frombuffer(data, dtype="<f4", count=N * stride // 4, offset=off).reshape(N, stride // 4)
    col = lambda byte_off: raw[:, byte_off // 4]
    means = np.zeros((N, 3), np.float32)
    if L["pos"][0] is not None:
        for c in range(3):
            if L["pos"][c] is not None:
                means[:, c] = col(L["pos"][c])

    def sh_block(start, count, default_coeffs):
        # extract_sh_coefficients (ply.cpp:446-476): value j of the block goes to (channel j // B, basis j % B)
        if count > 0 and count % 3 == 0 and start is not None:
            B = count // 3
            out = np.zeros((N, B, 3), np.float32)
            for j in range(count):
                out[:, j % B, j // B] = raw[:, start // 4 + j]
            return out
        return np.zeros((N, default_coeffs, 3), np.float32)

    sh0 = sh_block(L["dc_start"], L["dc_count"], 1)
    shN = sh_block(L["rest_start"], L["rest_count"], 15)
    opacity = np.zeros(N, np.float32)
    if L["opacity"] is not None:
        opacity[:] = col(L["opacity"])
    scaling = np.zeros((N, 3), np.float32)
    if L["scale"][0] is not None:
        for c in range(3):
            if L["scale"][c] is not None:
                scaling[:, c] = col(L["scale"][c])
    else:
        scaling[:] = -5.0
    rotation = np.zeros((N, 4), np.float32)
    if L["rot"][0] is not None:
        for c in range(4):
            if L["rot"][c] is not None:
                rotation[:, c] = col(L["rot"][c])
    else:
        rotation[:, 0] = 1.0
    sh_degree = int(np.sqrt(shN.shape[1] + 1)) - 1
    return dict(means=means, shs=np.concatenate([sh0, shN], 1), opacity=opacity, scaling=scaling, rotation=rotation,
                sh_degree=sh_degree)
