"""ctypes binding of libgsx.so (the gfx950 kernels + C ABI of include/gsx.h).

The library must have been built (python lichtfeld-studio_amd/build.py); loading fails loudly otherwise -
there is no CPU or PyTorch fallback for any operator.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgsx.so")

c_f = ctypes.c_float
c_i = ctypes.c_int
c_u32 = ctypes.c_uint32
c_i64 = ctypes.c_int64
c_sz = ctypes.c_size_t
c_p = ctypes.c_void_p

GSX_OK = 0
GSX_ERR_INVALID_ARGUMENT = -1
GSX_ERR_UNSUPPORTED = -2
GSX_ERR_WORKSPACE = -3
GSX_ERR_HIP = -4
GSX_ERR_OVERFLOW = -5

PINHOLE, ORTHO, FISHEYE, EQUIRECTANGULAR = 0, 1, 2, 3
ROLLING_TOP_TO_BOTTOM, ROLLING_LEFT_TO_RIGHT, ROLLING_BOTTOM_TO_TOP, ROLLING_RIGHT_TO_LEFT, GLOBAL = 0, 1, 2, 3, 4
ADAM_MAX_TENSORS = 8


class UTParams(ctypes.Structure):
    """gsplat/Cameras.h:27-44 UnscentedTransformParameters"""
    _fields_ = [("alpha", c_f), ("beta", c_f), ("kappa", c_f), ("in_image_margin_factor", c_f),
                ("require_all_sigma_points_valid", ctypes.c_int32)]

    def __init__(self, alpha=0.1, beta=2.0, kappa=0.0, in_image_margin_factor=0.1,
                 require_all_sigma_points_valid=True):
        super().__init__(alpha, beta, kappa, in_image_margin_factor, 1 if require_all_sigma_points_valid else 0)


class AdamGroup(ctypes.Structure):
    _fields_ = [("param", c_p), ("exp_avg", c_p), ("exp_avg_sq", c_p), ("grad", c_p), ("n", c_i64), ("lr", c_f),
                ("beta1", c_f), ("beta2", c_f), ("eps", c_f), ("bias_correction1_rcp", c_f),
                ("bias_correction2_sqrt_rcp", c_f), ("period", c_u32), ("split", c_u32), ("lr2", c_f),
                ("skip2", ctypes.c_int32)]


class RowTensor(ctypes.Structure):
    """gsx_row_tensor"""
    _fields_ = [("data", c_p), ("row_floats", c_u32), ("is_optimizer_state", ctypes.c_int32)]


class PlyLayout(ctypes.Structure):
    """gsx_ply_layout"""
    _fields_ = [("vertex_count", ctypes.c_uint64), ("data_offset", ctypes.c_uint64),
                ("stride_floats", ctypes.c_uint32), ("pos", ctypes.c_int32 * 3), ("opacity", ctypes.c_int32),
                ("scale", ctypes.c_int32 * 3), ("rot", ctypes.c_int32 * 4), ("dc_start", ctypes.c_int32),
                ("dc_count", ctypes.c_int32), ("rest_start", ctypes.c_int32), ("rest_count", ctypes.c_int32)]


class UpdateArgs(ctypes.Structure):
    """gsx_update_args"""
    _fields_ = ([("N", c_u32), ("K", c_u32), ("sh_degree", c_u32)] +
                [(n, c_p) for n in ("means", "opacity_raw", "scaling_raw", "rotation_raw", "shs", "m_means",
                                    "m_opacity", "m_scaling", "m_rotation", "m_shs", "v_means", "v_opacity",
                                    "v_scaling", "v_rotation", "v_shs", "radii", "colors", "viewmat",
                                    "accumulators")] +
                [(n, c_f) for n in ("lr_means", "lr_sh0", "lr_shN", "lr_scaling", "lr_rotation", "lr_opacity",
                                    "beta1", "beta2", "eps", "bias_correction1_rcp",
                                    "bias_correction2_sqrt_rcp")] +
                [("skip_shN", ctypes.c_int32), ("reg_scaling", c_f), ("reg_opacity", c_f), ("hold", c_p),
                 ("step_scalars", c_p), ("hold_report", c_p)])


class GsxError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"gsx status {status}: {message}")
        self.status = status


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python lichtfeld-studio_amd/build.py` (hipcc, gfx950). "
                "There is no fallback implementation.")
        L = ctypes.CDLL(LIB_PATH)
        L.gsx_last_error.restype = ctypes.c_char_p
        L.gsx_status_string.restype = ctypes.c_char_p
        L.gsx_n_bits.restype = c_u32
        L.gsx_image_loss_blocks.restype = c_u32
        L.gsx_photometric_partials.restype = c_u32
        L.gsx_l1_regularization_partials.restype = c_u32
        L.gsx_ply_row_floats.restype = c_u32
        L.gsx_ply_layout_sh_coeffs.restype = c_u32
        L.gsx_ply_format_header.restype = ctypes.c_int64
        L.gsx_ut_defaults.restype = UTParams
        for name in ("gsx_intersect_tile_count_workspace_bytes", "gsx_radix_sort_pairs_workspace_bytes",
                     "gsx_rasterize_bwd_workspace_bytes", "gsx_mcmc_relocate_workspace_bytes",
                     "gsx_raster_records_bytes", "gsx_rasterize_bwd_accum_bytes", "gsx_tile_order_bytes",
                     "gsx_intersect_tile_count_ordered_workspace_bytes", "gsx_tile_lists_workspace_bytes",
                     "gsx_rasterize_bwd_workspace_bytes_for", "gsx_rasterize_bwd_accum_bytes_for"):
            getattr(L, name).restype = c_sz
        L.gsx_tile_lists_counts.restype = c_p
        L.gsx_radix_sort_pairs_error.restype = c_p
        L.gsx_tile_lists_error.restype = c_p
        _lib = L
    return _lib


def check(status):
    if status != GSX_OK:
        raise GsxError(status, lib().gsx_last_error().decode())


def torch_ext():
    """gsx_torch_ext: the pybind11 module over the C++ host layer (csrc/host/*.cpp), built in-tree by build_ext.py.
    Fails loudly when it has not been built."""
    import importlib
    import sys
    import torch  # noqa: F401  (LibTorch must be loaded first)
    if _HERE not in sys.path:
        sys.path.insert(0, _HERE)
    return importlib.import_module("gsx_torch_ext")
