"""ctypes binding of libinpc_hip.so (declarations: include/inpc_hip.h).

The library is the product: there is no CPU or PyTorch fallback. Loading fails loudly when the
shared object has not been built (python -m inpc_amd.build).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "libinpc_hip.so"

INPC_OK = 0
E_INVALID_ARGUMENT, E_WORKSPACE, E_UNSUPPORTED, E_HIP, E_DEVICE = -1, -2, -3, -4, -5
FEAT_SH36_F16 = 0
FEAT_DIRECT_F32 = 1
FEAT_DIRECT_F16 = 2
FEAT_RAW37_F16 = 3
RASTER_INFERENCE = 1
RASTER_KEEP_GEOMETRY = 2
CULL_IF_COMPLETE = 0xFFFFFFFF  # INPC_CULL_IF_COMPLETE
CDF_HEAD_MIN_FLOATS = 16384  # INPC_CDF_HEAD_MIN_FLOATS: the smallest CDF head; inpc_cdf_head_floats(n_leaves) sizes one


class Camera(C.Structure):
    _fields_ = [
        ("width", C.c_int32),
        ("height", C.c_int32),
        ("focal_x", C.c_float),
        ("focal_y", C.c_float),
        ("center_x", C.c_float),
        ("center_y", C.c_float),
        ("near_plane", C.c_float),
        ("far_plane", C.c_float),
    ]


class RasterConfig(C.Structure):
    _fields_ = [
        ("n_points", C.c_uint32),
        ("tile", C.c_int32),
        ("channels", C.c_int32),
        ("feature_mode", C.c_int32),
        ("flags", C.c_uint32),
        ("cam", Camera),
        ("max_instances", C.c_uint32),
    ]


class RasterLayout(C.Structure):
    _fields_ = [
        ("total_bytes", C.c_size_t),
        ("counters", C.c_size_t),
        ("bin_start", C.c_size_t),
        ("point_record", C.c_size_t),
        ("instance_points", C.c_size_t),
        ("tile_ranges", C.c_size_t),
        ("debug_geometry", C.c_size_t),
        ("record_stride", C.c_uint32),
        ("grid_width", C.c_uint32),
        ("grid_height", C.c_uint32),
        ("n_tiles", C.c_uint32),
        ("end_bit", C.c_uint32),
        ("depth_key_bias", C.c_uint32),
        ("max_instances", C.c_uint32),
        ("reserved", C.c_uint32),
    ]


class GaussianConfig(C.Structure):
    _fields_ = [
        ("base", RasterConfig),
        ("sigma_world", C.c_float),
        ("sigma_cutoff", C.c_float),
        ("max_instances", C.c_uint32),
        ("reserved", C.c_uint32),
    ]


class GaussianLayout(C.Structure):
    _fields_ = [
        ("total_bytes", C.c_size_t),
        ("counters", C.c_size_t),
        ("point_touched", C.c_size_t),
        ("point_bounds", C.c_size_t),
        ("point_record", C.c_size_t),
        ("depth_keys", C.c_size_t),
        ("instance_points", C.c_size_t),
        ("tile_ranges", C.c_size_t),
        ("record_stride", C.c_uint32),
        ("grid_width", C.c_uint32),
        ("grid_height", C.c_uint32),
        ("n_tiles", C.c_uint32),
        ("end_bit", C.c_uint32),
        ("depth_key_bias", C.c_uint32),
        ("max_instances", C.c_uint32),
        ("reserved", C.c_uint32),
    ]


class TimingRecord(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ms", C.c_float)]


# name -> (restype, argtypes); every symbol include/inpc_hip.h declares
_P = C.c_void_p
_U32 = C.c_uint32
_F = C.c_float
_SZ = C.c_size_t
_CAM = C.POINTER(Camera)
_CFG = C.POINTER(RasterConfig)
_GCFG = C.POINTER(GaussianConfig)
SIGNATURES = {
    "inpc_last_error": (C.c_char_p, []),
    "inpc_abi_version": (C.c_int, []),
    "inpc_pcg32_seed": (None, [_P, C.c_uint64, C.c_uint64]),
    "inpc_pcg32_next_uint": (_U32, [_P]),
    "inpc_pcg32_next_float": (_F, [_P]),
    "inpc_pcg32_advance": (None, [_P, C.c_int64]),
    "inpc_leaf_weights": (C.c_int, [_P, _P, _P, _P, _P, _P, _U32, _CAM, _F, _P]),
    "inpc_sampler_workspace_bytes": (_SZ, [_U32]),
    "inpc_build_cdf": (C.c_int, [_P, _P, _SZ, _P, _SZ, _U32, _P]),
    "inpc_build_cdf_static": (C.c_int, [_P, _P, _SZ, _U32, _P]),
    "inpc_sample": (C.c_int, [_P, _P, _P, _SZ, _P, _P, _U32, _U32, _P, _P]),
    "inpc_cull_workspace_bytes": (_SZ, [_U32]),
    "inpc_cull_begin": (C.c_int, [_P, _SZ, _P]),
    "inpc_sample_cull_compact": (C.c_int, [_P, _P, _P, _SZ, _P, _P, _P, C.c_int, _U32, _U32, _U32, _U32, _CAM, _P, _P,
                                           _SZ, _P]),
    "inpc_cull_read_counts": (C.c_int, [_P, C.POINTER(_U32), C.POINTER(_U32), _P]),
    "inpc_cull_finish": (C.c_int, [_P, _P, _P, C.c_int, _U32, _U32, _P, _P, _SZ, _P]),
    "inpc_widen_ids": (C.c_int, [_P, _P, _U32, _P]),
    "inpc_expected_counts": (C.c_int, [_P, _P, _P, _U32, _P, _SZ, _U32, _P]),
    "inpc_expected_samples": (C.c_int, [_P, _P, _P, _P, _P, _U32, _U32, _U32, _F, _P, _P]),
    "inpc_raster_layout_query": (C.c_int, [_CFG, C.POINTER(RasterLayout)]),
    "inpc_raster_forward": (C.c_int, [_CFG, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "inpc_side_stream_policy": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int]),
    "inpc_raster_backward": (C.c_int, [_CFG, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "inpc_raster_read_counters": (C.c_int, [_CFG, _P, C.POINTER(_U32 * 3), _P]),
    "inpc_gaussian_layout_query": (C.c_int, [_GCFG, C.POINTER(GaussianLayout)]),
    "inpc_gaussian_forward": (C.c_int, [_GCFG, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "inpc_gaussian_backward": (C.c_int, [_GCFG, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "inpc_gaussian_read_counters": (C.c_int, [_GCFG, _P, C.POINTER(_U32 * 4), _P]),
    "inpc_field_update_workspace_bytes": (_SZ, [_U32]),
    "inpc_field_update": (C.c_int, [_P, _P, _U32, _P, _P, _U32, _F, _P, _SZ, _P]),
    "inpc_field_update_check": (C.c_int, [_P, _P]),
    "inpc_spherical_contraction": (C.c_int, [_P, _P, _U32, _P]),
    "inpc_opacity_forward": (C.c_int, [_P, _P, _SZ, _P]),
    "inpc_opacity_backward": (C.c_int, [_P, _P, _P, _SZ, _P]),
    "inpc_field_select_workspace_bytes": (C.c_size_t, [_U32]),
    "inpc_field_select_count": (C.c_int, [_P, _P, _U32, C.c_float, C.c_int, _P, _P, C.c_size_t, _P]),
    "inpc_field_prune": (C.c_int, [_P, _P, _P, _P, _U32, C.c_float, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "inpc_field_subdivide": (C.c_int, [_P, _P, _P, _P, _U32, C.c_float, C.c_int, C.POINTER(C.c_float), _P, _P, _P, _P,
                                       _P, _P, C.c_size_t, _P]),
    "inpc_cdf_head_floats": (C.c_size_t, [_U32]),
    "inpc_extract_global_workspace_bytes": (C.c_size_t, [_U32]),
    "inpc_extract_global": (C.c_int, [_P, _P, _P, _U32, C.POINTER(C.c_float), _P, _U32, _P, C.c_size_t, _P]),
    "inpc_extract_global_check": (C.c_int, [_P, _U32, _P]),
    "inpc_morton_workspace_bytes": (C.c_size_t, []),
    "inpc_morton_encode": (C.c_int, [_P, _U32, _P, _P, C.c_size_t, _P]),
    "inpc_weight_decay_grads": (C.c_int, [_P, _P, _U32, C.c_int, _P]),
    "inpc_cauchy_loss": (C.c_int, [_P, _P, _P, _U32, _P]),
    "inpc_cauchy_loss_backward": (C.c_int, [_P, _P, _P, _P, _U32, _P]),
    "inpc_timing_enable": (None, [C.c_int]),
    "inpc_timing_collect": (C.c_int, [C.POINTER(TimingRecord), C.c_int]),
    "inpc_calibration_copy": (C.c_int, [_P, _P, _SZ, _P]),
}

_lib = None


# how the library gets built: in the tree, or into an installed package (setup.py runs the same build)
BUILD_COMMAND = ["python", "-m", "inpc_amd.build"]
INSTALL_COMMAND = ["pip", "install", str(LIB_PATH.parent.parent), "--no-build-isolation"]


class ExtensionError(ImportError):
    """The native library is missing. Carries the package name and the command that builds it, like the
    Framework.ExtensionError the reference raises for its extension module (INPCCudaBackend/__init__.py:7-23)."""

    def __init__(self, name: str, install_command: list[str], detail: str = ""):
        super().__init__(f"extension '{name}' is not built{detail}; build it with `{' '.join(BUILD_COMMAND)}` "
                         f"(hipcc, gfx950) or install it with `{' '.join(install_command)}`. "
                         "inpc_amd has no fallback path.", name=name)
        self.install_command = install_command


class BackendError(RuntimeError):
    """A call into libinpc_hip.so failed (the counterpart of the RuntimeError pybind11 raises for
    the reference's C++ exceptions)."""


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ExtensionError("inpc_amd", INSTALL_COMMAND, f": {LIB_PATH} is missing")
        handle = C.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the symbol is not exported
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc != INPC_OK:
        msg = lib().inpc_last_error()
        raise BackendError(f"{what} failed with code {rc}: {msg.decode() if msg else ''}")


def ptr(t) -> C.c_void_p:
    """Device pointer of a tensor (None -> NULL)."""
    return C.c_void_p(None if t is None else t.data_ptr())


def current_stream() -> C.c_void_p:
    import torch

    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def make_camera(camera) -> Camera:
    return Camera(int(camera.width), int(camera.height), float(camera.focal_x), float(camera.focal_y),
                  float(camera.center_x), float(camera.center_y), float(camera.near_plane), float(camera.far_plane))


class KernelTimer:
    """Context manager around the library's per-launch HIP-event timing. After exit, `.records`
    is a list of (kernel name, milliseconds) in launch order."""

    def __init__(self):
        self.records = []

    def __enter__(self):
        lib().inpc_timing_enable(1)
        return self

    def __exit__(self, *exc):
        buf = (TimingRecord * 4096)()
        n = lib().inpc_timing_collect(buf, 4096)
        self.records = [(buf[i].name.decode(), float(buf[i].ms)) for i in range(n)]
        lib().inpc_timing_enable(0)
        return False
