"""ctypes binding of the CPU oracle (oracle/inpc_oracle.cpp).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py as the checker / the timed CPU baseline. The product package
(inpc_amd) never imports this module.

Every function takes and returns numpy arrays (host memory) and mirrors one exported function
of the oracle; the reference lines each one follows are cited in inpc_oracle.cpp.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "liboracle.so"

FEAT_SH36_F16 = 0
FEAT_DIRECT_F32 = 1
FEAT_DIRECT_F16 = 2
FEAT_RAW37_F16 = 3
RASTER_INFERENCE = 1


def build(force: bool = False) -> Path:
    """Compile liboracle.so with g++ (make decides whether anything is stale)."""
    if force and _LIB_PATH.exists():
        _LIB_PATH.unlink()
    subprocess.run(["make", "-C", str(_DIR), "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


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
        ("max_instances", C.c_uint32),   # capacity of the HIP library's buffers; the oracle ignores it
    ]


class _RasterDebug(C.Structure):
    _fields_ = [
        ("n_touched", C.c_void_p),
        ("bounds", C.c_void_p),
        ("screen_xy", C.c_void_p),
        ("depth", C.c_void_p),
        ("features_view", C.c_void_p),
        ("opacity", C.c_void_p),
        ("counts", C.c_void_p),
        ("depth_keys", C.c_void_p),
        ("depth_order", C.c_void_p),
        ("instance_keys", C.c_void_p),
        ("instance_points", C.c_void_p),
        ("tile_ranges", C.c_void_p),
        ("conic", C.c_void_p),
    ]


class GaussianConfig(C.Structure):
    _fields_ = [
        ("base", RasterConfig),
        ("sigma_world", C.c_float),
        ("sigma_cutoff", C.c_float),
        ("max_instances", C.c_uint32),
        ("reserved", C.c_uint32),
    ]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            build()
        _lib = C.CDLL(str(_LIB_PATH))
        _lib.oracle_pcg32_next_uint.restype = C.c_uint32
        _lib.oracle_pcg32_next_float.restype = C.c_float
        _lib.oracle_blocked_total.restype = C.c_float
        _lib.oracle_cdf_search.restype = C.c_uint32
        _lib.oracle_cdf_search.argtypes = [C.c_void_p, C.c_float, C.c_uint32]
        _lib.oracle_training_samples.restype = C.c_uint32
        _lib.oracle_expected_counts.restype = C.c_uint32
        _lib.oracle_float_to_half.restype = C.c_uint16
        _lib.oracle_float_to_half.argtypes = [C.c_float]
        _lib.oracle_half_to_float.restype = C.c_float
        _lib.oracle_half_to_float.argtypes = [C.c_uint16]
        _lib.oracle_now.restype = C.c_double
        _lib.oracle_num_threads.restype = C.c_int
        _lib.oracle_footprint_exp.restype = C.c_float
        _lib.oracle_footprint_exp.argtypes = [C.c_float]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def make_camera(width, height, fx, fy, cx=None, cy=None, near=0.01, far=100.0) -> Camera:
    return Camera(int(width), int(height), float(fx), float(fy),
                  float(width / 2 if cx is None else cx), float(height / 2 if cy is None else cy),
                  float(near), float(far))


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def set_num_threads(n: int) -> None:
    lib().oracle_set_num_threads(C.c_int(int(n)))


def now() -> float:
    return float(lib().oracle_now())


# ----------------------------------------------------------------------------------------------
# pcg32
# ----------------------------------------------------------------------------------------------
class Pcg32:
    """Host generator; `state` is a uint64[2] numpy array {state, inc}."""

    def __init__(self, initstate: int, initseq: int = 1):
        self.state = np.zeros(2, dtype=np.uint64)
        lib().oracle_pcg32_seed(_p(self.state), C.c_uint64(initstate & (2**64 - 1)), C.c_uint64(initseq))

    def copy(self) -> "Pcg32":
        other = Pcg32.__new__(Pcg32)
        other.state = self.state.copy()
        return other

    def next_uint(self) -> int:
        return int(lib().oracle_pcg32_next_uint(_p(self.state)))

    def next_float(self) -> float:
        return float(lib().oracle_pcg32_next_float(_p(self.state)))

    def advance(self, delta: int) -> None:
        lib().oracle_pcg32_advance(_p(self.state), C.c_int64(delta))


def float_to_half(f: float) -> int:
    return int(lib().oracle_float_to_half(C.c_float(f)))


def half_to_float(h: int) -> float:
    return float(lib().oracle_half_to_float(C.c_uint16(h)))


# ----------------------------------------------------------------------------------------------
# sampler
# ----------------------------------------------------------------------------------------------
def leaf_weights(centers, levels, weights, w2c, cam: Camera, initial_size: float) -> np.ndarray:
    centers, levels, weights, w2c = _f32(centers), _i32(levels), _f32(weights), _f32(w2c)
    out = np.empty(len(levels), dtype=np.float32)
    lib().oracle_leaf_weights(_p(centers), _p(levels), _p(weights), _p(w2c), _p(out), C.c_uint32(len(levels)),
                              C.byref(cam), C.c_float(initial_size))
    return out


def blocked_total(w) -> np.float32:
    w = _f32(w)
    return np.float32(lib().oracle_blocked_total(_p(w), C.c_uint32(len(w))))


def blocked_inclusive_scan(w) -> np.ndarray:
    out = _f32(w).copy()
    lib().oracle_blocked_inclusive_scan(_p(out), C.c_uint32(len(out)))
    return out


def build_cdf(w):
    """Returns (ok, cdf, sum)."""
    out = _f32(w).copy()
    s = C.c_float(0)
    ok = lib().oracle_build_cdf(_p(out), C.c_uint32(len(out)), C.byref(s))
    return bool(ok), out, np.float32(s.value)


def cdf_search(cdf, sample: float) -> int:
    cdf = _f32(cdf)
    return int(lib().oracle_cdf_search(_p(cdf), C.c_float(sample), C.c_uint32(len(cdf))))


def sample(centers, levels, cdf, n_samples: int, initial_size: float, rng: Pcg32):
    """Returns (positions (n,3), leaf ids (n,)); advances rng by 4*n."""
    centers, levels, cdf = _f32(centers), _i32(levels), _f32(cdf)
    pos = np.empty((n_samples, 3), dtype=np.float32)
    ids = np.empty(n_samples, dtype=np.int32)
    lib().oracle_sample(_p(centers), _p(levels), _p(cdf), _p(pos), _p(ids), C.c_uint32(n_samples),
                        C.c_uint32(len(levels)), C.c_float(initial_size), _p(rng.state))
    return pos, ids


def sample_cull_compact(centers, levels, cdf, w2c, cam: Camera, initial_size: float, rng: Pcg32, capacity: int,
                        k0: int, n_candidates: int, positions=None, ids=None, accepted: int = 0):
    """One round. Returns (positions, ids, accepted, consumed)."""
    centers, levels, cdf, w2c = _f32(centers), _i32(levels), _f32(cdf), _f32(w2c)
    if positions is None:
        positions = np.zeros((capacity, 3), dtype=np.float32)
        ids = np.full(capacity, -1, dtype=np.int32)
    acc = C.c_uint32(accepted)
    cons = C.c_uint32(0)
    lib().oracle_sample_cull_compact(_p(centers), _p(levels), _p(cdf), _p(w2c), _p(positions), _p(ids),
                                     C.c_uint32(capacity), C.c_uint32(k0), C.c_uint32(n_candidates),
                                     C.c_uint32(len(levels)), C.byref(cam), C.c_float(initial_size), _p(rng.state),
                                     C.byref(acc), C.byref(cons))
    return positions, ids, int(acc.value), int(cons.value)


def training_samples(centers, levels, weights, w2c, cam: Camera, initial_size: float, rng: Pcg32, n_samples: int):
    """Whole draw. Returns (positions, ids int32, consumed); advances rng by 4*consumed."""
    centers, levels, weights, w2c = _f32(centers), _i32(levels), _f32(weights), _f32(w2c)
    pos = np.empty((n_samples, 3), dtype=np.float32)
    ids = np.empty(n_samples, dtype=np.int32)
    consumed = lib().oracle_training_samples(_p(centers), _p(levels), _p(weights), _p(w2c), _p(pos), _p(ids),
                                             C.c_uint32(n_samples), C.c_uint32(len(levels)), C.byref(cam),
                                             C.c_float(initial_size), _p(rng.state))
    return pos, ids, int(consumed)


def expected_counts(weights, n_samples: int):
    """Returns (offsets int32 (L,), n_created, sum)."""
    weights = _f32(weights)
    offs = np.zeros(len(weights), dtype=np.int32)
    s = C.c_float(0)
    n = lib().oracle_expected_counts(_p(weights), _p(offs), C.c_uint32(n_samples), C.c_uint32(len(weights)),
                                     C.byref(s))
    return offs, int(n), np.float32(s.value)


def expected_samples(centers, levels, offsets, n_created: int, n_multi: int, initial_size: float, rng: Pcg32):
    centers, levels, offsets = _f32(centers), _i32(levels), _i32(offsets)
    pos = np.empty((n_created * n_multi, 3), dtype=np.float32)
    lib().oracle_expected_samples(_p(centers), _p(levels), _p(offsets), _p(pos), C.c_uint32(n_created),
                                  C.c_uint32(n_multi), C.c_uint32(len(levels)), C.c_float(initial_size),
                                  _p(rng.state))
    return pos


# ----------------------------------------------------------------------------------------------
# rasterizer
# ----------------------------------------------------------------------------------------------
def make_config(n_points: int, cam: Camera, tile: int = 16, channels: int = 4, feature_mode: int = FEAT_DIRECT_F32,
                flags: int = 0) -> RasterConfig:
    return RasterConfig(int(n_points), int(tile), int(channels), int(feature_mode), int(flags), cam)


def _features_array(features, feature_mode):
    if feature_mode == FEAT_DIRECT_F32:
        return _f32(features)
    return np.ascontiguousarray(features, dtype=np.float16)


def raster_forward(cfg: RasterConfig, positions, features, opacities, w2c, cam_position=None, debug: bool = False,
                   gaussian: "GaussianConfig | None" = None, scales=None, n_instances_hint: int = 0):
    """Returns dict(image (C,H,W), alpha (1,H,W), blending_weights (N,) | depth_image (1,H,W), + debug buffers).
    With `gaussian` (whose base is `cfg`) the Gaussian footprint is drawn instead of the bilinear one."""
    n = cfg.n_points
    W, H = cfg.cam.width, cfg.cam.height
    sh = cfg.feature_mode in (FEAT_SH36_F16, FEAT_RAW37_F16)
    Cn = 4 if sh else cfg.channels
    positions, w2c = _f32(positions), _f32(w2c)
    features = _features_array(features, cfg.feature_mode)
    opacities = None if opacities is None else _f32(opacities).reshape(-1)
    cam_position = _f32(np.zeros(3) if cam_position is None else cam_position)
    inference = bool(cfg.flags & RASTER_INFERENCE)
    image = np.zeros((Cn, H, W), dtype=np.float32)
    alpha = np.zeros((1, H, W), dtype=np.float32)
    bw = None if inference else np.zeros(n, dtype=np.float32)
    depth_image = np.zeros((1, H, W), dtype=np.float32) if inference else None
    out = {"image": image, "alpha": alpha, "blending_weights": bw, "depth_image": depth_image}
    dbg_ptr = None
    if debug:
        T = cfg.tile
        n_tiles = ((W + T - 1) // T) * ((H + T - 1) // T)
        bufs = {
            "n_touched": np.zeros(n, np.uint32),
            "bounds": np.zeros((n, 4), np.uint16),
            "screen_xy": np.zeros((n, 2), np.float32),
            "depth": np.zeros(n, np.float32),
            "features_view": np.zeros((n, Cn), np.float32),
            "opacity": np.zeros(n, np.float32),
            "counts": np.zeros(2, np.uint32),
            "depth_keys": np.zeros(n, np.uint32),
            "depth_order": np.zeros(n, np.uint32),
            "instance_keys": np.zeros(max(4 * n, n_instances_hint), np.uint16),
            "instance_points": np.zeros(max(4 * n, n_instances_hint), np.uint32),
            "tile_ranges": np.zeros((n_tiles, 2), np.uint32),
            "conic": np.zeros((n, 3), np.float32),
        }
        dbg = _RasterDebug(*[_p(bufs[name]) for name, _ in _RasterDebug._fields_])
        dbg_ptr = C.byref(dbg)
        out.update(bufs)
    if gaussian is not None:
        scales = None if scales is None else _f32(scales).reshape(-1)
        rc = lib().oracle_gaussian_forward(C.byref(gaussian), _p(positions), _p(features), _p(opacities), _p(scales),
                                           _p(w2c), _p(cam_position), _p(image), _p(alpha), _p(bw), _p(depth_image),
                                           dbg_ptr)
    else:
        rc = lib().oracle_raster_forward(C.byref(cfg), _p(positions), _p(features), _p(opacities), _p(w2c),
                                         _p(cam_position), _p(image), _p(alpha), _p(bw), _p(depth_image), dbg_ptr)
    if rc != 0:
        raise RuntimeError(f"oracle raster forward failed with {rc}")
    if debug:
        v, i = int(out["counts"][0]), int(out["counts"][1])
        out["n_visible"], out["n_instances"] = v, i
        for name in ("depth_keys", "depth_order"):
            out[name] = out[name][:v]
        for name in ("instance_keys", "instance_points"):
            out[name] = out[name][:i]
    return out


def gaussian_instance_count(gcfg: GaussianConfig, positions, w2c, scales=None) -> int:
    """Number of (point, tile) instances of a Gaussian-footprint call (sizes the debug buffers)."""
    cfg = gcfg.base
    n = cfg.n_points
    counts = np.zeros(2, np.uint32)
    fields = {name: None for name, _ in _RasterDebug._fields_}
    fields["counts"] = counts
    dbg = _RasterDebug(*[_p(fields[name]) for name, _ in _RasterDebug._fields_])
    W, H = cfg.cam.width, cfg.cam.height
    sh = cfg.feature_mode in (FEAT_SH36_F16, FEAT_RAW37_F16)
    Cn = 4 if sh else cfg.channels
    width = {FEAT_SH36_F16: 36, FEAT_RAW37_F16: 37}.get(cfg.feature_mode, Cn)
    feats = np.zeros((n, width), np.float32 if cfg.feature_mode == FEAT_DIRECT_F32 else np.float16)
    image = np.zeros((Cn, H, W), np.float32)
    alpha = np.zeros((1, H, W), np.float32)
    third = np.zeros(max(n, H * W), np.float32)
    scales = None if scales is None else _f32(scales).reshape(-1)
    rc = lib().oracle_gaussian_forward(C.byref(gcfg), _p(_f32(positions)), _p(feats), _p(np.zeros(n, np.float32)),
                                       _p(scales), _p(_f32(w2c)), _p(np.zeros(3, np.float32)), _p(image), _p(alpha),
                                       _p(third), _p(third), C.byref(dbg))
    if rc != 0:
        raise RuntimeError(f"oracle_gaussian_forward failed with {rc}")
    return int(counts[1])


def footprint_exp(x):
    """exp(x), x <= 0, as the Gaussian footprint evaluates it (elementwise, float32)."""
    x = np.asarray(x, np.float32)
    out = np.empty_like(x)
    f = lib().oracle_footprint_exp
    flat_in, flat_out = x.reshape(-1), out.reshape(-1)
    for i in range(flat_in.size):
        flat_out[i] = f(float(flat_in[i]))
    return out


class _GradAudit(C.Structure):
    _fields_ = [("view64", C.c_void_p), ("opacity64", C.c_void_p), ("view_abs", C.c_void_p), ("opacity_abs", C.c_void_p)]


def raster_backward(cfg: RasterConfig, grad_image, grad_alpha, image, alpha, positions, features, opacities, w2c,
                    cam_position=None, gaussian: "GaussianConfig | None" = None, audit: bool = False):
    """Returns (grad_features, grad_opacities (N,), grad_view (N,C)); with `audit` a fourth value, a dict of float64
    arrays: view64 (N,C) / opacity64 (N) = the gradients with every term evaluated and added in double precision,
    view_abs / opacity_abs = the sums of the magnitudes of what the terms are made of (the conditioning of each sum)."""
    n = cfg.n_points
    sh = cfg.feature_mode in (FEAT_SH36_F16, FEAT_RAW37_F16)
    Cn = 4 if sh else cfg.channels
    positions, w2c = _f32(positions), _f32(w2c)
    features = _features_array(features, cfg.feature_mode)
    opacities = _f32(opacities).reshape(-1)
    cam_position = _f32(np.zeros(3) if cam_position is None else cam_position)
    grad_image, grad_alpha, image, alpha = _f32(grad_image), _f32(grad_alpha), _f32(image), _f32(alpha)
    if cfg.feature_mode == FEAT_SH36_F16:
        gf = np.zeros((n, 36), dtype=np.float16)
    elif cfg.feature_mode == FEAT_DIRECT_F16:
        gf = np.zeros((n, Cn), dtype=np.float16)
    else:
        gf = np.zeros((n, Cn), dtype=np.float32)
    go = np.zeros(n, dtype=np.float32)
    gv = np.zeros((n, Cn), dtype=np.float32)
    if audit:
        extra = {"view64": np.zeros((n, Cn)), "opacity64": np.zeros(n), "view_abs": np.zeros((n, Cn)),
                 "opacity_abs": np.zeros(n)}
        record = _GradAudit(*(_p(extra[k]) for k in ("view64", "opacity64", "view_abs", "opacity_abs")))
        fn = lib().oracle_raster_backward_audit if gaussian is None else lib().oracle_gaussian_backward_audit
        rc = fn(C.byref(cfg if gaussian is None else gaussian), _p(grad_image), _p(grad_alpha), _p(image), _p(alpha),
                _p(positions), _p(features), _p(opacities), _p(w2c), _p(cam_position), _p(gf), _p(go), _p(gv),
                C.byref(record))
        if rc != 0:
            raise RuntimeError(f"oracle_raster_backward_audit failed with {rc}")
        return gf, go, gv, extra
    fn = lib().oracle_raster_backward if gaussian is None else lib().oracle_gaussian_backward
    rc = fn(C.byref(cfg if gaussian is None else gaussian), _p(grad_image), _p(grad_alpha), _p(image), _p(alpha),
            _p(positions), _p(features), _p(opacities), _p(w2c), _p(cam_position), _p(gf), _p(go), _p(gv))
    if rc != 0:
        raise RuntimeError(f"oracle_raster_backward failed with {rc}")
    return gf, go, gv


def raster_forward_backward(cfg: RasterConfig, positions, features, opacities, w2c, grad_image, grad_alpha,
                            cam_position=None):
    """One training step on shared state. Returns (image, alpha, blending_weights, grad_features, grad_opacities)."""
    n = cfg.n_points
    W, H = cfg.cam.width, cfg.cam.height
    sh = cfg.feature_mode in (FEAT_SH36_F16, FEAT_RAW37_F16)
    Cn = 4 if sh else cfg.channels
    positions, w2c = _f32(positions), _f32(w2c)
    features = _features_array(features, cfg.feature_mode)
    opacities = _f32(opacities).reshape(-1)
    cam_position = _f32(np.zeros(3) if cam_position is None else cam_position)
    grad_image, grad_alpha = _f32(grad_image), _f32(grad_alpha)
    image = np.zeros((Cn, H, W), dtype=np.float32)
    alpha = np.zeros((1, H, W), dtype=np.float32)
    bw = np.zeros(n, dtype=np.float32)
    if cfg.feature_mode == FEAT_SH36_F16:
        gf = np.zeros((n, 36), dtype=np.float16)
    elif cfg.feature_mode == FEAT_DIRECT_F16:
        gf = np.zeros((n, Cn), dtype=np.float16)
    else:
        gf = np.zeros((n, Cn), dtype=np.float32)
    go = np.zeros(n, dtype=np.float32)
    rc = lib().oracle_raster_forward_backward(C.byref(cfg), _p(positions), _p(features), _p(opacities), _p(w2c),
                                              _p(cam_position), _p(grad_image), _p(grad_alpha), _p(image), _p(alpha),
                                              _p(bw), _p(gf), _p(go))
    if rc != 0:
        raise RuntimeError(f"oracle_raster_forward_backward failed with {rc}")
    return image, alpha, bw, gf, go


# ----------------------------------------------------------------------------------------------
# probability-field statistics (Modules/ProbabilityField.py:146-157 of the reference), plain numpy
# ----------------------------------------------------------------------------------------------
def field_update(leaf_weights, leaf_scores, indices, weights, decay=0.9968):
    """Returns the updated (leaf_weights, leaf_scores) as new float32 arrays. Follows the reference line by line:
    decay (float32 multiply), per-leaf maximum / minimum of the sampled weights with 0 for leaves without samples
    (scatter_reduce_ amax / amin, include_self=False), maximum with the decayed values, clamped spread."""
    lw = np.asarray(leaf_weights, np.float32) * np.float32(decay)
    ls = np.asarray(leaf_scores, np.float32) * np.float32(decay)
    idx = np.asarray(indices, np.int64)
    w = np.asarray(weights, np.float32).reshape(-1)
    n = lw.shape[0]
    if idx.size and (idx.min() < 0 or idx.max() >= n):
        raise IndexError("sample index outside the leaf range")
    max_sampled = np.full(n, -np.inf, np.float32)
    min_sampled = np.full(n, np.inf, np.float32)
    np.maximum.at(max_sampled, idx, w)
    np.minimum.at(min_sampled, idx, w)
    hit = np.zeros(n, bool)
    hit[idx] = True
    max_sampled[~hit] = 0.0
    min_sampled[~hit] = 0.0
    lw = np.maximum(lw, max_sampled)
    ls = np.maximum(ls, np.clip(max_sampled - min_sampled, np.float32(0.0), np.float32(1.0)))
    return lw.astype(np.float32), ls.astype(np.float32)


# ----------------------------------------------------------------------------------------------
# element-wise steps between sampler and rasterizer, plain numpy in float32
# ----------------------------------------------------------------------------------------------
def field_prune(centers, levels, weights, scores, threshold):
    """Modules/ProbabilityField.py:159-165: the leaves with weight > threshold, in order."""
    w = np.asarray(weights, np.float32)
    keep = w > np.float32(threshold)
    return (np.asarray(centers, np.float32)[keep], np.asarray(levels, np.int32)[keep], w[keep],
            np.asarray(scores, np.float32)[keep])


def field_subdivide(centers, levels, weights, scores, initial_size, threshold, max_level=6, max_leaves=16_777_216):
    """Modules/ProbabilityField.py:217-257, leaf by leaf: the leaves that stay, in order, then eight children per
    split leaf. None when the octree would exceed max_leaves."""
    centers, levels = np.asarray(centers, np.float32), np.asarray(levels, np.int32)
    weights, scores = np.asarray(weights, np.float32), np.asarray(scores, np.float32)
    size = np.broadcast_to(np.asarray(initial_size, np.float32).reshape(-1), (3,))
    split = (scores > np.float32(threshold)) & (levels < max_level)
    n_split, n = int(split.sum()), len(levels)
    if n_split * 8 + (n - n_split) > max_leaves:
        return None
    out_c = [centers[~split]]
    out_l = [levels[~split]]
    out_w = [weights[~split]]
    out_s = [scores[~split]]
    kids_c = np.empty((n_split, 8, 3), np.float32)
    kids_l = np.empty((n_split, 8), np.int32)
    kids_w = np.empty((n_split, 8), np.float32)
    for r, i in enumerate(np.flatnonzero(split)):
        level = int(levels[i]) + 1
        offset = (size / np.float32(2.0 ** (level + 1))).astype(np.float32)
        for c in range(8):
            sign = np.array([1 if c & 1 else -1, 1 if c & 2 else -1, 1 if c & 4 else -1], np.float32)
            kids_c[r, c] = centers[i] + sign * offset
        kids_l[r] = level
        kids_w[r] = weights[i]
    out_c.append(kids_c.reshape(-1, 3))
    out_l.append(kids_l.reshape(-1))
    out_w.append(kids_w.reshape(-1))
    out_s.append(np.zeros(n_split * 8, np.float32))
    return np.concatenate(out_c), np.concatenate(out_l), np.concatenate(out_w), np.concatenate(out_s)


def halton_base(index: int, base: int) -> float:
    """utils.py:36-45."""
    result, f, i = 0.0, 1.0 / base, index
    while i > 0:
        result += f * (i % base)
        i //= base
        f /= base
    return result


def extract_global_samples(centers, levels, initial_size, counts):
    """Modules/ProbabilityField.py:131-140 with utils.py:36-64, sample by sample."""
    centers, levels = np.asarray(centers, np.float32), np.asarray(levels, np.int32)
    counts = np.asarray(counts, np.int64)
    size0 = np.broadcast_to(np.asarray(initial_size, np.float32).reshape(-1), (3,))
    out = np.empty((int(counts.sum()), 3), np.float32)
    s = 0
    for leaf in np.flatnonzero(counts):
        c = int(counts[leaf])
        if c == 1:
            out[s] = centers[leaf]
        else:
            size = (size0 / np.float32(2 ** int(levels[leaf]))).astype(np.float32)
            corner = (centers[leaf] - size / np.float32(2.0)).astype(np.float32)
            for h in range(c):
                coords = np.array([halton_base(h + 1, 2), halton_base(h + 1, 3), halton_base(h + 1, 5)]).astype(np.float32)
                out[s + h] = corner + (coords * size).astype(np.float32)
        s += c
    return out


def morton_encode(positions):
    """63-bit Z-order codes of the positions in their bounding cube, bit by bit: cell = min(uint((p - lo) *
    (2^21 / largest extent)), 2^21 - 1) per axis in float32, bit k of the x / y / z cell at bit 3k / 3k+1 / 3k+2.
    Stands where Modules/ProbabilityField.py:142 calls CudaUtils.MortonEncoding.morton_encode, whose source is not in
    the reference tree (parity with it unpinned; pinned as a Morton code by tests/test_oracle_field.py)."""
    p = np.asarray(positions, np.float32).reshape(-1, 3)
    if len(p) == 0:
        return np.zeros(0, np.int64)
    lo = p.min(0)
    extent = np.float32((p.max(0) - lo).max())
    scale = np.float32(2 ** 21) / extent if extent > 0 else np.float32(0.0)
    q = ((p - lo) * np.float32(scale)).astype(np.float32)
    cells = np.minimum(q.astype(np.uint64), np.uint64(2 ** 21 - 1))
    codes = np.zeros(len(p), np.uint64)
    for k in range(21):
        for axis in range(3):
            codes |= ((cells[:, axis] >> np.uint64(k)) & np.uint64(1)) << np.uint64(3 * k + axis)
    return codes.astype(np.int64)


def spherical_contraction(positions):
    """B/misc/src/misc_kernels.cu:49-66, every operation rounded to float32 in the written order."""
    p = np.asarray(positions, np.float32).reshape(-1, 3)
    f = np.float32
    x, y, z = p[:, 0], p[:, 1], p[:, 2]
    length_sq = np.maximum((x * x + y * y) + z * z, f(1.0))
    scale = (np.sqrt(length_sq) * f(2.0) - f(1.0)) / length_sq * f(0.25)
    return np.clip(scale[:, None] * p + f(0.5), f(0.0), f(1.0)).astype(np.float32)


def feature_to_opacity(raw):
    """utils.py:31-33: -expm1(-exp(x))."""
    x = np.asarray(raw, np.float32)
    return (-np.expm1(-np.exp(x))).astype(np.float32)


def feature_to_opacity_backward(grad, raw):
    """Gradient of the same expression with TruncExp's backward (utils.py:24-28)."""
    x = np.asarray(raw, np.float32)
    g = np.asarray(grad, np.float32)
    return ((g * np.exp(-np.exp(x))) * np.exp(np.clip(x, np.float32(-15.0), np.float32(15.0)))).astype(np.float32)


_DECAY_LEVELS = [177362944, 143808512, 110254080, 76699648, 43145216, 9590784, 1202176, 153600, 22528, 6144]
_DECAY_ENDS = [210917376] + _DECAY_LEVELS[:-1]


def weight_decay_grads(weights, offset=0):
    """B/misc/src/misc_kernels.cu:6-47 for the flat indices offset .. offset + len(weights) - 1."""
    w = np.asarray(weights, np.float32)
    idx = np.arange(w.shape[0], dtype=np.int64) + offset
    factor = np.zeros(w.shape[0], np.float32)
    for begin, end in zip(reversed(_DECAY_LEVELS), reversed(_DECAY_ENDS)):   # ascending thresholds: later ones win
        f = np.float32(np.float32(0.1) * np.float32(2.0)) / np.float32(end - begin)
        factor[idx >= begin] = f
    return (factor * w).astype(np.float32)


def cauchy_loss(input, target):
    d = np.asarray(input, np.float32) - np.asarray(target, np.float32)
    n = np.float32(d.size)
    return (np.log1p(d * d * np.float32(12.5)) / n).astype(np.float32)


def cauchy_loss_backward(grad, input, target):
    d = np.asarray(input, np.float32) - np.asarray(target, np.float32)
    n = np.float32(d.size)
    den = n * (np.float32(12.5) * d * d + np.float32(1.0))
    return (np.float32(25.0) * d / np.maximum(den, np.float32(1e-12)) * np.float32(grad)).astype(np.float32)
