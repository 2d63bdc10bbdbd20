"""Thin test-side wrappers that call libinpc_hip.so through its C ABI with torch device buffers and
return numpy arrays shaped like the oracle's outputs."""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from inpc_amd import _lib

# Where the wrappers below put their buffers when the caller names no device. The simulator tier (tests/cpu_sim)
# sets it to "cpu" while the kernels compiled for the host are the loaded library.
DEVICE = "cuda:0"


def device_of(device=None):
    return torch.device(DEVICE if device is None else device)


def dev(a, device=None):
    """A tensor on the device with a copy of `a` (a copy also where the device is the host: the kernels write into
    their arguments, and the caller keeps comparing against `a`)."""
    device = device_of(device)
    host = torch.from_numpy(np.ascontiguousarray(a))
    return host.clone() if device.type == "cpu" else host.to(device)


def poisoned_bytes(n_bytes: int, device) -> torch.Tensor:
    """n_bytes of random bytes on `device`, 256-byte aligned like every allocation of the GPU's allocator (a host
    allocation is only 64-byte aligned: a slice that starts at the next multiple of 256 is taken)."""
    raw = torch.randint(0, 256, (n_bytes + 256,), dtype=torch.uint8, device=device)
    skip = (-raw.data_ptr()) % 256
    return raw[skip:skip + n_bytes]


def cam_struct(camera) -> _lib.Camera:
    return _lib.make_camera(camera)


def stream():
    return _lib.current_stream()


def make_rng(seed: int, device=None):
    host = (C.c_uint64 * 2)()
    _lib.lib().inpc_pcg32_seed(host, C.c_uint64(seed), C.c_uint64(1))
    signed = [int(v) - 2**64 if int(v) >= 2**63 else int(v) for v in host]
    return torch.tensor(signed, dtype=torch.int64, device=device_of(device))


def rng_values(rng_dev):
    s, i = rng_dev.cpu().tolist()
    return s % 2**64, i % 2**64


def leaf_weights(oct, hv, device=None):
    device = device_of(device)
    lib = _lib.lib()
    n = len(oct.levels)
    out = torch.empty(n, dtype=torch.float32, device=device)
    cam = cam_struct(hv.camera)
    # keep the uploads alive until the launch is queued: a temporary's memory is recycled at once
    centers, levels, weights, w2c = dev(oct.centers), dev(oct.levels), dev(oct.weights), dev(hv.w2c)
    _lib.check(lib.inpc_leaf_weights(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(weights), _lib.ptr(w2c),
                                     _lib.ptr(out), None, n, C.byref(cam), oct.initial_size, stream()),
               "inpc_leaf_weights")
    return out


def leaf_boxes(oct, hv=None, device=None):
    """(L, 4) device tensor {centre, edge length} as inpc_leaf_weights writes it for the sampling calls
    (the camera does not enter it)."""
    from inpc_amd import synthetic

    if hv is None:
        hv = synthetic.camera_on_z(8, 8, 8.0, 1.0)
    device = device_of(device)
    lib = _lib.lib()
    n = len(oct.levels)
    out = torch.empty(n, dtype=torch.float32, device=device)
    boxes = torch.full((n, 4), float("nan"), dtype=torch.float32, device=device)
    cam = cam_struct(hv.camera)
    centers, levels, weights, w2c = dev(oct.centers), dev(oct.levels), dev(oct.weights), dev(hv.w2c)
    _lib.check(lib.inpc_leaf_weights(_lib.ptr(centers), _lib.ptr(levels), _lib.ptr(weights), _lib.ptr(w2c),
                                     _lib.ptr(out), _lib.ptr(boxes), n, C.byref(cam), oct.initial_size, stream()),
               "inpc_leaf_weights")
    return boxes


def build_cdf(w_dev):
    lib = _lib.lib()
    n = w_dev.numel()
    cdf = w_dev.clone()
    ws_bytes = int(lib.inpc_sampler_workspace_bytes(n))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=w_dev.device)
    total = torch.zeros(int(lib.inpc_cdf_head_floats(n)), dtype=torch.float32, device=w_dev.device)  # [0] = total
    _lib.check(lib.inpc_build_cdf(_lib.ptr(cdf), _lib.ptr(total), total.numel(), _lib.ptr(ws), ws_bytes, n, stream()),
               "inpc_build_cdf")
    return cdf, total


def sample(oct, cdf, total, n_samples, rng_dev):
    lib = _lib.lib()
    device = cdf.device
    pos = torch.full((n_samples, 3), float("nan"), dtype=torch.float32, device=device)
    ids = torch.full((n_samples,), -7, dtype=torch.int32, device=device)
    boxes = leaf_boxes(oct)
    _lib.check(lib.inpc_sample(_lib.ptr(boxes), _lib.ptr(cdf), _lib.ptr(total), total.numel(), _lib.ptr(pos),
                               _lib.ptr(ids), n_samples, len(oct.levels), _lib.ptr(rng_dev), stream()), "inpc_sample")
    return pos.cpu().numpy(), ids.cpu().numpy()


class CullDraw:
    """One training draw made of explicit rounds."""

    def __init__(self, oct, hv, cdf, total, rng_dev, capacity, max_round, ids_int64=False):
        self.lib = _lib.lib()
        self.ids_int64 = int(ids_int64)
        self.oct, self.hv, self.cdf, self.total, self.rng = oct, hv, cdf, total, rng_dev
        self.capacity = capacity
        device = cdf.device
        self.boxes, self.w2c = leaf_boxes(oct, hv), dev(hv.w2c)
        self.pos = torch.full((capacity, 3), float("nan"), dtype=torch.float32, device=device)
        self.ids = torch.full((capacity,), -7, dtype=torch.int64 if ids_int64 else torch.int32, device=device)
        self.ws_bytes = int(self.lib.inpc_cull_workspace_bytes(max_round))
        # poisoned: the round that starts at candidate 0 clears the state of the draw itself
        self.ws = poisoned_bytes(self.ws_bytes, device)
        self.cam = cam_struct(hv.camera)
        self.k0 = 0

    def round(self, n_candidates):
        _lib.check(self.lib.inpc_sample_cull_compact(
            _lib.ptr(self.boxes), _lib.ptr(self.cdf), _lib.ptr(self.total), self.total.numel(), _lib.ptr(self.w2c),
            _lib.ptr(self.pos), _lib.ptr(self.ids), self.ids_int64, self.capacity, self.k0, n_candidates,
            len(self.oct.levels), C.byref(self.cam), _lib.ptr(self.rng), _lib.ptr(self.ws), self.ws_bytes, stream()),
            "inpc_sample_cull_compact")
        self.k0 += n_candidates
        return self.counts()

    def counts(self):
        a, c = C.c_uint32(0), C.c_uint32(0)
        _lib.check(self.lib.inpc_cull_read_counts(_lib.ptr(self.ws), C.byref(a), C.byref(c), stream()),
                   "inpc_cull_read_counts")
        return int(a.value), int(c.value)

    def finish(self):
        _lib.check(self.lib.inpc_cull_finish(_lib.ptr(self.total), _lib.ptr(self.pos), _lib.ptr(self.ids), self.ids_int64,
                                             self.capacity, self.k0, _lib.ptr(self.rng), _lib.ptr(self.ws),
                                             self.ws_bytes, stream()), "inpc_cull_finish")


FEATURE_DTYPES = {_lib.FEAT_SH36_F16: np.float16, _lib.FEAT_DIRECT_F32: np.float32, _lib.FEAT_DIRECT_F16: np.float16,
                  _lib.FEAT_RAW37_F16: np.float16}


class RasterRun:
    """inpc_raster_forward (+ backward) through the C ABI on numpy inputs."""

    def __init__(self, hv, positions, features, opacities, tile=16, channels=4, feature_mode=_lib.FEAT_DIRECT_F32,
                 inference=False, device=None, max_instances=None, keep_geometry=True):
        self.lib = _lib.lib()
        self.hv = hv
        self.n = len(positions)
        sh = feature_mode in (_lib.FEAT_SH36_F16, _lib.FEAT_RAW37_F16)
        self.C = 4 if sh else channels
        flags = (_lib.RASTER_INFERENCE if inference else 0) | (_lib.RASTER_KEEP_GEOMETRY if keep_geometry else 0)
        # room for every possible instance unless a test asks for less
        capacity = max(4 * self.n, 1) if max_instances is None else max_instances
        self.cfg = _lib.RasterConfig(self.n, tile, self.C, feature_mode, flags, cam_struct(hv.camera), capacity)
        self.layout = _lib.RasterLayout()
        _lib.check(self.lib.inpc_raster_layout_query(C.byref(self.cfg), C.byref(self.layout)), "layout")
        self.inference = inference
        self.device = device = device_of(device)
        self.positions = dev(np.asarray(positions, np.float32).reshape(-1, 3), device)
        self.features = dev(np.asarray(features, FEATURE_DTYPES[feature_mode]), device)
        self.opacities = None if opacities is None else dev(np.asarray(opacities, np.float32).reshape(-1), device)
        self.w2c = dev(hv.w2c, device)
        self.cam_position = dev(hv.position, device)
        H, W = hv.camera.height, hv.camera.width
        self.image = torch.full((self.C, H, W), float("nan"), dtype=torch.float32, device=device)
        self.alpha = torch.full((1, H, W), float("nan"), dtype=torch.float32, device=device)
        self.bw = None if inference else torch.full((max(self.n, 1),), float("nan"), dtype=torch.float32, device=device)
        self.depth_image = torch.full((1, H, W), float("nan"), dtype=torch.float32, device=device) if inference else None
        # poisoned: nothing may depend on what the workspace held before the call
        self.ws = poisoned_bytes(self.layout.total_bytes, device)

    def forward(self):
        _lib.check(self.lib.inpc_raster_forward(
            C.byref(self.cfg), _lib.ptr(self.positions), _lib.ptr(self.features), _lib.ptr(self.opacities),
            _lib.ptr(self.w2c), _lib.ptr(self.cam_position), _lib.ptr(self.image), _lib.ptr(self.alpha),
            _lib.ptr(self.bw), _lib.ptr(self.depth_image), _lib.ptr(self.ws), self.layout.total_bytes, stream()),
            "inpc_raster_forward")
        return self

    def counters(self):
        out = (C.c_uint32 * 3)()
        _lib.check(self.lib.inpc_raster_read_counters(C.byref(self.cfg), _lib.ptr(self.ws), C.byref(out), stream()),
                   "inpc_raster_read_counters")
        return int(out[0]), int(out[1])

    def _buf(self, offset, count, dtype):
        nbytes = count * np.dtype(dtype).itemsize
        return self.ws[offset:offset + nbytes].cpu().numpy().view(dtype)

    def debug(self):
        """Intermediate buffers decoded into the oracle's shapes. Needs keep_geometry."""
        L, n = self.layout, self.n
        v, i = self.counters()
        assert L.debug_geometry != 0, "RasterRun(keep_geometry=True) keeps the projection for inspection"
        geo = self._buf(L.debug_geometry, 4 * n, np.float32).reshape(n, 4)
        info = geo.view(np.uint32)[:, 3]
        drawn = ((info >> 18) & 1).astype(bool)
        assert int(drawn.sum()) == v, "the visible count differs from the number of drawn points"
        tile0 = info & 0xFFFF
        nx = ((info >> 16) & 1) + 1
        ny = ((info >> 17) & 1) + 1
        x0, y0 = tile0 % L.grid_width, tile0 // L.grid_width
        n_touched = np.where(drawn, nx * ny, 0).astype(np.uint32)
        bounds = np.where(drawn[:, None], np.stack([x0, x0 + nx, y0, y0 + ny], axis=1), 0).astype(np.uint16)
        xy = np.where(drawn[:, None], geo[:, :2], 0).astype(np.float32)
        depth = np.where(drawn, geo[:, 2], 0).astype(np.float32)
        assert int(n_touched.sum()) == i, "the instance count differs from the sum of the touched tiles"
        # blend records: one per drawn point, at the point's index
        stride = L.record_stride
        raw = self._buf(L.point_record, n * stride, np.uint8).reshape(n, stride)
        head = raw[:, :32].copy().view(np.float32).reshape(n, 8)
        head_u = head.view(np.uint32)
        tag = head_u[:, 5]
        assert ((tag & 0x0FFFFFFF)[drawn] == np.nonzero(drawn)[0]).all(), "a record does not name its own point"
        assert ((((tag >> 29) & 3) == ((info >> 16) & 3)) | ~drawn).all(), "span bits of a record differ from its bounds"
        if not self.inference:
            assert ((((tag >> 28) & 1) == (n_touched > 1)) | ~drawn).all(), "several-tiles flag of a record is wrong"
        # footprint weights against the float expressions of the reference's blend (kernels.cu:284-287) at the two
        # candidate pixels per axis, from the kept screen position
        left = (head_u[:, 6] & 0xFFFF).astype(np.int64) - 1
        top = (head_u[:, 6] >> 16).astype(np.int64) - 1
        for axis, first, w0, w1 in ((0, left, head[:, 0], head[:, 1]), (1, top, head[:, 2], head[:, 3])):
            s_ = geo[:, axis]
            with np.errstate(invalid="ignore"):   # points that are not drawn may have any screen position
                expect_first = np.floor((s_ - np.float32(0.5)).astype(np.float32)).astype(np.int64)
            assert (first[drawn] == expect_first[drawn]).all(), "left / top candidate pixel of a record is wrong"
            for k, w in ((0, w0), (1, w1)):
                d = np.abs(s_ - ((first + k).astype(np.float32) + np.float32(0.5))).astype(np.float32)
                expect = np.where(d >= 1, np.float32(0), np.clip(np.float32(1) - d, 0, 1)).astype(np.float32)
                assert (w.view(np.uint32)[drawn] == expect.view(np.uint32)[drawn]).all(), "footprint weight of a record is wrong"
        opacity = np.where(drawn, head[:, 4], 0).astype(np.float32)
        feat_dtype = np.float16 if self.cfg.feature_mode == _lib.FEAT_DIRECT_F16 else np.float32
        feats = raw[:, 32:32 + self.C * np.dtype(feat_dtype).itemsize].copy().view(feat_dtype).reshape(n, self.C)
        features_view = np.where(drawn[:, None], feats.astype(np.float32), 0).astype(np.float32)
        bin_start = self._buf(L.bin_start, L.n_tiles + 1, np.uint32)
        assert bin_start[0] == 0 and bin_start[-1] == i and (np.diff(bin_start.astype(np.int64)) >= 0).all()
        points = self._buf(L.instance_points, max(i, 1), np.uint32)[:i]
        keys = np.repeat(np.arange(L.n_tiles, dtype=np.uint16), np.diff(bin_start.astype(np.int64)))
        return {
            "n_visible": v, "n_instances": i, "n_touched": n_touched, "bounds": bounds, "screen_xy": xy,
            "opacity": opacity, "depth": depth, "features_view": features_view,
            "instance_keys": keys, "instance_points": points,
            # depth key of every instance, in final order: what the per-tile sort ordered by
            "instance_depth_keys": geo.view(np.uint32)[points, 2],
            "tile_ranges": self._buf(L.tile_ranges, 2 * L.n_tiles, np.uint32).reshape(-1, 2),
        }

    def outputs(self):
        out = {"image": self.image.cpu().numpy(), "alpha": self.alpha.cpu().numpy()}
        if self.inference:
            out["depth_image"] = self.depth_image.cpu().numpy()
        else:
            out["blending_weights"] = self.bw.cpu().numpy()[:self.n]
        return out

    def backward_async(self, gi, ga):
        """Enqueues the backward pass on the current stream; device tensors in, device tensors out. The scratch
        buffer is kept on the object so that it outlives the call."""
        mode = self.cfg.feature_mode
        n, Cn = self.n, self.C
        device = self.device
        self._scratch = None
        if mode == _lib.FEAT_SH36_F16:
            gf = torch.full((n, 36), float("nan"), dtype=torch.float16, device=device)
            self._scratch = torch.empty((n, 4), dtype=torch.float32, device=device)
        elif mode == _lib.FEAT_DIRECT_F16:
            gf = torch.full((n, Cn), float("nan"), dtype=torch.float16, device=device)
            self._scratch = torch.empty((n, Cn), dtype=torch.float32, device=device)
        else:
            gf = torch.full((n, Cn), float("nan"), dtype=torch.float32, device=device)
        go = torch.full((n,), float("nan"), dtype=torch.float32, device=device)
        self._grads_in = (gi, ga)
        _lib.check(self.lib.inpc_raster_backward(
            C.byref(self.cfg), _lib.ptr(gi), _lib.ptr(ga), _lib.ptr(self.image), _lib.ptr(self.alpha),
            _lib.ptr(self.positions), _lib.ptr(self.cam_position), _lib.ptr(gf), _lib.ptr(go), _lib.ptr(self._scratch),
            _lib.ptr(self.ws), self.layout.total_bytes, stream()),
            "inpc_raster_backward")
        return gf, go

    def backward(self, grad_image, grad_alpha):
        device = self.device
        gf, go = self.backward_async(dev(np.asarray(grad_image, np.float32), device),
                                     dev(np.asarray(grad_alpha, np.float32), device))
        return gf.cpu().numpy(), go.cpu().numpy()


class GaussianRun:
    """inpc_gaussian_forward (+ backward) through the C ABI on numpy inputs."""

    def __init__(self, hv, positions, features, opacities, tile=8, channels=4, feature_mode=_lib.FEAT_DIRECT_F32,
                 inference=False, scales=None, sigma_world=0.0, sigma_cutoff=3.0, max_instances=0, device=None):
        self.lib = _lib.lib()
        self.n = len(positions)
        sh = feature_mode in (_lib.FEAT_SH36_F16, _lib.FEAT_RAW37_F16)
        self.C = 4 if sh else channels
        base = _lib.RasterConfig(self.n, tile, self.C, feature_mode, _lib.RASTER_INFERENCE if inference else 0,
                                 cam_struct(hv.camera))
        self.cfg = _lib.GaussianConfig(base, sigma_world, sigma_cutoff, max_instances, 0)
        self.layout = _lib.GaussianLayout()
        _lib.check(self.lib.inpc_gaussian_layout_query(C.byref(self.cfg), C.byref(self.layout)), "layout")
        self.inference = inference
        self.device = device = device_of(device)
        self.positions = dev(np.asarray(positions, np.float32).reshape(-1, 3), device)
        self.features = dev(np.asarray(features, FEATURE_DTYPES[feature_mode]), device)
        self.opacities = None if opacities is None else dev(np.asarray(opacities, np.float32).reshape(-1), device)
        self.scales = None if scales is None else dev(np.asarray(scales, np.float32).reshape(-1), device)
        self.w2c = dev(hv.w2c, device)
        self.cam_position = dev(hv.position, device)
        H, W = hv.camera.height, hv.camera.width
        self.image = torch.full((self.C, H, W), float("nan"), dtype=torch.float32, device=device)
        self.alpha = torch.full((1, H, W), float("nan"), dtype=torch.float32, device=device)
        self.bw = None if inference else torch.full((max(self.n, 1),), float("nan"), dtype=torch.float32, device=device)
        self.depth_image = torch.full((1, H, W), float("nan"), dtype=torch.float32, device=device) if inference else None
        # poisoned: nothing may depend on what the workspace held before the call
        self.ws = poisoned_bytes(self.layout.total_bytes, device)

    def forward(self):
        _lib.check(self.lib.inpc_gaussian_forward(
            C.byref(self.cfg), _lib.ptr(self.positions), _lib.ptr(self.features), _lib.ptr(self.opacities),
            _lib.ptr(self.scales), _lib.ptr(self.w2c), _lib.ptr(self.cam_position), _lib.ptr(self.image),
            _lib.ptr(self.alpha), _lib.ptr(self.bw), _lib.ptr(self.depth_image), _lib.ptr(self.ws),
            self.layout.total_bytes, stream()), "inpc_gaussian_forward")
        return self

    def counters(self, check=True):
        """(return code, [n_visible, n_instances, error flag, instances drawn])"""
        out = (C.c_uint32 * 4)()
        rc = self.lib.inpc_gaussian_read_counters(C.byref(self.cfg), _lib.ptr(self.ws), C.byref(out), stream())
        if check:
            _lib.check(rc, "inpc_gaussian_read_counters")
        return rc, [int(v) for v in out]

    def _buf(self, offset, count, dtype):
        nbytes = count * np.dtype(dtype).itemsize
        return self.ws[offset:offset + nbytes].cpu().numpy().view(dtype)

    def debug(self):
        """Intermediate buffers in the oracle's shapes."""
        L, n = self.layout, self.n
        _, (v, i, _, kept) = self.counters()
        assert kept == i
        touched = self._buf(L.point_touched, n, np.uint32).copy()
        vis = touched > 0
        packed = self._buf(L.point_bounds, 2 * n, np.uint32).reshape(n, 2)
        bounds = np.stack([packed[:, 0] & 0xFFFF, packed[:, 0] >> 16, packed[:, 1] & 0xFFFF, packed[:, 1] >> 16],
                          axis=1).astype(np.uint16)
        bounds[~vis] = 0
        stride = L.record_stride
        raw = self._buf(L.point_record, n * stride, np.uint8).reshape(n, stride)
        head = raw[:, :32].copy().view(np.float32).reshape(n, 8)
        word = head.view(np.uint32)[:, 7]
        assert (word[vis] & 0x0FFFFFFF == np.flatnonzero(vis)).all(), "a record names another point"
        assert ((word[vis] >> 31) == (touched[vis] > 1)).all(), "the several-tiles flag differs from the tile count"
        columns = (bounds[:, 1].astype(np.int64) - bounds[:, 0])[vis]
        assert (((word[vis] >> 28) & 7) == np.minimum(columns, 7)).all(), "the tile-column bits differ from the bounds"
        feats = raw[:, 32:32 + 4 * self.C].copy().view(np.float32).reshape(n, self.C)

        def drawn(a):
            a = a.copy()
            a[~vis] = 0
            return a

        # the depth of a point as the sort saw it (the record's depth word of a point that touches several tiles is
        # reused by the training configurations); the order the reference's depth sort would give: by (key, point)
        point_keys = self._buf(L.depth_keys, n, np.uint32).copy()
        assert (point_keys[~vis] == 0xFFFFFFFF).all(), "a point that is not drawn has a depth key"
        depth_order = np.flatnonzero(vis)[np.argsort(point_keys[vis], kind="stable")].astype(np.uint32)
        depth_keys = (point_keys[depth_order] + np.uint32(L.depth_key_bias)).astype(np.uint32)
        depth = np.zeros(n, np.float32)
        depth[depth_order] = depth_keys.view(np.float32)
        single = vis & (touched == 1)
        assert (head[single, 6].view(np.uint32) == depth[single].view(np.uint32)).all(), "record depth differs from the key"
        if self.inference:
            assert (head[vis, 6].view(np.uint32) == depth[vis].view(np.uint32)).all(), "record depth differs from the key"

        # the tiles' lists lie one after the other in tile order
        ranges = self._buf(L.tile_ranges, 2 * L.n_tiles, np.uint32).reshape(-1, 2).copy()
        lengths = (ranges[:, 1].astype(np.int64) - ranges[:, 0]).astype(np.int64)
        filled = lengths > 0
        assert int(lengths.sum()) == i, "the tile ranges do not add up to the instance count"
        starts = np.concatenate([[0], np.cumsum(lengths)[:-1]])
        assert (ranges[filled, 0] == starts[filled]).all(), "the tile ranges leave gaps or overlap"
        instance_keys = np.repeat(np.arange(L.n_tiles, dtype=np.uint16), lengths)
        points = self._buf(L.instance_points, max(i, 1), np.uint32)[:i].copy()
        return {
            "n_visible": v, "n_instances": i, "n_touched": touched, "bounds": bounds,
            "screen_xy": drawn(head[:, :2]), "opacity": drawn(head[:, 2]), "conic": drawn(head[:, 3:6]),
            "depth": depth, "features_view": drawn(feats),
            "depth_keys": depth_keys, "depth_order": depth_order,
            "instance_keys": instance_keys,
            "instance_points": points,
            # depth key of every instance, in final order: what the per-tile sort ordered by
            "instance_depth_keys": (point_keys[points] + np.uint32(L.depth_key_bias)).astype(np.uint32),
            "tile_ranges": ranges,
        }

    outputs = RasterRun.outputs

    def backward_async(self, gi, ga):
        """Enqueues the backward pass on the current stream; device tensors in, device tensors out."""
        mode = self.cfg.base.feature_mode
        n, Cn = self.n, self.C
        device = self.device
        self._scratch = None
        if mode == _lib.FEAT_SH36_F16:
            gf = torch.full((n, 36), float("nan"), dtype=torch.float16, device=device)
            self._scratch = torch.empty((n, 4), dtype=torch.float32, device=device)
        elif mode == _lib.FEAT_DIRECT_F16:
            gf = torch.full((n, Cn), float("nan"), dtype=torch.float16, device=device)
            self._scratch = torch.empty((n, Cn), dtype=torch.float32, device=device)
        else:
            gf = torch.full((n, Cn), float("nan"), dtype=torch.float32, device=device)
        go = torch.full((n,), float("nan"), dtype=torch.float32, device=device)
        self._grads_in = (gi, ga)
        _lib.check(self.lib.inpc_gaussian_backward(
            C.byref(self.cfg), _lib.ptr(gi), _lib.ptr(ga), _lib.ptr(self.image), _lib.ptr(self.alpha),
            _lib.ptr(self.positions), _lib.ptr(self.cam_position), _lib.ptr(gf), _lib.ptr(go), _lib.ptr(self._scratch),
            _lib.ptr(self.ws), self.layout.total_bytes, stream()), "inpc_gaussian_backward")
        return gf, go

    def backward(self, grad_image, grad_alpha):
        device = self.device
        gf, go = self.backward_async(dev(np.asarray(grad_image, np.float32), device),
                                     dev(np.asarray(grad_alpha, np.float32), device))
        return gf.cpu().numpy(), go.cpu().numpy()


# A gradient of the rasterizer is a sum of one term per (instance, pixel), of both signs for most points: evaluated in
# fp32, in whatever order, it is good to a few rounding units (2^-24) of the sum of the magnitudes its terms are made
# of, however small the sum itself comes out. kGradUnits is how many of those units a result may be away from the same
# sum taken in double precision, on top of the 1e-4 relative tolerance of the comparison. Sixteen: a term of the
# opacity gradient goes through a dot product over the channels and two running sums before it is added; over 2,500
# random scenes the CPU oracle's own fp32 sums needed up to 9.6 units and the HIP kernels' up to 11.5 (feature
# gradients: 1.7 and 1.9).
kGradUnits = 16.0


def assert_gradient_close(actual, audit, name, what="", rtol=1e-4, units=kGradUnits):
    """|actual - f64| <= rtol * |f64| + units * 2^-24 * (sum of magnitudes), element by element; `audit` is the fourth
    value of oracle.raster_backward(..., audit=True) and `name` is "view" or "opacity". Returns the largest number of
    rounding units any element needed beyond the relative tolerance."""
    actual = np.asarray(actual, np.float64)
    exact, magnitude = audit[name + "64"], audit[name + "_abs"]
    assert actual.shape == exact.shape, f"{what}: shape {actual.shape} vs {exact.shape}"
    assert np.isfinite(actual).all(), f"{what}: {int((~np.isfinite(actual)).sum())} non-finite elements"
    err = np.abs(actual - exact)
    unit = 2.0 ** -24 * magnitude
    beyond = np.maximum(err - rtol * np.abs(exact), 0.0)
    bad = beyond > units * unit
    if bad.any():
        idx = np.unravel_index(np.argmax(beyond - units * unit), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} elements differ; worst at {idx}: "
                             f"{actual[idx]!r} vs {exact[idx]!r} (|err|={err[idx]:.3e}, sum of magnitudes "
                             f"{magnitude[idx]:.3e}: {beyond[idx] / max(unit[idx], 1e-300):.1f} rounding units)")
    with np.errstate(divide="ignore", invalid="ignore"):
        used = np.where(unit > 0, beyond / unit, 0.0)
    return float(used.max(initial=0.0))


def assert_close(actual, expected, rtol=1e-4, atol=1e-6, what=""):
    """allclose with a report of the worst element."""
    actual, expected = np.asarray(actual, np.float64), np.asarray(expected, np.float64)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} vs {expected.shape}"
    err = np.abs(actual - expected)
    tol = atol + rtol * np.abs(expected)
    bad = err > tol
    if bad.any() or not np.isfinite(actual).all():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} elements differ; worst at {idx}: "
                             f"{actual[idx]!r} vs {expected[idx]!r} (|err|={err[idx]:.3e}); "
                             f"non-finite: {int((~np.isfinite(actual)).sum())}")


def extreme_positions(hv, n, seed):
    """Points of a cube around the origin of which four tenths are extreme: a coordinate that is NaN, infinite, huge
    (1e30, 3e38) or denormal-small, and depths on, just inside and just outside zero and the two clipping planes."""
    from inpc_amd import synthetic

    rng = np.random.default_rng(seed)
    pos = synthetic.cube_points(n, 2.0, seed)
    k = max(1, n // 10)
    order = rng.permutation(n)
    specials = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 3e38, 1e-30, -1e-30, 0.0], np.float32)
    for j in range(3):
        chosen = order[j * k:(j + 1) * k]
        pos[chosen, rng.integers(0, 3, len(chosen))] = specials[rng.integers(0, len(specials), len(chosen))]
    chosen = order[3 * k:4 * k]
    depths = np.array([0.0, 1e-9, -1e-9, 0.01, 0.0099999, 0.0100001, 100.0, 99.9999, 100.0001], np.float32)
    # synthetic.camera_on_z looks along +z from (0, 0, -distance): camera-space depth = z - position.z
    pos[chosen, 2] = (rng.choice(depths, len(chosen)) + np.float32(hv.position[2])).astype(np.float32)
    return pos
