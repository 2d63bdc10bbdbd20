"""Seeded synthetic scenes for tests and benchmarks (numpy only, host memory).

The workloads follow the benchmark configurations of this repository: a pinhole camera on the -z axis
looking at the origin (row-major 4x4 world-to-camera matrix, +z forward, x right, y down, principal
point at the image centre, near 0.01, far 100), an octree of same-level leaves with log-normal
probabilities, and point clouds with random features. Everything is drawn from
numpy.random.Generator(PCG64(seed)).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .views import PerspectiveCamera


@dataclass
class HostView:
    """A view in host memory; `to_view(device)` uploads it for the operator API."""
    camera: PerspectiveCamera
    w2c: np.ndarray       # (4,4) float32
    position: np.ndarray  # (3,) float32

    def to_view(self, device="cuda"):
        import torch

        from .views import View

        return View(self.camera, torch.from_numpy(self.w2c).to(device), torch.from_numpy(self.position).to(device))


def camera_on_z(width: int, height: int, focal: float, distance: float, near: float = 0.01,
                far: float = 100.0) -> HostView:
    """Camera at (0, 0, -distance) looking along +z at the origin."""
    cam = PerspectiveCamera(int(width), int(height), float(focal), float(focal), width / 2.0, height / 2.0, near, far)
    w2c = np.eye(4, dtype=np.float32)
    w2c[2, 3] = np.float32(distance)
    return HostView(cam, w2c, np.array([0.0, 0.0, -distance], dtype=np.float32))


def rotated_camera(width: int, height: int, focal: float, distance: float, yaw: float, pitch: float,
                   near: float = 0.01, far: float = 100.0) -> HostView:
    """Camera orbiting the origin at `distance`, looking at it; yaw about y, pitch about x (radians)."""
    cy, sy, cp, sp = np.cos(yaw), np.sin(yaw), np.cos(pitch), np.sin(pitch)
    ry = np.array([[cy, 0, sy], [0, 1, 0], [-sy, 0, cy]])
    rx = np.array([[1, 0, 0], [0, cp, -sp], [0, sp, cp]])
    rot = rx @ ry                      # world -> camera rotation
    pos = rot.T @ np.array([0.0, 0.0, -distance])
    w2c = np.eye(4)
    w2c[:3, :3] = rot
    w2c[:3, 3] = -rot @ pos
    cam = PerspectiveCamera(int(width), int(height), float(focal), float(focal), width / 2.0, height / 2.0, near, far)
    return HostView(cam, w2c.astype(np.float32), pos.astype(np.float32))


@dataclass
class Octree:
    centers: np.ndarray  # (L,3) float32
    levels: np.ndarray   # (L,) int32
    weights: np.ndarray  # (L,) float32, normalised probabilities
    initial_size: float


def octree_leaves(n_leaves: int, level: int, initial_size: float = 4.0, sigma: float = 1.5, seed: int = 0) -> Octree:
    """`n_leaves` distinct cells of the 2^level grid over [-size/2, size/2]^3 with log-normal(0, sigma)
    probabilities, normalised."""
    rng = np.random.default_rng(seed)
    side = 1 << level
    total = side ** 3
    if n_leaves > total:
        raise ValueError("more leaves than cells")
    picked = np.empty(0, dtype=np.int64)
    while picked.size < n_leaves:  # distinct cells without materialising the population
        extra = rng.integers(0, total, size=int((n_leaves - picked.size) * 1.1) + 16, dtype=np.int64)
        picked = np.unique(np.concatenate([picked, extra]))
    picked = rng.permutation(picked)[:n_leaves]
    picked.sort()
    ix, iy, iz = picked % side, (picked // side) % side, picked // (side * side)
    cell = initial_size / side
    centers = (np.stack([ix, iy, iz], axis=1).astype(np.float64) + 0.5) * cell - initial_size / 2.0
    prob = np.exp(rng.normal(0.0, sigma, size=n_leaves))
    prob /= prob.sum()
    return Octree(centers.astype(np.float32), np.full(n_leaves, level, dtype=np.int32), prob.astype(np.float32),
                  float(initial_size))


def cube_points(n: int, side: float = 1.0, seed: int = 0) -> np.ndarray:
    """n points uniform in a cube of the given side centred at the origin, float32 (n,3)."""
    rng = np.random.default_rng(seed)
    return ((rng.random((n, 3)) - 0.5) * side).astype(np.float32)


def point_attributes(n: int, channels: int, kind: str = "normal", seed: int = 1, dtype=np.float32):
    """(features (n,channels), opacities (n,)). kind "uniform": features ~U(0,1), opacity ~U(0.05,0.95);
    kind "normal": features ~N(0,1), opacity = sigmoid(N(0,1))."""
    rng = np.random.default_rng(seed)
    if kind == "uniform":
        feats = rng.random((n, channels))
        opac = rng.uniform(0.05, 0.95, size=n)
    else:
        feats = rng.normal(size=(n, channels))
        opac = 1.0 / (1.0 + np.exp(-rng.normal(size=n)))
    return feats.astype(dtype), opac.astype(np.float32)


def sh_features(n: int, seed: int = 2) -> np.ndarray:
    """(n,36) fp16 SH coefficients with a dominant DC term, as an appearance field would emit."""
    rng = np.random.default_rng(seed)
    f = rng.normal(scale=0.2, size=(n, 36))
    f[:, :4] += 1.0
    return f.astype(np.float16)
