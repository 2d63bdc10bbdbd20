"""Duck-typed stand-ins for the camera / view objects the operator API receives.

The reference unpacks `view.w2c`, `view.position` and `view.camera.{width, height, focal_x, focal_y,
center_x, center_y, near_plane, far_plane, distortion}` (B/torch_bindings/sampling.py:16-33,
B/torch_bindings/rasterization.py:105-128). Those objects come from the NeRFICG framework, which is
not a dependency of this package: anything with the same attributes works, and these two small classes
provide them for tests, benchmarks and stand-alone use.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

_CAMERA_FIELDS = ("width", "height", "focal_x", "focal_y", "center_x", "center_y", "near_plane", "far_plane")


@dataclass
class PerspectiveCamera:
    width: int
    height: int
    focal_x: float
    focal_y: float
    center_x: float
    center_y: float
    near_plane: float = 0.01
    far_plane: float = 100.0
    distortion: Optional[Any] = None


@dataclass
class View:
    camera: Any
    w2c: Any        # (4,4) float32 tensor on the GPU, row-major, +z forward, x right, y down
    position: Any   # (3,) float32 tensor on the GPU: camera centre in world space


_framework_camera = False   # False: not looked up yet; None: the framework is not importable


def _framework_camera_class():
    """The NeRFICG framework's PerspectiveCamera, or None; looked up once (a failing import is not cached by
    Python and costs a walk over sys.path every time)."""
    global _framework_camera
    if _framework_camera is False:
        try:  # pragma: no cover - only with the NeRFICG framework on the path
            from Cameras.Perspective import PerspectiveCamera as FrameworkCamera

            _framework_camera = FrameworkCamera
        except ImportError:
            _framework_camera = None
    return _framework_camera


def is_perspective(camera) -> bool:
    """True for a pinhole camera: the framework's PerspectiveCamera when it is importable, else any
    object that carries the pinhole scalars."""
    framework = _framework_camera_class()
    if framework is not None and isinstance(camera, framework):
        return True
    return all(hasattr(camera, f) for f in _CAMERA_FIELDS)
