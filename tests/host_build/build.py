"""Builds tests/host_build/geometry_host.hip (the rasterizer's per-point arithmetic compiled for the host) with hipcc
and binds it with ctypes. Test infrastructure: nothing of the product imports this."""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
SOURCE = HERE / "geometry_host.hip"
LIB = HERE / "libgeometry_host.so"
DEPS = [SOURCE, ROOT / "inpc_amd" / "csrc" / "geometry.hpp", ROOT / "inpc_amd" / "csrc" / "common.hpp",
        ROOT / "include" / "inpc_hip.h"]

_lib = None


def lib() -> C.CDLL:
    """The host build of geometry.hpp; compiled when a source is newer than it (same flags as the product: no
    contraction of multiply-adds, no packed fp32)."""
    global _lib
    if _lib is None:
        if not LIB.exists() or any(LIB.stat().st_mtime < d.stat().st_mtime for d in DEPS):
            cmd = ["hipcc", "-O2", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-ffp-contract=off", "-Xclang",
                   "-target-feature", "-Xclang", "-packed-fp32-ops", "-shared", str(SOURCE), "-o", str(LIB)]
            done = subprocess.run(cmd, capture_output=True, text=True, stdin=subprocess.DEVNULL, timeout=600)
            if done.returncode != 0:
                raise RuntimeError(f"hipcc failed on {SOURCE}:\n{done.stderr[-4000:]}")
        _lib = C.CDLL(str(LIB))
    return _lib
