"""Build libinpc_hip.so (the gfx950 kernels and their C ABI) in-tree with hipcc.

Usage: python -m inpc_amd.build [--force]
"""
from __future__ import annotations

import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libinpc_hip.so"
SOURCES = ["runtime.hip", "sampler.hip", "raster.hip", "field.hip", "misc.hip"]
HEADERS = ["common.hpp", "geometry.hpp", "blend.hpp", "tilesort.hpp", "gaussian.hpp"]

# -ffp-contract=off: tile bounds, depth keys, leaf picks and cull decisions must be bit-identical to
#   a CPU evaluation of the same expressions, so nothing may be fused behind the source's back.
# -packed-fp32-ops is switched off so the compiler never forms packed fp32 arithmetic.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build(force: bool = False, verbose: bool = False) -> Path:
    """Compile every source and link the shared library. Always recompiles when force is set,
    otherwise only when a source or header is newer than the library."""
    deps = [CSRC / s for s in SOURCES + HEADERS] + [PKG_DIR.parent / "include" / "inpc_hip.h"]
    if not force and LIB_PATH.exists() and all(LIB_PATH.stat().st_mtime >= d.stat().st_mtime for d in deps):
        return LIB_PATH
    objects = []
    procs = []
    for src in SOURCES:
        obj = CSRC / (Path(src).stem + ".o")
        cmd = ["hipcc", *HIPCC_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objects.append(str(obj))
    failed = False
    for src, proc in procs:
        out, _ = proc.communicate()
        if proc.returncode != 0:
            failed = True
            sys.stderr.write(f"--- hipcc failed on {src} ---\n{out}\n")
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("hipcc failed; see messages above")
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *objects]
    subprocess.run(link, check=True)
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, verbose=True)
    print(f"built {path}")
