"""Build libinpc_hip.so (the gfx950 kernels and their C ABI) in-tree with hipcc.

Usage: python -m inpc_amd.build [--force]
"""
from __future__ import annotations

import json
import re
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libinpc_hip.so"
RESOURCES_PATH = PKG_DIR / "kernel_resources.json"   # what the compiler reports per kernel, written with the library
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
    "-Rpass-analysis=kernel-resource-usage",   # registers, scratch, LDS and occupancy of every kernel (remarks)
]

_REMARKS = (("vgprs", r" VGPRs: (\d+)"), ("agprs", r" AGPRs: (\d+)"), ("sgprs", r" SGPRs: (\d+)"),
            ("scratch_bytes_per_lane", r"ScratchSize \[bytes/lane\]: (\d+)"),
            ("occupancy_waves_per_simd", r"Occupancy \[waves/SIMD\]: (\d+)"),
            ("lds_bytes_per_block", r"LDS Size \[bytes/block\]: (\d+)"))


def _kernel_resources(compiler_output: str) -> tuple[dict, str]:
    """The compiler's resource remarks as {mangled kernel name: figures}, and the output without them."""
    kernels, current, rest = {}, None, []
    for line in compiler_output.splitlines():
        if "[-Rpass-analysis=kernel-resource-usage]" not in line:
            rest.append(line)
            continue
        name = re.search(r"Function Name: (\S+)", line)
        if name:
            current = kernels.setdefault(name.group(1), {})
            continue
        for key, pattern in _REMARKS:
            found = re.search(pattern, line)
            if found and current is not None:
                current[key] = int(found.group(1))
    return kernels, "\n".join(rest)


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
    resources = {}
    for src, proc in procs:
        out, _ = proc.communicate()
        kernels, out = _kernel_resources(out)
        resources[src] = kernels
        if proc.returncode != 0:
            failed = True
            sys.stderr.write(f"--- hipcc failed on {src} ---\n{out}\n")
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("hipcc failed; see messages above")
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *objects]
    subprocess.run(link, check=True)
    RESOURCES_PATH.write_text(json.dumps(resources, indent=1, sort_keys=True))
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, verbose=True)
    print(f"built {path}")
