"""Builds the library's own sources (inpc_amd/csrc/*.hip) with g++ against the simulator's stand-in for the HIP
runtime (tests/cpu_sim/hip/, tests/cpu_sim/sim.cpp) into tests/cpu_sim/libinpc_sim.so: the same C ABI, kernels run
on the CPU one block after the other (see sim.hpp). TEST INFRASTRUCTURE ONLY: nothing of the product imports this,
and the product itself still refuses to run without its HIP library."""
from __future__ import annotations

import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
CSRC = ROOT / "inpc_amd" / "csrc"
LIB = HERE / "libinpc_sim.so"
SOURCES = ["runtime.hip", "sampler.hip", "raster.hip", "field.hip", "misc.hip"]
FLAGS = ["-x", "c++", "-std=c++17", "-O2", "-fPIC", "-ffp-contract=off", "-Wno-unknown-pragmas", f"-I{HERE}"]


def _stale() -> bool:
    if not LIB.exists():
        return True
    built = LIB.stat().st_mtime
    deps = list(CSRC.glob("*.hip")) + list(CSRC.glob("*.hpp")) + [ROOT / "include" / "inpc_hip.h", HERE / "sim.cpp",
                                                                  HERE / "sim.hpp", HERE / "hip" / "hip_runtime.h",
                                                                  HERE / "hip" / "hip_fp16.h"]
    return any(d.stat().st_mtime > built for d in deps)


def _compile(src: Path, obj: Path, flags: list[str]) -> None:
    done = subprocess.run(["g++", *flags, "-c", str(src), "-o", str(obj)], capture_output=True, text=True,
                          stdin=subprocess.DEVNULL, timeout=1200)
    if done.returncode != 0:
        raise RuntimeError(f"g++ failed on {src}:\n{done.stderr[-4000:]}")


def build(force: bool = False) -> Path:
    if not force and not _stale():
        return LIB
    objdir = HERE / "obj"
    objdir.mkdir(exist_ok=True)
    jobs = [(CSRC / s, objdir / (Path(s).stem + ".o"), FLAGS) for s in SOURCES]
    jobs.append((HERE / "sim.cpp", objdir / "sim.o", ["-std=c++17", "-O2", "-fPIC"]))
    with ThreadPoolExecutor(max_workers=6) as pool:
        list(pool.map(lambda job: _compile(*job), jobs))
    done = subprocess.run(["g++", "-shared", "-o", str(LIB), *[str(obj) for _, obj, _ in jobs]], capture_output=True,
                          text=True, stdin=subprocess.DEVNULL, timeout=600)
    if done.returncode != 0:
        raise RuntimeError(f"linking {LIB} failed:\n{done.stderr[-4000:]}")
    return LIB


if __name__ == "__main__":
    print(build(force=True))
