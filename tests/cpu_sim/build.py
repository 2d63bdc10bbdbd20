"""Builds the library's own sources (inpc_amd/csrc/*.hip) with a host compiler against the simulator's stand-in for the HIP
runtime (tests/cpu_sim/hip/, tests/cpu_sim/sim.cpp) into tests/cpu_sim/libinpc_sim.so: the same C ABI, kernels run
on the CPU one block after the other (see sim.hpp). TEST INFRASTRUCTURE ONLY: nothing of the product imports this,
and the product itself still refuses to run without its HIP library.

`sanitize=True` (or `python tests/cpu_sim/build.py --sanitize`) builds libinpc_sim_asan.so with AddressSanitizer and
UndefinedBehaviorSanitizer: every load and store of every kernel is then checked against the bounds of the buffer it
lands in (the tensors of the tests are heap allocations) and against the alignment of its type (a float4 access needs
16 bytes, as the 128-bit LDS and memory instructions do), every shift against the width of its operand, every signed
operation against overflow, every conversion of a float to an integer against the integer's range (where x86 and the
GPU give different results); the first finding ends the process. The process has to start with the sanitizer's
runtime preloaded:

    LD_PRELOAD=$(gcc -print-file-name=libasan.so) ASAN_OPTIONS=detect_leaks=0 INPC_SIM_SANITIZE=1 \\
        python -m pytest tests/test_sim_kernels.py -q
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
CSRC = ROOT / "inpc_amd" / "csrc"
LIB = HERE / "libinpc_sim.so"
LIB_SANITIZE = HERE / "libinpc_sim_asan.so"
SOURCES = ["runtime.hip", "sampler.hip", "raster.hip", "field.hip", "misc.hip"]
COMMON = ["-std=c++17", "-fPIC"]
OPTIMIZE = ["-O2"]
SANITIZE = ["-O1", "-g", "-fsanitize=address,undefined,float-cast-overflow", "-fno-sanitize-recover=undefined,float-cast-overflow", "-fno-omit-frame-pointer"]
KERNEL_FLAGS = ["-x", "c++", "-ffp-contract=off", "-Wno-unknown-pragmas", f"-I{HERE}"]
# The host compiler: INPC_SIM_CXX if set; else ROCm's clang++ for the plain build (it is there wherever hipcc is) and
# g++ for the sanitizer build (whose runtime the command above preloads), g++ for both where there is no clang++.
# Unlike g++, clang++ also puts the __shared__ variables of function templates into the section that the simulator
# fills with a byte pattern before every block (hip/hip_runtime.h), so with it no kernel can count on what an earlier
# block left in any of its LDS.
def _compiler(sanitize: bool) -> str:
    chosen = os.environ.get("INPC_SIM_CXX")
    if chosen:
        return chosen
    if not sanitize:
        for candidate in (shutil.which("clang++"), "/opt/rocm/lib/llvm/bin/clang++"):
            if candidate and Path(candidate).exists():
                return candidate
    return "g++"


def _stale(lib: Path) -> bool:
    if not lib.exists():
        return True
    built = lib.stat().st_mtime
    deps = list(CSRC.glob("*.hip")) + list(CSRC.glob("*.hpp")) + [ROOT / "include" / "inpc_hip.h", HERE / "sim.cpp",
                                                                  HERE / "sim.hpp", HERE / "hip" / "hip_runtime.h",
                                                                  HERE / "hip" / "hip_fp16.h", Path(__file__)]
    return any(d.stat().st_mtime > built for d in deps)


def _compile(cxx: str, src: Path, obj: Path, flags: list[str]) -> None:
    done = subprocess.run([cxx, *flags, "-c", str(src), "-o", str(obj)], capture_output=True, text=True,
                          stdin=subprocess.DEVNULL, timeout=1800)
    if done.returncode != 0:
        raise RuntimeError(f"{cxx} failed on {src}:\n{done.stderr[-4000:]}")


def build(force: bool = False, sanitize: bool = False) -> Path:
    lib = LIB_SANITIZE if sanitize else LIB
    if not force and not _stale(lib):
        return lib
    mode = SANITIZE if sanitize else OPTIMIZE
    cxx = _compiler(sanitize)
    objdir = HERE / ("obj_asan" if sanitize else "obj")
    objdir.mkdir(exist_ok=True)
    jobs = [(CSRC / s, objdir / (Path(s).stem + ".o"), [*COMMON, *mode, *KERNEL_FLAGS]) for s in SOURCES]
    jobs.append((HERE / "sim.cpp", objdir / "sim.o", [*COMMON, *mode]))
    with ThreadPoolExecutor(max_workers=6) as pool:
        list(pool.map(lambda job: _compile(cxx, *job), jobs))
    link = [cxx, "-shared", *(["-fsanitize=address,undefined"] if sanitize else []), "-o", str(lib)]
    done = subprocess.run([*link, *[str(obj) for _, obj, _ in jobs]], capture_output=True, text=True,
                          stdin=subprocess.DEVNULL, timeout=600)
    if done.returncode != 0:
        raise RuntimeError(f"linking {lib} failed:\n{done.stderr[-4000:]}")
    return lib


SELFTEST_LIB = HERE / "libsim_selftest.so"


def build_selftest() -> Path:
    """selftest.cpp (kernels that check the simulator itself) with the simulator core, as a library of its own."""
    deps = [HERE / "selftest.cpp", HERE / "sim.cpp", HERE / "sim.hpp", HERE / "hip" / "hip_runtime.h"]
    if SELFTEST_LIB.exists() and all(SELFTEST_LIB.stat().st_mtime >= d.stat().st_mtime for d in deps):
        return SELFTEST_LIB
    done = subprocess.run([_compiler(False), *COMMON, *OPTIMIZE, "-ffp-contract=off", f"-I{HERE}", "-shared", "-o", str(SELFTEST_LIB),
                           str(HERE / "selftest.cpp"), str(HERE / "sim.cpp")], capture_output=True, text=True,
                          stdin=subprocess.DEVNULL, timeout=600)
    if done.returncode != 0:
        raise RuntimeError(f"building {SELFTEST_LIB} failed:\n{done.stderr[-4000:]}")
    return SELFTEST_LIB


MSAN_DRIVER = HERE / "msan_driver"
MSAN_FLAGS = ["-O1", "-g", "-fsanitize=memory", "-fsanitize-memory-track-origins=2", "-fno-omit-frame-pointer"]


def clang() -> str | None:
    """A clang++ (MemorySanitizer is clang's): INPC_SIM_CXX if it is one, one on the PATH, or ROCm's."""
    for candidate in (os.environ.get("INPC_SIM_CXX"), shutil.which("clang++"), "/opt/rocm/lib/llvm/bin/clang++"):
        if candidate and "clang" in Path(candidate).name and Path(candidate).exists():
            return candidate
    return None


def build_msan_driver() -> Path:
    """msan_driver.cpp, the library's sources and the simulator as one executable under MemorySanitizer."""
    cxx = clang()
    if cxx is None:
        raise RuntimeError("MemorySanitizer needs clang++")
    deps = list(CSRC.glob("*.hip")) + list(CSRC.glob("*.hpp")) + [ROOT / "include" / "inpc_hip.h", HERE / "sim.cpp",
                                                                  HERE / "sim.hpp", HERE / "hip" / "hip_runtime.h",
                                                                  HERE / "hip" / "hip_fp16.h", HERE / "msan_driver.cpp",
                                                                  Path(__file__)]
    if MSAN_DRIVER.exists() and all(MSAN_DRIVER.stat().st_mtime >= d.stat().st_mtime for d in deps):
        return MSAN_DRIVER
    objdir = HERE / "obj_msan"
    objdir.mkdir(exist_ok=True)
    jobs = [(CSRC / s, objdir / (Path(s).stem + ".o"), [*COMMON, *MSAN_FLAGS, *KERNEL_FLAGS]) for s in SOURCES]
    jobs.append((HERE / "sim.cpp", objdir / "sim.o", [*COMMON, *MSAN_FLAGS]))
    jobs.append((HERE / "msan_driver.cpp", objdir / "msan_driver.o", [*COMMON, *MSAN_FLAGS, f"-I{HERE}"]))
    with ThreadPoolExecutor(max_workers=7) as pool:
        list(pool.map(lambda job: _compile(cxx, *job), jobs))
    done = subprocess.run([cxx, "-fsanitize=memory", "-o", str(MSAN_DRIVER), *[str(obj) for _, obj, _ in jobs]],
                          capture_output=True, text=True, stdin=subprocess.DEVNULL, timeout=600)
    if done.returncode != 0:
        raise RuntimeError(f"linking {MSAN_DRIVER} failed:\n{done.stderr[-4000:]}")
    return MSAN_DRIVER


if __name__ == "__main__":
    print(build(force=True, sanitize="--sanitize" in sys.argv[1:]))
