"""Builds and packages inpc_amd: `pip install . --no-build-isolation` compiles libinpc_hip.so for gfx950 with hipcc
(inpc_amd/build.py) and installs it inside the package, the way the reference's setup.py builds its extension module
(INPCCudaBackend/setup.py:1-54). An in-tree build needs no install: `python -m inpc_amd.build`."""
import importlib.util
from pathlib import Path

from setuptools import setup
from setuptools.command.build_py import build_py

ROOT = Path(__file__).parent.resolve()


def _hip_build():
    # loaded from its file: importing the package itself would pull in torch and the library that is not built yet
    spec = importlib.util.spec_from_file_location("_inpc_amd_build", ROOT / "inpc_amd" / "build.py")
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


class BuildWithHip(build_py):
    """Compiles the HIP library (when a source is newer than it) before the Python files are collected."""

    def run(self):
        path = _hip_build().build(force=False, verbose=True)
        print(f"built {path}")
        super().run()


setup(
    name="inpc_amd",
    version="0.3.0",
    description="MI355X (gfx950) implementation of the INPCCudaBackend hot path: octree point sampler and tile-based "
                "differentiable point rasterizer behind a C ABI",
    packages=["inpc_amd"],
    package_data={"inpc_amd": ["libinpc_hip.so", "csrc/*.hip", "csrc/*.hpp"]},
    python_requires=">=3.10",
    cmdclass={"build_py": BuildWithHip},
)
