"""What the compiler reports for every kernel of libinpc_hip.so (inpc_amd/build.py keeps hipcc's
-Rpass-analysis=kernel-resource-usage remarks next to the library): no kernel spills registers to scratch memory, the
static LDS of each fits a workgroup, and the kernels whose occupancy the design counts on keep it. Checked without a
GPU: these are properties of the code object."""
import json
import subprocess

import pytest

from inpc_amd import build

LDS_PER_WORKGROUP = 160 * 1024   # gfx950


@pytest.fixture(scope="module")
def kernels():
    if not build.RESOURCES_PATH.exists():
        build.build(force=True)
    by_source = json.loads(build.RESOURCES_PATH.read_text())
    mangled = [name for source in by_source.values() for name in source]
    plain = subprocess.run(["c++filt", *mangled], capture_output=True, text=True, stdin=subprocess.DEVNULL, timeout=60,
                           check=True).stdout.splitlines()
    out = {}
    for (source, table) in by_source.items():
        for name in table:
            readable = plain[mangled.index(name)].replace("inpc::(anonymous namespace)::", "").replace("void ", "")
            out[readable.split("(")[0]] = dict(table[name], source=source)
    return out


def test_every_source_reported_its_kernels(kernels):
    sources = {k["source"] for k in kernels.values()}
    assert sources == set(build.SOURCES)
    assert len(kernels) > 120
    for name in ("blend::k_blend_forward<16, 8, false, false>", "blend::k_blend_backward<16, 8, false>",
                 "tilesort::k_tile_sort<512>", "k_sample_cull<long>", "k_cdf_finish", "gaussian::k_blend_backward<16, 16>"):
        assert name in kernels, name


def test_no_kernel_uses_scratch_memory(kernels):
    spilling = {name: k["scratch_bytes_per_lane"] for name, k in kernels.items() if k["scratch_bytes_per_lane"] != 0}
    assert not spilling, spilling


def test_static_lds_fits_a_workgroup(kernels):
    for name, k in kernels.items():
        assert k["lds_bytes_per_block"] <= LDS_PER_WORKGROUP, (name, k)


def test_occupancy_the_design_counts_on(kernels):
    # the large tile sort runs two 512-thread blocks per compute unit (four waves per SIMD: at most 128 registers);
    # the bilinear blends of the benchmark's shape keep at least four waves per SIMD by registers
    for name, at_least in (("tilesort::k_tile_sort<512>", 4), ("tilesort::k_tile_sort<128>", 4),
                           ("blend::k_blend_forward<16, 8, false, false>", 4), ("blend::k_blend_backward<16, 8, false>", 4),
                           ("k_sample_cull<long>", 4), ("k_sample_cull<int>", 4)):
        assert kernels[name]["occupancy_waves_per_simd"] >= at_least, (name, kernels[name])
        assert kernels[name]["agprs"] == 0
