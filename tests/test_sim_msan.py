"""The library's entry points on workspaces and outputs that nobody has initialised, under MemorySanitizer
(tests/cpu_sim/msan_driver.cpp: the kernels' own sources, the simulator and a driver as one clang++ -fsanitize=memory
executable): sampler, CDF, expected counts, training draw, field update and bookkeeping, element-wise operators, and forward + backward + inference of both
footprints with both tile sizes and in the spherical-harmonics modes. It ends at the first branch, address or output that depends on a byte nothing has
written. Building it takes a minute and a half, so the test only runs when INPC_SIM_MSAN=1 is set:

    INPC_SIM_MSAN=1 python -m pytest tests/test_sim_msan.py -q
"""
import os
import subprocess

import pytest


@pytest.mark.skipif(os.environ.get("INPC_SIM_MSAN", "") in ("", "0"), reason="set INPC_SIM_MSAN=1 (needs clang++, ~2 min)")
def test_nothing_reads_what_nothing_has_written():
    from tests.cpu_sim import build

    if build.clang() is None:
        pytest.skip("MemorySanitizer needs clang++")
    driver = build.build_msan_driver()
    done = subprocess.run([str(driver)], capture_output=True, text=True, stdin=subprocess.DEVNULL, timeout=1200)
    assert done.returncode == 0, (done.stdout + done.stderr)[-6000:]
    assert "no use of uninitialised memory" in done.stdout
    assert done.stdout.count("footprint") == 6 and "field bookkeeping" in done.stdout
