"""The simulator of tests/cpu_sim checked on its own (tests/cpu_sim/selftest.cpp): what its wave and block operations
return against their definitions, restated here in numpy (DPP row shifts and broadcasts through an inclusive wave
scan that must equal cumsum; ballots, shuffles, quad permutations; barrier counts with threads that have left;
atomics), and the negative control for the thread orders: a hand-off between lanes without a barrier must give
different results under INPC_SIM_ORDER=forward and =reverse, the same hand-off behind a barrier must not."""
import ctypes as C
import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def selftest():
    from tests.cpu_sim import build

    return C.CDLL(str(build.build_selftest()))


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def test_wave_and_block_operations(selftest):
    rng = np.random.default_rng(0)
    n = 192   # three waves
    v = rng.integers(0, 1000, n).astype(np.uint32)
    scan, shuffled, quads, counted = (np.full(n, 0xDEAD, np.uint32) for _ in range(4))
    ballots = np.zeros(3, np.uint64)
    selftest.selftest_wave_ops(_ptr(v), _ptr(scan), _ptr(ballots), _ptr(shuffled), _ptr(quads), _ptr(counted))
    lanes = np.arange(n) % 64
    waves = np.arange(n) // 64
    # inclusive sum inside each wave
    want = np.concatenate([np.cumsum(v[w * 64:(w + 1) * 64], dtype=np.uint64) for w in range(3)]).astype(np.uint32)
    np.testing.assert_array_equal(scan, want)
    for w in range(3):
        bits = sum(1 << l for l in range(64) if v[w * 64 + l] & 1)
        assert int(ballots[w]) == bits
    base = waves * 64
    up = np.where(lanes >= 2, v[np.maximum(np.arange(n) - 2, 0)], v)   # no source: the lane's own value
    want = v[base + ((lanes * 7 + 3) & 63)] + 1000 * v[base + (lanes ^ 5)] + 1000000 * up
    np.testing.assert_array_equal(shuffled, want.astype(np.uint32))
    front = np.where(lanes > 0, v[np.maximum(np.arange(n) - 1, 0)], 77)   # wave_shr:1: lane 0 keeps `old`
    want = v[np.arange(n) ^ 1] + 100000 * front
    np.testing.assert_array_equal(quads, want.astype(np.uint32))
    stays = np.arange(n) % 5 != 0
    count = int(((v & 2) != 0)[stays].sum())
    np.testing.assert_array_equal(counted[stays], np.uint32(count + 0 + 100000))
    np.testing.assert_array_equal(counted[~stays], np.uint32(0xDEAD))   # left before the barriers, wrote nothing


def test_atomics(selftest):
    counter = np.zeros(2, np.uint32)
    slots = np.zeros(5 * 128, np.uint32)
    total = np.zeros(1, np.float32)
    selftest.selftest_atomics(_ptr(counter), _ptr(slots), _ptr(total))
    assert counter[0] == 5 * (127 * 128 // 2) and counter[1] == 5 * 128 - 1
    np.testing.assert_array_equal(slots, 1)
    assert total[0] == 0.5 * 5 * 128


_SCRIPT = """
import ctypes as C, json, sys
import numpy as np
lib = C.CDLL(sys.argv[1])
out = {}
for with_barrier in (0, 1):
    a = np.zeros(3 * 256, np.uint32)
    lib.selftest_handoff(a.ctypes.data_as(C.c_void_p), with_barrier)
    out[str(with_barrier)] = a.tolist()
print(json.dumps(out))
"""


def _handoff(selftest_path, order):
    env = dict(os.environ, INPC_SIM_ORDER=order)
    done = subprocess.run([sys.executable, "-c", _SCRIPT, str(selftest_path)], env=env, capture_output=True, text=True,
                          stdin=subprocess.DEVNULL, timeout=300, check=True)
    return {k: np.array(v, np.uint32) for k, v in json.loads(done.stdout).items()}


def test_a_missing_barrier_shows_under_another_thread_order(selftest):
    from tests.cpu_sim import build

    t = np.arange(256)
    right = np.tile((3 * (255 - t) + 1).astype(np.uint32), 3)
    results = {order: _handoff(build.SELFTEST_LIB, order) for order in ("forward", "reverse", "shuffle")}
    for order, got in results.items():
        np.testing.assert_array_equal(got["1"], right, err_msg=f"with the barrier, order {order}")
    # without it thread t reads what thread 255 - t has written so far, which is a matter of the order: no order gets
    # all of it right, and two orders get different parts of it right
    wrong = {order: got["0"] != right for order, got in results.items()}
    for order in wrong:
        assert wrong[order].any(), order
        assert set(np.unique(results[order]["0"][wrong[order]])) == {0}   # what is wrong is the cleared value
    assert (wrong["forward"] != wrong["reverse"]).any()
