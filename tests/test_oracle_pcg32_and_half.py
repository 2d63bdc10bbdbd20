"""Pins the oracle's PCG32 and fp16 conversions against published / library answers (CPU only)."""
import ctypes as C

import numpy as np

MASK64 = (1 << 64) - 1
MULT = 0x5851F42D4C957F2D


class PyPcg32:
    """Independent restatement of PCG32 XSH-RR 64/32 from the published algorithm (pcg-random.org, pcg32 demo)."""

    def __init__(self, initstate, initseq=1):
        self.state = 0
        self.inc = ((initseq << 1) | 1) & MASK64
        self.next_uint()
        self.state = (self.state + initstate) & MASK64
        self.next_uint()

    def next_uint(self):
        old = self.state
        self.state = (old * MULT + self.inc) & MASK64
        xorshifted = (((old >> 18) ^ old) >> 27) & 0xFFFFFFFF
        rot = old >> 59
        return ((xorshifted >> rot) | (xorshifted << ((-rot) & 31))) & 0xFFFFFFFF

    def next_float(self):
        bits = np.uint32((self.next_uint() >> 9) | 0x3F800000)
        return np.float32(bits.view(np.float32) - np.float32(1.0))


def test_published_known_answer(oracle):
    # first outputs of the pcg32 demo generator seeded with (42, 54)
    r = oracle.Pcg32(42, 54)
    assert [r.next_uint() for _ in range(6)] == [0xA15C02B7, 0x7B47F409, 0xBA1D3330, 0x83D2F293, 0xBFA4784B,
                                                 0xCBED606E]


def test_matches_independent_restatement(oracle):
    for seed, seq in [(0, 1), (1234, 1), (2**63 + 17, 5), (2**64 - 1, 2**40)]:
        a, b = oracle.Pcg32(seed, seq), PyPcg32(seed, seq)
        assert (int(a.state[0]), int(a.state[1])) == (b.state, b.inc)
        assert [a.next_uint() for _ in range(50)] == [b.next_uint() for _ in range(50)]
        fa = [a.next_float() for _ in range(50)]
        fb = [float(b.next_float()) for _ in range(50)]
        assert fa == fb


def test_advance_is_repeated_stepping_and_composes(oracle):
    base = oracle.Pcg32(99)
    for k in (0, 1, 2, 3, 7, 64, 1000, 12345):
        stepped = base.copy()
        for _ in range(k):
            stepped.next_uint()
        jumped = base.copy()
        jumped.advance(k)
        assert int(jumped.state[0]) == int(stepped.state[0]), k
    a = base.copy()
    a.advance(123456789)
    a.advance(987654321)
    b = base.copy()
    b.advance(123456789 + 987654321)
    assert int(a.state[0]) == int(b.state[0])
    c = base.copy()
    c.advance(5000)
    c.advance(-5000)  # going back is going the long way round
    assert int(c.state[0]) == int(base.state[0])


def test_next_float_range_and_grid(oracle):
    r = oracle.Pcg32(7)
    v = np.array([r.next_float() for _ in range(20000)], dtype=np.float64)
    assert (v >= 0).all() and (v < 1).all()
    assert np.all(v * 2**23 == np.round(v * 2**23))  # multiples of 2^-23
    assert abs(v.mean() - 0.5) < 0.01


def test_library_host_helpers_match_oracle(oracle):
    # the host-side PCG32 helpers of the product library run without a GPU
    from inpc_amd import _lib

    lib = _lib.lib()
    for seed in (0, 5, 2**40 + 3):
        host = (C.c_uint64 * 2)()
        lib.inpc_pcg32_seed(host, C.c_uint64(seed), C.c_uint64(1))
        ref = oracle.Pcg32(seed, 1)
        assert (int(host[0]), int(host[1])) == (int(ref.state[0]), int(ref.state[1]))
        assert [lib.inpc_pcg32_next_uint(host) for _ in range(10)] == [ref.next_uint() for _ in range(10)]
        lib.inpc_pcg32_advance(host, C.c_int64(4 * 8388608))
        ref.advance(4 * 8388608)
        assert int(host[0]) == int(ref.state[0])
        assert float(lib.inpc_pcg32_next_float(host)) == ref.next_float()


def test_half_conversions_match_numpy(oracle):
    halfs = np.arange(65536, dtype=np.uint16)
    as_float = halfs.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 7):
        f = oracle.half_to_float(h)
        assert np.float32(f).tobytes() == as_float[h].tobytes() or (np.isnan(f) and np.isnan(as_float[h]))
    rng = np.random.default_rng(0)
    values = np.concatenate([
        (rng.standard_normal(20000) * 10.0 ** rng.integers(-9, 6, 20000)).astype(np.float32),
        rng.integers(0, 2**32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        as_float[np.isfinite(as_float)][::13],
        np.array([65504.0, 65519.9, 65520.0, 1e-8, 2.0**-25, 2.0**-24, 2.0**-24 * 1.5, 0.0, -0.0], np.float32),
    ])
    values = values[~np.isnan(values)]
    with np.errstate(over="ignore"):
        expect = values.astype(np.float16).view(np.uint16)
    got = np.array([oracle.float_to_half(float(v)) for v in values], dtype=np.uint16)
    np.testing.assert_array_equal(got, expect)
