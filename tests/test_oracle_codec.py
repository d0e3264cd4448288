"""fp16 codec of the oracle, pinned exhaustively against numpy.float16
(an IEEE-754 binary16 library routine) -- QW/src/utils.cpp:497-564."""
import numpy as np

from oracle_lib import lib


def test_f16_to_f32_all_encodings():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.orc_f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_roundtrip_and_midpoints():
    # every half value, the float just below/above it, and the exact midpoints
    # between neighbouring halves (ties must go to even)
    bits = np.arange(0x7C00, dtype=np.uint16)            # finite positives
    h = bits.view(np.float16).astype(np.float64)
    nxt = np.arange(1, 0x7C01, dtype=np.uint16).view(np.float16).astype(np.float64)
    nxt[-1] = 65536.0                                     # the would-be next binade
    mid = (h + nxt) / 2
    cases = np.concatenate([h, mid, np.nextafter(mid.astype(np.float32), np.float32(0)).astype(np.float64),
                            np.nextafter(mid.astype(np.float32), np.float32(1e9)).astype(np.float64)])
    cases = np.concatenate([cases, -cases]).astype(np.float32)
    want = cases.astype(np.float16).view(np.uint16)
    got = np.array([lib.orc_f32_to_f16(float(c)) for c in cases], np.uint16)
    assert np.array_equal(got, want)


def test_f32_to_f16_random_and_specials():
    rng = np.random.default_rng(1)
    u = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    f = u.view(np.float32)
    f = f[np.isfinite(f)]
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([lib.orc_f32_to_f16(float(c)) for c in f], np.uint16)
    assert np.array_equal(got, want)
    assert lib.orc_f32_to_f16(float("inf")) == 0x7C00
    assert lib.orc_f32_to_f16(float("-inf")) == 0xFC00
    assert lib.orc_f32_to_f16(70000.0) == 0x7C00            # saturates to Inf
    assert (lib.orc_f32_to_f16(float("nan")) & 0x7C00) == 0x7C00
    assert (lib.orc_f32_to_f16(float("nan")) & 0x03FF) != 0


def test_f64_to_f16_single_rounding():
    # a double that rounds differently when it passes through float32 first:
    # 1 + 2^-11 + 2^-30 is above the half midpoint, float32 rounds it onto the midpoint
    d = 1.0 + 2.0**-11 + 2.0**-30
    assert lib.orc_f64_to_f16(d) == np.float16(d).view(np.uint16) == 0x3C01
    assert np.float32(d).astype(np.float16).view(np.uint16) == 0x3C00
    rng = np.random.default_rng(2)
    x = rng.standard_normal(100000) * 10.0 ** rng.uniform(-9, 5, 100000)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([lib.orc_f64_to_f16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)


def test_expf_close_to_libm():
    xs = np.linspace(-87, 88, 70001).astype(np.float32)
    got = np.array([lib.orc_expf_export(float(v)) for v in xs], np.float32)
    want = np.exp(xs.astype(np.float64))
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got.astype(np.float64) - want) / ulp) <= 2.0
