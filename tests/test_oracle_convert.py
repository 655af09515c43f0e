"""Pins the CPU checker's bf16 / f16 converters (no GPU needed): exhaustive widening of all
65,536 encodings against numpy, narrowing against a committed fixture produced by torch and
numpy (tests/golden/make_convert_fixture.py) and against live numpy conversion of random bits."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "convert_f32_to_half.npz")


def test_widen_every_f16_encoding(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = oracle.widen("f16", h)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    # NaNs keep sign and payload, shifted into the wider mantissa
    assert np.array_equal(got.view(np.uint32)[nan] & 0x7fffff, (h[nan].astype(np.uint32) & 0x3ff) << 13)


def test_widen_every_bf16_encoding(oracle):
    h = np.arange(65536, dtype=np.uint16)
    got = oracle.widen("bf16", h)
    assert np.array_equal(got.view(np.uint32), h.astype(np.uint32) << 16)


def test_narrow_matches_fixture(oracle):
    z = np.load(GOLDEN)
    f = z["f32_bits"].view(np.float32)
    nan = np.isnan(f)
    for dtype, key, quiet in (("bf16", "bf16_bits", 0x0040), ("f16", "f16_bits", 0x0200)):
        got, want = oracle.narrow(dtype, f), z[key]
        assert np.array_equal(got[~nan], want[~nan]), dtype
        # NaN in -> quiet NaN out, sign kept
        exp_mask = 0x7f80 if dtype == "bf16" else 0x7c00
        assert np.all((got[nan] & exp_mask) == exp_mask) and np.all(got[nan] & quiet)
        assert np.array_equal(got[nan] >> 15, (z["f32_bits"][nan] >> 31).astype(np.uint16))


def test_narrow_f16_random_bits_vs_numpy(oracle):
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    # concentrate half of them where f16 is finite (exponents -26 .. 16)
    e = rng.integers(127 - 26, 127 + 17, size=1_000_000, dtype=np.uint32)
    bits[:1_000_000] = (bits[:1_000_000] & np.uint32(0x807fffff)) | (e << 23)
    f = bits.view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = oracle.narrow("f16", f)
    ok = ~np.isnan(f)
    assert np.array_equal(got[ok], want[ok])


def test_narrow_bf16_random_bits_vs_integer_rule(oracle):
    """Independent statement of round-to-nearest-even on the dropped 16 bits, in numpy integers."""
    rng = np.random.default_rng(6)
    bits = rng.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    ok = ~np.isnan(f)
    b = bits[ok].astype(np.uint64)
    low, top = b & 0xffff, b >> 16
    up = (low > 0x8000) | ((low == 0x8000) & ((top & 1) == 1))
    want = (top + up).astype(np.uint16)
    assert np.array_equal(oracle.narrow("bf16", f)[ok], want)


def test_round_trip_is_identity(oracle):
    h = np.arange(65536, dtype=np.uint16)
    for dtype in ("bf16", "f16"):
        w = oracle.widen(dtype, h)
        back = oracle.narrow(dtype, w)
        nan = np.isnan(w)
        assert np.array_equal(back[~nan], h[~nan]), dtype


def test_rng_streams(oracle):
    a = oracle.fill_uniform_f32(100000, 0, 0, -1.0, 1.0)
    b = oracle.fill_uniform_f32(100000, 0, 1, -1.0, 1.0)
    assert a.min() >= -1.0 and a.max() < 1.0 and abs(float(a.mean())) < 0.02
    assert not np.array_equal(a, b)
    assert np.array_equal(a, oracle.fill_uniform_f32(100000, 0, 0, -1.0, 1.0))
    assert np.array_equal(a[:10], oracle.fill_uniform_f32(10, 0, 0, -1.0, 1.0)), "counter-based: prefix-stable"
    n = oracle.widen("bf16", oracle.fill_normal("bf16", 400000, 2, 3, 0.0, 1e-2))
    assert abs(float(n.mean())) < 1e-4 and abs(float(n.std()) - 1e-2) < 2e-4
    i = oracle.fill_int32(100000, 3, 0)
    assert i.min() >= -(1 << 20) and i.max() <= (1 << 20)
