"""Pins the CPU checker's bf16 / f16 converters (no GPU needed): exhaustive widening of all
65,536 encodings against numpy, narrowing against a committed fixture produced by torch and
numpy (tests/golden/make_convert_fixture.py) and against live numpy conversion of random bits.
The 8-bit floats are pinned the same way against torch.float8_e4m3fn / torch.float8_e5m2 (all
256 encodings, narrowing wherever torch's non-saturating conversion is finite) and against the
closed form of the formats elsewhere."""
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


# ---- 8-bit floats ------------------------------------------------------------------------
F8 = {"f8e4m3": dict(man=3, bias=7, max=448.0, max_code=0x7e),
      "f8e5m2": dict(man=2, bias=15, max=57344.0, max_code=0x7b)}


def _torch_f8(dtype):
    import torch
    return {"f8e4m3": torch.float8_e4m3fn, "f8e5m2": torch.float8_e5m2}[dtype]


def _closed_form_f8(code, man, bias):
    """Value of one encoding from the format definition (finite encodings only)."""
    s = -1.0 if code & 0x80 else 1.0
    e, m = (code & 0x7f) >> man, code & ((1 << man) - 1)
    if e == 0:
        return s * m * 2.0 ** (1 - bias - man)
    return s * (1 + m / (1 << man)) * 2.0 ** (e - bias)


def test_widen_every_f8_encoding(oracle):
    import torch
    codes = np.arange(256, dtype=np.uint8)
    for dtype, f in F8.items():
        got = oracle.widen(dtype, codes)
        want = torch.from_numpy(codes.copy()).view(_torch_f8(dtype)).to(torch.float32).numpy()
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan), dtype
        assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan]), dtype
        # and against the definition of the format, which torch is not needed for
        for c in range(256):
            if dtype == "f8e4m3" and (c & 0x7f) == 0x7f:
                assert np.isnan(got[c])
            elif dtype == "f8e5m2" and (c & 0x7f) >= 0x7c:
                assert (np.isinf(got[c]) and (got[c] < 0) == bool(c & 0x80)) if (c & 0x7f) == 0x7c else np.isnan(got[c])
            else:
                assert got[c] == np.float32(_closed_form_f8(c, f["man"], f["bias"])), (dtype, c)
                assert np.signbit(got[c]) == bool(c & 0x80)


def test_narrow_f8_vs_torch_where_finite(oracle):
    import torch
    rng = np.random.default_rng(8)
    for dtype, f in F8.items():
        bits = rng.integers(0, 1 << 32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
        # exponents from far below the smallest subnormal to the top binade of the format
        top = int(np.log2(f["max"]))
        e = rng.integers(127 - f["bias"] - f["man"] - 6, 127 + top + 1, size=bits.size, dtype=np.uint32)
        bits = (bits & np.uint32(0x807fffff)) | (e << 23)
        x = bits.view(np.float32)
        # ties and neighbours of ties at every step of the format
        codes = np.arange(256, dtype=np.uint8)
        vals = oracle.widen(dtype, codes)
        vals = vals[np.isfinite(vals)].astype(np.float64)
        vs = np.sort(vals)
        mid = ((vs[:-1] + vs[1:]) / 2).astype(np.float32)
        ties = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                               vals.astype(np.float32)])
        x = np.concatenate([x, ties])
        x = x[np.abs(x) <= f["max"]]
        want = torch.from_numpy(x.copy()).to(_torch_f8(dtype)).view(torch.uint8).numpy()
        got = oracle.narrow(dtype, x)
        assert np.array_equal(got, want), dtype


def test_narrow_f8_saturates(oracle):
    for dtype, f in F8.items():
        mx = np.float32(f["max"])
        x = np.array([mx, np.nextafter(mx, np.float32(np.inf)), mx * 1.03, mx * 1.07, mx * 2, 3e38],
                     dtype=np.float32)
        assert np.all(oracle.narrow(dtype, x) == f["max_code"]), dtype
        assert np.all(oracle.narrow(dtype, -x) == (0x80 | f["max_code"])), dtype
        nan = oracle.narrow(dtype, np.array([np.nan, -np.nan], dtype=np.float32))
        assert np.all((nan & 0x7f) == 0x7f), dtype
        # true infinities: kept by the format that has them, NaN in the one that has none; as torch
        import torch
        inf = np.array([np.inf, -np.inf], dtype=np.float32)
        want = torch.from_numpy(inf).to(_torch_f8(dtype)).view(torch.uint8).numpy()
        assert np.array_equal(oracle.narrow(dtype, inf), want), dtype
        assert want.tolist() == ([0x7c, 0xfc] if dtype == "f8e5m2" else [0x7f, 0xff])
        # the smallest subnormal step: exactly half rounds to even (zero), just above rounds up
        step = np.float32(2.0 ** (1 - f["bias"] - f["man"]))
        x = np.array([step / 2, np.nextafter(step / 2, np.float32(1)), step * 1.5, -step / 2, 0.0, -0.0, 1e-40],
                     dtype=np.float32)
        assert oracle.narrow(dtype, x).tolist() == [0, 1, 2, 0x80, 0, 0x80, 0], dtype


def test_f8_round_trip_is_identity(oracle):
    codes = np.arange(256, dtype=np.uint8)
    for dtype in F8:
        f = oracle.widen(dtype, codes)
        keep = np.isfinite(f)
        assert np.array_equal(oracle.narrow(dtype, f[keep]), codes[keep]), dtype


def test_f8_reduce_small_brute_force(oracle):
    """The reduce of 8-bit floats equals: widen exactly, fold in binary32 in input order,
    narrow once -- stated here with numpy float32 arithmetic and the pinned converters."""
    rng = np.random.default_rng(9)
    for dtype, f in F8.items():
        ins = [rng.integers(0, 256, size=5000, dtype=np.uint64).astype(np.uint8) for _ in range(5)]
        ok = np.ones(5000, dtype=bool)
        for a in ins:
            ok &= np.isfinite(oracle.widen(dtype, a))
        ins = [a[ok] for a in ins]
        acc = oracle.widen(dtype, ins[0])
        for a in ins[1:]:
            acc = (acc + oracle.widen(dtype, a)).astype(np.float32)
        assert np.array_equal(oracle.reduce(dtype, "sum", ins), oracle.narrow(dtype, acc)), dtype
