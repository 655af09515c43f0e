"""Writes tests/golden/convert_f32_to_half.npz: float32 inputs and their bf16 / f16 bit patterns
as produced by torch and numpy (library conversions, round-to-nearest-even), used to pin the CPU
checker's converters.  The reference holds no fixtures for this path (it has no tests), so the
expected values come from these two independent library implementations.

Run from the repository root:  python tests/golden/make_convert_fixture.py
"""
import os

import numpy as np
import torch


def main():
    rng = np.random.default_rng(20240607)
    parts = []
    # every bf16 and f16 tie / near-tie around a spread of exponents
    for e in list(range(-30, 31, 3)) + [-126, -127, -133, -140, -149, 15, 16, 127]:
        base = np.float32(2.0) ** np.float32(max(e, -126))
        for frac in (0, 1, 2, 3, 0x7fff, 0x8000, 0x8001, 0xffff, 0x10000, 0x17fff, 0x18000, 0x18001, 0xfff, 0x1000,
                     0x1001, 0x2fff, 0x3000, 0x3001, 0x7fffff, 0x7f8000, 0x7fefff, 0x7ff000):
            bits = (np.float32(base).view(np.uint32) & np.uint32(0xff800000)) | np.uint32(frac)
            parts.append(np.array([bits, bits | np.uint32(0x80000000)], dtype=np.uint32))
    special = np.array([0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0xffc00000, 0x7f800001,
                        0x7fbfffff, 0x7fffffff, 0x00000001, 0x007fffff, 0x00800000, 0x33000000, 0x33000001,
                        0x32ffffff, 0x33800000, 0x38800000, 0x387fffff, 0x387fe000, 0x387ff000, 0x477fe000,
                        0x477fefff, 0x477ff000, 0x477fffff, 0x47800000, 0x7f7fffff, 0x7f7f8000, 0x7f7f7fff],
                       dtype=np.uint32)
    parts.append(special)
    parts.append(rng.integers(0, 1 << 32, size=6000, dtype=np.uint64).astype(np.uint32))
    bits = np.concatenate(parts)
    f = bits.view(np.float32)
    t = torch.from_numpy(f.copy())
    bf16 = t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    with np.errstate(over="ignore", invalid="ignore"):
        f16 = f.astype(np.float16).view(np.uint16)
    f16_torch = t.to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(f)
    assert np.array_equal(f16[~nan], f16_torch[~nan]), "numpy and torch disagree on f32 -> f16"
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "convert_f32_to_half.npz")
    np.savez_compressed(out, f32_bits=bits, bf16_bits=bf16, f16_bits=f16)
    print("wrote", out, bits.size, "values")


if __name__ == "__main__":
    main()
