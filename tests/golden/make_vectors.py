"""Writes the committed known-answer vectors of the MXFP8 quantizer (`mx_vectors.npz`).

    python tests/golden/make_vectors.py

The expected bytes come from the slow, definition-level routines in `tests/_independent.py`
(an enumeration of all 256 e4m3 codes with nearest-value search and ties to the even code; the
block exponent as the smallest e with 2^e * 448 >= amax found by an exact-arithmetic loop),
which share no code with the oracle or the kernels. The inputs gather the edge cases the
reference's own tests use (`tests/quant/test_fp8_formats.py:85-106`: amax on both sides of
the 1.75 mantissa threshold, subnormal amax, all-zero blocks, +-448 saturation, signed
zeros) plus seeded blocks spanning the bf16 exponent range.

Arrays: `x_bits` uint16 [R, 128] (bf16 bit patterns), `codes` uint8 [R, 128], `scales` uint8
[R, 4]; `w_int8_in` fp32 / `w_int8_q` int8 / `w_int8_scale` fp32: the per-row int8 weight
quantizer's half-to-even known answers (`tests/kernels/quant/test_int8_linear.py:142-148`).
"""

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from tests._independent import mx_quantize  # noqa: E402


def bf16_bits(v: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns, round to nearest even (inputs here are finite)."""
    b = v.astype(np.float32).view(np.uint32).astype(np.uint64)
    return (((b + 0x7FFF + ((b >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def bf16_value(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def build_inputs() -> np.ndarray:
    rng = np.random.default_rng(20240229)
    rows = []
    # seeded blocks over the exponent range, four different magnitudes per row
    for e in range(-126, 120, 6):
        r = rng.standard_normal(128).astype(np.float32)
        r *= np.repeat(np.float32(2.0) ** np.array([e, e + 1, e + 3, min(e + 7, 126)], dtype=np.float32), 32)
        rows.append(r)
    # amax just below / at / above the mantissa threshold 1.75 at several exponents
    for e in (-20, -1, 0, 5):
        r = rng.uniform(-1, 1, 128).astype(np.float32) * np.float32(2.0**e)
        for blk, top in enumerate((1.7421875, 1.75, 1.7578125, 1.9921875)):
            r[blk * 32 + 7] = np.float32(top * 2.0**e) * (-1 if blk % 2 else 1)
        rows.append(r)
    # all-zero blocks with signed zeros, a subnormal-only block, saturation, tiny amax
    r = np.zeros(128, dtype=np.float32)
    r[1] = -0.0
    r[32:64] = np.float32(2.0**-133) * rng.integers(-3, 4, 32)
    r[64:96] = np.float32(448.0) * rng.choice([-1, 1], 32)
    r[96:128] = np.float32(1e-30) * rng.uniform(-1, 1, 32)
    rows.append(r)
    # one huge element among small ones (everything else flushes to zero codes)
    r = rng.standard_normal(128).astype(np.float32) * np.float32(1e-3)
    r[5], r[40], r[70], r[100] = 3e38, -6e4, 57344.0, 1.0
    rows.append(r)
    # every e4m3 rounding midpoint neighbourhood at unit scale (amax 448 -> e = 0)
    mids = np.array([448.0, 17.0, 18.0, 19.0, 0.001953125 * 0.5, 0.001953125 * 1.5, 0.0009765625, 0.0087890625, 27.0, 29.0, 432.0, 400.0], dtype=np.float32)
    r = np.zeros(128, dtype=np.float32)
    for blk in range(4):
        r[blk * 32] = 448.0
        r[blk * 32 + 1 : blk * 32 + 1 + len(mids)] = mids * (-1 if blk % 2 else 1)
        r[blk * 32 + 14 : blk * 32 + 32] = rng.uniform(-30, 30, 18)
    rows.append(r)
    return bf16_bits(np.stack(rows))


def main() -> None:
    x_bits = build_inputs()
    x = bf16_value(x_bits)
    codes, scales = mx_quantize(x)
    w = np.array([[127.0, 0.5, 1.5, -2.5, -127.0], [0.0, 0.0, 0.0, 0.0, 0.0], [63.5, -31.75, 0.25, 0.75, -0.25]], dtype=np.float32)
    amax = np.maximum(np.abs(w).max(1), np.float32(1e-12)).astype(np.float32)
    scale = (amax / np.float32(127.0)).astype(np.float32)
    q = np.clip(np.rint((w / scale[:, None]).astype(np.float32)), -127, 127).astype(np.int8)
    out = Path(__file__).with_name("mx_vectors.npz")
    np.savez_compressed(out, x_bits=x_bits, codes=codes.astype(np.uint8), scales=scales.astype(np.uint8), w_int8_in=w, w_int8_q=q, w_int8_scale=scale)
    print(f"wrote {out}: x_bits {x_bits.shape}, codes {codes.shape}, scales {scales.shape}")


if __name__ == "__main__":
    main()
