"""Independent formulas the oracle is pinned against: written from the format
definitions (bit layout of e4m3fn, the MX scale definition), sharing no code with
`oracle/` or with the kernels."""

from fractions import Fraction

import numpy as np


def e4m3_code_values() -> np.ndarray:
    """fp64 value of every e4m3fn byte 0..255 (NaN for 0x7F / 0xFF)."""
    out = np.zeros(256, np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp, man = (code >> 3) & 0xF, code & 7
        if exp == 0xF and man == 7:
            out[code] = np.nan
        elif exp == 0:
            out[code] = sign * man * 2.0**-9
        else:
            out[code] = sign * (8 + man) * 2.0 ** (exp - 10)
    return out


CODE_VALUES = e4m3_code_values()
_POSITIVE = CODE_VALUES[:0x7F]  # ascending, 0 .. 448


def nearest_e4m3(v: np.ndarray) -> np.ndarray:
    """e4m3fn byte of every fp32 value: clamp to +-448, nearest representable value,
    a tie goes to the even byte; the sign bit is the input's; NaN -> 0x7F | sign."""
    v = np.asarray(v, np.float32)
    a = np.minimum(np.abs(v.astype(np.float64)), 448.0)
    dist = np.abs(a.reshape(-1, 1) - _POSITIVE.reshape(1, -1))
    best = dist.min(axis=1, keepdims=True)
    tied = dist == best
    first = tied.argmax(axis=1)
    last = tied.shape[1] - 1 - tied[:, ::-1].argmax(axis=1)
    code = np.where(first % 2 == 0, first, last)  # at most two candidates, adjacent
    code = np.where(np.isnan(a).reshape(-1), 0x7F, code).reshape(v.shape)
    sign = (v.view(np.uint32) >> 24) & 0x80
    return (code | sign).astype(np.uint8)


def mx_exponent(amax: float) -> int:
    """Smallest e >= -127 with 2^e * 448 >= max(amax, fp32(1e-30)), in exact arithmetic."""
    a = max(Fraction(float(amax)), Fraction(float(np.float32(1e-30))))
    e = -127
    while Fraction(2) ** e * 448 < a:
        e += 1
    return e


def mx_quantize(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """(e4m3 bytes, E8M0 bytes) of an fp32 [rows, K] array, block by block."""
    rows, k = x.shape
    q = np.zeros((rows, k), np.uint8)
    s = np.zeros((rows, k // 32), np.uint8)
    for r in range(rows):
        for b in range(k // 32):
            blk = x[r, 32 * b : 32 * b + 32].astype(np.float32)
            e = mx_exponent(np.abs(blk).max())
            s[r, b] = e + 127
            scaled = (blk.astype(np.float64) * 2.0**-e).astype(np.float32)
            q[r, 32 * b : 32 * b + 32] = nearest_e4m3(scaled)
    return q, s


def fp32_scale(amax: np.ndarray) -> np.ndarray:
    return (np.maximum(np.float32(amax), np.float32(1e-12)) / np.float32(448.0)).astype(np.float32)


def swizzle_index(r: int, c: int, col_tiles: int) -> int:
    tile = (r // 128) * col_tiles + c // 4
    return tile * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + c % 4
