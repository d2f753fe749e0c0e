"""Second, independent statement of the quantization scheme in plain Python.

No numpy, no torch: binary32 / binary16 rounding is done with ``struct`` (pack 'f' / 'e'
round to nearest even), division and subtraction in Python doubles then rounded once to
binary32 (for binary32 operands the double result rounded to binary32 equals the correctly
rounded binary32 result), ``round()`` is Python's round-half-to-even.  Used only to pin the
numpy oracle on small inputs.
"""

from __future__ import annotations

import struct


def f32(v: float) -> float:
    return struct.unpack("<f", struct.pack("<f", v))[0]


def f16(v: float) -> float:
    try:
        return struct.unpack("<e", struct.pack("<e", v))[0]
    except OverflowError:
        return float("inf") if v > 0 else float("-inf")


def f16_bits(v: float) -> int:
    return struct.unpack("<H", struct.pack("<e", v))[0]


def clamp(v: float, lo: float, hi: float) -> float:
    return lo if v < lo else hi if v > hi else v


def quantize_w8_row(row: list[float]) -> tuple[list[int], float]:
    amax = max(abs(f32(v)) for v in row)
    scale = f16(f32(amax / 127.0))
    d = scale if scale != 0.0 else 1.0
    q = [int(clamp(round(f32(f32(v) / d)), -127, 127)) for v in row]
    return q, scale


def quantize_w4_group(group: list[float]) -> tuple[list[int], float, int]:
    assert len(group) == 128
    vals = [f32(v) for v in group]
    mn, mx = min(vals), max(vals)
    scale = f16(f32(f32(mx - mn) / 15.0))
    d = scale if scale != 0.0 else 1.0
    zero = clamp(round(f32(-mn / d)), 0, 15)
    q = [int(clamp(f32(round(f32(v / d)) + zero), 0, 15)) for v in vals]
    return q, scale, int(zero)


def pack_word(nibbles: list[int]) -> int:
    assert len(nibbles) == 8
    word = 0
    for j, v in enumerate(nibbles):
        assert 0 <= v <= 15
        word |= v << (4 * j)
    return word - (1 << 32) if word >= (1 << 31) else word  # two's-complement int32
