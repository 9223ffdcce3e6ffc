"""Bit-level OCP FP8 E4M3 ("e4m3fn") encode/decode in numpy, written from the format
definition (OCP 8-bit Floating Point Specification, section 5: 1 sign, 4 exponent bits with
bias 7, 3 mantissa bits, subnormals at exponent 0, no infinities, S.1111.111 = NaN,
largest finite 448).

TEST INFRASTRUCTURE ONLY: an independent second implementation against which both
torch's `.to(torch.float8_e4m3fn)` (what the reference calls, src/inference/attention.py:
109-110) and the HIP encoder are checked.  It rounds by exact rational comparison against
the table of representable values instead of by bit tricks, so a mistake in a rounding
constant cannot be shared with the implementations under test.

Overflow follows the cast the reference relies on: no saturation; a magnitude whose
round-to-nearest-even result would exceed 448 (i.e. >= 464 after rounding ties to even,
464 itself rounds to 448), infinities and NaN become NaN (0x7F | sign).
"""
import numpy as np


def decode_table():
    """float64 value of each of the 256 byte codes (NaN for 0x7F and 0xFF)."""
    out = np.empty(256, dtype=np.float64)
    for b in range(256):
        sign = -1.0 if b & 0x80 else 1.0
        e = (b >> 3) & 0xF
        m = b & 0x7
        if e == 0xF and m == 0x7:
            out[b] = np.nan
        elif e == 0:
            out[b] = sign * (m / 8.0) * 2.0 ** -6
        else:
            out[b] = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return out


_TABLE = decode_table()
_POS = _TABLE[:0x7F]            # 0 .. 448 ascending, codes 0x00..0x7E


def decode(bytes_u8):
    """uint8 array -> float32 array (exact)."""
    return _TABLE[np.asarray(bytes_u8, dtype=np.uint8)].astype(np.float32)


def encode(x):
    """float array -> uint8 e4m3fn codes, round-to-nearest-even, NaN on overflow."""
    x = np.asarray(x, dtype=np.float32)
    flat = x.reshape(-1)
    a = np.abs(flat).astype(np.float64)
    sign = (np.signbit(flat)).astype(np.uint8) << 7
    # nearest representable magnitude by search in the sorted table
    hi = np.searchsorted(_POS, a, side="left")          # first code with value >= a
    hi = np.clip(hi, 0, len(_POS) - 1)
    lo = np.clip(hi - 1, 0, len(_POS) - 1)
    d_hi = np.abs(_POS[hi] - a)
    d_lo = np.abs(a - _POS[lo])
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = np.where(pick_lo, lo, hi).astype(np.int64)
    # beyond the largest finite value: the next grid point would be 480 (mantissa 111 at the
    # top exponent, which is the NaN code); ties-to-even at the midpoint 464 stays on 448
    over = a > 448.0
    code = np.where(over & (a <= 464.0), 0x7E, code)
    code = np.where(over & (a > 464.0), 0x7F, code)
    code = np.where(np.isnan(a), 0x7F, code)
    return (code.astype(np.uint8) | sign).reshape(x.shape)
