"""TEST ORACLE, not product code: OCP e4m3 ("fn": finite only, max 448, NaN = 0x7f) codec in numpy.

Restates FP32toFP8E4M3FN / FP8E4M3FNtoFP32 (src/utils/fp8_utils.h:111-155) as arithmetic:
round to nearest even onto the grid {m/8 * 2^-6 (subnormal), (1 + m/8) * 2^(e-7)}, saturating
to +-448 (infinities included), NaN -> 0x7f. Pinned in tests/test_oracle_nn.py against the
reference functions compiled into oracle/_ref and against a brute-force nearest-code search.
"""
import numpy as np


def e4m3_table():
    """float32[256]: value of every code (NaN for 0x7f / 0xff)."""
    codes = np.arange(256)
    e = (codes >> 3) & 15
    m = (codes & 7).astype(np.float64)
    mag = np.where(e == 0, m / 8.0 * 2.0 ** -6, (1.0 + m / 8.0) * 2.0 ** (e - 7.0))
    mag = np.where((codes & 0x7F) == 0x7F, np.nan, mag)
    return np.where(codes & 0x80, -mag, mag).astype(np.float32)


_TABLE = e4m3_table()


def e4m3_decode(codes):
    return _TABLE[np.asarray(codes, np.uint8)]


def e4m3_encode(x):
    """float array -> uint8 codes, round to nearest even, saturating."""
    x = np.asarray(x, np.float32)
    sign = np.signbit(x).astype(np.uint8) << 7
    with np.errstate(invalid="ignore"):
        a = np.abs(x).astype(np.float64)
    nan = np.isnan(a)
    a = np.where(nan, 0.0, np.minimum(a, 448.0))
    # exponent of the grid the value falls on: subnormals share the spacing 2^-9 of the first binade
    with np.errstate(divide="ignore"):
        ex = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    ex = np.clip(ex, -6, 8)
    step = 2.0 ** (ex - 3)
    q = np.rint(a / step)              # numpy rint is round-half-even; a/step is exact (power-of-two divisor)
    mag = q * step                     # may carry into the next binade, which is still on the grid
    # code from magnitude
    with np.errstate(divide="ignore"):
        e2 = np.floor(np.log2(np.where(mag > 0, mag, 1.0)))
    e2 = np.clip(e2, -6, 8)
    sub = mag < 2.0 ** -6
    mant = np.where(sub, mag / 2.0 ** -9, (mag / 2.0 ** e2 - 1.0) * 8.0)
    code = np.where(sub, mant, (e2 + 7) * 8 + mant).astype(np.uint8)
    code = np.where(nan, 0x7F, code).astype(np.uint8)
    return (code | sign).astype(np.uint8)


def quantize_rows(w):
    """Per-row weight quantisation: scale = absmax / 448 (1 for an all-zero row).
    Returns (codes uint8 [N,K], scale float32 [N])."""
    w = np.asarray(w, np.float32)
    amax = np.abs(w).max(axis=1)
    scale = np.where(amax > 0, amax / np.float32(448.0), 1.0).astype(np.float32)
    return e4m3_encode(w / scale[:, None]), scale
