"""E4M3FN codec in integer arithmetic (numpy). Test infrastructure only.

Format (reference tests/e4m3_vectors.py:17-22): byte s eeee mmm, bias 7; e == 0 is subnormal m * 2^-9, otherwise
(8 + m) * 2^(e - 10); 0x7F and 0xFF are NaN; the largest finite value is 0x7E = 448; there are no infinities.
"""
import numpy as np


def decode(codes):
    """uint8 codes -> float32 values, exactly (reference kernels/core/python/crit_kcore/formats.py:49-58; NaN codes
    decode to NaN here rather than to +-480)."""
    b = np.asarray(codes, dtype=np.uint8).astype(np.int32)
    e = (b >> 3) & 15
    m = (b & 7).astype(np.float32)
    unit = ((e + 117) << 23).astype(np.int32).view(np.float32)      # 2^(e - 10)
    mag = np.where(e == 0, m * np.float32(2.0 ** -9), (m + np.float32(8.0)) * unit).astype(np.float32)
    mag = np.where((b & 0x7F) == 0x7F, np.float32(np.nan), mag)
    return np.where((b & 0x80) != 0, -mag, mag).astype(np.float32)


def magnitude(byte):
    """|value| of one E4M3FN byte from its fields alone, None for NaN (reference tests/e4m3_vectors.py:17-22)."""
    exponent, mantissa = (byte >> 3) & 15, byte & 7
    if exponent == 15 and mantissa == 7:
        return None
    return mantissa * 2.0 ** -9 if exponent == 0 else (8 + mantissa) * 2.0 ** (exponent - 10)


def encode(x):
    """float32 values -> uint8 codes: clamp to [-448, 448], then round to the nearest code with ties to even
    (reference formats.py:61-79 for the rounding; inference/attention-state/code/pages.py:444 for the clamp before it).
    The sign comes from the sign bit, so -0.0 and negatives that round to zero give 0x80. NaN gives 0x7F | sign."""
    x = np.asarray(x, dtype=np.float32)
    nan = np.isnan(x)
    with np.errstate(invalid="ignore"):
        c = np.where(nan, np.float32(0), np.clip(x, np.float32(-448.0), np.float32(448.0))).astype(np.float32)
    a = np.abs(c)
    bits = a.view(np.int32)
    ex = (bits >> 23) - 127
    # Normal codes: scale the magnitude into [1, 2) exactly, round the mantissa to 3 bits with rint (ties to even).
    safe_ex = np.clip(ex, -126, 127)
    frac = a * ((127 - safe_ex) << 23).astype(np.int32).view(np.float32)
    mant = np.rint((frac - np.float32(1.0)) * np.float32(8.0)).astype(np.int32)
    carry = mant == 8
    ex = np.where(carry, ex + 1, ex)
    mant = np.where(carry, 0, mant)
    normal = ((ex + 7) << 3) | mant
    # Below 2^-6 the codes are subnormal, multiples of 2^-9 (code 8, the smallest normal, falls out of the rounding).
    sub = np.rint(a * np.float32(512.0)).astype(np.int32)
    code = np.where(a < np.float32(0.015625), sub, normal)
    code = np.where(nan, 0x7F, code)
    sign = (x.view(np.int32) >> 24) & 0x80
    return (code | sign).astype(np.uint8)
