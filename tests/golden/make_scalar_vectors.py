"""Writes tests/golden/scalar_vectors.npz: decode tables and per-element known answers.

Everything here is computed with exact rationals and Python integers from the format definitions (OCP FP8 E4M3 /
E5M2, FP6 E3M2 / E2M3) and from the bit-level rules of the reference kernel, independently of the C oracle and of the
HIP library:

  decode_<fmt>      value of every code (fp32 bits); E4M3 0x7F / 0xFF and E5M2 exponent 31 are not finite
  cast_x            fp32 inputs: every grid point, every midpoint, midpoint +/- 1 ulp, the overflow edges
  cast_sw_<fmt>     software cast (FQ:125-215): nearest even, zero result +0, E4M3 above 464 and E5M2 from 61440
                    upward give the NaN pattern 0x7FFFFFFF, E3M2 / E2M3 saturate at 28 / 7.5
  cast_hw_<fmt>     hardware cast model (FQ:218-245): nearest even, saturating, the sign of a zero result is kept
  sqdd_x, sqdd_s    bf16 inputs (as bits) and fp32 scales (as bits) for scale -> cast -> descale
  sqdd_fp32_<fmt>   bf16 bits of fp32_to_bf16(cast_hw(x * s) / s), IEEE fp32 arithmetic (FQ:310-316, 46-60)
  sqdd_e8_<fmt>     the same with the scale's exponent added to / subtracted from the exponent field, clamped at 0
                    with the mantissa kept (FQ:283-305): a zero cast result comes back as 2^(-e8-127) when e8 < 0

Usage: python tests/golden/make_scalar_vectors.py
"""
import os
import struct
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# name -> (exponent bits, mantissa bits, bias, number of finite non-negative codes)
FORMATS = {"e4m3": (4, 3, 7, 127), "e5m2": (5, 2, 15, 124), "e3m2": (3, 2, 3, 32), "e2m3": (2, 3, 1, 32)}
NAN_BITS = 0x7FFFFFFF


def f2b(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def b2f(b):
    return struct.unpack("<f", struct.pack("<I", b & 0xFFFFFFFF))[0]


def code_value(fmt, code):
    """Exact value of a non-negative code, also one step past the largest finite code (the overflow neighbour)."""
    eb, mb, bias, _ = FORMATS[fmt]
    e, m = code >> mb, code & ((1 << mb) - 1)
    if e == 0:
        return Fraction(m, 1 << mb) * Fraction(2) ** (1 - bias)
    return (1 + Fraction(m, 1 << mb)) * Fraction(2) ** (e - bias)


def decode_table(fmt):
    eb, mb, bias, nfinite = FORMATS[fmt]
    ncodes = 1 << (1 + eb + mb)
    out = np.zeros(ncodes, np.uint32)
    for c in range(ncodes):
        mag, sign = c & (ncodes // 2 - 1), c >> (eb + mb)
        if mag < nfinite:
            out[c] = f2b(float(code_value(fmt, mag))) | (sign << 31)
        elif fmt == "e5m2" and mag == 124:
            out[c] = 0x7F800000 | (sign << 31)
        else:
            out[c] = 0x7FC00000 | (sign << 31)
    return out


def nearest_even_code(fmt, a):
    """Index of the code nearest to the non-negative rational a (ties to the even code); may return the overflow
    neighbour nfinite."""
    n = FORMATS[fmt][3]
    lo, hi = 0, n
    while hi - lo > 1:
        mid = (lo + hi) // 2
        if code_value(fmt, mid) <= a:
            lo = mid
        else:
            hi = mid
    if a >= code_value(fmt, n):
        return n
    dlo, dhi = a - code_value(fmt, lo), code_value(fmt, hi) - a
    if dlo < dhi:
        return lo
    if dhi < dlo:
        return hi
    return lo if lo % 2 == 0 else hi


def cast(fmt, xbits, hw):
    """fp32 bits -> fp32 bits of the cast value (finite inputs)."""
    n = FORMATS[fmt][3]
    sign = xbits & 0x80000000
    a = Fraction(b2f(xbits & 0x7FFFFFFF))
    c = nearest_even_code(fmt, a)
    if c == n:
        if not hw and fmt in ("e4m3", "e5m2"):
            return NAN_BITS
        c = n - 1
    if c == 0:
        return sign if hw else 0
    return f2b(float(code_value(fmt, c))) | sign


def rhu_bf16(bits):
    """fp32 bits -> bf16 bits, half-up on the magnitude (FQ:46-60); an exponent carried past 255 gives 0x8000."""
    mag = (bits & 0x7FFFFFFF) + 0x8000
    if mag >> 31:
        return 0x8000
    return ((bits >> 16) & 0x8000) | (mag >> 16)


def mul32(a, b):
    return f2b(float(np.float32(b2f(a)) * np.float32(b2f(b))))


def div32(a, b):
    with np.errstate(all="ignore"):
        return f2b(float(np.float32(b2f(a)) / np.float32(b2f(b))))


def sqdd_fp32(fmt, x16, sbits):
    return rhu_bf16(div32(cast(fmt, mul32(x16 << 16, sbits), True), sbits))


def shift_exponent(bits, delta):
    e = ((bits >> 23) & 0xFF) + delta
    e = max(e, 0)
    assert e < 255
    return (bits & 0x807FFFFF) | (e << 23)


def sqdd_e8(fmt, x16, sbits):
    e8 = ((sbits >> 23) & 0xFF) - 127
    return rhu_bf16(shift_exponent(cast(fmt, shift_exponent(x16 << 16, e8), True), -e8))


def cast_inputs():
    xs = set()
    for fmt, (eb, mb, bias, n) in FORMATS.items():
        for c in range(n):
            a, b = code_value(fmt, c), code_value(fmt, c + 1)
            mid = f2b(float((a + b) / 2))
            for v in (f2b(float(a)), mid, mid - 1, mid + 1):
                xs.add(v)
                xs.add(v | 0x80000000)
    for v in (0.0, 1e-30, 2.0 ** -20, 463.0, 464.0, 465.0, 480.0, 61439.0, 61440.0, 65536.0, 1e6, 3e38, 7.75, 8.0, 29.0, 30.0):
        xs.add(f2b(v))
        xs.add(f2b(v) | 0x80000000)
    return np.array(sorted(xs), np.uint32)


def sqdd_inputs():
    rng = np.random.default_rng(20240)
    x = list(rng.integers(0, 0x7F80, 400)) + [0x0000, 0x8000, 0x0001, 0x007F, 0x0080, 0x3F80, 0xBF80, 0x43E0, 0x7F7F, 0x3A83, 0x2000]
    x = [int(v) | (int(rng.integers(0, 2)) << 15) if v not in (0x0000, 0x8000) else int(v) for v in x]
    scales = [448.0 / 240.0, 1.0, 0.448, 0.0004, 7.5 / 300.0, 57344.0 / 3.0, 448.0 / 1e-3, 2.0 ** -12, 2.0 ** 20, 3.9999, 448.0 / 0.0123]
    xs, ss = [], []
    for s in scales:
        sb = f2b(float(np.float32(s)))
        for v in x:
            e = (v >> 7) & 0xFF
            e8 = ((sb >> 23) & 0xFF) - 127
            if e + e8 >= 200:                       # keep clear of the exponent-field overflow the kernel never guards
                continue
            xs.append(v)
            ss.append(sb)
    return np.array(xs, np.uint16), np.array(ss, np.uint32)


def main():
    out = {}
    for fmt in FORMATS:
        out[f"decode_{fmt}"] = decode_table(fmt)
    cx = cast_inputs()
    out["cast_x"] = cx
    for fmt in FORMATS:
        out[f"cast_sw_{fmt}"] = np.array([cast(fmt, int(v), False) for v in cx], np.uint32)
    for fmt in ("e4m3", "e5m2"):
        out[f"cast_hw_{fmt}"] = np.array([cast(fmt, int(v), True) for v in cx], np.uint32)
    sx, ss = sqdd_inputs()
    out["sqdd_x"], out["sqdd_s"] = sx, ss
    for fmt in ("e4m3", "e5m2"):
        out[f"sqdd_fp32_{fmt}"] = np.array([sqdd_fp32(fmt, int(a), int(b)) for a, b in zip(sx, ss)], np.uint16)
        out[f"sqdd_e8_{fmt}"] = np.array([sqdd_e8(fmt, int(a), int(b)) for a, b in zip(sx, ss)], np.uint16)
    np.savez_compressed(os.path.join(HERE, "scalar_vectors.npz"), **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
