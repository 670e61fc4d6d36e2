"""Host-side packing of bf16 / f8E4M3FN / f8E5M2 values into their storage bytes.

numpy has no such dtypes; arrays of these types travel as uint16 / uint8 bit
patterns (what Julia's BFloat16s / Float8s / DLFP8Types arrays hold in memory;
type map in the reference: src/PrimitiveTypes.jl:6-48, ext/ReactantFloat8sExt.jl:6).
Conversions round to nearest even; f8E4M3FN has no infinity and overflows to NaN.
"""
import numpy as np


def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _f8_table(ebits, mbits, bias, fn):
    t = np.zeros(256, dtype=np.float32)
    for c in range(256):
        e = (c >> mbits) & ((1 << ebits) - 1)
        m = c & ((1 << mbits) - 1)
        s = -1.0 if c & 0x80 else 1.0
        top = (1 << ebits) - 1
        if fn and e == top and m == (1 << mbits) - 1:
            t[c] = np.nan
        elif not fn and e == top:
            t[c] = s * np.inf if m == 0 else np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** (1 - bias - mbits)
        else:
            t[c] = s * (1 + m / (1 << mbits)) * 2.0 ** (e - bias)
    return t


_E4M3 = _f8_table(4, 3, 7, True)
_E5M2 = _f8_table(5, 2, 15, False)


def f8e4m3fn_bits_to_f32(b):
    return _E4M3[np.asarray(b, dtype=np.uint8)]


def f8e5m2_bits_to_f32(b):
    return _E5M2[np.asarray(b, dtype=np.uint8)]


def _to_f8(x, table, nan_code, overflow_code):
    """Nearest-even rounding by searching the sorted table of finite positives."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    codes = np.array([c for c in range(128) if np.isfinite(table[c])], dtype=np.int64)
    vals = table[codes].astype(np.float64)
    idx = np.clip(np.searchsorted(vals, a), 1, len(vals) - 1)
    lo, hi = vals[idx - 1], vals[idx]
    pick_hi = (a - lo > hi - a) | ((a - lo == hi - a) & (codes[idx] % 2 == 0))
    c = np.where(pick_hi, codes[idx], codes[idx - 1])
    # beyond the largest finite value: halfway to the next (absent) step still rounds down
    vmax = vals[-1]
    step = vals[-1] - vals[-2]
    c = np.where(a > vmax, np.where((a - vmax < step / 2) | ((a - vmax == step / 2) & (codes[-1] % 2 == 0)),
                                    codes[-1], overflow_code), c)
    c = np.where(np.isinf(a), overflow_code, c)
    c = np.where(np.isnan(a), nan_code, c)
    return (c.astype(np.uint8) | (np.signbit(x).astype(np.uint8) << 7)).astype(np.uint8)


def f32_to_f8e4m3fn_bits(x):
    return _to_f8(x, _E4M3, 0x7F, 0x7F)


def f32_to_f8e5m2_bits(x):
    return _to_f8(x, _E5M2, 0x7F, 0x7C)
