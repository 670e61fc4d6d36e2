"""TEST INFRASTRUCTURE (oracle) -- not part of the product path.

Narrow floating-point formats restated in numpy integer arithmetic.

* bf16: upper 16 bits of IEEE binary32, round-to-nearest-even on conversion
  (StableHLO `convert` semantics; dtype code BF16=16 in the reference's
  src/xla/Utils.jl:18-40).
* f8E4M3FN (OCP e4m3): 1 sign, 4 exponent (bias 7), 3 mantissa, no infinity,
  0x7F/0xFF are NaN, max finite 448 (dtype code F8E4M3FN=20; the reference maps
  Float8s/DLFP8Types onto it in ext/ReactantFloat8sExt.jl:6 and
  ext/ReactantDLFP8TypesExt.jl:14-17, promotion rules src/PrimitiveTypes.jl:6-48).
* f8E5M2: 1/5/2, bias 15, has inf/NaN (truncated binary16).

Values are carried as float32 arrays that only hold representable numbers;
`*_to_bits` / `*_from_bits` give the storage bytes.

Pinned by tests/test_oracle_lowfloat.py against (a) the closed-form 256-entry
decode tables from the OCP FP8 specification and (b) torch CPU casts as an
independent library.
"""
import numpy as np


def f32_to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = (u + 0x7FFF + lsb) >> 16
    r = r.astype(np.uint16)
    nan = np.isnan(x)
    if np.any(nan):
        r = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)
    return r


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def round_bf16(x):
    return bf16_bits_to_f32(f32_to_bf16_bits(x)).reshape(np.shape(x))


def _decode_table(ebits, mbits, bias, fn):
    out = np.zeros(256, dtype=np.float32)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> mbits) & ((1 << ebits) - 1)
        m = code & ((1 << mbits) - 1)
        if fn:
            if e == (1 << ebits) - 1 and m == (1 << mbits) - 1:
                out[code] = np.nan
                continue
        else:
            if e == (1 << ebits) - 1:
                out[code] = s * np.inf if m == 0 else np.nan
                continue
        if e == 0:
            v = m * 2.0 ** (1 - bias - mbits)
        else:
            v = (1.0 + m / float(1 << mbits)) * 2.0 ** (e - bias)
        out[code] = s * v
    return out


E4M3FN_TABLE = _decode_table(4, 3, 7, True)
E5M2_TABLE = _decode_table(5, 2, 15, False)


def _f32_to_f8_bits(x, ebits, mbits, bias, fn):
    """Round-to-nearest-even f32 -> 8-bit float.  Overflow after rounding gives
    NaN for the FN (no-infinity) format and inf for the IEEE-like one."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    shape = x.shape
    xf = x.reshape(-1).astype(np.float64)
    sign = np.signbit(xf)
    a = np.abs(xf)
    out = np.zeros(a.shape, dtype=np.uint8)
    nan = np.isnan(a)
    inf = np.isinf(a)
    fin = ~(nan | inf)
    av = np.where(fin, a, 0.0)
    # quantum of the binade holding |x|
    min_norm_exp = 1 - bias
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(av > 0, av, 1.0))).astype(np.int64)
    # guard against log2 rounding at binade edges
    e = np.where(2.0 ** e > av, e - 1, e)
    e = np.where(2.0 ** (e + 1) <= av, e + 1, e)
    e = np.maximum(e, min_norm_exp)
    q = 2.0 ** (e - mbits)
    n = av / q  # exact in f64
    r = np.rint(n)  # ties to even
    v = r * q
    # re-derive the code from the rounded value
    with np.errstate(divide="ignore"):
        e2 = np.floor(np.log2(np.where(v > 0, v, 1.0))).astype(np.int64)
    e2 = np.where(2.0 ** e2 > v, e2 - 1, e2)
    e2 = np.where(2.0 ** (e2 + 1) <= v, e2 + 1, e2)
    sub = v < 2.0 ** min_norm_exp
    mant_sub = np.rint(v / 2.0 ** (min_norm_exp - mbits)).astype(np.int64)
    mant_norm = np.rint((v / 2.0 ** e2 - 1.0) * (1 << mbits)).astype(np.int64)
    expf = np.where(sub, 0, e2 + bias)
    mant = np.where(sub, mant_sub, mant_norm)
    code = (expf << mbits) | mant
    emax_field = (1 << ebits) - 1
    if fn:
        max_code = (emax_field << mbits) | ((1 << mbits) - 2)
        nan_code = 0x7F
        over = code > max_code
        code = np.where(over, nan_code, code)
        code = np.where(inf | nan, nan_code, code)
    else:
        inf_code = emax_field << mbits
        over = code >= inf_code
        code = np.where(over | inf, inf_code, code)
        code = np.where(nan, inf_code | 1 | (1 << (mbits - 1)), code)
    code = np.where(v == 0, np.where(inf | nan, code, 0), code)
    out = code.astype(np.uint8) | (sign.astype(np.uint8) << 7)
    return out.reshape(shape)


def f32_to_e4m3fn_bits(x):
    return _f32_to_f8_bits(x, 4, 3, 7, True)


def f32_to_e5m2_bits(x):
    return _f32_to_f8_bits(x, 5, 2, 15, False)


def e4m3fn_bits_to_f32(b):
    return E4M3FN_TABLE[np.asarray(b, dtype=np.uint8)]


def e5m2_bits_to_f32(b):
    return E5M2_TABLE[np.asarray(b, dtype=np.uint8)]


def round_e4m3fn(x):
    return e4m3fn_bits_to_f32(f32_to_e4m3fn_bits(x))


def round_e5m2(x):
    return e5m2_bits_to_f32(f32_to_e5m2_bits(x))


def f32_to_f16_bits(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)
