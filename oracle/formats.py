"""Number formats on the path, as closed forms over all codes (numpy, CPU; test infrastructure).

Format constants follow the reference type table (python/triton/language/core.py:352-363:
fp8e4nv = 1-4-3 bias 7, fp8e5 = 1-5-2 bias 15; fp16 bias 15, bf16 bias 127) and the table in its
conversion test (python/test/unit/language/test_conversions.py:295-303: (exp_bits, mant_bits,
bias, max_repr) = (4,3,7,0x7e) / (5,2,15,0x7b)).  e2m1 and e8m0 are OCP MX v1.0 formats that the
reference snapshot does not contain.
"""
from __future__ import annotations

import numpy as np

# (exponent_bits, mantissa_bits, bias, max finite code) - test_conversions.py:295-303
FP8_FORMATS = {"e4m3": (4, 3, 7, 0x7E), "e5m2": (5, 2, 15, 0x7B)}


def fp8_table(fmt: str) -> np.ndarray:
    """float32[256]: value of every code, from (-1)^s * 2^(e-bias) * (1 + m/2^mb), subnormals
    2^(1-bias) * m/2^mb.  e4m3: S.1111.111 is NaN and there is no infinity; e5m2 is IEEE-like."""
    eb, mb, bias, _ = FP8_FORMATS[fmt]
    out = np.empty(256, dtype=np.float64)
    for c in range(256):
        s = -1.0 if c >> 7 else 1.0
        e = (c >> mb) & ((1 << eb) - 1)
        m = c & ((1 << mb) - 1)
        if fmt == "e4m3" and e == 15 and m == 7:
            v = np.nan
        elif fmt == "e5m2" and e == 31:
            v = np.inf if m == 0 else np.nan
        elif e == 0:
            v = 2.0 ** (1 - bias) * (m / 2.0 ** mb)
        else:
            v = 2.0 ** (e - bias) * (1 + m / 2.0 ** mb)
        out[c] = s * v if not np.isnan(v) else np.nan
    return out.astype(np.float32)


def fp8_upcast_emulated(codes: np.ndarray, fmt: str) -> np.ndarray:
    """The reference test's bit-level emulation (test_conversions.py:178-209): place sign,
    exponent and mantissa into an fp32 pattern and multiply by 2^(127-bias).  Valid for finite
    codes (it has no inf/NaN special cases, like the kernel it restates)."""
    eb, mb, bias, _ = FP8_FORMATS[fmt]
    x = codes.astype(np.uint32)
    mant = x & ((1 << mb) - 1)
    exp = (x >> mb) & ((1 << eb) - 1)
    sign = x >> 7
    y = ((sign << 31) | (exp << 23) | (mant << (23 - mb))).astype(np.uint32).view(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        return (y.astype(np.float64) * 2.0 ** (127 - bias)).astype(np.float32)


def fp8_upcast_interpreter(codes: np.ndarray, fmt: str) -> np.ndarray:
    """Restatement of the interpreter's up-cast to fp16 (`_convert_float`,
    python/triton/runtime/interpreter.py:130-191, the path `create_dot` uses for fp8 operands,
    :542-549): subnormals are renormalised by locating the top mantissa bit (:141-158), the
    exponent is re-biased and clamped (:160-161), the mantissa shifted up (:172-174).  Returns the
    fp16 BIT PATTERNS as uint16, exactly as that function does.

    Two quirks of that function are reproduced here and NOT adopted by the build: e4m3fn NaN
    (0x7F) comes out as 480.0 (no NaN case), and e5m2 subnormals come out as 0 or 2^-15 (their
    re-biased exponent clamps to 0 and the final underflow fix-up :175-189 only covers inputs with
    a non-zero exponent field).  It agrees with the closed form on every other finite code."""
    eb, mb, bias, _ = FP8_FORMATS[fmt]
    ob, om, obias = 5, 10, 15  # fp16
    x = codes.astype(np.uint8)
    sign = (x >> 7) & 1
    significand = (x & ((1 << mb) - 1)).astype(np.uint8)
    exponent = ((x >> mb) & ((1 << eb) - 1)).astype(np.int32)
    sub = exponent == 0
    bit_pos = np.zeros(x.shape, dtype=np.int32)
    for i in range(mb):
        bit = (significand >> i) & 1
        bit_pos[bit == 1] = mb - i
    zero_sig = significand == 0
    exponent = exponent.copy()
    exponent[sub] = 1 - bit_pos[sub]
    exponent[zero_sig & sub] = bias - obias
    significand = significand.copy()
    significand[sub] = (significand[sub].astype(np.int32) << bit_pos[sub]) & ((1 << mb) - 1)
    exp_out = np.maximum(0, np.minimum(exponent - bias + obias, (1 << ob) - 1)).astype(np.uint16)
    sig_out = (significand.astype(np.uint16) << (om - mb)) & ((1 << om) - 1)
    return (sign.astype(np.uint16) << 15) | (exp_out << om) | sig_out


def e2m1_table() -> np.ndarray:
    """float32[16]: OCP e2m1 codes 0..7 -> {0, .5, 1, 1.5, 2, 3, 4, 6}; bit 3 is the sign."""
    mag = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
    return np.concatenate([mag, -mag])


def e8m0_table() -> np.ndarray:
    """float32[256]: OCP e8m0 scale byte b -> 2^(b-127); 255 -> NaN (2^-127 is an fp32 subnormal)."""
    out = np.ldexp(np.float64(1.0), np.arange(255) - 127).astype(np.float32)
    out = np.concatenate([out, np.array([np.nan], dtype=np.float32)])
    return out


def unpack_fp4(packed: np.ndarray) -> np.ndarray:
    """uint8 [..., K/2] -> codes uint8 [..., K]: element 2i in the low nibble, 2i+1 in the high one."""
    lo = packed & 15
    hi = packed >> 4
    return np.stack([lo, hi], axis=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def pack_fp4(codes: np.ndarray) -> np.ndarray:
    c = codes.reshape(*codes.shape[:-1], codes.shape[-1] // 2, 2).astype(np.uint8)
    return (c[..., 0] | (c[..., 1] << 4)).astype(np.uint8)


def round_bf16(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 (round to nearest even, the default cast: python/triton/language/semantic.py:752-755),
    returned as the fp32 value of the rounded number."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = np.isnan(x)
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16
    out = r.view(np.float32).copy()
    out[nan] = np.nan
    return out


def round_fp16(x: np.ndarray) -> np.ndarray:
    """fp32 -> fp16 RTNE (`ndarray.astype(np.float16)`, interpreter.py:385-393), as an fp32 value."""
    with np.errstate(over="ignore"):
        return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "fp16":
        return round_fp16(x)
    if dtype == "bf16":
        return round_bf16(x)
    if dtype == "fp32":
        return np.asarray(x, dtype=np.float32)
    if dtype in FP8_FORMATS:
        # `x.to(tl.float8e5)` / `.to(tl.float8e4nv)`: RTNE, saturating (see encode_fp8)
        return fp8_table(dtype)[encode_fp8(np.asarray(x, dtype=np.float32), dtype)].astype(np.float32)
    raise ValueError(dtype)


def encode_fp8(x: np.ndarray, fmt: str) -> np.ndarray:
    """fp32 -> fp8 codes, round to nearest even, overflow saturates to the largest finite code
    (the down-cast maxima of test_conversions.py:307-329: 448 for e4m3fn, 57344 for e5m2).
    Brute force over the table (nearest value, ties to the even code), so it shares no logic
    with the bit-twiddling encoders it is used to check."""
    eb, mb, bias, max_code = FP8_FORMATS[fmt]
    tab = fp8_table(fmt).astype(np.float64)
    pos = tab[: max_code + 1]  # non-negative finite codes, increasing
    a = np.abs(np.asarray(x, dtype=np.float64))
    idx = np.searchsorted(pos, a, side="left")
    idx = np.clip(idx, 1, max_code)
    lo, hi = pos[idx - 1], pos[idx]
    pick_hi = (a - lo > hi - a) | ((a - lo == hi - a) & ((idx & 1) == 0))
    code = np.where(pick_hi, idx, idx - 1)
    code = np.where(a >= pos[max_code], max_code, code)
    code = np.where(a == 0, 0, code).astype(np.uint8)
    sign = (np.signbit(x).astype(np.uint8)) << 7
    out = code | sign
    return np.where(np.isnan(x), np.uint8(0x7F), out).astype(np.uint8)
