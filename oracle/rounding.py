"""Single-rounding conversions used by the oracle.  Test infrastructure only.

All "T-typed" tensors of the oracle are numpy float32 arrays whose values are
exactly representable in T (bf16 or fp16).  These helpers round an exact
binary64 (or binary32) value ONCE, to nearest-even, into such a value.

Pinned by tests/test_oracle_rounding.py against library routines:
``torch.Tensor.to(torch.bfloat16)`` / ``numpy.float16`` on fp32-representable
inputs, hand-built double-rounding traps, and an exhaustive comparison of
``f32_to_e4m3fn`` with ``torch.float8_e4m3fn`` over every fp16 value in range
(the reference's ``cvt.rn.satfinite.e4m3x2.f32``, csrc/numeric_conversion.cuh:48-63).
"""
import numpy as np

BF16 = "bf16"
FP16 = "fp16"

_BF16_MAX = float((2.0 - 2.0 ** -7) * 2.0 ** 127)
_BF16_OVF = float((2.0 - 2.0 ** -8) * 2.0 ** 127)  # ties-to-even goes to inf from here


def f64_to_bf16(x):
    """Round binary64 -> bf16 directly (one rounding, RNE).  Returns float32."""
    x = np.asarray(x, dtype=np.float64)
    ax = np.abs(x)
    with np.errstate(invalid="ignore", over="ignore"):
        bits = ax.view(np.uint64) if ax.flags.c_contiguous else np.ascontiguousarray(ax).view(np.uint64)
        lsb = (bits >> np.uint64(45)) & np.uint64(1)
        r = ((bits + np.uint64((1 << 44) - 1) + lsb) >> np.uint64(45)) << np.uint64(45)
        y = r.view(np.float64).reshape(ax.shape)
        sub = ax < 2.0 ** -126
        y = np.where(sub, np.rint(ax * 2.0 ** 133) * 2.0 ** -133, y)
        y = np.where(ax >= _BF16_OVF, np.inf, y)
        y = np.where(np.isnan(x), np.nan, y)
        y = np.copysign(y, x)
    return y.astype(np.float32)


def f64_to_f16(x):
    """Round binary64 -> fp16 directly (numpy converts with one rounding)."""
    with np.errstate(over="ignore"):
        return np.asarray(x, dtype=np.float64).astype(np.float16).astype(np.float32)


def round_to(x, dtype):
    """Round exact binary64 values once to T in {bf16, fp16}; result as float32."""
    if dtype == BF16:
        return f64_to_bf16(x)
    if dtype == FP16:
        return f64_to_f16(x)
    raise ValueError(f"unknown dtype tag {dtype!r}")


def bits16(x, dtype):
    """16-bit pattern of T-typed values (given as float32)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == BF16:
        return (x.view(np.uint32) >> np.uint32(16)).astype(np.uint16)
    if dtype == FP16:
        return x.astype(np.float16).view(np.uint16)
    raise ValueError(dtype)


def from_bits16(b, dtype):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    if dtype == BF16:
        return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)
    if dtype == FP16:
        return b.view(np.float16).astype(np.float32)
    raise ValueError(dtype)


# --------------------------------------------------------------------------
# OCP FP8 e4m3fn (1-4-3, bias 7, max 448, no inf, NaN = 0x7f/0xff)
# --------------------------------------------------------------------------

def _e4m3_table():
    t = np.zeros(256, dtype=np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 7
        if e == 15 and m == 7:
            v = np.nan
        elif e == 0:
            v = m * 2.0 ** -9
        else:
            v = (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[c] = s * v
    return t


E4M3_VALUES = _e4m3_table()


def f32_to_e4m3fn(x):
    """fp32 -> e4m3fn code (uint8): RNE, saturate-to-finite (+-448), NaN -> 0x7f|sign."""
    x = np.asarray(x, dtype=np.float32)
    ax = np.abs(x).astype(np.float64)
    with np.errstate(invalid="ignore", divide="ignore"):
        _, ex = np.frexp(ax)               # ax = m * 2**ex, m in [0.5, 1)
        e = np.maximum(ex - 1, -6)         # exponent of the binade, clamped to the subnormal one
        q = np.ldexp(1.0, e - 3)           # spacing of representable values in that binade
        y = np.rint(ax / q) * q            # RNE (ax/q is exact: power-of-two divide)
        y = np.minimum(y, 448.0)
        _, ey = np.frexp(y)
        ey = ey - 1
        normal = y >= 2.0 ** -6
        code_n = ((ey + 7).astype(np.int64) << 3) | np.rint((y / np.ldexp(1.0, ey) - 1.0) * 8.0).astype(np.int64)
        code_s = np.rint(y * 2.0 ** 9).astype(np.int64)
        code = np.where(normal, code_n, code_s)
        code = np.where(np.isnan(ax), 0x7F, code)
    sign = (np.signbit(x).astype(np.int64)) << 7
    return (code | sign).astype(np.uint8)


def e4m3fn_to_f32(code):
    return E4M3_VALUES[np.asarray(code, dtype=np.uint8)]
