"""OCP FP8 e4m3fn (finite + NaN, max 448) encode / decode on the CPU.

Oracle code: test infrastructure only.

The reference stores activations with ``__nv_cvt_float_to_fp8(v, __NV_SATFINITE,
__NV_E4M3)`` after clamping to +-448
(batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_ops.cu:99-103), i.e.
round-to-nearest-even into e4m3fn.  ``e4m3fn_encode`` restates that rounding
with integer arithmetic on the fp32 bit pattern; it does not call torch's cast,
so the test that compares the two pins it to a library routine.
"""
from __future__ import annotations

import numpy as np

E4M3_MAX = np.float32(448.0)


def e4m3fn_decode_table() -> np.ndarray:
    """All 256 byte values -> float32 (0x7F / 0xFF are NaN)."""
    out = np.empty(256, dtype=np.float32)
    for b in range(256):
        sign = -1.0 if (b & 0x80) else 1.0
        exp = (b >> 3) & 0xF
        man = b & 0x7
        if exp == 0xF and man == 0x7:
            v = float("nan")
        elif exp == 0:
            v = sign * man * 2.0 ** -9          # subnormal: man/8 * 2^-6
        else:
            v = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
        out[b] = v
    return out


_DECODE = e4m3fn_decode_table()


def e4m3fn_decode(b: np.ndarray) -> np.ndarray:
    return _DECODE[np.asarray(b, dtype=np.uint8)]


def e4m3fn_encode(x: np.ndarray) -> np.ndarray:
    """float32 -> e4m3fn byte, round-to-nearest-even, saturating at +-448.

    NaN -> 0x7F.  The callers on the path clamp to +-448 first, so saturation
    is only exercised by the tests.
    """
    x = np.asarray(x, dtype=np.float32)
    sign = (x.view(np.uint32) >> 31).astype(np.uint8) << 7
    a = np.abs(x).astype(np.float64)
    nan = np.isnan(a)
    a = np.where(nan, 0.0, a)
    a = np.minimum(a, 448.0)
    # subnormal range |x| < 2^-6 : units of 2^-9, RNE (np.rint is half-to-even)
    sub = np.rint(a * 512.0)                       # 0..8 ; 8 == 0x08 == 2^-6
    # normal range
    m, e = np.frexp(np.where(a > 0, a, 1.0))       # a = m * 2^e, m in [0.5,1)
    e = e - 1                                      # a = (2m) * 2^e, 2m in [1,2)
    man = np.rint((2.0 * m - 1.0) * 8.0)           # 0..8
    carry = man == 8
    e = np.where(carry, e + 1, e)
    man = np.where(carry, 0, man)
    norm = ((e + 7).astype(np.int64) << 3) | man.astype(np.int64)
    code = np.where(a < 2.0 ** -6, sub.astype(np.int64), norm)
    code = np.minimum(code, 0x7E).astype(np.uint8)
    out = code | sign
    out = np.where(nan, np.uint8(0x7F), out).astype(np.uint8)
    return out
