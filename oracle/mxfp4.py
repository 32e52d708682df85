"""MXFP4 (e2m1 values + one e8m0 scale per 32 along K) on the CPU.  Oracle
code: test infrastructure only.

``dequant`` restates ``mxfp4_dequantize_oracle``
(batchgen/moe/mxfp4_oracle_vector.py:80-115): low nibble = even K element,
high nibble = odd; nibble bit 3 = sign, bits 0-2 index
[0, .5, 1, 1.5, 2, 3, 4, 6]; scale = 2^(byte - 127), no clamp.

``quantize`` has no counterpart in the reference (it holds no MXFP4 quantiser:
its tests draw random nibbles and scale bytes, tests/kimi_k3_harness.py:427-448);
parity unpinned there.  It follows the OCP Microscaling v1.0 closed form:
shared exponent = floor(log2(amax)) - 2 (2 = emax of e2m1), elements rounded to
nearest-even e2m1 with saturation at +-6.  Scale bytes are kept inside
[1, 254]: 0x00 and 0xFF are forbidden by the reference loader
(mxfp4_oracle_vector.py:55).
"""
from __future__ import annotations

import numpy as np

F32 = np.float32
E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
LUT16 = np.concatenate([E2M1, -E2M1]).astype(np.float32)
GROUP = 32


def dequant(packed: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """packed [..., K/2] uint8, scales [..., K/32] uint8 -> float32 [..., K]."""
    packed = np.asarray(packed, dtype=np.uint8)
    scales = np.asarray(scales, dtype=np.uint8)
    lo = LUT16[packed & 0x0F]
    hi = LUT16[packed >> 4]
    vals = np.empty(packed.shape[:-1] + (packed.shape[-1] * 2,), dtype=np.float32)
    vals[..., 0::2] = lo
    vals[..., 1::2] = hi
    exp = scales.astype(np.int32) - 127
    exp = np.repeat(exp, GROUP, axis=-1)
    return np.ldexp(vals.astype(np.float64), exp).astype(np.float32)


def _e2m1_code(a: np.ndarray) -> np.ndarray:
    """|value| (already divided by the scale) -> code 0..7, round-to-nearest-even."""
    code = np.zeros(a.shape, dtype=np.uint8)
    # midpoints; a tie goes to the neighbour with an even code
    for mid, tie_up in ((0.25, False), (0.75, True), (1.25, False), (1.75, True),
                        (2.5, False), (3.5, True), (5.0, False)):
        code += ((a >= mid) if tie_up else (a > mid)).astype(np.uint8)
    return code


def quantize(w: np.ndarray):
    """w [..., K] fp32 (K % 32 == 0) -> (packed [..., K/2] u8, scales [..., K/32] u8)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    *lead, k = w.shape
    assert k % GROUP == 0
    g = w.reshape(*lead, k // GROUP, GROUP)
    amax = np.abs(g).max(axis=-1)
    _, e = np.frexp(np.where(amax > 0, amax, 1.0))       # amax = m*2^e, m in [.5,1)
    shared = (e - 1) - 2
    byte = np.clip(shared + 127, 1, 254)
    byte = np.where(amax > 0, byte, 127).astype(np.int32)  # all-zero group: scale 1.0
    scale = np.ldexp(1.0, byte - 127)
    v = g.astype(np.float64) / scale[..., None]
    code = _e2m1_code(np.abs(v))
    code = code | ((np.signbit(g)).astype(np.uint8) << 3)
    code = code.reshape(*lead, k)
    packed = (code[..., 0::2] | (code[..., 1::2] << 4)).astype(np.uint8)
    return packed, byte.astype(np.uint8)
