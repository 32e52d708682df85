"""Fused residual add + RMSNorm + per-token 128-block FP8 cast on the CPU.  Oracle code: test
infrastructure only.

Restates ``add_rmsnorm_bf16_6144_fp8_quant_kernel``
(batchgen_kernels/src/attention/csrc/add_rmsnorm_fp8_quant.cu:242-384), one row per block, thread t owning
columns 8t..8t+7:

    sum_i      = float(residual_i) + (row_valid ? float(hidden_i) : 0)            :303-307
    residual_i = bf16(sum_i)                      (stored back)                    :308, :311
    sum_sq_t   = fmaf(sum_i, sum_i, sum_sq_t)     over the thread's 8 columns      :309
    total      = block tree: 32-lane shuffle-down trees (offsets 16..1) per warp, then the warp sums
                 through the same tree in lanes 0..nwarps-1 of warp 0 (other lanes 0)   :179-209
    inv_rms    = rsqrt(total / H + eps)                                            :315
    normed_i   = bf16( float(residual_i as stored) * inv_rms * float(weight_i) )   :322-327
    then the 1-D quantiser over normed (bf16-rounded):                             :340-376
    amax = max(max|normed|, 2^-16);  scale = max(amax * (1/448), 1e-12)
    q = clamp(normed / scale, +-448) -> e4m3fn RNE;  rows >= quant_num_valid: bytes 0, scales 1e-12

Two operations of the reference are approximate CUDA instructions and therefore not functions that another
machine can reproduce: ``rsqrtf`` (:315) and Triton's ``div.full.f32`` (:211-228).  This build defines them
as the correctly rounded ones -- inv_rms = float32(1 / sqrt(float64(v))), q = IEEE fp32 division -- on the
device and here alike, which keeps the reference's own contract (fused == norm followed by the standalone
quantiser, bit for bit) while differing from the CUDA bytes by at most the last place of inv_rms.

The reference fixes H = 6144 (768 threads); the same thread/tree structure is used here for any H that is a
multiple of 128 up to 8192 (H/8 threads, ceil(H/256) warps).
"""
from __future__ import annotations

import numpy as np

from .quant import act_quant, as_f32, bf16_round

F32 = np.float32
F64 = np.float64


def fma_f32(a, b, c) -> np.ndarray:
    """Correctly rounded float32 fma(a, b, c) for float32 arrays.

    a*b is exact in float64.  s = fl64(p + c) with its exact error e (TwoSum); rounding s to float32 is the
    correctly rounded result unless s sits exactly on a float32 rounding boundary and e != 0, in which case
    the tie is broken by the sign of e.
    """
    a = np.asarray(a, dtype=F32).astype(F64)
    b = np.asarray(b, dtype=F32).astype(F64)
    c = np.asarray(c, dtype=F32).astype(F64)
    p = a * b
    s = p + c
    bb = s - p
    e = (p - (s - bb)) + (c - bb)                      # TwoSum: p + c == s + e exactly
    r = s.astype(F32)
    bits = np.abs(s).view(np.uint64)
    tie = ((bits & np.uint64(0x1FFFFFFF)) == np.uint64(0x10000000)) & (e != 0) & np.isfinite(s)
    if np.any(tie):
        lo = np.nextafter(r, F32(-np.inf))
        hi = np.nextafter(r, F32(np.inf))
        # r was rounded to even from the tie point s; the exact value lies on the side of e
        below = np.where(r.astype(F64) > s, lo, r)     # float32 neighbour just below s
        above = np.where(r.astype(F64) > s, r, hi)     # float32 neighbour just above s
        r = np.where(tie, np.where(e > 0, above, below), r)
    return r.astype(F32)


def _tree32(v: np.ndarray) -> np.ndarray:
    """Lane 0 of a 32-lane shuffle-down tree (offsets 16, 8, 4, 2, 1) over the last axis."""
    off = 16
    while off >= 1:
        v = (v[..., :off] + v[..., off:2 * off]).astype(F32)
        off //= 2
    return v[..., 0]


def rsqrt_cr(v: np.ndarray) -> np.ndarray:
    with np.errstate(divide="ignore", invalid="ignore"):
        return (1.0 / np.sqrt(np.asarray(v, dtype=F32).astype(F64))).astype(F32)


def add_rmsnorm(residual, hidden, weight, eps: float, row_valid_mask=None, num_valid_tokens=None):
    """-> (normed bf16-as-f32 [M,H], new residual bf16-as-f32 [M,H]).  Rows >= num_valid_tokens keep their
    residual and get NaN in ``normed`` here to mark "not written"."""
    res = as_f32(residual)
    hid = as_f32(hidden)
    w = as_f32(weight).reshape(-1)
    m, h = res.shape
    assert h % 8 == 0 and h // 8 <= 1024
    if row_valid_mask is not None:
        valid = as_f32(row_valid_mask).reshape(-1) != 0
        hid = np.where(valid[:, None], hid, F32(0.0))
    s = (res + hid).astype(F32)
    new_res = bf16_round(s)
    threads = h // 8
    cols = s.reshape(m, threads, 8)
    sq = np.zeros((m, threads), dtype=F32)
    for i in range(8):
        sq = fma_f32(cols[:, :, i], cols[:, :, i], sq)
    nwarps = (threads + 31) // 32
    lanes = np.zeros((m, nwarps * 32), dtype=F32)
    lanes[:, :threads] = sq
    warp_sums = _tree32(lanes.reshape(m, nwarps, 32))
    stage2 = np.zeros((m, 32), dtype=F32)
    stage2[:, :nwarps] = warp_sums
    total = _tree32(stage2)
    inv = rsqrt_cr((total / F32(h)).astype(F32) + F32(eps))
    normed = bf16_round(((new_res * inv[:, None]).astype(F32) * w[None, :]).astype(F32))
    if num_valid_tokens is not None:
        nv = int(num_valid_tokens)
        new_res[nv:] = bf16_round(res)[nv:]
        normed[nv:] = np.nan
    return normed, new_res


def quant_1d(normed, num_valid_tokens=None):
    """The 1-D quantiser with the padding-row branch (fp8_quantize.py:305-331)."""
    y, s = act_quant(normed, form="A")
    if num_valid_tokens is not None:
        nv = int(num_valid_tokens)
        y[nv:] = 0
        s[nv:] = F32(1e-12)
    return y, s


def add_rmsnorm_fp8_quant(residual, hidden, weight, eps: float, norm_num_valid_tokens=None,
                          quant_num_valid_tokens=None, row_valid_mask=None):
    """-> (normed, new residual, fp8 bytes [M,H] uint8, scales [M,H/128] fp32)."""
    normed, new_res = add_rmsnorm(residual, hidden, weight, eps, row_valid_mask, norm_num_valid_tokens)
    y, s = quant_1d(np.nan_to_num(normed, nan=0.0) if norm_num_valid_tokens is not None else normed,
                    quant_num_valid_tokens)
    return normed, new_res, y, s
