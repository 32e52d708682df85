"""Block-scaled grouped GEMM on the CPU: fp32 dequantise-then-matmul.  Oracle
code: test infrastructure only.

Restates what the reference tests use as ground truth for the grouped FP8
GEMMs: dequantise activations (per row, per 128-K scale) and weights (per
128x128 block scale) to fp32, then a plain fp32 matmul per expert
(``_dequant_rows``, tests/test_moe_compact_ragged_fp8.py:312-318;
``masked_reference``, tests/test_glm52_deepgemm_masked_parity_gpu.py:111-125).
The mathematical definition is
Y[r,n] = sum_kb ( sum_{k in kb} Xq[r,k]*Wq[e,n,k] ) * xs[r,kb] * ws[e,n/128,kb]
(batchgen/moe/grouped_fp8_blockwise_moe.py:292-327).
"""
from __future__ import annotations

import numpy as np
import torch

from .quant import act_dequant, act_quant, bf16_round, swiglu_bf16, weight_block_dequant
from . import mxfp4 as _mx
from . import situ as _situ

F32 = np.float32


def _mm(a: np.ndarray, b_t: np.ndarray) -> np.ndarray:
    """a [M,K] @ b_t[N,K]^T in fp32 (torch CPU, multi-threaded)."""
    return (torch.from_numpy(np.ascontiguousarray(a)) @ torch.from_numpy(np.ascontiguousarray(b_t)).T).numpy()


def grouped_gemm_fp8(xq, xs, wq, ws, seqlens, cu_seqlens, to_bf16=True):
    """xq [M,K] bytes, xs [M,K/128]; wq [E,N,K] bytes, ws [E,N/128,K/128(+pad)].

    Rows [cu[e], cu[e]+seqlens[e]) belong to expert e; other rows of the
    result are 0.  Returns float32 [M,N] (bf16-rounded when to_bf16).
    """
    m, k = xq.shape
    e, n, _ = wq.shape
    kb = k // 128
    xd = act_dequant(xq, xs[:, :kb])
    out = np.zeros((m, n), dtype=F32)
    for g in range(e):
        c = int(seqlens[g])
        if c == 0:
            continue
        r0 = int(cu_seqlens[g])
        wd = weight_block_dequant(wq[g], ws[g][:, :kb])
        out[r0:r0 + c] = _mm(xd[r0:r0 + c], wd)
    return bf16_round(out) if to_bf16 else out


def grouped_gemm_fp8_blockpromote(xq, xs, wq, ws, seqlens, cu_seqlens):
    """Same product accumulated the way the kernels do it: an exact-ish partial
    sum per 128-K block, scaled by xs*ws, added in fp32 in ascending kb.  Used
    to show that the kernel-vs-oracle gap is accumulation order only."""
    from .fp8 import e4m3fn_decode
    m, k = xq.shape
    e, n, _ = wq.shape
    kb = k // 128
    xv = e4m3fn_decode(xq)
    out = np.zeros((m, n), dtype=F32)
    for g in range(e):
        c = int(seqlens[g])
        if c == 0:
            continue
        r0 = int(cu_seqlens[g])
        wv = e4m3fn_decode(wq[g])
        acc = np.zeros((c, n), dtype=F32)
        for b in range(kb):
            part = _mm(xv[r0:r0 + c, b * 128:(b + 1) * 128], wv[:, b * 128:(b + 1) * 128])
            sc = (xs[r0:r0 + c, b:b + 1] * np.repeat(ws[g][:, b], 128)[None, :]).astype(F32)
            acc = (acc + part * sc).astype(F32)
        out[r0:r0 + c] = acc
    return out


def expert_mlp_fp8(xq, xs, gate_q, gate_s, up_q, up_s, down_q, down_s, seqlens, cu_seqlens, variant="i"):
    """gate_up -> SwiGLU -> requant -> down, with the intermediate rounded the way ``variant`` says:

    "i"    fp32 gate and up, fp32 SiLU, ONE bf16 round, requant form C: the reference's Triton stage 1
           (w8a8_grouped_gemm_stage_1.py:1023-1026) and what the HIP kernels compute;
    "ii"   the reference's CuTe fused stage 1 (``oracle.quant.swiglu_cute_bf16``) + requant form C
           (``act_quant_ragged`` on its bf16 output, glm5/model.py:2560-2573);
    "iii"  the reference's DeepGEMM chains: gate and up leave the first GEMM as bf16, then
           ``silu_mul_{masked,ragged}_group_quant`` (bf16 SiLU, bf16 product, requant form D,
           moe_masked_act_quant.py:96-104);
    "fp32" no rounding that the semantics do not ask for: SwiGLU in fp32 fed straight to the requant
           (form C), the down product left in fp32 -- the yardstick the variants' errors are measured against.

    Returns (y [M,H] float32 -- bf16-valued except for "fp32" --, h [M,I], hq bytes, hs scales).
    """
    from .quant import silu_f32, silu_mul_group_quant, swiglu_cute_bf16
    g = grouped_gemm_fp8(xq, xs, gate_q, gate_s, seqlens, cu_seqlens, to_bf16=False)
    u = grouped_gemm_fp8(xq, xs, up_q, up_s, seqlens, cu_seqlens, to_bf16=False)
    if variant == "i":
        h = swiglu_bf16(g, u)
        hq, hs = act_quant(h)
    elif variant == "ii":
        h = swiglu_cute_bf16(g, u)
        hq, hs = act_quant(h)
    elif variant == "iii":
        hq, hs, h = silu_mul_group_quant(bf16_round(g), bf16_round(u), "D")
    elif variant == "fp32":
        h = (silu_f32(g) * u.astype(F32)).astype(F32)
        hq, hs = act_quant(h)
    else:
        raise ValueError(f"unknown SwiGLU rounding variant {variant!r}")
    y = grouped_gemm_fp8(hq, hs, down_q, down_s, seqlens, cu_seqlens, to_bf16=variant != "fp32")
    return y, h, hq, hs


def grouped_gemm_mxfp4(x_bf16, w_packed, w_scales, seqlens, cu_seqlens, to_bf16=True):
    """W4A16: x [M,K] bf16-valued fp32; w_packed [E,N,K/2], w_scales [E,N,K/32]."""
    m, k = x_bf16.shape
    e, n, _ = w_packed.shape
    out = np.zeros((m, n), dtype=F32)
    for g in range(e):
        c = int(seqlens[g])
        if c == 0:
            continue
        r0 = int(cu_seqlens[g])
        wd = _mx.dequant(w_packed[g], w_scales[g])
        out[r0:r0 + c] = _mm(x_bf16[r0:r0 + c], wd)
    return bf16_round(out) if to_bf16 else out


def expert_mlp_mxfp4(x, gate_p, gate_s, up_p, up_s, down_p, down_s, seqlens, cu_seqlens, activation="swiglu"):
    """bf16 activations, MXFP4 weights, a bf16 intermediate: SwiGLU on the fp32 products, or SiTU on the
    bf16-rounded ones (``oracle.situ.situ_fused``)."""
    g = grouped_gemm_mxfp4(x, gate_p, gate_s, seqlens, cu_seqlens, to_bf16=False)
    u = grouped_gemm_mxfp4(x, up_p, up_s, seqlens, cu_seqlens, to_bf16=False)
    h = _situ.situ_fused(g, u) if activation == "situ" else swiglu_bf16(g, u)
    y = grouped_gemm_mxfp4(h, down_p, down_s, seqlens, cu_seqlens, to_bf16=True)
    return y, h


def rel_frobenius(a: np.ndarray, b: np.ndarray) -> float:
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
