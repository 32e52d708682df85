"""Per-token, per-128 FP8 activation quantisation and 128x128 weight block
quantisation on the CPU.  Oracle code: test infrastructure only.

Canonical activation form ("form C"), restating ``act_quant_3d`` /
``act_quant_ragged``
(batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_ops.cu:39-111, 151-252):

    amax  = max |x| over the 128-block (columns past K count as 0)
    s     = fmaxf(amax, 1e-12f) * (1.0f / 448.0f)
    q     = fmaxf(fminf(x / s, 448), -448)      (IEEE fp32 division)
    byte  = e4m3fn RNE (q)

fminf/fmaxf ignore a NaN operand (C semantics), which np.fmin/np.fmax also do,
so a NaN input becomes +448 exactly as in the reference kernel.
"""
from __future__ import annotations

import numpy as np

from .fp8 import e4m3fn_decode, e4m3fn_encode

F32 = np.float32
BLOCK = 128
INV448 = F32(1.0) / F32(448.0)
EPS = F32(1e-12)


def as_f32(x) -> np.ndarray:
    """torch (bf16/fp32) or numpy -> contiguous numpy float32."""
    if hasattr(x, "detach"):
        x = x.detach().cpu().float().numpy()
    return np.ascontiguousarray(x, dtype=np.float32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest-even bfloat16, returned as float32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = np.isnan(x)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32)
    return np.where(nan, np.float32("nan"), out).astype(np.float32)


def _blocks(x: np.ndarray):
    m, k = x.shape
    kb = (k + BLOCK - 1) // BLOCK
    pad = kb * BLOCK - k
    xp = np.pad(x, ((0, 0), (0, pad))) if pad else x
    return xp.reshape(m, kb, BLOCK), kb


def act_quant(x, form: str = "C"):
    """x [M, K] -> (bytes uint8 [M, K], scale fp32 [M, ceil(K/128)]).

    form "C": the ``batchgen_kernels.moe`` quantiser (canonical here).
    form "A": Triton 1-D quantiser (batchgen_kernels/triton/fp8_quantize.py:276-331):
              amax floored at 2^-16, scale = max(amax*(1/448), 1e-12), non-finite q -> 0.
    form "B": ``fused_silu_quant_3d`` (fp8_blockwise_ops.cu:495-504):
              s = fmaxf(amax,1e-12)/448 ; q = x * (1/s).
    form "D": DeepGEMM-chain activation (batchgen_kernels/triton/moe_masked_act_quant.py:100-104):
              s = max(amax,1e-10)/448 ; q = x / s.
    """
    x = as_f32(x)
    m, k = x.shape
    xb, kb = _blocks(x)
    amax = np.fmax.reduce(np.abs(xb), axis=2, initial=F32(0.0)).astype(F32)
    if form == "C":
        s = np.fmax(amax, EPS) * INV448
        q = xb / s[:, :, None]
    elif form == "A":
        amax = np.fmax(amax, F32(2.0 ** -16))
        s = np.fmax(amax * INV448, EPS)
        q = xb / s[:, :, None]
        # clamp first, then |q| < 1e30 else 0 (fp8_quantize.py:321-325): with min/max that drop a NaN
        # operand the guard never fires (NaN and +-inf have become +-448 by then)
        with np.errstate(invalid="ignore"):
            q = np.fmax(np.fmin(q.astype(F32), F32(448.0)), F32(-448.0))
        q = np.where(np.abs(q) < F32(1e30), q, F32(0.0))
    elif form == "B":
        s = np.fmax(amax, EPS) / F32(448.0)
        q = xb * (F32(1.0) / s)[:, :, None]
    elif form == "D":
        s = np.fmax(amax, F32(1e-10)) / F32(448.0)
        q = xb / s[:, :, None]
    else:
        raise ValueError(form)
    with np.errstate(invalid="ignore"):
        q = np.fmax(np.fmin(q.astype(F32), F32(448.0)), F32(-448.0))
    y = e4m3fn_encode(q).reshape(m, kb * BLOCK)[:, :k]
    return np.ascontiguousarray(y), s.astype(F32)


def act_dequant(y: np.ndarray, s: np.ndarray) -> np.ndarray:
    """bytes [M,K] + scale [M,KB] -> float32 [M,K]."""
    m, k = y.shape
    v = e4m3fn_decode(y)
    return v * np.repeat(s, BLOCK, axis=1)[:, :k]


def pad_row_scale() -> np.float32:
    """Scale written for an all-zero (alignment pad) row."""
    return np.fmax(F32(0.0), EPS) * INV448


def act_quant_masked(x, tokens_per_expert):
    """``act_quant_3d``: x [E, S, K]; rows >= tokens_per_expert[e] untouched.

    Returns (y [E,S,K] uint8, scale [E,S,KB] fp32, written [E,S] bool).
    Unwritten entries are returned as 0 and must be ignored by the caller.
    """
    x = as_f32(x)
    e, s_, k = x.shape
    y, sc = act_quant(x.reshape(e * s_, k))
    y = y.reshape(e, s_, k)
    sc = sc.reshape(e, s_, -1)
    cnt = np.asarray(tokens_per_expert).reshape(e, 1)
    written = np.arange(s_)[None, :] < cnt
    y = np.where(written[:, :, None], y, 0).astype(np.uint8)
    sc = np.where(written[:, :, None], sc, F32(0)).astype(F32)
    return y, sc, written


def act_quant_ragged_model(x, seqlens, cu_seqlens, row_align: int):
    """Write-set model of ``act_quant_ragged`` (fp8_blockwise_ops.cu:130-139;
    executable form in the reference's tests/test_act_quant_ragged_fixed_grid.py:80-123).

    x [max_rows, K].  Returns (y [max_rows,K], scale_t [KB, max_rows],
    written [max_rows] bool, valid [max_rows] bool).  Row r is owned by
    o = max{e : cu[e] <= r}; written iff cu[0] <= r < cu[E] and
    r - cu[o] < align(seqlens[o]); valid iff also r - cu[o] < seqlens[o].
    Pad rows (written, not valid): bytes 0, scale = pad_row_scale().
    """
    x = as_f32(x)
    max_rows, k = x.shape
    seqlens = np.asarray(seqlens, dtype=np.int64)
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    ne = len(seqlens)
    rows = np.arange(max_rows, dtype=np.int64)
    owner = np.searchsorted(cu[:ne], rows, side="right") - 1
    owner_c = np.clip(owner, 0, ne - 1)
    rel = rows - cu[owner_c]
    span = (seqlens[owner_c] + row_align - 1) // row_align * row_align
    written = (rows >= cu[0]) & (rows < cu[ne]) & (owner >= 0) & (rel < span)
    valid = written & (rel < seqlens[owner_c])
    xz = np.where(valid[:, None], x, F32(0))
    y, sc = act_quant(xz)
    y = np.where(written[:, None], y, 0).astype(np.uint8)
    sc = np.where(written[:, None], sc, F32(0)).astype(F32)
    return y, np.ascontiguousarray(sc.T), written, valid


# ----------------------------------------------------------------------------
# weights: 128x128 block quantisation (inputs of the path, not a kernel)
# ----------------------------------------------------------------------------
def weight_block_quant(w):
    """w [..., N, K] fp32 -> (bytes [..., N, K], scale [..., N/128, K/128]).

    scale = max(amax,1e-10)/448 ; q = clamp(w/scale) -> e4m3fn
    (the reference tests' weight recipe, tests/test_glm52_deepgemm_masked_parity_gpu.py:80-87).
    """
    w = as_f32(w)
    *lead, n, k = w.shape
    assert n % BLOCK == 0 and k % BLOCK == 0
    wb = w.reshape(*lead, n // BLOCK, BLOCK, k // BLOCK, BLOCK)
    amax = np.abs(wb).max(axis=(-3, -1)).astype(F32)
    s = np.fmax(amax, F32(1e-10)) / F32(448.0)
    q = wb / s[..., :, None, :, None]
    q = np.fmax(np.fmin(q.astype(F32), F32(448.0)), F32(-448.0))
    y = e4m3fn_encode(q).reshape(*lead, n, k)
    return y, s.astype(F32)


def weight_block_dequant(y: np.ndarray, s: np.ndarray, to_bf16: bool = False) -> np.ndarray:
    """``deepseek_v3_dequantization`` (batchgen_kernels/triton/fp8_quantize.py:624-656):
    float(Wq).view(nb,128,kb,128) * s[:,None,:,None]; optionally rounded to bf16."""
    *lead, n, k = y.shape
    v = e4m3fn_decode(y).reshape(*lead, n // BLOCK, BLOCK, k // BLOCK, BLOCK)
    out = (v * s[..., :, None, :, None]).astype(F32).reshape(*lead, n, k)
    return bf16_round(out) if to_bf16 else out


# ----------------------------------------------------------------------------
# SwiGLU between the two GEMMs
# ----------------------------------------------------------------------------
def silu_f32(g: np.ndarray) -> np.ndarray:
    g = g.astype(np.float64)
    return (g / (1.0 + np.exp(-g))).astype(F32)


def swiglu_bf16(gate_f32: np.ndarray, up_f32: np.ndarray) -> np.ndarray:
    """Rounding variant (i): fp32 gate, fp32 up, fp32 silu, ONE bf16 round
    (batchgen_kernels/triton/w8a8_grouped_gemm_stage_1.py:1023-1026)."""
    return bf16_round(silu_f32(gate_f32) * up_f32.astype(F32))


def swiglu_cute_bf16(gate_f32: np.ndarray, up_f32: np.ndarray) -> np.ndarray:
    """Rounding variant (ii), the reference's own fused stage-1 kernel
    (batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_s1_kernel.cuh:556-581): the gate accumulator is
    rounded to bf16 when it is parked in shared memory, ``sigmoid = 1.0f / (1.0f + __expf(-gate))``,
    ``(gate * sigmoid) * up`` with the fp32 up accumulator, one more bf16 round.

    ``__expf(x)`` is CUDA's ``ex2.approx(x * log2e)``: the argument product is rounded to fp32 and the
    hardware exp2 is accurate to about 2 ulp.  The emulation rounds the product exactly as the instruction
    sequence does and takes exp2 and the division correctly rounded -- an emulation of the kernel's rounding
    structure, not of the last bits of two approximate instructions."""
    g = bf16_round(gate_f32)
    t = (-g * F32(1.4426950408889634)).astype(F32)
    with np.errstate(over="ignore"):
        e = np.exp2(t.astype(np.float64)).astype(F32)
        sig = (F32(1.0) / (F32(1.0) + e).astype(F32)).astype(F32)
    return bf16_round(((g * sig).astype(F32) * as_f32(up_f32)).astype(F32))


def silu_torch_f32(g) -> np.ndarray:
    """PyTorch's fp32 SiLU, ``x / (1 + exp(-x))`` as three float32 operations -- the formula and precision the
    reference's fused activation quantisers restate (batchgen_kernels/triton/fp8_quantize.py:414-424: libdevice
    ``exp``, round-to-nearest division).  ``exp`` is taken correctly rounded (float64, rounded once)."""
    g = as_f32(g)
    with np.errstate(over="ignore"):
        e = np.exp(-g.astype(np.float64)).astype(F32)
        d = (F32(1.0) + e).astype(F32)
        return (g / d).astype(F32)


def silu_mul_bf16(gate, up) -> np.ndarray:
    """bf16( bf16(silu(gate)) * up ): SiLU cast back to the input dtype before the multiply, bf16 product
    (moe_masked_act_quant.py:96-99; fp8_quantize.py:425-426)."""
    s = bf16_round(silu_torch_f32(gate))
    return bf16_round((s * as_f32(up)).astype(F32))


def silu_mul_group_quant(gate, up, form: str):
    """[M, I] gate, up -> (bytes, scales, product): form "D" = ``silu_mul_{masked,ragged}_group_quant``
    (oracle ``act_reference``, tests/test_glm52_deepgemm_masked_parity_gpu.py:128-149), form "A" =
    ``silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d``."""
    p = silu_mul_bf16(gate, up)
    y, s = act_quant(p, form=form)
    return y, s, p

