"""The masked m-grouped routed GEMM chain of the DeepEP decode MoE path, with the reference's names, argument
lists and error policy (batchgen/models/glm/glm5/moe_deepgemm_masked.py:74-342):

    R1  : masked( (x, x_scales), (W_gate_up, S_gate_up) ) -> gu [E, S, 2I]
    act : quant(silu(gu[..., :I]) * gu[..., I:])          -> (a, a_scales)
    R2  : masked( (a, a_scales), (W_down, S_down) )       -> out [E, S, H]

``fp8_m_grouped_gemm_nt_masked`` is the entry of the third-party ``deep_gemm`` package that the reference calls
(:318-341); here it is this build's grouped FP8 GEMM, which reads the same operands: A ``[E, S, K]`` e4m3fn, its
scales MN-major (a contiguous ``[E, K/128, S]`` block viewed as ``[E, S, K/128]``), B ``[E, N, K]`` with exact
``[E, N/128, K/128]`` scales, D ``[E, S, N]`` bf16; only rows below ``masked_m[e]`` are read or written.
DeepGEMM's own accumulation order is not reproduced (the package is not in the reference tree); results are
pinned like the reference's own test does, against the fp32 dequantise-then-matmul of the live rows
(tests/test_glm52_deepgemm_masked_parity_gpu.py:111-125).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch

from .._lib import Fp8Act, Fp8Weight, check, lib, ptr, stream

FP8_DTYPE = torch.float8_e4m3fn
SCALE_BLOCK = 128
MASKED_BLOCK_M = 64
SCALE_TMA_ALIGN_FLOATS = 4


def fp8_m_grouped_gemm_nt_masked(lhs, rhs, d: torch.Tensor, masked_m: torch.Tensor, expected_m: int) -> None:
    """``d[e, :masked_m[e]] = dequant(a[e]) @ dequant(b[e]).T`` (bf16), the rest of ``d`` untouched.
    ``expected_m`` is a scheduling hint of the reference kernel: accepted and ignored (the kernel choice is
    made on the device from ``masked_m``)."""
    a, sa = lhs
    b, sb = rhs
    if a.dim() != 3 or b.dim() != 3 or d.dim() != 3:
        raise RuntimeError("masked GEMM takes A [E, S, K], B [E, N, K] and D [E, S, N]")
    e, s_, k = a.shape
    n = b.shape[1]
    if b.shape[0] != e or b.shape[2] != k or tuple(d.shape) != (e, s_, n):
        raise RuntimeError(f"masked GEMM shape mismatch: A {tuple(a.shape)}, B {tuple(b.shape)}, D {tuple(d.shape)}")
    if a.dtype != FP8_DTYPE or b.dtype != FP8_DTYPE or d.dtype != torch.bfloat16:
        raise RuntimeError(f"masked GEMM takes {FP8_DTYPE} operands and a bfloat16 output")
    if k % SCALE_BLOCK or n % SCALE_BLOCK:
        raise RuntimeError(f"masked GEMM is block-scaled: K {k} and N {n} must be multiples of {SCALE_BLOCK}")
    if not (a.is_contiguous() and b.is_contiguous() and d.is_contiguous()):
        raise RuntimeError("masked GEMM takes contiguous A, B and D")
    require_mn_major_tma_aligned(sa, "A scales")
    if tuple(sa.shape) != (e, s_, k // SCALE_BLOCK):
        raise RuntimeError(f"A scales must be [E, S, K // {SCALE_BLOCK}] = {(e, s_, k // SCALE_BLOCK)}; got "
                           f"{tuple(sa.shape)}")
    if tuple(sb.shape) != (e, n // SCALE_BLOCK, k // SCALE_BLOCK) or sb.dtype != torch.float32 or not sb.is_contiguous():
        raise RuntimeError(f"B scales must be contiguous f32 [E, N // {SCALE_BLOCK}, K // {SCALE_BLOCK}]; got "
                           f"{tuple(sb.shape)} {sb.dtype}")
    if tuple(masked_m.shape) != (e,) or masked_m.dtype != torch.int32:
        raise RuntimeError(f"masked_m must be int32 [{e}]")
    if e == 0 or s_ == 0:
        return
    kb = k // SCALE_BLOCK
    act = Fp8Act(ptr(a), ptr(sa), 1, s_, kb * s_)
    w = Fp8Weight(ptr(b), n * k, None, ptr(sb), (n // SCALE_BLOCK) * kb, kb, None, 0, 0)
    cu = _group_starts(e, s_, a.device)
    with torch.cuda.device(a.device):
        check(lib().bgmoe_fp8_grouped_gemm(C.byref(act), C.byref(w), ptr(masked_m), ptr(cu), e, e * s_, n, k, ptr(d),
                                           stream()))


_STARTS = {}


def _group_starts(e: int, s_: int, device) -> torch.Tensor:
    """cu_seqlens of the uniform-stride layout, e*S (one small tensor per (E, S, device), made once so that a
    captured call allocates nothing)."""
    key = (e, s_, str(device))
    t = _STARTS.get(key)
    if t is None:
        t = (torch.arange(e + 1, dtype=torch.int32, device=device) * s_).contiguous()
        _STARTS[key] = t
    return t


def masked_gemm_fn():
    """The masked m-grouped FP8 GEMM (in the reference: ``deep_gemm.fp8_m_grouped_gemm_nt_masked``)."""
    return fp8_m_grouped_gemm_nt_masked


def masked_act_quant_fn():
    """The masked ``quant(silu(gate) * up)`` kernel."""
    from ..kernels.triton.moe_masked_act_quant import silu_mul_masked_group_quant
    return silu_mul_masked_group_quant


def expected_m_per_expert(*, local_rows: int, world_size: int, topk: int, num_experts_global: int) -> int:
    """Mean routed rows per GLOBAL expert, rounded up: the masked kernel's row-count hint."""
    args = dict(local_rows=local_rows, world_size=world_size, topk=topk, num_experts_global=num_experts_global)
    bad = [k for k, v in args.items() if v <= 0]
    if bad:
        raise ValueError(f"expected_m_per_expert: {', '.join(bad)} must be positive ({args})")
    g = int(num_experts_global)
    return (int(local_rows) * int(world_size) * int(topk) + g) // g


def _mn_major_problem(scales: torch.Tensor):
    """None when ``scales`` is a [E, K/128, S] block seen as [E, S, K/128] with S a multiple of 4, else what is
    wrong with it."""
    if scales.dim() != 3:
        return f"expected a 3-D [E, S, K // {SCALE_BLOCK}] view, got shape {tuple(scales.shape)}"
    if scales.dtype != torch.float32:
        return f"expected float32, got {scales.dtype}"
    _e, rows, blocks = scales.shape
    if rows % SCALE_TMA_ALIGN_FLOATS:
        return f"row extent {rows} is not a multiple of {SCALE_TMA_ALIGN_FLOATS}"
    if scales.stride() != (blocks * rows, 1, rows):
        return (f"strides {tuple(scales.stride())} are not {(blocks * rows, 1, rows)} (transpose(1, 2) of a "
                f"contiguous [E, {blocks}, {rows}] block)")
    return None


def is_mn_major_tma_aligned(scales: torch.Tensor) -> bool:
    return _mn_major_problem(scales) is None


def require_mn_major_tma_aligned(scales: torch.Tensor, name: str) -> None:
    """Raise unless ``scales`` can be read in place (nothing is repacked here: that would allocate)."""
    problem = _mn_major_problem(scales)
    if problem is not None:
        raise RuntimeError(f"{name}: MN-major A-scales required; {problem}")


@dataclass(frozen=True)
class DeepGemmMaskedExpertWeights:
    """A routed layer's weights as the masked GEMM reads them: ``gate_up_w`` = fused ``[E, 2I, H]`` stack (gate
    rows first), ``down_w`` = ``[E, H, I]``, scales exact ``[E, N // 128, K // 128]`` (no padded axis)."""

    gate_up_w: torch.Tensor
    gate_up_scale: torch.Tensor
    down_w: torch.Tensor
    down_scale: torch.Tensor

    def validate(self, *, num_experts: int, hidden_size: int, intermediate_size: int) -> None:
        e, h, i = int(num_experts), int(hidden_size), int(intermediate_size)
        if h % SCALE_BLOCK or i % SCALE_BLOCK:
            raise RuntimeError(f"hidden {h} / intermediate {i}: both must be multiples of {SCALE_BLOCK}")
        b = SCALE_BLOCK
        wanted = (("gate_up_w", (e, 2 * i, h), FP8_DTYPE), ("down_w", (e, h, i), FP8_DTYPE),
                  ("gate_up_scale", (e, 2 * i // b, h // b), torch.float32),
                  ("down_scale", (e, h // b, i // b), torch.float32))
        for field, shape, dtype in wanted:
            t = getattr(self, field)
            if tuple(t.shape) != shape or t.dtype != dtype or not t.is_contiguous():
                raise RuntimeError(f"{field}: need contiguous {dtype} {shape}, got {t.dtype} {tuple(t.shape)} with "
                                   f"strides {tuple(t.stride())}")


def run_deepgemm_masked_moe(*, x_fp8: torch.Tensor, x_scales: torch.Tensor, weights: DeepGemmMaskedExpertWeights,
                            masked_m: torch.Tensor, expected_m: int, gate_up_out: torch.Tensor,
                            act_fp8: torch.Tensor, act_scales: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """Run one routed layer's masked chain into caller-owned buffers: allocates nothing, synchronises nothing,
    reads its per-step row counts from ``masked_m`` on the device."""
    if not isinstance(expected_m, int):
        raise RuntimeError(f"expected_m is a host constant of the capture and must be an int, not {type(expected_m).__name__}")
    e, s_ = x_fp8.shape[:2]
    two_i = int(weights.gate_up_w.shape[1])
    if two_i % 2:
        raise RuntimeError(f"gate_up_w {tuple(weights.gate_up_w.shape)}: the fused stack needs 2I rows per expert")
    inter = two_i // 2
    if tuple(gate_up_out.shape) != (e, s_, two_i) or gate_up_out.stride(-1) != 1:
        raise RuntimeError(f"gate_up_out must be [E, S, 2I] = {(e, s_, two_i)} with a contiguous last axis (its halves "
                           f"are read as strided views); got {tuple(gate_up_out.shape)}, strides "
                           f"{tuple(gate_up_out.stride())}")
    require_mn_major_tma_aligned(x_scales, "x_scales")
    require_mn_major_tma_aligned(act_scales, "act_scales")
    masked_gemm = masked_gemm_fn()
    act_quant = masked_act_quant_fn()
    masked_gemm((x_fp8, x_scales), (weights.gate_up_w, weights.gate_up_scale), gate_up_out, masked_m, expected_m)
    act_quant(gate_up_out[:, :, :inter], gate_up_out[:, :, inter:], act_fp8, act_scales, masked_m,
              group_size=SCALE_BLOCK)
    masked_gemm((act_fp8, act_scales), (weights.down_w, weights.down_scale), out, masked_m, expected_m)
    return out
