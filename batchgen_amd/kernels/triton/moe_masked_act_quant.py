"""``silu_mul_masked_group_quant`` / ``silu_mul_ragged_group_quant`` with the reference's signatures and
argument policy (batchgen_kernels/triton/moe_masked_act_quant.py:112-376): the activation between the two
grouped GEMMs of the DeepGEMM chains.  SiLU in fp32 cast back to bf16 before the multiply, bf16 product,
``absmax / 448`` group scale (absmax floored at 1e-10), clamped e4m3 store; rows at or beyond the live count
are neither read nor written; every buffer caller-owned, nothing allocates, nothing synchronises."""
from __future__ import annotations

import torch

from ..._lib import check, lib, ptr, stream

_FP8_DTYPE = torch.float8_e4m3fn


def _common(kind, gate, up, out, out_scale, group_size, dims):
    if gate.dim() != dims or up.dim() != dims or out.dim() != dims:
        raise ValueError(f"{kind} act/quant takes {'expert-major [E, S, I]' if dims == 3 else 'flat [m, I]'} gate, up "
                         f"and out; got {tuple(gate.shape)} / {tuple(up.shape)} / {tuple(out.shape)}")
    if gate.shape != up.shape or gate.shape != out.shape:
        raise ValueError(f"{kind} act/quant needs gate, up and out on the same extent; got {tuple(gate.shape)} / "
                         f"{tuple(up.shape)} / {tuple(out.shape)}")
    if gate.dtype != up.dtype:
        raise ValueError(f"{kind} act/quant needs one input dtype; got {gate.dtype} gate and {up.dtype} up")
    if gate.dtype != torch.bfloat16:
        raise ValueError(f"{kind} act/quant is built for bfloat16 inputs, got {gate.dtype}")
    if out.dtype != _FP8_DTYPE:
        raise ValueError(f"{kind} act/quant writes {_FP8_DTYPE}, not {out.dtype}")
    if out_scale.dtype != torch.float32:
        raise ValueError(f"{kind} act/quant writes f32 group scales, not {out_scale.dtype}")
    if group_size != 128:
        raise ValueError(f"{kind} act/quant is built for the quant group 128, got {group_size}")
    size_n = gate.shape[-1]
    if size_n % group_size != 0:
        raise ValueError(f"{kind} act/quant needs the intermediate size {size_n} to be a multiple of the quant group "
                         f"{group_size}")
    for name, tensor in (("gate", gate), ("up", up), ("out", out)):
        if tensor.stride(-1) != 1:
            raise ValueError(f"{kind} act/quant needs a contiguous last dim on {name}; got strides "
                             f"{tuple(tensor.stride())}")
    if gate.stride() != up.stride():
        raise ValueError(f"{kind} act/quant needs gate and up with equal strides (two halves of one GEMM output); got "
                         f"{tuple(gate.stride())} / {tuple(up.stride())}")
    if not (gate.is_cuda and up.is_cuda and out.is_cuda and out_scale.is_cuda):
        raise ValueError(f"{kind} act/quant needs CUDA tensors")
    return size_n


def silu_mul_masked_group_quant(gate, up, out, out_scale, masked_m, *, group_size: int = 128,
                                rows_per_launch: int = 0, num_stages: int = 6) -> None:
    """``out, out_scale = quant(silu(gate) * up)`` over the live rows only (``rows_per_launch`` and
    ``num_stages`` are launch hints of the reference kernel: accepted and ignored)."""
    size_n = _common("masked", gate, up, out, out_scale, group_size, 3)
    num_experts, rows, _ = gate.shape
    if out_scale.shape != (num_experts, rows, size_n // group_size):
        raise ValueError(f"masked act/quant needs out_scale on the logical [E, S, I // {group_size}] extent "
                         f"{(num_experts, rows, size_n // group_size)}; got {tuple(out_scale.shape)}")
    if masked_m.shape != (num_experts,):
        raise ValueError(f"masked act/quant needs masked_m [{num_experts}]; got {tuple(masked_m.shape)}")
    if masked_m.dtype != torch.int32:
        raise ValueError(f"masked act/quant needs an int32 masked_m; got {masked_m.dtype}")
    if num_experts == 0 or rows == 0:
        return
    with torch.cuda.device(gate.device):
        check(lib().bgmoe_silu_mul_group_quant(
            ptr(gate), ptr(up), gate.stride(0), gate.stride(1), ptr(masked_m), None, num_experts, rows, size_n, 1,
            ptr(out), out.stride(0), out.stride(1), ptr(out_scale), out_scale.stride(0), out_scale.stride(1),
            out_scale.stride(2), None, stream()))


def silu_mul_ragged_group_quant(gate, up, out, out_scale, counts, cu_seqlens, *, group_size: int = 128,
                                rows_per_launch: int = 0, num_stages: int = 6) -> None:
    """The flat-row sibling: expert ``e``'s live rows sit at ``[cu_seqlens[e], cu_seqlens[e] + counts[e])`` of
    2-D ``[m, I]`` buffers; ``out_scale`` is the row-major ``[m, I // group_size]`` matrix."""
    size_n = _common("ragged", gate, up, out, out_scale, group_size, 2)
    rows = gate.shape[0]
    if out_scale.shape != (rows, size_n // group_size):
        raise ValueError(f"ragged act/quant needs a row-major out_scale on the [m, I // {group_size}] extent "
                         f"{(rows, size_n // group_size)}; got {tuple(out_scale.shape)}")
    if out_scale.stride(-1) != 1:
        raise ValueError(f"ragged act/quant writes row-major scales; got strides {tuple(out_scale.stride())}")
    if counts.ndim != 1 or cu_seqlens.shape != (counts.numel() + 1,):
        raise ValueError(f"ragged act/quant needs counts [E] and cu_seqlens [E + 1]; got {tuple(counts.shape)} / "
                         f"{tuple(cu_seqlens.shape)}")
    if counts.dtype != torch.int32 or cu_seqlens.dtype != torch.int32:
        raise ValueError(f"ragged act/quant needs int32 counts and cu_seqlens; got {counts.dtype} / "
                         f"{cu_seqlens.dtype}")
    num_experts = counts.numel()
    if num_experts == 0 or rows == 0:
        return
    with torch.cuda.device(gate.device):
        # no group can own more rows than the buffer has: the row count bounds the per-group walk
        check(lib().bgmoe_silu_mul_group_quant(
            ptr(gate), ptr(up), 0, gate.stride(0), ptr(counts), ptr(cu_seqlens), num_experts, rows, size_n, 1,
            ptr(out), 0, out.stride(0), ptr(out_scale), 0, out_scale.stride(0), 1, None, stream()))
