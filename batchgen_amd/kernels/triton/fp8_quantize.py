"""The per-token 128-block FP8 casts of batchgen_kernels/triton/fp8_quantize.py with the reference's signatures:
``per_token_blocked_quantize_bf16_to_fp8_1d`` (:334-391, the 1-D quantiser) and
``silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d`` (:462-526): SiLU(gate) * up and the cast that feed a
down-projection GEMM, in one launch; bit-identical to the 1-D quantiser applied to ``bf16(bf16(silu(g)) * u)``."""
from __future__ import annotations

import torch

from ..._lib import check, lib, ptr, stream


def silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d(gate_up: torch.Tensor, block_size: int = 128,
                                                       num_warps: int = 4, num_stages: int = 2,
                                                       scale_tma_aligned: bool = False):
    """-> (out [M, I] float8_e4m3fn, scale [M, I / block] fp32; with ``scale_tma_aligned`` a view of an MN-major
    ``[num_blocks, align4(M)]`` allocation).  ``num_warps`` / ``num_stages`` are accepted and ignored."""
    if gate_up.dtype != torch.bfloat16:
        raise TypeError(f"gate_up must be bfloat16, got {gate_up.dtype}")
    if gate_up.dim() != 2:
        raise ValueError(f"gate_up must be 2D [M, 2 * I], got shape {tuple(gate_up.shape)}")
    if not gate_up.is_contiguous():
        raise ValueError("gate_up must be contiguous")
    m, width = gate_up.shape
    if width % 2 != 0:
        raise ValueError(f"gate_up width must be even (gate | up), got {width}")
    dim = width // 2
    if block_size != 128:
        raise ValueError(f"the scale block is 128 in this build, got {block_size}")
    if dim % block_size != 0:
        raise ValueError(f"half width {dim} must be a multiple of the scale block {block_size}: "
                         "a block straddling gate and up would quantize across both halves")
    if m == 0:
        raise ValueError("silu_mul quantize needs at least one row")
    if not gate_up.is_cuda:
        raise ValueError("gate_up must be a CUDA tensor")
    nb = dim // block_size
    out = torch.empty((m, dim), device=gate_up.device, dtype=torch.float8_e4m3fn)
    if scale_tma_aligned:
        scale = torch.empty((nb, (m + 3) // 4 * 4), device=gate_up.device, dtype=torch.float32).transpose(0, 1)[:m, :]
    else:
        scale = torch.empty((m, nb), device=gate_up.device, dtype=torch.float32)
    up = gate_up[:, dim:]
    with torch.cuda.device(gate_up.device):
        check(lib().bgmoe_silu_mul_group_quant(
            ptr(gate_up), up.data_ptr(), 0, width, None, None, 1, m, dim, 0, ptr(out), 0, dim, ptr(scale), 0,
            scale.stride(0), scale.stride(1), None, stream()))
    return out, scale


def per_token_blocked_quantize_bf16_to_fp8_1d(x: torch.Tensor, block_size: int = 128, num_warps: int = 4,
                                              num_stages: int = 2, num_valid_tokens: torch.Tensor | None = None,
                                              scale_tma_aligned: bool = False):
    """-> (out [M, dim] float8_e4m3fn, scale [M, ceil(dim / 128)] fp32; with ``scale_tma_aligned`` a view of an
    MN-major ``[num_blocks, align4(M)]`` allocation).  Rows at or past ``num_valid_tokens`` (device int32 scalar)
    get zero bytes and scale 1e-12.  ``num_warps`` / ``num_stages`` are accepted and ignored."""
    assert x.dtype == torch.bfloat16
    assert x.is_contiguous()
    assert x.dim() == 2, f"Expected 2D tensor got {x.dim()}D with shape {x.shape}"
    if block_size != 128:
        raise ValueError(f"the scale block is 128 in this build, got {block_size}")
    if num_valid_tokens is not None:
        if num_valid_tokens.device != x.device:
            raise ValueError("num_valid_tokens must be on the same device as x")
        if num_valid_tokens.dtype != torch.int32:
            raise TypeError(f"num_valid_tokens must be int32, got {num_valid_tokens.dtype}")
        if num_valid_tokens.numel() != 1:
            raise ValueError(f"num_valid_tokens must contain one element, got {tuple(num_valid_tokens.shape)}")
    m, dim = x.shape
    nb = (dim + block_size - 1) // block_size
    out = torch.empty((m, dim), device=x.device, dtype=torch.float8_e4m3fn)
    if scale_tma_aligned:
        scale = torch.empty((nb, (m + 3) // 4 * 4), device=x.device, dtype=torch.float32).transpose(0, 1)[:m, :]
    else:
        scale = torch.empty((m, nb), device=x.device, dtype=torch.float32)
    if m == 0 or dim == 0:
        return out, scale
    with torch.cuda.device(x.device):
        check(lib().bgmoe_act_quant_rows_1d(ptr(x), m, dim, ptr(out), ptr(scale), scale.stride(0), scale.stride(1),
                                            ptr(num_valid_tokens) if num_valid_tokens is not None else None,
                                            stream()))
    return out, scale
