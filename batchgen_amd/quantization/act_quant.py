"""``act_quant`` of batchgen/quantization/act_quant.py:78-128: the bf16 -> blockwise e4m3fn cast of activations,
which the reference routes to the 1-D quantiser for bf16 / block 128 inputs.  Only that route exists here; the
reference's legacy Triton path for other dtypes or block sizes is not built and raises."""
from __future__ import annotations

from typing import Tuple

import torch

from ..kernels.triton.fp8_quantize import per_token_blocked_quantize_bf16_to_fp8_1d


def act_quant(x: torch.Tensor, block_size: int = 128, eps: float = 1e-12,
              num_valid_tokens: torch.Tensor | None = None,
              scale_tma_aligned: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [..., N] bf16 -> (y float8_e4m3fn, same shape; scale fp32 [..., ceil(N / 128)])."""
    assert x.is_contiguous(), 'Input must be contiguous'
    if x.dtype != torch.bfloat16 or block_size != 128 or eps != 1e-12:
        raise NotImplementedError("act_quant: bfloat16 input, block_size 128 and eps 1e-12 only")
    shape = x.shape
    flat = x.view(-1, shape[-1])
    if flat.shape[0] == 0:
        nb = (shape[-1] + 127) // 128
        return (torch.empty(shape, dtype=torch.float8_e4m3fn, device=x.device),
                torch.empty((*shape[:-1], nb), dtype=torch.float32, device=x.device))
    if scale_tma_aligned and x.dim() != 2:
        raise ValueError("scale_tma_aligned act_quant currently requires a 2D input")
    y, scale = per_token_blocked_quantize_bf16_to_fp8_1d(flat, block_size=block_size, num_valid_tokens=num_valid_tokens,
                                                         scale_tma_aligned=scale_tma_aligned)
    return y.view(*shape), scale if scale_tma_aligned else scale.view(*shape[:-1], scale.size(-1))
