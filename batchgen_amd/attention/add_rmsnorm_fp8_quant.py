"""Python entry point of the fused add + RMSNorm + FP8-quantise producer, with the reference's signature
(batchgen_kernels/attention/add_rmsnorm_fp8_quant.py:33-83)."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..kernels import load_extension

_ext = None


def _get_ext():
    global _ext
    if _ext is None:
        _ext = load_extension("batchgen_kernels.attention._C_add_rmsnorm_fp8_quant")
    return _ext


def preload_add_rmsnorm_fp8_quant_kernel():
    """Resolve the library before graph capture."""
    return _get_ext()


def cuda_add_rmsnorm_fp8_quant(residual: torch.Tensor, hidden: torch.Tensor, weight: torch.Tensor,
                               eps: float = 1e-5, norm_num_valid_tokens: Optional[torch.Tensor] = None,
                               quant_num_valid_tokens: Optional[torch.Tensor] = None,
                               row_valid_mask: Optional[torch.Tensor] = None,
                               scale_tma_aligned: bool = False
                               ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``residual`` is updated in place.  Returns ``(normed, residual, x_fp8, x_scale)``: the unfused
    add + RMSNorm's ``normed``/``residual`` and the standalone 1-D quantiser's bytes and scales of
    ``normed``.  ``x_fp8``/``x_scale`` can be handed to the FP8 expert GEMMs as they are."""
    r = _get_ext().add_rmsnorm_fp8_quant_forward(residual, hidden, weight, eps, norm_num_valid_tokens,
                                                 quant_num_valid_tokens, row_valid_mask, scale_tma_aligned)
    return r[0], r[1], r[2], r[3]
