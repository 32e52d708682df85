"""gfx950 implementation of the reference extension
``batchgen_kernels.attention._C_add_rmsnorm_fp8_quant``
(binding: batchgen_kernels/src/attention/csrc/add_rmsnorm_fp8_quant.cu:553-566)."""
from __future__ import annotations

import torch

from ..._lib import check, lib, ptr, stream
from .. import _checks as ck


def _num_valid(t, name):
    ck.gpu(t, name)
    if t.dtype != torch.int32:
        ck.fail(f"{name} must be int32, got {t.dtype}")
    if t.numel() != 1:
        ck.fail(f"{name} must contain one element, got {t.numel()}")
    return t


def add_rmsnorm_fp8_quant_forward(residual, hidden, weight, eps, norm_num_valid_tokens=None,
                                  quant_num_valid_tokens=None, row_valid_mask=None, scale_tma_aligned=False):
    """Fused add + RMSNorm + per-token 128-block e4m3fn cast.  Returns
    [normed_out, residual, quant_out, quant_scale]; ``residual`` is updated in place when it is contiguous
    (add_rmsnorm_fp8_quant.cu:414-541)."""
    for t, name in ((residual, "residual"), (hidden, "hidden"), (weight, "weight")):
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            ck.fail(f"{name} must be CUDA")
        if t.dtype != torch.bfloat16:
            ck.fail(f"fused add+RMSNorm+FP8 requires bf16 {name}, got {t.dtype}")
    residual = residual.contiguous()
    hidden = hidden.contiguous()
    weight = weight.contiguous()
    h = residual.size(-1)
    if h % 128 != 0 or not 128 <= h <= 8192:
        ck.fail(f"fused add+RMSNorm+FP8 handles hidden sizes that are multiples of 128 up to 8192; got "
                f"hidden_size={h}")
    if residual.numel() != hidden.numel():
        ck.fail(f"residual and hidden must have the same number of elements ({residual.numel()} vs "
                f"{hidden.numel()})")
    if weight.numel() != h:
        ck.fail(f"weight must hold {h} elements, got {weight.numel()}")
    rows = residual.numel() // h
    dev = residual.device
    blocks = h // 128
    normed = torch.empty_like(residual)
    quant = torch.empty((rows, h), dtype=torch.float8_e4m3fn, device=dev)
    if scale_tma_aligned:
        aligned = (rows + 3) // 4 * 4
        scale = torch.empty((blocks, aligned), dtype=torch.float32, device=dev).transpose(0, 1)[:rows]
    else:
        scale = torch.empty((rows, blocks), dtype=torch.float32, device=dev)
    if rows == 0:
        return [normed, residual, quant, scale]
    nnv = _num_valid(norm_num_valid_tokens, "norm_num_valid_tokens") if norm_num_valid_tokens is not None else None
    qnv = _num_valid(quant_num_valid_tokens, "quant_num_valid_tokens") if quant_num_valid_tokens is not None else None
    if nnv is not None and (qnv is None or nnv.data_ptr() != qnv.data_ptr()):
        ck.fail("norm_num_valid_tokens requires quant_num_valid_tokens to be the SAME tensor: a row the norm "
                "skips has undefined normed_out bytes, so its FP8 output cannot be reproduced")
    mask = None
    if row_valid_mask is not None:
        if not row_valid_mask.is_cuda:
            ck.fail("row_valid_mask must be CUDA")
        if row_valid_mask.dtype != residual.dtype:
            ck.fail("row_valid_mask dtype must match residual dtype")
        if row_valid_mask.numel() != rows:
            ck.fail(f"row_valid_mask must have one entry per row (expected {rows}, got {row_valid_mask.numel()})")
        mask = row_valid_mask.contiguous()
    with torch.cuda.device(dev):
        check(lib().bgmoe_add_rmsnorm_fp8_quant(
            ptr(residual), ptr(hidden), ptr(weight), rows, h, float(eps), ptr(normed), ptr(quant), ptr(scale),
            scale.stride(0), scale.stride(1), ptr(nnv), ptr(qnv), ptr(mask), stream()))
    return [normed, residual, quant, scale]
