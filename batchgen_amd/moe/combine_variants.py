"""The remaining weighted-combine helpers of the reference's model files, as thin callers of the combine kernel
(``out[t] = sum_k float(row_k) * w[t, k]``, fp32 accumulation in ascending k, `csrc/combine.hip`):

* ``moe_weighted_sum_triton`` / ``_v2`` / ``moe_weighted_sum_v3`` (batchgen_kernels/triton/moe_weighted_sum.py:159-210,
  262-330, 607-632): dense ``[T, K, H]`` expert results times ``[T, K]`` weights -> ``[T, H]`` in the input dtype;
* ``build_inverse_mapping`` / ``scatter_weight_reduce_optimized``
  (batchgen/models/deepseek/deepseekv3/modeling_deepseek_v3.py:1474-1542): sparse ``[nnz, H]`` results with the
  (token, slot) of every row -> fp32 ``[T, H]``;
* ``moe_fp32_accum_triton_v2`` (:1034-1065): expert-sorted rows and their sorting permutation -> ``[T, H]``.

The block-size and version arguments select among the reference's Triton kernels, which all compute the same sum:
accepted and ignored.
"""
from __future__ import annotations

import torch

from .._lib import check, lib, ptr, stream

_MAX_K = 32
_IDENTITY = {}


def _identity_pos(n: int, device) -> torch.Tensor:
    key = (str(device),)
    t = _IDENTITY.get(key)
    if t is None or t.numel() < n:
        t = torch.arange(max(n, 1 << 16), dtype=torch.int32, device=device)
        _IDENTITY[key] = t
    return t


def _dense_sum(global_results: torch.Tensor, topk_weight: torch.Tensor) -> torch.Tensor:
    if global_results.dim() != 3:
        raise ValueError("global_results must be [num_tokens, topk, hidden_size]")
    t, k, h = global_results.shape
    if tuple(topk_weight.shape) != (t, k):
        raise ValueError(f"Shape mismatch: {tuple(topk_weight.shape)} vs {(t, k)}")
    if global_results.dtype != torch.bfloat16 or not global_results.is_cuda or not global_results.is_contiguous():
        raise ValueError("global_results must be a contiguous CUDA bfloat16 tensor")
    if not 1 <= k <= _MAX_K:
        raise ValueError(f"topk must be in [1, {_MAX_K}], got {k}")
    out = torch.empty((t, h), dtype=global_results.dtype, device=global_results.device)
    if t == 0 or h == 0:
        return out
    w = topk_weight.to(torch.float32).contiguous()
    with torch.cuda.device(global_results.device):
        check(lib().bgmoe_reduce_weighted_scatter(ptr(global_results), ptr(_identity_pos(t * k, global_results.device)),
                                                  ptr(w), t, h, k, ptr(out), -1, None, 0, stream()))
    return out


def moe_weighted_sum_triton(global_results, topk_weight, use_optimized=True, version="v1"):
    return _dense_sum(global_results, topk_weight)


def moe_weighted_sum_triton_v2(global_results, topk_weight):
    return _dense_sum(global_results, topk_weight)


def moe_weighted_sum_v3(global_results, topk_weight, block_size_tokens=None, block_size_hidden=None, debug=False):
    return _dense_sum(global_results, topk_weight)


def build_inverse_mapping(global_indices: torch.Tensor, token_topk_pos: torch.Tensor, num_tokens: int,
                          num_experts_per_tok: int) -> torch.Tensor:
    """``[num_tokens, num_experts_per_tok]`` int64: the row of ``res`` that holds token t's slot k, -1 when none."""
    mapping = torch.full((num_tokens, num_experts_per_tok), -1, dtype=torch.int64, device=global_indices.device)
    if global_indices.numel():
        mapping[global_indices.long(), token_topk_pos.long()] = torch.arange(global_indices.numel(), dtype=torch.int64,
                                                                             device=global_indices.device)
    return mapping


def scatter_weight_reduce_optimized(res: torch.Tensor, global_indices: torch.Tensor, token_topk_pos: torch.Tensor,
                                    topk_weight: torch.Tensor, num_tokens: int, num_experts_per_tok: int) -> torch.Tensor:
    """fp32 ``[num_tokens, hidden]``; ``global_indices`` / ``token_topk_pos`` may be longer than ``res`` has rows."""
    if topk_weight.dtype != torch.float32 or tuple(topk_weight.shape) != (num_tokens, num_experts_per_tok):
        raise ValueError(f"topk_weight must be float32 ({num_tokens}, {num_experts_per_tok}), got {topk_weight.dtype} "
                         f"{tuple(topk_weight.shape)}")
    nnz, hidden = res.shape
    out = torch.zeros((num_tokens, hidden), dtype=torch.float32, device=res.device)
    if nnz == 0 or num_tokens == 0:
        return out
    if res.dtype != torch.bfloat16 or not res.is_contiguous() or not 1 <= num_experts_per_tok <= _MAX_K:
        raise ValueError(f"res must be contiguous bfloat16 and num_experts_per_tok in [1, {_MAX_K}]")
    pos = build_inverse_mapping(global_indices[:nnz], token_topk_pos[:nnz], num_tokens,
                                num_experts_per_tok).to(torch.int32).contiguous()
    with torch.cuda.device(res.device):
        check(lib().bgmoe_reduce_weighted_scatter_fp32(ptr(res), ptr(pos), ptr(topk_weight.contiguous()), num_tokens,
                                                       hidden, num_experts_per_tok, ptr(out), stream()))
    return out


def moe_fp32_accum_triton_v2(outs: torch.Tensor, idxs: torch.Tensor, topk_weights: torch.Tensor) -> torch.Tensor:
    """The prefill combine of ``DeepseekV3MoE_Prefill.moe_infer``
    (batchgen/models/deepseek/deepseekv3/modeling_deepseek_v3.py:1034-1065): ``outs`` [T * K, H] are the expert
    outputs in expert-sorted order, ``idxs`` the sorting permutation (sorted row j came from flat (token, k) index
    ``idxs[j]``); returns ``[T, H]`` in the dtype of ``outs``, fp32 accumulation over k ascending.  Each term is one
    fused multiply-add here, as in the CUDA combine kernels; whether the reference's Triton kernel contracts the
    product and the sum is decided by its compiler (parity unpinned at the last fp32 bit, before the bf16
    rounding)."""
    t, k = topk_weights.shape
    if outs.dim() != 2 or outs.shape[0] != t * k or idxs.numel() != t * k:
        raise ValueError(f"outs must be [{t * k}, H] and idxs [{t * k}]; got {tuple(outs.shape)} and {tuple(idxs.shape)}")
    if outs.dtype != torch.bfloat16 or not outs.is_cuda or not outs.is_contiguous() or not 1 <= k <= _MAX_K:
        raise ValueError(f"outs must be a contiguous CUDA bfloat16 tensor and topk in [1, {_MAX_K}]")
    h = outs.shape[1]
    out = torch.empty((t, h), dtype=outs.dtype, device=outs.device)
    if t == 0 or h == 0:
        return out
    pos = torch.empty(t * k, dtype=torch.int32, device=outs.device)
    pos[idxs.reshape(-1).long()] = torch.arange(t * k, dtype=torch.int32, device=outs.device)
    w = topk_weights.to(torch.float32).contiguous()
    with torch.cuda.device(outs.device):
        check(lib().bgmoe_reduce_weighted_scatter(ptr(outs), ptr(pos), ptr(w), t, h, k, ptr(out), -1, None, 0, stream()))
    return out
