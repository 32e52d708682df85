"""Masked / ragged dispatch and weighted reduce with the reference's frozen
signatures (batchgen/moe/dispatch_scatter_3d.py:76-232;
tests/contracts/test_pin_moe.py:63-140)."""
from __future__ import annotations

from ..kernels import load_extension

_ext = None


def _get_ext():
    global _ext
    if _ext is None:
        _ext = load_extension("batchgen_kernels.moe._C_dispatch_scatter_3d")
    return _ext


def dispatch_scatter_3d(x, topk_indices, act_buffer, expert_start, num_local_experts, max_tokens_padded,
                        expert_counts, expert_counters, topk_pos):
    """-> (expert_counts, topk_pos); rows land in act_buffer[e*max_tokens_padded + slot]."""
    r = _get_ext().dispatch_scatter_3d(x, topk_indices, act_buffer, expert_start, num_local_experts,
                                       max_tokens_padded, expert_counts, expert_counters, topk_pos)
    return r[0], r[1]


def dispatch_scatter_ragged(x, topk_indices, act_buffer, expert_start, num_local_experts, expert_counts,
                            expert_counters, topk_pos, cu_seqlens, row_align=64):
    """-> (expert_counts, cu_seqlens, topk_pos); expert e owns rows [cu[e], cu[e]+count[e])."""
    r = _get_ext().dispatch_scatter_ragged(x, topk_indices, act_buffer, expert_start, num_local_experts,
                                           expert_counts, expert_counters, topk_pos, cu_seqlens, row_align)
    return r[0], r[1], r[2]


def reduce_weighted_scatter(expert_output, topk_pos, topk_weights, N, H, K, output=None):
    return _get_ext().reduce_weighted_scatter(expert_output, topk_pos, topk_weights, N, H, K, output)


def reduce_weighted_scatter_fp32(expert_output, topk_pos, topk_weights, N, H, K, output):
    return _get_ext().reduce_weighted_scatter_fp32(expert_output, topk_pos, topk_weights, N, H, K, output)


def reduce_weighted_scatter_bf16_ordered(expert_output, topk_pos, topk_indices, topk_weights, N, H, K, output):
    return _get_ext().reduce_weighted_scatter_bf16_ordered(expert_output, topk_pos, topk_indices,
                                                           topk_weights, N, H, K, output)


def ragged_row_capacity(num_tokens: int, top_k: int, num_local_experts: int, row_align: int = 64) -> int:
    """Worst-case rows of the ragged buffer (batchgen_kernels/src/moe/dispatch_scatter_3d.cu:229-243)."""
    nk = num_tokens * top_k
    return (nk + (row_align - 1) * min(num_local_experts, nk)) // row_align * row_align
