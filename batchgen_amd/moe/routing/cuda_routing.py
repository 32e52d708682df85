"""Routing wrappers with the reference's signatures and argument policy
(batchgen/moe/routing/cuda_routing.py:102-432): ValueError / TypeError for
argument policy, RuntimeError from the op's own checks."""
from __future__ import annotations

import torch

from ...kernels import load_extension

GATE_SIGMOID_TOPK_WARP_MAX_EXPERTS = 256
_ext = None


def _get_ext():
    global _ext
    if _ext is None:
        _ext = load_extension("batchgen_kernels.moe._C_routing")
    return _ext


def _check_gate_padding_args(num_valid_tokens, rank_token_counts, rows_per_rank):
    """cuda_routing.py:102-121."""
    if rank_token_counts is not None:
        if num_valid_tokens is not None:
            raise ValueError("rank_token_counts and num_valid_tokens are mutually exclusive "
                             "padding descriptions; pass exactly one")
        if rows_per_rank is None:
            raise ValueError("rows_per_rank is required when rank_token_counts is given")
        if int(rows_per_rank) <= 0:
            raise ValueError(f"rows_per_rank must be positive, got {rows_per_rank}")
    elif rows_per_rank is not None:
        raise ValueError("rows_per_rank is only meaningful together with rank_token_counts")


def gate_sigmoid_topk_cuda(router_logits, e_score_correction, k=8, routed_scaling_factor=2.5,
                           topk_indices=None, topk_weights=None, num_valid_tokens=None, latent_out=None,
                           latent_offset=None, rank_token_counts=None, rows_per_rank=None):
    """Fused sigmoid + top-k + normalise + scale (cuda_routing.py:124-222)."""
    _check_gate_padding_args(num_valid_tokens, rank_token_counts, rows_per_rank)
    if (latent_out is None) != (latent_offset is None):
        raise ValueError("latent_out and latent_offset must be given together")
    if router_logits.dtype != torch.float32:
        router_logits = router_logits.float()
    n = router_logits.shape[0]
    dev = router_logits.device
    if topk_indices is None:
        topk_indices = torch.empty(n, k, dtype=torch.int32, device=dev)
    if topk_weights is None:
        topk_weights = torch.empty(n, k, dtype=torch.float32, device=dev)
    opts = {}
    if num_valid_tokens is not None:
        opts["num_valid_tokens"] = num_valid_tokens
    if latent_out is not None:
        opts["latent_out"] = latent_out
        opts["latent_offset"] = int(latent_offset)
    if rank_token_counts is not None:
        opts["rank_token_counts"] = rank_token_counts
        opts["rows_per_rank"] = int(rows_per_rank)
    r = _get_ext().gate_sigmoid_topk(router_logits, e_score_correction, k, routed_scaling_factor,
                                     topk_indices, topk_weights, **opts)
    return r[0], r[1]


def gate_sigmoid_topk_warp_cuda(router_logits, e_score_correction, k=8, routed_scaling_factor=2.5,
                                topk_indices=None, topk_weights=None, num_valid_tokens=None,
                                rank_token_counts=None, rows_per_rank=None):
    """E <= 256 form, int32 or int64 ids (cuda_routing.py:225-304)."""
    _check_gate_padding_args(num_valid_tokens, rank_token_counts, rows_per_rank)
    if router_logits.dtype != torch.float32:
        raise TypeError(f"gate_sigmoid_topk_warp_cuda takes FP32 router_logits, got {router_logits.dtype}")
    if e_score_correction.dtype != torch.float32:
        raise TypeError("gate_sigmoid_topk_warp_cuda takes an FP32 e_score_correction, got "
                        f"{e_score_correction.dtype}")
    if router_logits.dim() != 2 or router_logits.shape[1] > GATE_SIGMOID_TOPK_WARP_MAX_EXPERTS:
        raise ValueError(f"gate_sigmoid_topk_warp_cuda handles [N, E <= {GATE_SIGMOID_TOPK_WARP_MAX_EXPERTS}] "
                         f"logits, got {tuple(router_logits.shape)}; use gate_sigmoid_topk_cuda")
    if topk_indices is not None and topk_indices.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"topk_indices must be int32 or int64, got {topk_indices.dtype}")
    n = router_logits.shape[0]
    dev = router_logits.device
    if topk_indices is None:
        topk_indices = torch.empty(n, k, dtype=torch.int32, device=dev)
    if topk_weights is None:
        topk_weights = torch.empty(n, k, dtype=torch.float32, device=dev)
    opts = {}
    if num_valid_tokens is not None:
        opts["num_valid_tokens"] = num_valid_tokens
    if rank_token_counts is not None:
        opts["rank_token_counts"] = rank_token_counts
        opts["rows_per_rank"] = int(rows_per_rank)
    r = _get_ext().gate_sigmoid_topk_warp(router_logits, e_score_correction, k, routed_scaling_factor,
                                          topk_indices, topk_weights, **opts)
    return r[0], r[1]


def glm5_router_gemm_cuda(hidden_states, router_weight, router_logits=None, rank_token_counts=None,
                          bucket_size=0, world_size=1):
    """``hidden_states @ router_weight.T`` as fp32 logits from bf16 operands, graph-safe: with
    ``rank_token_counts`` the rows are rank-major ``[world_size, bucket_size]`` and padding rows are zeroed
    on the device (cuda_routing.py:318-366)."""
    if hidden_states.dtype != torch.bfloat16:
        hidden_states = hidden_states.to(torch.bfloat16)
    if router_weight.dtype != torch.bfloat16:
        router_weight = router_weight.to(torch.bfloat16)
    if not hidden_states.is_contiguous():
        hidden_states = hidden_states.contiguous()
    if not router_weight.is_contiguous():
        router_weight = router_weight.contiguous()
    n = hidden_states.shape[0]
    e = router_weight.shape[0]
    dev = hidden_states.device
    if router_logits is None:
        router_logits = torch.empty(n, e, dtype=torch.float32, device=dev)
    elif not router_logits.is_contiguous():
        raise ValueError("router_logits must be contiguous")
    if rank_token_counts is None:
        rank_token_counts = torch.empty(0, dtype=torch.int64, device=dev)
    else:
        if rank_token_counts.dtype != torch.int64:
            rank_token_counts = rank_token_counts.to(torch.int64)
        if not rank_token_counts.is_contiguous():
            rank_token_counts = rank_token_counts.contiguous()
    return _get_ext().glm5_router_gemm(hidden_states, router_weight, rank_token_counts, router_logits,
                                       int(bucket_size), int(world_size))


def router_gemm_gate_sigmoid_topk(hidden_states, router_weight, e_score_correction, k=8,
                                  routed_scaling_factor=2.5, topk_indices=None, topk_weights=None,
                                  n_group=0, topk_group=0, rank_token_counts=None, rows_per_rank=None):
    """``glm5_router_gemm_cuda`` then ``gate_sigmoid_topk_cuda`` (or, with ``n_group >= 1``, the
    group-limited gate on the sigmoided logits) as one call that never writes the logits; ids and weights
    are identical to the two-call sequence.  No counterpart in the reference, which runs the two ops back
    to back (batchgen/models/glm5/model.py:1119-1161)."""
    _check_gate_padding_args(None, rank_token_counts, rows_per_rank)
    if hidden_states.dtype != torch.bfloat16:
        hidden_states = hidden_states.to(torch.bfloat16)
    if router_weight.dtype != torch.bfloat16:
        router_weight = router_weight.to(torch.bfloat16)
    r = _get_ext().router_gemm_gate(hidden_states.contiguous(), router_weight.contiguous(), e_score_correction,
                                    k, routed_scaling_factor, topk_indices, topk_weights, n_group, topk_group,
                                    rank_token_counts, rows_per_rank)
    return r[0], r[1]


def dispatch_count_gather_cuda(x, topk_indices, expert_start, num_local_experts, expert_counts=None,
                               expert_offsets=None, expert_counters=None, dispatched_x=None, topk_pos=None,
                               num_valid_tokens=-1):
    """Tight dispatch -> (dispatched_x, expert_counts, expert_offsets, topk_pos) (cuda_routing.py:369-432)."""
    if topk_indices.dtype != torch.int32:
        topk_indices = topk_indices.to(torch.int32)
    n, k = topk_indices.shape
    h = x.shape[1]
    dev = x.device
    e = num_local_experts
    if expert_counts is None:
        expert_counts = torch.zeros(e, dtype=torch.int32, device=dev)
    if expert_offsets is None:
        expert_offsets = torch.empty(e + 1, dtype=torch.int32, device=dev)
    if expert_counters is None:
        expert_counters = torch.zeros(e, dtype=torch.int32, device=dev)
    if topk_pos is None:
        topk_pos = torch.full((n * k,), -1, dtype=torch.int32, device=dev)
    if dispatched_x is None:
        dispatched_x = torch.empty(max(n * k, 1), h, dtype=x.dtype, device=dev)
    r = _get_ext().dispatch_count_gather(x, topk_indices, expert_start, num_local_experts, expert_counts,
                                         expert_offsets, expert_counters, dispatched_x, topk_pos,
                                         num_valid_tokens)
    return dispatched_x, r[0], r[1], r[2]


def reduce_weighted_scatter_cuda(expert_output, topk_pos, topk_weights, N, H, K, output=None,
                                 num_valid_tokens=-1):
    """cuda_routing.py:435-470."""
    return _get_ext().reduce_weighted_scatter(expert_output, topk_pos, topk_weights, N, H, K, output,
                                              num_valid_tokens)
