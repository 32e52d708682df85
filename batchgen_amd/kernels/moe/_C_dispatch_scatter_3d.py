"""gfx950 implementation of the reference extension ``batchgen_kernels.moe._C_dispatch_scatter_3d``
(bindings: batchgen_kernels/src/moe/dispatch_scatter_3d.cu:671-683)."""
from __future__ import annotations

import torch

from ..._lib import check, lib, ptr, stream
from .. import _checks as ck
from .._workspace import dispatch_workspace

_INT32_MAX = 2147483647


def dispatch_scatter_3d(x, topk_indices, act_buffer, expert_start, num_local_experts, max_tokens_padded,
                        expert_counts, expert_counters, topk_pos):
    """Masked [E_local, max_tokens_padded, H] layout (dispatch_scatter_3d.cu:88-137).
    Returns [expert_counts, topk_pos]."""
    ck.cuda_tensor(None, x, torch.bfloat16, "x")
    if x.dim() != 2:
        ck.fail("x must be BF16 [N, H]")
    n, h = x.shape
    ck.gpu(topk_indices, "topk_indices")
    if topk_indices.dim() != 2 or topk_indices.size(0) != n:
        ck.fail(f"topk_indices must be int32 [N = {n}, K]")
    if num_local_experts <= 0 or max_tokens_padded <= 0:
        ck.fail("num_local_experts and max_tokens_padded must be positive")
    k = topk_indices.size(1)
    flat = topk_indices.reshape(-1).contiguous()
    ck.cuda_tensor(x, flat, torch.int32, "topk_indices")
    ck.cuda_tensor(x, act_buffer, torch.bfloat16, "act_buffer")
    if act_buffer.numel() < num_local_experts * max_tokens_padded * h:
        ck.fail("act_buffer is smaller than [E_local * max_tokens_padded, H]")
    for t, name in ((expert_counts, "expert_counts"), (expert_counters, "expert_counters"),
                    (topk_pos, "topk_pos")):
        ck.cuda_tensor(x, t, torch.int32, name)
    if topk_pos.numel() < n * k:
        ck.fail("topk_pos must have N*K elements")
    if expert_counts.numel() < num_local_experts or expert_counters.numel() < num_local_experts:
        ck.fail(f"expert_counts / expert_counters must hold E_local = {num_local_experts} elements")
    ws, ws_bytes = dispatch_workspace(x.device, n * k, num_local_experts)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_dispatch_scatter_3d(ptr(x), ptr(flat), n, k, h, ptr(act_buffer), int(expert_start),
                                              int(num_local_experts), int(max_tokens_padded), ptr(expert_counts),
                                              ptr(expert_counters), ptr(topk_pos), ptr(ws), ws_bytes, stream()))
    return [expert_counts, topk_pos]


def dispatch_scatter_ragged(x, topk_indices, act_buffer, expert_start, num_local_experts, expert_counts,
                            expert_counters, topk_pos, cu_seqlens, row_align):
    """Contiguous ragged layout with device cu_seqlens (dispatch_scatter_3d.cu:255-358).
    Returns [expert_counts, cu_seqlens, topk_pos]."""
    row_align = int(row_align)
    if row_align <= 0 or (row_align & (row_align - 1)) != 0 or row_align > _INT32_MAX:
        ck.fail(f"row_align must be a positive power of two, got {row_align}")
    ck.gpu(x, "x")
    for t, name in ((x, "x"), (topk_indices, "topk_indices"), (act_buffer, "act_buffer"),
                    (expert_counts, "expert_counts"), (expert_counters, "expert_counters"),
                    (topk_pos, "topk_pos"), (cu_seqlens, "cu_seqlens")):
        ck.cuda_tensor(x, t, None, name)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        ck.fail("x must be BF16 [N, H]")
    if topk_indices.dim() != 2 or topk_indices.dtype != torch.int32 or topk_indices.size(0) != x.size(0):
        ck.fail("topk_indices must be int32 [N, K]")
    if act_buffer.dim() != 2 or act_buffer.dtype != torch.bfloat16 or act_buffer.size(1) != x.size(1):
        ck.fail("act_buffer must be BF16 [rows, H]")
    n, h = x.shape
    k = topk_indices.size(1)
    e = int(num_local_experts)
    if expert_start < 0 or expert_start + e > _INT32_MAX:
        ck.fail(f"expert_start out of range: {expert_start}")
    nk = n * k
    cap = (nk + (row_align - 1) * min(e, nk)) // row_align * row_align
    if not (cap <= act_buffer.size(0) <= _INT32_MAX):
        ck.fail(f"act_buffer rows ({act_buffer.size(0)}) must be in [{cap}, INT32_MAX]")
    if expert_counts.dtype != torch.int32 or expert_counts.dim() != 1 or expert_counts.size(0) != e:
        ck.fail("expert_counts must be int32 [E_local]")
    if expert_counters.dtype != torch.int32 or expert_counters.dim() != 1 or expert_counters.size(0) != e:
        ck.fail("expert_counters must be int32 [E_local]")
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.size(0) != e + 1:
        ck.fail("cu_seqlens must be int32 [E_local + 1]")
    if topk_pos.dtype != torch.int32 or topk_pos.dim() != 1 or topk_pos.size(0) != nk:
        ck.fail("topk_pos must be int32 [N * K]")
    ws, ws_bytes = dispatch_workspace(x.device, nk, e)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_dispatch_scatter_ragged(ptr(x), ptr(topk_indices), n, k, h, ptr(act_buffer),
                                                  act_buffer.size(0), int(expert_start), e, ptr(expert_counts),
                                                  ptr(expert_counters), ptr(topk_pos), ptr(cu_seqlens), row_align,
                                                  ptr(ws), ws_bytes, stream()))
    return [expert_counts, cu_seqlens, topk_pos]


def reduce_weighted_scatter(expert_output, topk_pos, topk_weights, N, H, K, output):
    """dispatch_scatter_3d.cu:527-556 (K in {2,4,8}; output allocated when empty)."""
    if K not in (2, 4, 8):
        ck.fail(f"Unsupported K={K}")
    ck.gpu(expert_output, "expert_output")
    if output is None or output.numel() == 0:
        output = torch.zeros((N, H), dtype=torch.bfloat16, device=expert_output.device)
    ck.combine_args(expert_output, topk_pos, topk_weights, output, int(N), int(H), int(K), torch.bfloat16)
    with torch.cuda.device(expert_output.device):
        check(lib().bgmoe_reduce_weighted_scatter(ptr(expert_output), ptr(topk_pos), ptr(topk_weights), int(N),
                                                  int(H), int(K), ptr(output), -1, None, 0, stream()))
    return output


def reduce_weighted_scatter_fp32(expert_output, topk_pos, topk_weights, N, H, K, output):
    """dispatch_scatter_3d.cu:558-597 (K == 16, fp32 output)."""
    if N <= 0 or H <= 0:
        ck.fail("N and H must be positive")
    if K != 16:
        ck.fail(f"K3 FP32 weighted combine requires K=16, got {K}")
    for t, dt, name in ((expert_output, torch.bfloat16, "expert_output"), (topk_pos, torch.int32, "topk_pos"),
                        (topk_weights, torch.float32, "topk_weights"), (output, torch.float32, "output")):
        ck.cuda_tensor(None, t, dt, name)
    if topk_pos.numel() < N * K or topk_weights.numel() < N * K:
        ck.fail("topk_pos / topk_weights is smaller than N*K")
    if output.dim() != 2 or output.size(0) < N or output.size(1) != H:
        ck.fail("output must have shape [N, H]")
    if expert_output.dim() != 2 or expert_output.size(1) != H:
        ck.fail("expert_output must have shape [rows, H]")
    with torch.cuda.device(expert_output.device):
        check(lib().bgmoe_reduce_weighted_scatter_fp32(ptr(expert_output), ptr(topk_pos), ptr(topk_weights),
                                                       int(N), int(H), int(K), ptr(output), stream()))
    return output


def reduce_weighted_scatter_bf16_ordered(expert_output, topk_pos, topk_indices, topk_weights, N, H, K, output):
    """dispatch_scatter_3d.cu:599-669 (K in {2,4,8}, H % 8 == 0)."""
    if N <= 0 or H <= 0:
        ck.fail("N and H must be positive")
    if K not in (2, 4, 8):
        ck.fail(f"ordered BF16 combine supports K=2,4,8, got {K}")
    if H % 8 != 0:
        ck.fail(f"ordered BF16 combine requires H % 8 == 0, got H={H}")
    for t, dt, name in ((expert_output, torch.bfloat16, "expert_output"), (topk_pos, torch.int32, "topk_pos"),
                        (topk_indices, torch.int32, "topk_indices"), (topk_weights, torch.float32, "topk_weights"),
                        (output, torch.bfloat16, "output")):
        ck.cuda_tensor(expert_output, t, dt, name)
    if topk_pos.numel() != N * K:
        ck.fail("topk_pos must contain N*K elements")
    if tuple(topk_indices.shape) != (N, K) or tuple(topk_weights.shape) != (N, K):
        ck.fail("topk_indices / topk_weights must have shape [N, K]")
    if tuple(output.shape) != (N, H):
        ck.fail("output must have shape [N, H]")
    with torch.cuda.device(expert_output.device):
        check(lib().bgmoe_reduce_weighted_scatter_bf16_ordered(ptr(expert_output), ptr(topk_pos),
                                                               ptr(topk_indices), ptr(topk_weights), int(N),
                                                               int(H), int(K), ptr(output), stream()))
    return output
