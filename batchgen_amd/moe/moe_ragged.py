"""The compact ragged workspace helpers of the GLM-5 grouped prefill and MoE decode, with the reference's names
and argument orders (batchgen/models/glm/glm5/moe_ragged.py:14-377), over this build's ops:

* sizing: ``gemm_tilem_avg`` (:24-28), ``gemm_tilem_avg_effective`` (:167-176; the reference's batch-level debug
  override does not exist here, so it is the formula), ``ragged_row_capacity`` (:222-233), ``make_quant_buffers``
  (:236-249);
* ops: ``dispatch_scatter_ragged`` (:252-276), ``act_quant_ragged`` (:279-295), ``silu_mul_quant_ragged``
  (:298-327), ``deepep_ll_scale_repack`` (:330-351), ``reduce_weighted_scatter_bf16_ordered`` (:354-377);
* the receive-count histogram diagnostic (:52-164): device-side accumulation that a captured graph may contain,
  and a host read-back that must stay outside any capture.
"""
from __future__ import annotations

import torch

from ..kernels import load_extension
from . import dispatch_scatter_3d as _dispatch

ROW_ALIGN = 64
QUANT_BLOCK = 128
_CAPACITY_BLOCK = 128


def gemm_tilem_avg(global_rows: int, topk: int, num_global_experts: int) -> int:
    """Mean rows per expert segment, at least 1: the grouped GEMM's row-count hint (a host constant per captured
    bucket).  The kernels here pick their tile on the device from the counts, so the value only travels."""
    if num_global_experts <= 0:
        raise ValueError("num_global_experts must be positive")
    return max(1, int(global_rows) * int(topk) // int(num_global_experts))


def gemm_tilem_avg_effective(global_rows: int, topk: int, num_global_experts: int) -> int:
    return gemm_tilem_avg(global_rows, topk, num_global_experts)


def ragged_row_capacity(max_global_tokens: int, topk: int, num_local_experts: int, row_align: int = ROW_ALIGN) -> int:
    """Static row capacity of the ragged buffers: every (token, k) pair live plus the worst alignment padding of
    every local expert, rounded up to 128 rows."""
    rows = int(max_global_tokens) * int(topk) + int(num_local_experts) * (int(row_align) - 1)
    return -(-rows // _CAPACITY_BLOCK) * _CAPACITY_BLOCK


def make_quant_buffers(rows: int, dim: int, device):
    """(bytes [rows, dim] uint8, scales [dim // 128, rows] fp32, zeroed): the quantised activations and their
    transposed scale matrix as the grouped GEMM reads them."""
    if dim % QUANT_BLOCK:
        raise ValueError(f"ragged quant dim must be a multiple of {QUANT_BLOCK}, got {dim}")
    return (torch.empty(rows, dim, dtype=torch.uint8, device=device),
            torch.zeros(dim // QUANT_BLOCK, rows, dtype=torch.float32, device=device))


def _ops():
    return load_extension("batchgen_kernels.moe._C_fp8_blockwise_ops")


def require_ragged_kernels():
    """(dispatch module, quantiser module); raises ImportError when the library is not built."""
    return load_extension("batchgen_kernels.moe._C_dispatch_scatter_3d"), _ops()


def dispatch_scatter_ragged(x, topk_indices, act_buffer, expert_start, num_local_experts, expert_counts,
                            expert_counters, cu_seqlens, topk_pos, row_align: int = ROW_ALIGN):
    """Note the order: ``cu_seqlens`` before ``topk_pos`` here, the other way round in the op underneath."""
    return _dispatch.dispatch_scatter_ragged(x, topk_indices, act_buffer, expert_start, num_local_experts,
                                             expert_counts, expert_counters, topk_pos, cu_seqlens, int(row_align))


def act_quant_ragged(x, seqlens, cu_seqlens, output, scale, row_align: int = ROW_ALIGN) -> None:
    _ops().act_quant_ragged(x, seqlens, cu_seqlens, output, scale, int(row_align))


def silu_mul_quant_ragged(gate, up, output, scale_rows, seqlens, cu_seqlens) -> None:
    """SiLU(gate) * up and the FP8 group cast of the live ragged rows in one pass; ``scale_rows`` is the row-major
    ``[m, I // 128]`` matrix."""
    from ..kernels.triton.moe_masked_act_quant import silu_mul_ragged_group_quant
    silu_mul_ragged_group_quant(gate, up, output, scale_rows, seqlens, cu_seqlens, group_size=QUANT_BLOCK)


def deepep_ll_scale_repack(recv_scales, recv_count, out, span_align: int) -> None:
    _ops().deepep_ll_scale_repack(recv_scales, recv_count, out, int(span_align))


def reduce_weighted_scatter_bf16_ordered(expert_output, topk_pos, topk_indices, topk_weights, num_tokens: int,
                                         hidden_size: int, topk: int, *, output):
    return _dispatch.reduce_weighted_scatter_bf16_ordered(expert_output, topk_pos, topk_indices, topk_weights,
                                                          num_tokens, hidden_size, topk, output)


# ---- receive-count histogram: slot 0 = accumulated layer-steps, slot 1 = routed rows, slot 2 + t = expert slots
# that needed t row tiles of block_m rows

def recv_count_histogram_width(stride: int, block_m: int) -> int:
    if int(stride) <= 0 or int(block_m) <= 0:
        raise ValueError(f"recv-count histogram needs positive stride/block_m; got {stride}/{block_m}")
    return 3 + -(-int(stride) // int(block_m))


def accumulate_recv_count_histogram(hist: torch.Tensor, recv_count: torch.Tensor, block_m: int) -> None:
    """Device work only (static shapes, no host read): safe inside a captured graph, cumulative over replays."""
    if hist.dtype != torch.int64:
        raise RuntimeError(f"recv-count histogram must be int64; got {hist.dtype}")
    if recv_count.dim() != 1:
        raise RuntimeError(f"recv_count must be the per-expert [E] row counts; got {tuple(recv_count.shape)}")
    rows = recv_count.to(torch.int64)
    tiles = ((rows + (int(block_m) - 1)) // int(block_m)).clamp_(0, hist.numel() - 3) + 2
    hist.index_add_(0, tiles, torch.ones_like(tiles))
    hist[0] += 1
    hist[1] += rows.sum()


def format_recv_count_histogram(hist: torch.Tensor, block_m: int) -> str:
    """One host read-back for a log line; refuses to run inside a graph capture."""
    if hist.is_cuda and torch.cuda.is_current_stream_capturing():
        raise RuntimeError("format_recv_count_histogram reads the histogram back to the host and must not be "
                           "called inside a CUDA graph capture; keep only accumulate_recv_count_histogram in the "
                           "captured forward")
    steps, rows, *buckets = (int(v) for v in hist.tolist())
    slots = sum(buckets)
    if slots == 0:
        return "recv-count histogram: no accumulation yet"
    over = sum(buckets[2:])
    parts = " ".join(f"{t}t={c}({100.0 * c / slots:.2f}%)" for t, c in enumerate(buckets) if c)
    return (f"recv-count histogram (block_m={block_m}): layer-steps={steps} expert-slots={slots} rows={rows} "
            f"mean_rows_per_slot={rows / slots:.2f} over_one_tile={over}({100.0 * over / slots:.3f}%) | {parts}")
