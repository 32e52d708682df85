"""Grouped FP8 block-scaled GEMM wrappers with the reference's signatures
(batchgen/moe/grouped_fp8_blockwise_moe.py:143-655)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from torch import Tensor

from ..kernels import load_extension

_MODULE_NAME = "batchgen_kernels.moe._C_fp8_blockwise_gemm"
_ext = None


def _get_module():
    global _ext
    if _ext is None:
        _ext = load_extension(_MODULE_NAME)
    return _ext


def grouped_fp8_tile_m(num_seq_per_group_avg: int) -> int:
    """The reference's TileM bucket for ``avg`` (<=16 -> 16, <=32 -> 32, else 64).  The gfx950 kernels
    choose their row tiling per group on the device; the value only keeps plan checks meaningful."""
    avg = int(num_seq_per_group_avg)
    if avg <= 16:
        return 16
    if avg <= 32:
        return 32
    return 64


@dataclass(frozen=True)
class GroupedFp8TmaPlan:
    """What one prepare call recorded for an S1/S3 pair (grouped_fp8_blockwise_moe.py:160-186).  There are
    no TMA descriptors on gfx950; the plan only pins which buffers it was made for."""
    s1_tma_desc: Optional[Tensor]
    s3_tma_desc: Optional[Tensor]
    tiles: Optional[Tensor]
    cu_tiles: Optional[Tensor]
    tile_m: int
    seqlens_ptr: int
    cu_seqlens_ptr: int
    s1_x_ptr: int
    s1_output_ptr: int
    s3_x_ptr: int
    s3_output_ptr: int
    m: int
    s1_k: int
    s1_n: int
    s3_k: int
    s3_n: int


def prepare_grouped_fp8_s1_s3_tma(s1_x, s1_output, s3_x, s3_output, seqlens, cu_seqlens,
                                  num_seq_per_group_avg, *, s1_tma_desc=None, s3_tma_desc=None, tiles=None,
                                  cu_tiles=None) -> GroupedFp8TmaPlan:
    _get_module().fp8_blockwise_prepare_s1_s3_tma(s1_x, s1_output, s3_x, s3_output, seqlens, cu_seqlens,
                                                  int(num_seq_per_group_avg), s1_tma_desc, s3_tma_desc, tiles,
                                                  cu_tiles)
    return GroupedFp8TmaPlan(
        s1_tma_desc=s1_tma_desc, s3_tma_desc=s3_tma_desc, tiles=tiles, cu_tiles=cu_tiles,
        tile_m=grouped_fp8_tile_m(num_seq_per_group_avg), seqlens_ptr=seqlens.data_ptr(),
        cu_seqlens_ptr=cu_seqlens.data_ptr(), s1_x_ptr=s1_x.data_ptr(), s1_output_ptr=s1_output.data_ptr(),
        s3_x_ptr=s3_x.data_ptr(), s3_output_ptr=s3_output.data_ptr(), m=int(s1_x.shape[0]),
        s1_k=int(s1_x.shape[1]), s1_n=int(s1_output.shape[1]), s3_k=int(s3_x.shape[1]),
        s3_n=int(s3_output.shape[1]))


def _check_plan(plan, stage, x_fp8, output, seqlens, cu_seqlens, num_seq_per_group_avg):
    """Refuse a plan prepared for other buffers, counts or TileM (grouped_fp8_blockwise_moe.py:250-289)."""
    if stage == "s1":
        want = (plan.s1_x_ptr, plan.s1_output_ptr, plan.s1_k, plan.s1_n)
    else:
        want = (plan.s3_x_ptr, plan.s3_output_ptr, plan.s3_k, plan.s3_n)
    if output is None:
        raise ValueError(f"grouped FP8 {stage}: a tma_plan needs the output buffer it was prepared for; "
                         "output=None would allocate a different one")
    got = (x_fp8.data_ptr(), output.data_ptr(), int(x_fp8.shape[1]), int(output.shape[1]))
    problems = []
    if got != want:
        problems.append(f"(x, output, K, N) {got} != prepared {want}")
    if int(x_fp8.shape[0]) != plan.m or int(output.shape[0]) != plan.m:
        problems.append(f"rows {int(x_fp8.shape[0])}/{int(output.shape[0])} != prepared {plan.m}")
    if (seqlens.data_ptr(), cu_seqlens.data_ptr()) != (plan.seqlens_ptr, plan.cu_seqlens_ptr):
        problems.append("seqlens / cu_seqlens are not the tensors the plan was prepared from")
    if grouped_fp8_tile_m(num_seq_per_group_avg) != plan.tile_m:
        problems.append(f"TileM {grouped_fp8_tile_m(num_seq_per_group_avg)} (avg {num_seq_per_group_avg}) != "
                        f"prepared {plan.tile_m}")
    if problems:
        raise ValueError(f"grouped FP8 {stage}: tma_plan does not match this call: " + "; ".join(problems))


def grouped_fp8_blockwise_gemm(x_fp8, weight_3d, seqlens, cu_seqlens, x_scale, w_scale_3d,
                               num_seq_per_group_avg, output=None, tma_desc=None, tma_plan=None):
    """[M,K] fp8 x [E,N,K] fp8 -> [M,N] bf16; x_scale transposed [K/128, M_pad]; w_scale [E,N/128,pad4(K/128)]."""
    if tma_plan is not None:
        if tma_desc is not None:
            raise ValueError("grouped FP8 gemm: tma_plan and tma_desc are exclusive")
        _check_plan(tma_plan, "s3", x_fp8, output, seqlens, cu_seqlens, num_seq_per_group_avg)
    return _get_module().fp8_blockwise_grouped_gemm(x_fp8, weight_3d, seqlens, cu_seqlens, x_scale, w_scale_3d,
                                                    int(num_seq_per_group_avg), output)


def grouped_fp8_blockwise_s3(x_fp8, weight_3d, seqlens, cu_seqlens, x_scale, w_scale_3d, num_seq_per_group_avg,
                             output=None, tma_desc=None, tma_plan=None):
    """The down projection: the single grouped GEMM under its stage name."""
    return grouped_fp8_blockwise_gemm(x_fp8, weight_3d, seqlens, cu_seqlens, x_scale, w_scale_3d,
                                      num_seq_per_group_avg, output, tma_desc, tma_plan)


def grouped_fp8_blockwise_fused_s1(x_fp8, gate_weight_3d, up_weight_3d, seqlens, cu_seqlens, x_scale,
                                   gate_w_scale_3d, up_w_scale_3d, num_seq_per_group_avg, output=None,
                                   tma_desc=None, tma_plan=None):
    """bf16( silu(gate GEMM) * up GEMM ) in one launch."""
    if tma_plan is not None:
        if tma_desc is not None:
            raise ValueError("grouped FP8 s1: tma_plan and tma_desc are exclusive")
        _check_plan(tma_plan, "s1", x_fp8, output, seqlens, cu_seqlens, num_seq_per_group_avg)
    return _get_module().fp8_blockwise_fused_s1(x_fp8, gate_weight_3d, up_weight_3d, seqlens, cu_seqlens,
                                                x_scale, gate_w_scale_3d, up_w_scale_3d,
                                                int(num_seq_per_group_avg), output)
