"""The two grouped GEMMs of the DeepSeek-V3 decode MoE on the masked 3-D layout, with the reference wrappers'
names and positional arguments (batchgen/models/deepseek/deepseekv3/grouped_gemm_kernel.py:253-361):

``fused_fp8_moe_stage_1_tma_wrapper``   bf16( silu(x Wg^T) * (x Wu^T) ), fp32 throughout, one rounding
                                        (batchgen_kernels/triton/w8a8_grouped_gemm_stage_1.py:1023-1026)
``fused_dequant_grouped_gemm_fp8_tma_wrapper``   bf16( x W^T )

Activations ``[E, M_max, K]`` e4m3fn with scales ``[E, M_max, K/128]`` (any strides), one row-major ``[N, K]``
weight and ``[N/128, K/128]`` scale tensor per expert, handed over as device pointer arrays, row counts in
``expert_token_counts``; rows at or beyond an expert's count are not written by the first wrapper.  The block
sizes, stage and warp counts are tuning knobs of the reference's Triton kernels: accepted and ignored.
"""
from __future__ import annotations

import ctypes as C

import torch

from .._lib import Fp8Act, Fp8Weight, check, lib, ptr, stream

_STARTS = {}


def _starts(e: int, m_max: int, device) -> torch.Tensor:
    key = (e, m_max, str(device))
    t = _STARTS.get(key)
    if t is None:
        t = (torch.arange(e + 1, dtype=torch.int32, device=device) * m_max).contiguous()
        _STARTS[key] = t
    return t


def _operands(x, x_scale, weight_list, w_ptrs, scale_list, s_ptrs, counts, num_local_experts, out, what):
    if x.dim() != 3 or x_scale.dim() != 3:
        raise RuntimeError(f"{what}: activations and their scales are [E, M_max, K] / [E, M_max, K/128]")
    e, m_max, k = x.shape
    n = int(weight_list[0].shape[0])
    if x.dtype != torch.float8_e4m3fn or not x.is_contiguous() or k % 128 or n % 128:
        raise RuntimeError(f"{what}: contiguous float8_e4m3fn activations with K ({k}) and N ({n}) multiples of 128")
    if tuple(x_scale.shape) != (e, m_max, k // 128) or x_scale.dtype != torch.float32:
        raise RuntimeError(f"{what}: activation scales must be f32 {(e, m_max, k // 128)}, got {tuple(x_scale.shape)}")
    if tuple(weight_list[0].shape) != (n, k) or not weight_list[0].is_contiguous() \
            or tuple(scale_list[0].shape) != (n // 128, k // 128):
        raise RuntimeError(f"{what}: each expert's weight is row-major [N, K] with scales [N/128, K/128]")
    if int(num_local_experts) != e:
        raise RuntimeError(f"{what}: num_local_experts ({num_local_experts}) must equal the leading extent {e}")
    for t, name in ((w_ptrs, "weight pointers"), (s_ptrs, "scale pointers")):
        if t.dtype != torch.int64 or not t.is_cuda or t.numel() < e or t.stride(0) != 1:
            raise RuntimeError(f"{what}: {name} must be a dense CUDA int64 tensor with one entry per expert")
    if counts.dtype != torch.int32 or counts.numel() < e:
        raise RuntimeError(f"{what}: expert_token_counts must be int32 [{e}]")
    if out is not None and (tuple(out.shape) != (e, m_max, n) or out.dtype != torch.bfloat16 or not out.is_contiguous()):
        raise RuntimeError(f"{what}: out must be contiguous bfloat16 {(e, m_max, n)}")
    act = Fp8Act(ptr(x), ptr(x_scale), x_scale.stride(1), x_scale.stride(2), x_scale.stride(0))
    w = Fp8Weight(None, 0, ptr(w_ptrs), None, 0, k // 128, ptr(s_ptrs), 0, 0)
    return e, m_max, k, n, act, w


def fused_fp8_moe_stage_1_tma_wrapper(hidden_states, hidden_states_scale, gate_weight_list, gate_ptrs_ptr,
                                      up_weight_list, up_ptrs_ptr, gate_scale_list, gate_scale_ptrs_ptr,
                                      up_scale_list, up_scale_ptrs_ptr, expert_token_counts, num_local_experts,
                                      gate_gemm_block_size=(64, 32, 128), scale_block_size=128, num_stages=3,
                                      num_warps=4, out=None):
    what = "fused_fp8_moe_stage_1"
    e, m_max, k, n, act, wg = _operands(hidden_states, hidden_states_scale, gate_weight_list, gate_ptrs_ptr,
                                        gate_scale_list, gate_scale_ptrs_ptr, expert_token_counts, num_local_experts,
                                        out, what)
    _, _, _, n2, _, wu = _operands(hidden_states, hidden_states_scale, up_weight_list, up_ptrs_ptr, up_scale_list,
                                   up_scale_ptrs_ptr, expert_token_counts, num_local_experts, out, what)
    if n2 != n:
        raise RuntimeError(f"{what}: gate and up weights differ in N ({n} / {n2})")
    if scale_block_size != 128:
        raise RuntimeError(f"{what}: the scale block is 128 in this build")
    output = out if out is not None else torch.empty((e, m_max, n), dtype=torch.bfloat16, device=hidden_states.device)
    with torch.cuda.device(hidden_states.device):
        check(lib().bgmoe_fp8_fused_s1(C.byref(act), C.byref(wg), C.byref(wu), ptr(expert_token_counts),
                                       ptr(_starts(e, m_max, hidden_states.device)), e, e * m_max, n, k, ptr(output),
                                       None, None, 0, 0, stream()))
    return output


def fused_dequant_grouped_gemm_fp8_tma_wrapper(lhs, lhs_scale, rhs_list, rhs_ptrs_ptr, rhs_scale_list,
                                               rhs_scale_ptrs_ptr, expert_token_counts, num_local_experts,
                                               gemm_block_size=(64, 32, 128), scale_block_size=(128, 128),
                                               num_stages=3, num_warps=4, out=None):
    what = "fused_dequant_grouped_gemm_fp8"
    e, m_max, k, n, act, w = _operands(lhs, lhs_scale, rhs_list, rhs_ptrs_ptr, rhs_scale_list, rhs_scale_ptrs_ptr,
                                       expert_token_counts, num_local_experts, out, what)
    if tuple(scale_block_size) != (128, 128):
        raise RuntimeError(f"{what}: the scale block is 128 x 128 in this build")
    # the reference allocates its own output zero-filled; rows beyond a count stay zero there and here
    output = out if out is not None else torch.zeros((e, m_max, n), dtype=torch.bfloat16, device=lhs.device)
    with torch.cuda.device(lhs.device):
        check(lib().bgmoe_fp8_grouped_gemm(C.byref(act), C.byref(w), ptr(expert_token_counts),
                                           ptr(_starts(e, m_max, lhs.device)), e, e * m_max, n, k, ptr(output), stream()))
    return output
