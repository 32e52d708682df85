"""gfx950 implementation of the MXFP4 ops of the reference extension
``batchgen_kernels.moe._C_marlin_grouped_gemm`` (Python callers:
batchgen/moe/marlin_grouped_moe.py:411-543).

The op names and positional argument orders are the reference's.  The pointer tables address weights
in THIS build's resident layout (tile-major by default, made by ``mxfp4_weight_repack`` from the
checkpoint layout packed ``[N, K/2]`` + scales ``[N, K/32]``); the reference's Marlin register layout is
an NVIDIA ``ldmatrix`` / ``mma.m16n8k16`` artefact and is not reproduced.  ``workspace``, ``n_tiles``
and ``max_m_tiles`` are accepted and ignored.  ``grouped_marlin_gemm_m16_s1_mxfp4_situ`` applies the
reference op's activation, SiTU with beta 4 / linear beta 25 on the bf16-rounded branches
(batchgen_kernels/src/moe/marlin_grouped_gemm.cu:243-256, :1055-1069); the stacked-weight form
``mxfp4_fused_s1`` takes ``activation="swiglu"`` (the benchmark's config) or ``"situ"``.  INT4 ops of that
extension are out of scope.
"""
from __future__ import annotations

import ctypes as C

import torch

from ..._lib import Mxfp4Weight, check, lib, ptr, stream
from .. import _checks as ck

_LAYOUT = {"row_major": 0, "tile_major": 1}
ACTIVATIONS = {"swiglu": 0, "situ": 1}      # BGMOE_ACT_SWIGLU, BGMOE_ACT_SITU


def mxfp4_weight_repack(w_packed, scales):
    """[G, N, K/2] uint8 + [G, N, K/32] uint8 (checkpoint layout) -> tile-major copies (one-time)."""
    ck.cuda_tensor(None, w_packed, torch.uint8, "w_packed")
    ck.cuda_tensor(w_packed, scales, torch.uint8, "scales")
    w = w_packed if w_packed.dim() == 3 else w_packed.unsqueeze(0)
    s = scales if scales.dim() == 3 else scales.unsqueeze(0)
    g, n, k2 = w.shape
    k = k2 * 2
    if tuple(s.shape) != (g, n, k // 32):
        ck.fail(f"scales must be [{g}, {n}, {k // 32}]")
    wo, so = torch.empty_like(w), torch.empty_like(s)
    with torch.cuda.device(w.device):
        check(lib().bgmoe_mxfp4_weight_repack(ptr(w), ptr(s), ptr(wo), ptr(so), g, n, k, stream()))
    return wo.view_as(w_packed), so.view_as(scales)


def _tbl(w_ptrs, s_ptrs, e, layout):
    for t, name in ((w_ptrs, "B_ptrs"), (s_ptrs, "scales_ptrs")):
        if t.dtype != torch.int64 or not t.is_cuda or t.numel() < e:
            ck.fail(f"{name} must be a CUDA int64 tensor with one device pointer per expert")
    return Mxfp4Weight(None, 0, ptr(w_ptrs), None, 0, ptr(s_ptrs), _LAYOUT[layout], 0)


def _counts(expert_starts, expert_counts, e):
    for t, name in ((expert_starts, "expert_starts"), (expert_counts, "expert_counts")):
        if t.dtype != torch.int32 or not t.is_cuda or t.numel() < e:
            ck.fail(f"{name} must be a CUDA int32 tensor with one entry per expert")


def grouped_marlin_gemm_m16_s1_mxfp4_situ(x, gate_B_ptrs, up_B_ptrs, C_ptrs, gate_scales_ptrs, up_scales_ptrs,
                                          expert_starts, expert_counts, E, N, K, workspace=None, n_tiles=None,
                                          max_m_tiles=None, weight_layout="tile_major"):
    """Fused gate + up + SiTU, bf16 result written through C_ptrs[e] (token t of expert e at
    C_ptrs[e] + t*N).  Zero-count experts are skipped on the device; the caller must not filter them."""
    ck.cuda_tensor(None, x, torch.bfloat16, "x")
    if x.dim() != 2 or x.size(1) != K:
        ck.fail(f"x must be BF16 [rows, {K}]")
    if N % 128 or K % 128:
        ck.fail(f"N ({N}) and K ({K}) must be multiples of 128")
    _counts(expert_starts, expert_counts, E)
    if C_ptrs.dtype != torch.int64 or not C_ptrs.is_cuda or C_ptrs.numel() < E:
        ck.fail("C_ptrs must be a CUDA int64 tensor with one device pointer per expert")
    wg = _tbl(gate_B_ptrs, gate_scales_ptrs, E, weight_layout)
    wu = _tbl(up_B_ptrs, up_scales_ptrs, E, weight_layout)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_mxfp4_fused_s1(ptr(x), C.byref(wg), C.byref(wu), ptr(expert_counts), ptr(expert_starts),
                                         int(E), x.size(0), int(N), int(K), None, ptr(C_ptrs), ACTIVATIONS["situ"],
                                         0, stream()))
    return None


def marlin_grouped_m16_mxfp4(A, B_ptrs, C_ptrs, scales_ptrs, expert_starts, expert_counts, num_experts, prob_n,
                             prob_k, workspace=None, num_matrices=1, n_tiles=None, max_m_tiles=None,
                             weight_layout="tile_major"):
    """Grouped W4A16 GEMM (the down projection), bf16 result through C_ptrs[e]."""
    ck.cuda_tensor(None, A, torch.bfloat16, "A")
    if A.dim() != 2 or A.size(1) != prob_k:
        ck.fail(f"A must be BF16 [rows, {prob_k}]")
    if prob_n % 128 or prob_k % 128:
        ck.fail(f"N ({prob_n}) and K ({prob_k}) must be multiples of 128")
    if num_matrices != 1:
        ck.fail("num_matrices != 1 is not built: call once per matrix")
    _counts(expert_starts, expert_counts, num_experts)
    w = _tbl(B_ptrs, scales_ptrs, num_experts, weight_layout)
    with torch.cuda.device(A.device):
        check(lib().bgmoe_mxfp4_grouped_gemm(ptr(A), C.byref(w), ptr(expert_counts), ptr(expert_starts),
                                             int(num_experts), A.size(0), int(prob_n), int(prob_k), None,
                                             ptr(C_ptrs), 0, stream()))
    return None


def _stack(wp, sc, layout):
    g, n, k2 = wp.shape
    return Mxfp4Weight(ptr(wp), n * k2, None, ptr(sc), sc.size(1) * sc.size(2), None, _LAYOUT[layout], 0)


def mxfp4_fused_s1(x, gate_p, gate_s, up_p, up_s, seqlens, cu_seqlens, output=None, weight_layout="row_major",
                   row_bound=0, activation="swiglu"):
    """Stacked-weight form: x [M,K] bf16; gate/up packed [G,N,K/2] + scales [G,N,K/32]; out [M,N] bf16,
    rows [cu[g], cu[g]+seqlens[g]) of group g."""
    if activation not in ACTIVATIONS:
        ck.fail(f"activation must be one of {sorted(ACTIVATIONS)}")
    ck.cuda_tensor(None, x, torch.bfloat16, "x")
    for t, name in ((gate_p, "gate_p"), (gate_s, "gate_s"), (up_p, "up_p"), (up_s, "up_s")):
        ck.cuda_tensor(x, t, torch.uint8, name)
    ck.cuda_tensor(x, seqlens, torch.int32, "seqlens")
    ck.cuda_tensor(x, cu_seqlens, torch.int32, "cu_seqlens")
    g, n, k2 = gate_p.shape
    m, k = x.shape
    if k != 2 * k2 or up_p.shape != gate_p.shape:
        ck.fail("x / gate / up shape mismatch")
    if output is None:
        output = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    wg, wu = _stack(gate_p, gate_s, weight_layout), _stack(up_p, up_s, weight_layout)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_mxfp4_fused_s1(ptr(x), C.byref(wg), C.byref(wu), ptr(seqlens), ptr(cu_seqlens), g, m, n, k,
                                         ptr(output), None, ACTIVATIONS[activation], int(row_bound), stream()))
    return output


def mxfp4_grouped_gemm(x, w_p, w_s, seqlens, cu_seqlens, output=None, weight_layout="row_major", row_bound=0):
    """Stacked-weight form of the single grouped GEMM."""
    ck.cuda_tensor(None, x, torch.bfloat16, "x")
    ck.cuda_tensor(x, w_p, torch.uint8, "w_p")
    ck.cuda_tensor(x, w_s, torch.uint8, "w_s")
    ck.cuda_tensor(x, seqlens, torch.int32, "seqlens")
    ck.cuda_tensor(x, cu_seqlens, torch.int32, "cu_seqlens")
    g, n, k2 = w_p.shape
    m, k = x.shape
    if k != 2 * k2:
        ck.fail("x / weight K mismatch")
    if output is None:
        output = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    w = _stack(w_p, w_s, weight_layout)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_mxfp4_grouped_gemm(ptr(x), C.byref(w), ptr(seqlens), ptr(cu_seqlens), g, m, n, k,
                                             ptr(output), None, int(row_bound), stream()))
    return output
