"""gfx950 implementation of the reference extension ``batchgen_kernels.moe._C_fp8_blockwise_gemm``
(bindings: batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_gemm.cu:1253-1299).

The TMA-descriptor / tile-table arguments of the reference ops are accepted and
ignored: the gfx950 kernels build their work list on the device from
``seqlens`` and need no descriptors.  ``num_seq_per_group_avg`` (the reference's
TileM hint) is accepted and ignored too: the kernels pick the row tiling per
group from the device-side count, so results never depend on the hint.
"""
from __future__ import annotations

import ctypes as C

import torch

from ..._lib import Fp8Act, Fp8Weight, check, lib, ptr, stream
from .. import _checks as ck

_MAX_GROUPS = 1024


def _check_inputs(x, weight, seqlens, cu_seqlens, x_scale, w_scale, output, wname="weight"):
    ck.gpu(x, "x")
    for t, name in ((x, "x"), (weight, wname), (seqlens, "seqlens"), (cu_seqlens, "cu_seqlens"),
                    (x_scale, "x_scale"), (w_scale, "w_scale")):
        ck.cuda_tensor(x, t, None, name)
    if x.dim() != 2 or x.dtype not in ck.FP8_BYTES:
        ck.fail("x must be float8_e4m3fn [m, K]")
    if weight.dim() != 3 or weight.dtype not in ck.FP8_BYTES:
        ck.fail(f"{wname} must be float8_e4m3fn [G, N, K]")
    if seqlens.dim() != 1 or seqlens.dtype != torch.int32:
        ck.fail("seqlens must be int32 [G]")
    if cu_seqlens.dim() != 1 or cu_seqlens.dtype != torch.int32:
        ck.fail("cu_seqlens must be int32 [G + 1]")
    if x_scale.dim() != 2 or x_scale.dtype != torch.float32:
        ck.fail("x_scale must be float32 [K/128, m_pad]")
    if w_scale.dim() != 3 or w_scale.dtype != torch.float32:
        ck.fail("w_scale must be float32 [G, N/128, pad4(K/128)]")
    m, k = x.shape
    g, n, k2 = weight.shape
    if not (0 < g <= _MAX_GROUPS):
        ck.fail(f"num_group must be in [1, {_MAX_GROUPS}], got {g}")
    if k2 != k:
        ck.fail("x and weight K mismatch")
    if k <= 0 or k % 128 or n <= 0 or n % 128:
        ck.fail(f"K ({k}) and N ({n}) must be positive multiples of 128")
    if seqlens.size(0) != g:
        ck.fail("seqlens and weight num_group mismatch")
    if cu_seqlens.size(0) != g + 1:
        ck.fail(f"cu_seqlens must have num_group + 1 entries, got {cu_seqlens.size(0)}")
    kb = k // 128
    if x_scale.size(0) != kb:
        ck.fail(f"x_scale must have K/128 = {kb} rows, got {x_scale.size(0)}")
    m_pad = x_scale.size(1)
    if not (m > 0 and 0 < m_pad <= m):
        ck.fail(f"x_scale columns (m_pad={m_pad}) must be in [1, x rows={m}]")
    if w_scale.size(0) != g or w_scale.size(1) != n // 128 or w_scale.size(2) < kb:
        ck.fail(f"w_scale must be [G, N/128, pad4(K/128)] = [{g}, {n // 128}, {(kb + 3) // 4 * 4}]")
    if output is not None:
        ck.cuda_tensor(x, output, torch.bfloat16, "output")
        if tuple(output.shape) != (m, n):
            ck.fail(f"output must be BF16 [m, N] = [{m}, {n}]")
    return m, n, k, m_pad, g


def _act(x, x_scale, m_pad):
    return Fp8Act(ptr(x), ptr(x_scale), 1, m_pad)


_LAYOUT = {"row_major": 0, "tile_major": 1}


def _stacked(weight, w_scale, layout="row_major"):
    g, n, k = weight.shape
    return Fp8Weight(ptr(weight), n * k, None, ptr(w_scale), w_scale.size(1) * w_scale.size(2),
                     w_scale.size(2), None, _LAYOUT[layout], 0)


def _table(proto_w, w_ptrs, proto_s, s_ptrs, layout="row_major"):
    return Fp8Weight(None, 0, ptr(w_ptrs), None, 0, proto_s.size(-1), ptr(s_ptrs), _LAYOUT[layout], 0)


def fp8_weight_repack(weight):
    """[G, N, K] row-major e4m3fn -> tile-major resident layout (one-time, at weight load).  No
    reference counterpart as an op; plays the role of its Marlin repack / TMA plan steps."""
    ck.cuda_tensor(None, weight, ck.FP8_BYTES, "weight")
    w = weight if weight.dim() == 3 else weight.unsqueeze(0)
    g, n, k = w.shape
    out = torch.empty_like(w)
    with torch.cuda.device(w.device):
        check(lib().bgmoe_fp8_weight_repack(ptr(w), ptr(out), g, n, k, stream()))
    return out.view_as(weight)


def fp8_blockwise_grouped_gemm(x, weight, seqlens, cu_seqlens, x_scale, w_scale, num_seq_per_group_avg,
                               output=None, tma_desc=None, tiles=None, cu_tiles=None, update_tma=True,
                               weight_layout="row_major", max_group_rows=0, workspace=None):
    """Y[r,n] = sum_kb (Xq[r,kb] . Wq[g,n,kb]) * xs[kb,r] * ws[g,n/128,kb] -> bf16 [m, N].
    ``max_group_rows`` / ``workspace`` (this build's additions): see ``streamk_workspace``."""
    m, n, k, m_pad, g = _check_inputs(x, weight, seqlens, cu_seqlens, x_scale, w_scale, output)
    if output is None:
        output = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    a, b = _act(x, x_scale, m_pad), _stacked(weight, w_scale, weight_layout)
    with torch.cuda.device(x.device):
        if workspace is not None:
            check(lib().bgmoe_fp8_grouped_gemm_balanced(C.byref(a), C.byref(b), ptr(seqlens), ptr(cu_seqlens), g, m, n,
                                                        k, ptr(output), int(max_group_rows), ptr(workspace),
                                                        workspace.numel() * workspace.element_size(), stream()))
        else:
            check(lib().bgmoe_fp8_grouped_gemm(C.byref(a), C.byref(b), ptr(seqlens), ptr(cu_seqlens), g, m, n, k,
                                               ptr(output), stream()))
    return output


def streamk_workspace(device):
    """A zeroed workspace for the balanced form of the grouped GEMMs (``workspace=`` of
    fp8_blockwise_grouped_gemm / fp8_blockwise_fused_s1_quant together with ``max_group_rows``, the caller's
    bound on the rows of any group).  Caller-owned; one per stream; calls leave its counters at zero."""
    with torch.cuda.device(device):
        check(lib().bgmoe_init())
        return torch.zeros(int(lib().bgmoe_fp8_streamk_workspace_bytes()), dtype=torch.uint8, device=device)


def fp8_blockwise_fused_s1(x, gate_weight, up_weight, seqlens, cu_seqlens, x_scale, gate_w_scale, up_w_scale,
                           num_seq_per_group_avg, output=None, tma_desc=None, tiles=None, cu_tiles=None,
                           update_tma=True, weight_layout="row_major"):
    """bf16( silu(X Wg^T) * (X Wu^T) ) -> [m, N]."""
    m, n, k, m_pad, g = _check_inputs(x, gate_weight, seqlens, cu_seqlens, x_scale, gate_w_scale, output,
                                      "gate_weight")
    _check_inputs(x, up_weight, seqlens, cu_seqlens, x_scale, up_w_scale, output, "up_weight")
    if up_weight.shape != gate_weight.shape:
        ck.fail("gate_weight and up_weight shape mismatch")
    if output is None:
        output = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    a = _act(x, x_scale, m_pad)
    wg, wu = _stacked(gate_weight, gate_w_scale, weight_layout), _stacked(up_weight, up_w_scale, weight_layout)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_fp8_fused_s1(C.byref(a), C.byref(wg), C.byref(wu), ptr(seqlens), ptr(cu_seqlens), g, m,
                                       n, k, ptr(output), None, None, 0, 0, stream()))
    return output


def fp8_blockwise_fused_s1_quant(x, gate_weight, up_weight, seqlens, cu_seqlens, x_scale, gate_w_scale,
                                 up_w_scale, out_q, out_scale_t, weight_layout="row_major", max_group_rows=0,
                                 workspace=None):
    """Fused S1 with the requant in the epilogue: out_q [m,N] bytes + TRANSPOSED scale [N/128, m].
    Same bytes as fp8_blockwise_fused_s1 followed by act_quant_ragged on the live rows."""
    m, n, k, m_pad, g = _check_inputs(x, gate_weight, seqlens, cu_seqlens, x_scale, gate_w_scale, None,
                                      "gate_weight")
    _check_inputs(x, up_weight, seqlens, cu_seqlens, x_scale, up_w_scale, None, "up_weight")
    ck.cuda_tensor(x, out_q, ck.FP8_BYTES, "out_q")
    ck.cuda_tensor(x, out_scale_t, torch.float32, "out_scale_t")
    if tuple(out_q.shape) != (m, n) or tuple(out_scale_t.shape) != (n // 128, m):
        ck.fail(f"out_q must be [{m}, {n}] and out_scale_t [{n // 128}, {m}]")
    a = _act(x, x_scale, m_pad)
    wg, wu = _stacked(gate_weight, gate_w_scale, weight_layout), _stacked(up_weight, up_w_scale, weight_layout)
    with torch.cuda.device(x.device):
        if workspace is not None:
            check(lib().bgmoe_fp8_fused_s1_balanced(C.byref(a), C.byref(wg), C.byref(wu), ptr(seqlens), ptr(cu_seqlens),
                                                    g, m, n, k, None, ptr(out_q), ptr(out_scale_t), 1, m,
                                                    int(max_group_rows), ptr(workspace),
                                                    workspace.numel() * workspace.element_size(), stream()))
        else:
            check(lib().bgmoe_fp8_fused_s1(C.byref(a), C.byref(wg), C.byref(wu), ptr(seqlens), ptr(cu_seqlens), g, m,
                                           n, k, None, ptr(out_q), ptr(out_scale_t), 1, m, stream()))
    return out_q, out_scale_t


def _check_ptrs(t, g, name):
    if t.dtype != torch.int64 or t.dim() != 1 or t.numel() != g or not t.is_cuda:
        ck.fail(f"{name} must be a CUDA int64 [{g}] tensor of device pointers")


def fp8_blockwise_grouped_gemm_ptrs(x, weight_prototype, weight_ptrs, seqlens, cu_seqlens, x_scale,
                                    w_scale_prototype, w_scale_ptrs, num_seq_per_group_avg, output=None,
                                    tma_desc=None, tiles=None, cu_tiles=None):
    """Pointer-array form: group g's weight [N,K] at weight_ptrs[g], its scales [N/128, pad4(K/128)] at
    w_scale_ptrs[g]; the prototypes only carry shape and dtype (fp8_blockwise_gemm.cu:617-660)."""
    g = seqlens.numel()
    _check_ptrs(weight_ptrs, g, "weight_ptrs")
    _check_ptrs(w_scale_ptrs, g, "w_scale_ptrs")
    n, k = weight_prototype.shape[-2:]
    m = x.size(0)
    if x.size(1) != k or k % 128 or n % 128:
        ck.fail("x / weight_prototype K, N mismatch or not multiples of 128")
    if output is None:
        output = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    a = _act(x, x_scale, x_scale.size(1))
    b = _table(weight_prototype, weight_ptrs, w_scale_prototype, w_scale_ptrs)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_fp8_grouped_gemm(C.byref(a), C.byref(b), ptr(seqlens), ptr(cu_seqlens), g, m, int(n),
                                           int(k), ptr(output), stream()))
    return output


def fp8_blockwise_fused_s1_ptrs(x, gate_weight_prototype, gate_weight_ptrs, up_weight_prototype, up_weight_ptrs,
                                seqlens, cu_seqlens, x_scale, gate_w_scale_prototype, gate_w_scale_ptrs,
                                up_w_scale_prototype, up_w_scale_ptrs, num_seq_per_group_avg, output=None,
                                tma_desc=None, tiles=None, cu_tiles=None):
    g = seqlens.numel()
    for t, name in ((gate_weight_ptrs, "gate_weight_ptrs"), (up_weight_ptrs, "up_weight_ptrs"),
                    (gate_w_scale_ptrs, "gate_w_scale_ptrs"), (up_w_scale_ptrs, "up_w_scale_ptrs")):
        _check_ptrs(t, g, name)
    n, k = gate_weight_prototype.shape[-2:]
    m = x.size(0)
    if x.size(1) != k or k % 128 or n % 128:
        ck.fail("x / gate_weight_prototype K, N mismatch or not multiples of 128")
    if output is None:
        output = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    a = _act(x, x_scale, x_scale.size(1))
    wg = _table(gate_weight_prototype, gate_weight_ptrs, gate_w_scale_prototype, gate_w_scale_ptrs)
    wu = _table(up_weight_prototype, up_weight_ptrs, up_w_scale_prototype, up_w_scale_ptrs)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_fp8_fused_s1(C.byref(a), C.byref(wg), C.byref(wu), ptr(seqlens), ptr(cu_seqlens), g, m,
                                       int(n), int(k), ptr(output), None, None, 0, 0, stream()))
    return output


def fp8_blockwise_prepare_s1_s3_tma(s1_x, s1_output, s3_x, s3_output, seqlens, cu_seqlens, num_seq_per_group_avg,
                                    s1_tma_desc, s3_tma_desc, tiles, cu_tiles):
    """The reference writes TMA descriptors and a tile table here (fp8_blockwise_gemm.cu:1100-1190).
    gfx950 needs neither; the call only validates its arguments so callers stay unchanged."""
    for t, name in ((s1_x, "s1_x"), (s1_output, "s1_output"), (s3_x, "s3_x"), (s3_output, "s3_output"),
                    (seqlens, "seqlens"), (cu_seqlens, "cu_seqlens")):
        ck.gpu(t, name)
    if s1_x.size(0) != s3_x.size(0) or s1_output.size(0) != s1_x.size(0):
        ck.fail("S1 and S3 must share one row space")
    return None
