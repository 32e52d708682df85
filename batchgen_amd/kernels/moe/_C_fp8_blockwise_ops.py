"""gfx950 implementation of the reference extension ``batchgen_kernels.moe._C_fp8_blockwise_ops``
(bindings: batchgen_kernels/src/moe/fp8_blockwise/fp8_blockwise_ops.cu:800-814)."""
from __future__ import annotations

import torch

from ..._lib import check, lib, ptr, stream
from .. import _checks as ck


def act_quant_3d(x, tokens_per_expert):
    """x [E, mtp, K] bf16 -> (y uint8 [E,mtp,K], scale fp32 [E,mtp,ceil(K/128)]); rows past
    tokens_per_expert[e] are left as allocated (fp8_blockwise_ops.cu:519-556)."""
    if x.dim() != 3:
        ck.fail("x must be 3D [E, mtp, K]")
    if x.dtype != torch.bfloat16:
        ck.fail("x must be BF16")
    if not x.is_contiguous():
        ck.fail("x must be contiguous")
    ck.gpu(x, "x")
    ck.cuda_tensor(x, tokens_per_expert, torch.int32, "tokens_per_expert")
    e, mtp, k = x.shape
    y = torch.empty((e, mtp, k), dtype=torch.uint8, device=x.device)
    scale = torch.empty((e, mtp, (k + 127) // 128), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_act_quant_3d(ptr(x), ptr(tokens_per_expert), e, mtp, k, ptr(y), ptr(scale), stream()))
    return y, scale


def act_quant_ragged(x, seqlens, cu_seqlens, y, scale, row_align):
    """Caller-owned y [max_rows,K] (uint8 or e4m3fn) and TRANSPOSED scale [ceil(K/128), max_rows]
    (fp8_blockwise_ops.cu:558-628)."""
    row_align = int(row_align)
    if row_align <= 0 or (row_align & (row_align - 1)) != 0:
        ck.fail(f"row_align must be a positive power of two, got {row_align}")
    ck.gpu(x, "x")
    for t, name in ((x, "x"), (seqlens, "seqlens"), (cu_seqlens, "cu_seqlens"), (y, "y"), (scale, "scale")):
        ck.cuda_tensor(x, t, None, name)
    if x.dim() != 2 or x.dtype != torch.bfloat16:
        ck.fail("x must be BF16 [max_rows, K]")
    max_rows, k = x.shape
    kb = (k + 127) // 128
    if seqlens.dtype != torch.int32 or seqlens.dim() != 1 or seqlens.numel() < 1:
        ck.fail("seqlens must be int32 [E]")
    e = seqlens.numel()
    if cu_seqlens.dtype != torch.int32 or cu_seqlens.dim() != 1 or cu_seqlens.numel() != e + 1:
        ck.fail("cu_seqlens must be int32 [E + 1]")
    if y.dtype not in ck.FP8_BYTES or tuple(y.shape) != (max_rows, k):
        ck.fail("y must be uint8 or float8_e4m3fn [max_rows, K]")
    if scale.dtype != torch.float32 or tuple(scale.shape) != (kb, max_rows):
        ck.fail(f"scale must be float32 [{kb}, {max_rows}]")
    with torch.cuda.device(x.device):
        check(lib().bgmoe_act_quant_ragged(ptr(x), ptr(seqlens), ptr(cu_seqlens), e, max_rows, k, ptr(y),
                                           ptr(scale), row_align, stream()))
    return y, scale


def silu_mul_3d(gate, up, tokens_per_expert):
    """bf16(silu(gate) * up) on [E, mtp, N] (fp8_blockwise_ops.cu:630-655)."""
    if gate.dim() != 3 or up.dim() != 3:
        ck.fail("Inputs must be 3D")
    if gate.shape != up.shape:
        ck.fail("Shape mismatch")
    if gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16:
        ck.fail("Must be BF16")
    ck.cuda_tensor(None, gate, None, "gate")
    ck.cuda_tensor(gate, up, None, "up")
    ck.cuda_tensor(gate, tokens_per_expert, torch.int32, "tokens_per_expert")
    e, mtp, n = gate.shape
    out = torch.empty_like(gate)
    with torch.cuda.device(gate.device):
        check(lib().bgmoe_silu_mul_3d(ptr(gate), ptr(up), ptr(tokens_per_expert), e, mtp, n, ptr(out), stream()))
    return out


def fused_silu_quant_3d(gate, up, tokens_per_expert):
    """-> (y uint8 [E,mtp,N], scale [E,mtp,ceil(N/128)]) (fp8_blockwise_ops.cu:657-684); same bytes
    as silu_mul_3d followed by act_quant_3d."""
    if gate.dim() != 3 or up.dim() != 3:
        ck.fail("Inputs must be 3D")
    if gate.shape != up.shape:
        ck.fail("Shape mismatch")
    ck.cuda_tensor(None, gate, torch.bfloat16, "gate")
    ck.cuda_tensor(gate, up, torch.bfloat16, "up")
    ck.cuda_tensor(gate, tokens_per_expert, torch.int32, "tokens_per_expert")
    e, mtp, n = gate.shape
    y = torch.empty((e, mtp, n), dtype=torch.uint8, device=gate.device)
    scale = torch.empty((e, mtp, (n + 127) // 128), dtype=torch.float32, device=gate.device)
    with torch.cuda.device(gate.device):
        check(lib().bgmoe_fused_silu_quant_3d(ptr(gate), ptr(up), ptr(tokens_per_expert), e, mtp, n, ptr(y),
                                              ptr(scale), stream()))
    return y, scale


def act_quant_rows(x, y=None, scale=None, scale_transposed=False):
    """Plain per-row quantiser (the 1-D ``act_quant`` of batchgen/quantization/act_quant.py:78-128):
    x [M,K] bf16 -> (y [M,K] e4m3fn, scale [M,K/128] or transposed [K/128,M])."""
    ck.cuda_tensor(None, x, torch.bfloat16, "x")
    if x.dim() != 2:
        ck.fail("x must be 2-D")
    m, k = x.shape
    kb = (k + 127) // 128
    if y is None:
        y = torch.empty((m, k), dtype=torch.float8_e4m3fn, device=x.device)
    if scale is None:
        scale = torch.empty((kb, m) if scale_transposed else (m, kb), dtype=torch.float32, device=x.device)
    ck.cuda_tensor(x, y, ck.FP8_BYTES, "y")
    ck.cuda_tensor(x, scale, torch.float32, "scale")
    srow, skb = (1, scale.size(1)) if scale_transposed else (scale.size(1), 1)
    with torch.cuda.device(x.device):
        check(lib().bgmoe_act_quant_rows(ptr(x), m, k, ptr(y), ptr(scale), srow, skb, stream()))
    return y, scale


_BAD_COUNT = {}


def deepep_ll_scale_repack_status(device) -> torch.Tensor:
    """int32 [1] on ``device``: becomes 1 when a ``deepep_ll_scale_repack`` call on that device met a receive
    count outside [0, S] (the reference traps the device there; here that expert is skipped and the flag is
    raised). Stays set until the caller zeroes it."""
    key = str(torch.device(device))
    t = _BAD_COUNT.get(key)
    if t is None:
        t = torch.zeros(1, dtype=torch.int32, device=device)
        _BAD_COUNT[key] = t
    return t


def deepep_ll_scale_repack(recv_scales, recv_count, out, span_align):
    """recv_scales: the exchange's [E, S, hidden/128] fp32 view (strides (KB*S, 1, S)) -> out [hidden/128, E*S],
    each expert's live span (rounded up to span_align) only (fp8_blockwise_ops.cu:744-797). Returns out."""
    ck.gpu(recv_scales, "recv_scales")
    ck.cuda_tensor(recv_scales, recv_count, None, "recv_count")
    ck.cuda_tensor(recv_scales, out, None, "out")
    if recv_scales.dim() != 3 or recv_scales.dtype != torch.float32:
        ck.fail("recv_scales must be float32 [E, S, hidden/128]")
    e, s_, kb = recv_scales.shape
    if e <= 0 or s_ <= 0 or kb <= 0:
        ck.fail("recv_scales must be non-empty")
    if tuple(recv_scales.stride()) != (kb * s_, 1, s_):
        ck.fail(f"recv_scales must be the (1, 2)-transposed view of a contiguous [E, hidden/128, S] block, i.e. "
                f"strides ({kb * s_}, 1, {s_}); got {tuple(recv_scales.stride())}")
    if recv_count.dim() != 1 or recv_count.dtype != torch.int32 or recv_count.shape[0] != e:
        ck.fail("recv_count must be int32 [E]")
    if out.dim() != 2 or out.dtype != torch.float32 or tuple(out.shape) != (kb, e * s_) or not out.is_contiguous():
        ck.fail(f"out must be float32 [hidden/128, E * S] = [{kb}, {e * s_}]")
    with torch.cuda.device(recv_scales.device):
        check(lib().bgmoe_deepep_ll_scale_repack(ptr(recv_scales), ptr(recv_count), ptr(out), e, kb, s_, int(span_align),
                                                 ptr(deepep_ll_scale_repack_status(recv_scales.device)), stream()))
    return out
