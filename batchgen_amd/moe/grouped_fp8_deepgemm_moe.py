"""The contiguous m-grouped FP8 GEMM of the streamed prefill, with the reference's names and argument lists
(batchgen/moe/grouped_fp8_deepgemm_moe.py:69-232): rows are described by a row -> group map instead of
(seqlens, cu_seqlens), activation scales are row-major ``[m, K/128]``, the weights one dense ``[G, N, K]`` stack
with exact ``[G, N/128, K/128]`` scales.

``m_grouped_fp8_gemm_nt_contiguous`` is the entry of the third-party ``deep_gemm`` package the reference calls
(:231); here it is this build's grouped FP8 GEMM behind a one-block kernel that turns the row map into segment
starts and lengths on the device.  DeepGEMM's accumulation order is not reproduced (the package is not in the
reference tree); the result is pinned against the fp32 dequantise-then-matmul of the live rows.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence

import torch
from torch import Tensor

from .._lib import Fp8Act, Fp8Weight, check, lib, ptr, stream

_QUANT_BLOCK = 128
_M_ALIGNMENT = 128          # what the reference's pinned deep_gemm build reports


def deepgemm_m_alignment() -> int:
    """Per-group row alignment of the contiguous layout (this build's kernels accept any start; the value is
    the reference backend's, so that layouts stay interchangeable)."""
    return _M_ALIGNMENT


def dense_group_view(members: Sequence[Tensor]) -> Tensor:
    """One ``[G, *shape]`` view over per-group tensors that lie back to back in one allocation; raises
    ``ValueError`` when they do not (different storage, shape, dtype, a gap, or not contiguous)."""
    if len(members) == 0:
        raise ValueError("dense_group_view needs at least one member")
    first = members[0]
    if not first.is_contiguous():
        raise ValueError("group member 0 is not contiguous")
    nbytes = first.numel() * first.element_size()
    storage = first.untyped_storage()
    for i, t in enumerate(members):
        if t.shape != first.shape or t.dtype != first.dtype or not t.is_contiguous():
            raise ValueError(f"group member {i}: shape, dtype and contiguity must match member 0")
        if t.untyped_storage().data_ptr() != storage.data_ptr():
            raise ValueError(f"group member {i} belongs to another allocation")
        off = t.data_ptr() - first.data_ptr()
        if off != i * nbytes:
            raise ValueError(f"group member {i} starts {off} B after member 0, a dense stack needs {i * nbytes} B")
    if first.data_ptr() + len(members) * nbytes > storage.data_ptr() + storage.nbytes():
        raise ValueError("the dense stack would run past its allocation")
    return first.as_strided((len(members), *first.shape), (first.numel(), *first.stride()))


def build_grouped_layout(seqlens: Tensor, cu_seqlens: Tensor, total_rows: int, alignment: Optional[int] = None,
                         validate: bool = True, group_ids: Optional[Tensor] = None) -> Tensor:
    """int32 ``[total_rows]``: row r -> ``group_ids[e]`` (or e) when ``cu_seqlens[e] <= r < cu_seqlens[e] +
    seqlens[e]``, else -1.  ``validate`` reads the starts back (a host synchronisation) to check the alignment
    and the extent; callers on a steady-state path pass ``validate=False``."""
    if alignment is None:
        alignment = deepgemm_m_alignment()
    if seqlens.ndim != 1 or cu_seqlens.ndim != 1:
        raise ValueError("seqlens and cu_seqlens must be 1-D")
    groups = seqlens.numel()
    if cu_seqlens.numel() != groups + 1:
        raise ValueError("cu_seqlens must have one more entry than seqlens")
    if group_ids is not None and (group_ids.ndim != 1 or group_ids.numel() != groups):
        raise ValueError("group_ids must map every expert segment")
    first = cu_seqlens[:groups].to(torch.int64)
    if validate:
        if bool((first % alignment != 0).any()):
            raise ValueError(f"a group start is not {alignment}-row aligned")
        if int(cu_seqlens[-1]) > total_rows:
            raise ValueError("cu_seqlens exceeds the reserved rows")
    dev = seqlens.device
    last = first + seqlens.to(torch.int64)                     # one past each segment's last live row
    rows = torch.arange(total_rows, dtype=torch.int64, device=dev)
    # the only segment that can own a row is the last one starting at or before it (starts never decrease, and of
    # several segments with one start all but the last are empty); the row is live if it lies before that
    # segment's end
    owner_c = (torch.searchsorted(first, rows, right=True) - 1).clamp_(min=0)
    inside = (rows >= first[owner_c]) & (rows < last[owner_c])
    ids = (group_ids.to(device=dev, dtype=torch.int32) if group_ids is not None
           else torch.arange(groups, dtype=torch.int32, device=dev))
    out = torch.full((total_rows,), -1, dtype=torch.int32, device=dev)
    out[inside] = ids[owner_c[inside]]
    return out


def _scale_rows_first(scale: Tensor, rows: int) -> Tensor:
    """fp32 ``[rows, K/128]`` from the engines' ``[K/128, rows]`` buffers (a small transposing copy)."""
    if scale.ndim != 2:
        raise ValueError("activation scale must be 2-D")
    if scale.shape[1] < rows:
        raise ValueError("activation scale has fewer rows than the batch")
    return scale[:, :rows].t().contiguous()


def m_grouped_fp8_gemm_nt_contiguous(lhs, rhs, d: Tensor, grouped_layout: Tensor) -> None:
    """``d[r] = dequant(a[r]) @ dequant(b[grouped_layout[r]]).T`` for rows with a group, bf16; rows mapped to -1
    are neither read nor written."""
    a, sfa = lhs
    b, sfb = rhs
    if a.dim() != 2 or b.dim() != 3 or d.dim() != 2:
        raise ValueError("contiguous grouped GEMM takes A [m, K], B [G, N, K] and D [m, N]")
    m, k = a.shape
    g, n, _ = b.shape
    kb = k // _QUANT_BLOCK
    if b.shape[2] != k or tuple(d.shape) != (m, n) or k % _QUANT_BLOCK or n % _QUANT_BLOCK:
        raise ValueError(f"shape mismatch: A {tuple(a.shape)}, B {tuple(b.shape)}, D {tuple(d.shape)} (K, N multiples "
                         f"of {_QUANT_BLOCK})")
    if a.dtype != torch.float8_e4m3fn or b.dtype != torch.float8_e4m3fn or d.dtype != torch.bfloat16:
        raise ValueError("contiguous grouped GEMM takes float8_e4m3fn operands and a bfloat16 output")
    if not (a.is_contiguous() and d.is_contiguous()) or b.stride() != (n * k, k, 1):
        raise ValueError("A and D must be contiguous and B a dense [G, N, K] stack (stride(0) == N*K)")
    if tuple(sfa.shape) != (m, kb) or sfa.dtype != torch.float32 or sfa.stride(-1) != 1:
        raise ValueError(f"SFA must be row-major f32 [m, K/{_QUANT_BLOCK}] = {(m, kb)}; got {tuple(sfa.shape)} strides "
                         f"{tuple(sfa.stride())}")
    if tuple(sfb.shape) != (g, n // _QUANT_BLOCK, kb) or sfb.dtype != torch.float32 or not sfb.is_contiguous():
        raise ValueError(f"SFB must be contiguous f32 [G, N/{_QUANT_BLOCK}, K/{_QUANT_BLOCK}]; got {tuple(sfb.shape)}")
    if tuple(grouped_layout.shape) != (m,) or grouped_layout.dtype != torch.int32:
        raise ValueError(f"grouped_layout must be int32 [{m}]")
    if not 1 <= g <= 1024:
        raise ValueError(f"between 1 and 1024 groups, got {g}")
    if m == 0:
        return
    seg = torch.empty(2 * g + 2, dtype=torch.int32, device=a.device)        # seqlens [g] | starts [g + 1]
    act = Fp8Act(ptr(a), ptr(sfa), sfa.stride(0), 1, 0)
    w = Fp8Weight(ptr(b), n * k, None, ptr(sfb), (n // _QUANT_BLOCK) * kb, kb, None, 0, 0)
    with torch.cuda.device(a.device):
        check(lib().bgmoe_layout_to_segments(ptr(grouped_layout), m, g, ptr(seg), seg.data_ptr() + 4 * g, None, stream()))
        check(lib().bgmoe_fp8_grouped_gemm(C.byref(act), C.byref(w), ptr(seg), seg.data_ptr() + 4 * g, g, m, n, k, ptr(d),
                                           stream()))


def grouped_fp8_deepgemm_gemm(x_fp8: Tensor, x_scale: Tensor, b: Tensor, sfb: Tensor, *, output: Tensor,
                              grouped_layout: Tensor, x_scale_rows_major: bool = False) -> Tensor:
    """One m-grouped contiguous GEMM over a dense weight stack into ``output`` (bf16 ``[m, N]``).  ``x_scale`` is the
    engines' ``[K/128, rows]`` buffer unless ``x_scale_rows_major`` says it already is ``[rows, K/128]``."""
    rows = output.shape[0]
    if grouped_layout.shape[0] != rows:
        raise ValueError("grouped_layout rows must match the output rows")
    if x_scale_rows_major:
        if x_scale.ndim != 2 or x_scale.stride(-1) != 1:
            raise ValueError(f"a rows-major activation scale must be 2-D with a contiguous last dim; got strides "
                             f"{tuple(x_scale.stride())}")
        if x_scale.shape[0] < rows:
            raise ValueError("rows-major activation scale has fewer rows than the batch")
        sfa = x_scale[:rows]
    else:
        sfa = _scale_rows_first(x_scale, rows)
    m_grouped_fp8_gemm_nt_contiguous((x_fp8[:rows], sfa), (b, sfb), output, grouped_layout)
    return output
