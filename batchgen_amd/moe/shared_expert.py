"""The dense FP8 expert (shared expert, dense-layer MLP) as the reference's model code runs it
(batchgen/models/glm/glm5/wrappers.py:251-463, batchgen/attention/mla/fa3_backend.py:525-590):

    fused   : quantise(x) -> ONE GEMM over the stacked [gate; up] weight -> SiLU(gate) * up + quantise -> down GEMM
    unfused : quantise(x) once -> gate GEMM, up GEMM -> bf16 SiLU * up -> quantise -> down GEMM

``fp8_gemm_nt`` stands where the reference calls ``deep_gemm.fp8_gemm_nt``: here it is this build's grouped FP8
GEMM run with one group, so gate and up columns of the fused product are the separate products bit for bit (same
K order, same block scales), and the two chains give identical bytes.  Inside ``Fp8MoELayer`` the shared expert
does not go through this module: it runs as one more group of the routed launch.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from .._lib import Fp8Act, Fp8Weight, check, lib, ptr, stream
from ..kernels.triton.fp8_quantize import (per_token_blocked_quantize_bf16_to_fp8_1d,
                                           silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d)
from ..quantization.act_quant import act_quant

FP8_DTYPE = torch.float8_e4m3fn
BLOCK = 128
DENSE_MAX_ROWS = 64        # up to here the K-split dense kernel for any N (measured cross-overs against the
DENSE_MAX_ROWS_NARROW = 512  # grouped GEMM with one group), up to here for N <= DENSE_NARROW_N
DENSE_NARROW_N = 8192

_ROWS = {}


def _one_group(m: int, device):
    """Device pointers to cu_seqlens = [0, m] and seqlens = [m] inside one table per device
    ([0, 0, 0, 1, 0, 2, ...]; grown by doubling, so steady-state calls allocate nothing)."""
    key = str(device)
    t = _ROWS.get(key)
    if t is None or t.numel() < 2 * (m + 1):
        size = 1 << max(12, (m + 1).bit_length())
        t = torch.stack([torch.zeros(size, dtype=torch.int32), torch.arange(size, dtype=torch.int32)], dim=1)
        t = t.reshape(-1).to(device)
        _ROWS[key] = t
    base = t.data_ptr() + 8 * m
    return base, base + 4


def _workspace(nbytes: int, device):
    """Split-K partial sums: per device and stream, never freed once handed out (kernels/_workspace.py)."""
    from ..kernels._workspace import dense_gemm_workspace
    return dense_gemm_workspace(device, nbytes)


def fp8_gemm_nt(lhs, rhs, d: torch.Tensor, weight_layout: str = "row_major") -> None:
    """``d = dequant(a) @ dequant(b).T`` (bf16).  a [M, K] e4m3fn with scales [M, K/128] fp32, row-major or
    MN-major (any strides); b [N, K] with block scales [N/128, K/128].  ``weight_layout="tile_major"`` (no reference
    counterpart) takes ``b`` in the resident layout of ``fp8_weight_repack``."""
    a, sa = lhs
    b, sb = rhs
    if a.dim() != 2 or b.dim() != 2 or d.dim() != 2:
        raise RuntimeError("fp8_gemm_nt takes A [M, K], B [N, K] and D [M, N]")
    m, k = a.shape
    n = b.shape[0]
    if b.shape[1] != k or tuple(d.shape) != (m, n):
        raise RuntimeError(f"fp8_gemm_nt shape mismatch: A {tuple(a.shape)}, B {tuple(b.shape)}, D {tuple(d.shape)}")
    if a.dtype != FP8_DTYPE or b.dtype != FP8_DTYPE or d.dtype != torch.bfloat16:
        raise RuntimeError(f"fp8_gemm_nt takes {FP8_DTYPE} operands and a bfloat16 output")
    if k % BLOCK or n % BLOCK:
        raise RuntimeError(f"fp8_gemm_nt is block-scaled: K {k} and N {n} must be multiples of {BLOCK}")
    if not (a.is_contiguous() and b.is_contiguous() and d.is_contiguous()):
        raise RuntimeError("fp8_gemm_nt takes contiguous A, B and D")
    kb = k // BLOCK
    if tuple(sa.shape) != (m, kb) or sa.dtype != torch.float32:
        raise RuntimeError(f"A scales must be f32 [M, K // {BLOCK}] = {(m, kb)}; got {tuple(sa.shape)} {sa.dtype}")
    if tuple(sb.shape) != (n // BLOCK, kb) or sb.dtype != torch.float32 or not sb.is_contiguous():
        raise RuntimeError(f"B scales must be contiguous f32 [N // {BLOCK}, K // {BLOCK}]; got {tuple(sb.shape)} "
                           f"{sb.dtype}")
    if m == 0:
        return
    layout = {"row_major": 0, "tile_major": 1}[weight_layout]
    act = Fp8Act(ptr(a), ptr(sa), sa.stride(0), sa.stride(1), 0)
    with torch.cuda.device(a.device):
        if m <= DENSE_MAX_ROWS or (m <= DENSE_MAX_ROWS_NARROW and n <= DENSE_NARROW_N):
            need = lib().bgmoe_fp8_dense_gemm_workspace(m, n, k, layout)
            ws = _workspace(need, a.device)
            check(lib().bgmoe_fp8_dense_gemm(C.byref(act), ptr(b), ptr(sb), kb, layout, m, n, k, ptr(d), ptr(ws), need,
                                             stream()))
            return
        w = Fp8Weight(ptr(b), n * k, None, ptr(sb), (n // BLOCK) * kb, kb, None, layout, 0)
        cu, seqlens = _one_group(m, a.device)
        check(lib().bgmoe_fp8_grouped_gemm(C.byref(act), C.byref(w), seqlens, cu, 1, m, n, k, ptr(d), stream()))


def w8a16_gemm_act_quant(activation_bf16: torch.Tensor):
    """The (fp8, scale) pair ``w8a16_gemm`` would make of ``activation_bf16`` itself: quantise once, feed several
    GEMMs (fa3_backend.py:498-522)."""
    return act_quant(activation_bf16.view(-1, activation_bf16.size(-1)))


def w8a16_gemm(weight_data_fp8: torch.Tensor, weight_scale_inv_fp32: torch.Tensor, activation_bf16: torch.Tensor,
               x_fp8=None) -> torch.Tensor:
    """FP8 weight [n, k] x FP8-quantised activation ([m, k] or [g, l, k] bf16) -> bf16 (w8a8 despite the name,
    as in the reference)."""
    assert weight_data_fp8.dim() == 2
    assert activation_bf16.dim() in (2, 3)
    x = activation_bf16.view(-1, activation_bf16.size(-1))
    m, k = x.shape
    n = weight_data_fp8.size(0)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    if x_fp8 is None:
        x_fp8 = act_quant(x)
    else:
        q, s = x_fp8
        if (q.dtype != FP8_DTYPE or tuple(q.shape) != (m, k) or s.dtype != torch.float32
                or tuple(s.shape) != (m, (k + BLOCK - 1) // BLOCK) or q.device != x.device or s.device != x.device):
            raise ValueError(f"x_fp8 must be the act_quant pair of the activation: fp8 ({m}, {k}) and f32 "
                             f"({m}, {(k + BLOCK - 1) // BLOCK}) on {x.device}")
    fp8_gemm_nt(x_fp8, (weight_data_fp8, weight_scale_inv_fp32), out)
    return out.view(*activation_bf16.shape[:-1], n) if activation_bf16.dim() == 3 else out


class Fp8DenseExpert:
    """gate / up / down FP8 weights of one dense expert with the reference wrapper's two forward chains.  ``gate``
    and ``up`` must be the row halves of ONE contiguous ``gate_up`` [2I, K] allocation for the fused chain
    (the loader stores them that way: `weight_loader.py`)."""

    def __init__(self, gate, gate_scale, up, up_scale, down, down_scale, gate_up: Optional[torch.Tensor] = None,
                 layer_idx: int = 0):
        self.layer_idx = layer_idx
        self.gate, self.gate_scale = gate, gate_scale
        self.up, self.up_scale = up, up_scale
        self.down, self.down_scale = down, down_scale
        self.gate_up = None
        self.gate_up_scale = None
        if gate_up is not None:
            self.bind_fused_gate_up(gate_up)

    def bind_fused_gate_up(self, gate_up: torch.Tensor) -> None:
        """Every assumption that makes ``[gate; up] @ x`` equal to the two products is checked once, here."""
        who = f"Layer {self.layer_idx}"
        inter, hidden = self.gate.shape
        if (gate_up.dim() != 2 or tuple(gate_up.shape) != (2 * inter, hidden) or tuple(self.up.shape) != (inter, hidden)
                or not gate_up.is_contiguous() or gate_up.dtype != FP8_DTYPE):
            raise RuntimeError(f"{who}: the fused weight must be a contiguous {FP8_DTYPE} [2I, K] = "
                               f"{(2 * inter, hidden)} over gate {tuple(self.gate.shape)} and up "
                               f"{tuple(self.up.shape)}; got {tuple(gate_up.shape)} {gate_up.dtype}")
        if self.gate.data_ptr() != gate_up.data_ptr() or self.up.data_ptr() != gate_up[inter:].data_ptr():
            raise RuntimeError(f"{who}: gate and up are not the row halves of the fused allocation; the fused GEMM "
                               "would read other bytes than the per-projection GEMMs")
        if inter % BLOCK or hidden % BLOCK:
            raise RuntimeError(f"{who}: I={inter} and K={hidden} must be multiples of the {BLOCK}-wide scale block (a "
                               "block must not straddle gate and up)")
        want = (inter // BLOCK, hidden // BLOCK)
        for name, s in (("gate", self.gate_scale), ("up", self.up_scale)):
            if s is None or tuple(s.shape) != want or s.dtype != torch.float32 or s.device != gate_up.device:
                raise RuntimeError(f"{who}: {name} block scales must be fp32 {want} on {gate_up.device}; got "
                                   f"{None if s is None else (tuple(s.shape), s.dtype, s.device)}")
        self.gate_up = gate_up
        self.gate_up_scale = torch.cat([self.gate_scale, self.up_scale], dim=0).contiguous()

    def forward(self, hidden_states, out=None, x_fp8=None, x_scale=None):
        if self.gate_up is not None:
            return self.forward_fused_gate_up(hidden_states, out, x_fp8, x_scale)
        if out is not None:
            raise ValueError(f"Layer {self.layer_idx}: out= requires the fused gate/up binding")
        if x_fp8 is not None or x_scale is not None:
            raise ValueError(f"Layer {self.layer_idx}: x_fp8/x_scale require the fused gate/up binding")
        return self.forward_unfused(hidden_states)

    __call__ = forward

    def forward_unfused(self, hidden_states):
        x_fp8 = w8a16_gemm_act_quant(hidden_states)
        gate = w8a16_gemm(self.gate, self.gate_scale, hidden_states, x_fp8=x_fp8)
        up = w8a16_gemm(self.up, self.up_scale, hidden_states, x_fp8=x_fp8)
        return w8a16_gemm(self.down, self.down_scale, torch.nn.functional.silu(gate) * up)

    def _gate_up_activation_from_partials(self, x_fp8, x_scale, rows, hidden):
        """When the [gate; up] GEMM runs in its block-split form, the activation kernel adds the K-slices itself
        (same bits as GEMM -> bf16 -> activation, one launch and one round trip less); None when the GEMM takes
        another form."""
        two_i = self.gate_up.shape[0]
        if not (rows <= DENSE_MAX_ROWS or (rows <= DENSE_MAX_ROWS_NARROW and two_i <= DENSE_NARROW_N)):
            return None
        need = lib().bgmoe_fp8_dense_gemm_workspace(rows, two_i, hidden, 0)
        if need <= 0 or x_fp8.dtype != FP8_DTYPE or not x_fp8.is_contiguous():
            return None
        inter = two_i // 2
        ws = _workspace(need, x_fp8.device)
        act = Fp8Act(ptr(x_fp8), ptr(x_scale), x_scale.stride(0), x_scale.stride(1), 0)
        slices = C.c_int32(0)
        h_fp8 = torch.empty((rows, inter), device=x_fp8.device, dtype=FP8_DTYPE)
        h_scale = torch.empty((inter // BLOCK, (rows + 3) // 4 * 4), device=x_fp8.device,
                              dtype=torch.float32).transpose(0, 1)[:rows, :]
        with torch.cuda.device(x_fp8.device):
            check(lib().bgmoe_fp8_dense_gemm_partials(C.byref(act), ptr(self.gate_up), ptr(self.gate_up_scale),
                                                      hidden // BLOCK, 0, rows, two_i, hidden, ptr(ws), need,
                                                      C.byref(slices), stream()))
            check(lib().bgmoe_silu_mul_group_quant_partials(ptr(ws), slices.value, rows * two_i, rows, inter, 0,
                                                            ptr(h_fp8), inter, ptr(h_scale), h_scale.stride(0),
                                                            h_scale.stride(1), stream()))
        return h_fp8, h_scale

    def deepgemm_forward(self, x, scale=None):
        """``DeepseekV3MLP.deepgemm_forward(x, scale)`` (batchgen/models/deepseek/deepseekv3/
        modeling_deepseek_v3.py:630-637): the per-projection chain, block scales optionally taken from a dict with
        the checkpoint's ``{gate,up,down}_proj.weight_scale_inv`` keys."""
        if scale is None:
            return self.forward_unfused(x)
        x_fp8 = w8a16_gemm_act_quant(x)
        up = w8a16_gemm(self.up, scale["up_proj.weight_scale_inv"], x, x_fp8=x_fp8)
        gate = w8a16_gemm(self.gate, scale["gate_proj.weight_scale_inv"], x, x_fp8=x_fp8)
        return w8a16_gemm(self.down, scale["down_proj.weight_scale_inv"], torch.nn.functional.silu(gate) * up)

    def forward_fused_gate_up(self, hidden_states, out=None, x_fp8=None, x_scale=None):
        who = f"Layer {self.layer_idx}"
        if hidden_states.dtype != torch.bfloat16:
            raise TypeError(f"{who}: fused shared expert takes bf16 input, got {hidden_states.dtype}")
        x = hidden_states.view(-1, hidden_states.size(-1))
        rows, hidden = x.shape
        n_out = self.down.shape[0]
        if out is None:
            out = torch.empty((rows, n_out), dtype=torch.bfloat16, device=x.device)
        elif (tuple(out.shape) != (rows, n_out) or out.dtype != torch.bfloat16 or not out.is_contiguous()
              or out.device != x.device):
            raise ValueError(f"{who}: shared-expert out must be a contiguous bf16 [{rows}, {n_out}] tensor on "
                             f"{x.device}, got {tuple(out.shape)}/{out.dtype}/contiguous={out.is_contiguous()}")
        shaped = (lambda t: t) if hidden_states.dim() == 2 else (lambda t: t.view(*hidden_states.shape[:-1], n_out))
        if rows == 0:
            return shaped(out)
        if x_fp8 is None and x_scale is None:
            x_fp8, x_scale = per_token_blocked_quantize_bf16_to_fp8_1d(x, scale_tma_aligned=True)
        elif x_fp8 is None or x_scale is None:
            raise ValueError(f"{who}: x_fp8 and x_scale must be given together, got "
                             f"{'x_scale' if x_fp8 is None else 'x_fp8'} alone")
        else:
            blocks, aligned = hidden // BLOCK, (rows + 3) // 4 * 4
            if x_fp8.dtype != FP8_DTYPE:
                raise TypeError(f"{who}: x_fp8 must be float8_e4m3fn, got {x_fp8.dtype}")
            if tuple(x_fp8.shape) != (rows, hidden):
                raise ValueError(f"{who}: x_fp8 must be ({rows}, {hidden}), got {tuple(x_fp8.shape)}")
            if x_scale.dtype != torch.float32:
                raise TypeError(f"{who}: x_scale must be fp32, got {x_scale.dtype}")
            if tuple(x_scale.shape) != (rows, blocks):
                raise ValueError(f"{who}: x_scale must be ({rows}, {blocks}), got {tuple(x_scale.shape)}")
            if x_scale.stride() != (1, aligned):
                raise ValueError(f"{who}: x_scale must carry the scale_tma_aligned MN-major layout (stride "
                                 f"(1, {aligned})), got {x_scale.stride()}")
        h = self._gate_up_activation_from_partials(x_fp8, x_scale, rows, hidden)
        if h is None:
            gate_up = torch.empty((rows, self.gate_up.shape[0]), dtype=torch.bfloat16, device=x.device)
            fp8_gemm_nt((x_fp8, x_scale), (self.gate_up, self.gate_up_scale), gate_up)
            h = silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d(gate_up, scale_tma_aligned=True)
        h_fp8, h_scale = h
        fp8_gemm_nt((h_fp8, h_scale), (self.down, self.down_scale), out)
        return shaped(out)
