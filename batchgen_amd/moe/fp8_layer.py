"""FP8 MoE layer forward on one GPU's share of the experts.

Host-side counterpart of the reference's layer glue: the abstract template
``MoEBase`` (batchgen/moe/moe_base.py:188-264: gate -> expert compute -> shared
expert) with the buffer discipline of ``Glm5MoE3DBuffers``
(batchgen/models/glm/glm5/model.py:1241-1428): every buffer is allocated once
at construction, the forward allocates nothing and never synchronises.
The collectives of the reference template are out of scope (one GPU).
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from .. import _lib
from .._lib import Fp8Weight, check, lib, ptr, stream
from ..workloads import MoEConfig
from .dispatch_scatter_3d import ragged_row_capacity

vp, i32, i64, f32, sz = _lib.vp, _lib.i32, _lib.i64, _lib.f32, _lib.sz


class LayerStruct(C.Structure):
    """bgmoe_moe_fp8_layer (include/bgmoe.h)"""
    _fields_ = [
        ("n", i32), ("h", i32), ("inter", i32), ("e_total", i32), ("e_local", i32), ("expert_start", i32),
        ("top_k", i32), ("n_group", i32), ("topk_group", i32), ("rsf", f32),
        ("layout", i32), ("max_tokens", i32), ("row_align", i32),
        ("has_shared", i32), ("shared_folded", i32), ("shared_inter", i32), ("shared_mode", i32),
        ("cap_rows", i64),
        ("x", vp), ("logits", vp), ("bias", vp),
        ("gate", Fp8Weight), ("up", Fp8Weight), ("down", Fp8Weight),
        ("sh_gate", Fp8Weight), ("sh_up", Fp8Weight), ("sh_down", Fp8Weight),
        ("topk_ids", vp), ("topk_weights", vp), ("expert_counts", vp), ("cu_seqlens", vp), ("topk_pos", vp),
        ("xq", vp), ("xs", vp), ("hq", vp), ("hs", vp), ("shq", vp), ("shs", vp), ("y", vp),
        ("workspace", vp), ("workspace_bytes", sz), ("out", vp),
        ("x_fp8", vp), ("x_scale", vp), ("x_scale_row_stride", i64), ("x_scale_kb_stride", i64),
        ("router_weight", vp), ("router_hidden", vp), ("router_workspace", vp), ("router_workspace_bytes", sz),
        ("routes_given", i32),
        ("gemm_workspace", vp), ("gemm_workspace_bytes", sz),
    ]


_lib.register("bgmoe_moe_fp8_layer_forward", i32, [C.POINTER(LayerStruct), vp])
ROUTES_GIVEN, ROUTES_GIVEN_DISTINCT = 1, 2          # bgmoe_moe_fp8_layer.routes_given (include/bgmoe.h)


W_ROW_MAJOR, W_TILE_MAJOR = 0, 1
STREAMK_MAX_TOKENS = 256      # no group of such a batch exceeds the weight-streaming kernel's row limit


def _check_stack(q: torch.Tensor, s: torch.Tensor):
    """Stacks may be views (one half of a fused gate/up block, scales with a padded trailing axis): each
    expert's [N, K] bytes must be dense and its scale rows unit-stride."""
    e, n, k = q.shape
    if q.stride(2) != 1 or q.stride(1) != k or s.stride(2) != 1:
        raise RuntimeError(f"expert weights must be dense [N, K] per expert with unit-stride scale rows; got "
                           f"strides {q.stride()} / {s.stride()}")


def _stack_desc(q: torch.Tensor, s: torch.Tensor, layout: int = W_ROW_MAJOR) -> Fp8Weight:
    _check_stack(q, s)
    return Fp8Weight(ptr(q), q.stride(0), None, ptr(s), s.stride(0), s.stride(1), None, layout, 0)


def repack_tile_major(q: torch.Tensor) -> torch.Tensor:
    """[..., N, K] e4m3fn row-major -> the same bytes in the tile-major resident layout (see
    include/bgmoe.h).  One-time, at weight load."""
    if q.dim() == 2:
        q = q.unsqueeze(0)
    e, n, k = q.shape
    out = torch.empty((e, n, k), dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        if q.is_contiguous():
            check(lib().bgmoe_fp8_weight_repack(ptr(q), ptr(out), e, n, k, stream()))
        else:                                        # a strided stack of dense experts: one expert at a time
            if q.stride(2) != 1 or q.stride(1) != k:
                raise RuntimeError("each expert's weight must be a dense [N, K] block")
            for i in range(e):
                check(lib().bgmoe_fp8_weight_repack(ptr(q[i]), ptr(out[i]), 1, n, k, stream()))
    return out


class Fp8MoELayer:
    """forward(hidden_states [N,H] bf16, router_logits [N,E] fp32) -> [N,H] bf16.

    ``weights``: dict(gate_q [E_l,I,H] e4m3fn, gate_s [E_l,I/128,H/128] fp32, up_q, up_s,
    down_q [E_l,H,I], down_s); ``shared``: same keys with one leading group, or None.
    ``bias``: the router's score-correction bias [E] fp32.
    """

    def __init__(self, cfg: MoEConfig, weights, shared, bias: torch.Tensor, max_tokens_in: Optional[int] = None,
                 shared_mode: str = "bf16_add", fold_shared: bool = True, weight_layout: str = "tile_major",
                 router_weight: Optional[torch.Tensor] = None, balanced_gemm: bool = False,
                 weights_repacked: bool = False):
        """``weights_repacked``: the ``*_q`` tensors already hold the tile-major bytes (``repack_tile_major``), e.g.
        because two layers share one resident copy; the layer then takes them as they are."""
        self.cfg = cfg
        dev = weights["gate_q"].device
        with torch.cuda.device(dev):
            check(lib().bgmoe_init())          # first-launch queries now, so that forward() is capturable at once
        if weight_layout not in ("tile_major", "row_major"):
            raise ValueError(f"unknown weight_layout {weight_layout!r}")
        self.layout = W_TILE_MAJOR if weight_layout == "tile_major" else W_ROW_MAJOR
        if weights_repacked and self.layout != W_TILE_MAJOR:
            raise ValueError("weights_repacked needs weight_layout='tile_major'")
        if self.layout == W_TILE_MAJOR and not weights_repacked:
            # resident copy in the streaming layout; the caller may drop the row-major tensors
            weights = dict(weights)
            shared = dict(shared) if shared is not None else None
            for d in (weights, shared):
                if d is not None:
                    for name in ("gate_q", "up_q", "down_q"):
                        d[name] = repack_tile_major(d[name])
        self.device = dev
        self.n_max = int(max_tokens_in or cfg.n_tokens)
        n, h, inter, el, k = self.n_max, cfg.hidden, cfg.inter, cfg.e_local, cfg.top_k
        self.weights, self.shared = weights, shared
        self.bias = bias.to(dev, torch.float32).contiguous()
        self.masked = cfg.layout == "masked"
        self.cap_rows = el * cfg.max_tokens if self.masked else ragged_row_capacity(n, k, el, cfg.row_align)
        has_shared = shared is not None
        self.folded = bool(has_shared and fold_shared and cfg.shared_inter == inter)
        rows = self.cap_rows + (n if has_shared else 0)
        e8, f4, i4, b2 = torch.uint8, torch.float32, torch.int32, torch.bfloat16
        self.topk_ids = torch.empty((n, k), dtype=i4, device=dev)
        self.topk_weights = torch.empty((n, k), dtype=f4, device=dev)
        self.expert_counts = torch.zeros(el + 1, dtype=i4, device=dev)
        self.cu_seqlens = torch.zeros(el + 2, dtype=i4, device=dev)
        self.topk_pos = torch.empty(n * k, dtype=i4, device=dev)
        self.xq = torch.zeros((rows, h), dtype=e8, device=dev)
        self.xs = torch.zeros((rows, h // 128), dtype=f4, device=dev)
        self.hq = torch.zeros((rows, inter), dtype=e8, device=dev)
        self.hs = torch.zeros((rows, inter // 128), dtype=f4, device=dev)
        self.y = torch.zeros((rows, h), dtype=b2, device=dev)
        self.out = torch.empty((n, h), dtype=b2, device=dev)
        self.shq = self.shs = None
        if has_shared and not self.folded:
            self.shq = torch.zeros((n, cfg.shared_inter), dtype=e8, device=dev)
            self.shs = torch.zeros((n, cfg.shared_inter // 128), dtype=f4, device=dev)
        ws_bytes = int(lib().bgmoe_dispatch_workspace_bytes(n * k, el))
        self.workspace = torch.empty(max(ws_bytes, 16), dtype=e8, device=dev)

        L = LayerStruct()
        L.h, L.inter, L.e_total, L.e_local, L.expert_start = h, inter, cfg.n_experts, el, cfg.expert_start
        L.top_k, L.n_group, L.topk_group, L.rsf = k, cfg.n_group, cfg.topk_group, cfg.rsf
        L.layout, L.max_tokens, L.row_align = (0 if self.masked else 1), cfg.max_tokens, max(cfg.row_align, 1)
        L.has_shared, L.shared_folded, L.shared_inter = int(has_shared), int(self.folded), cfg.shared_inter
        L.shared_mode = {"bf16_add": 0, "fp32_add": 1}[shared_mode]
        L.cap_rows = self.cap_rows
        L.bias = ptr(self.bias)
        if self.folded:
            # one pointer table per matrix: local experts then the shared expert
            self._tables = {}
            for name in ("gate", "up", "down"):
                q, s = weights[name + "_q"], weights[name + "_s"]
                sq, ss = shared[name + "_q"], shared[name + "_s"]
                wp = [q[i].data_ptr() for i in range(el)] + [sq[0].data_ptr()]
                sp = [s[i].data_ptr() for i in range(el)] + [ss[0].data_ptr()]
                tw = torch.tensor(wp, dtype=torch.int64, device=dev)
                ts = torch.tensor(sp, dtype=torch.int64, device=dev)
                self._tables[name] = (tw, ts)
                _check_stack(q, s)
                if sq.stride(1) != q.size(2) or ss.stride(1) != s.stride(1):
                    raise RuntimeError("a folded shared expert must use the routed experts' scale row stride")
                setattr(L, name, Fp8Weight(None, 0, ptr(tw), None, 0, s.stride(1), ptr(ts), self.layout, 0))
        else:
            for name in ("gate", "up", "down"):
                setattr(L, name, _stack_desc(weights[name + "_q"], weights[name + "_s"], self.layout))
            if has_shared:
                for name in ("gate", "up", "down"):
                    setattr(L, "sh_" + name, _stack_desc(shared[name + "_q"], shared[name + "_s"], self.layout))
                L.shq, L.shs = ptr(self.shq), ptr(self.shs)
        L.topk_ids, L.topk_weights = ptr(self.topk_ids), ptr(self.topk_weights)
        L.expert_counts, L.cu_seqlens, L.topk_pos = ptr(self.expert_counts), ptr(self.cu_seqlens), ptr(self.topk_pos)
        L.xq, L.xs, L.hq, L.hs, L.y = ptr(self.xq), ptr(self.xs), ptr(self.hq), ptr(self.hs), ptr(self.y)
        L.workspace, L.workspace_bytes = ptr(self.workspace), self.workspace.numel()
        L.out = ptr(self.out)
        self.gemm_workspace = None
        if balanced_gemm and self.layout == W_TILE_MAJOR and n <= STREAMK_MAX_TOKENS:
            # decode-sized batches: both grouped GEMMs in their balanced form (its counters start at zero)
            gb = int(lib().bgmoe_fp8_streamk_workspace_bytes())
            self.gemm_workspace = torch.zeros(gb, dtype=e8, device=dev)
            L.gemm_workspace, L.gemm_workspace_bytes = ptr(self.gemm_workspace), gb
        self.router_weight = None
        if router_weight is not None:
            # the layer then routes from the hidden states: router GEMM + gate, no logits tensor
            if router_weight.dtype != torch.bfloat16 or tuple(router_weight.shape) != (cfg.n_experts, h):
                raise RuntimeError(f"router_weight must be BF16 [{cfg.n_experts}, {h}]")
            self.router_weight = router_weight.contiguous()
            rb = int(lib().bgmoe_router_gemm_workspace_bytes(n, h, cfg.n_experts))
            self.router_workspace = torch.empty(max(rb, 16), dtype=e8, device=dev)
            L.router_weight = ptr(self.router_weight)
            L.router_workspace, L.router_workspace_bytes = ptr(self.router_workspace), self.router_workspace.numel()
        self._L = L
        self._fn = lib().bgmoe_moe_fp8_layer_forward

    def forward(self, hidden_states: torch.Tensor, router_logits: Optional[torch.Tensor] = None,
                x_fp8: Optional[torch.Tensor] = None, x_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``router_logits=None`` routes from ``hidden_states`` through the layer's ``router_weight``.
        ``x_fp8``/``x_scale`` (``[N,H]`` e4m3fn or uint8, ``[N,H/128]`` fp32 of any strides) are the tokens
        already quantised by the producer upstream (``cuda_add_rmsnorm_fp8_quant``); both or neither, as in
        the reference's hand-down (batchgen/models/glm/glm5/wrappers.py:416-447)."""
        cfg = self.cfg
        if hidden_states.dtype != torch.bfloat16 or hidden_states.dim() != 2 or hidden_states.size(1) != cfg.hidden:
            raise RuntimeError(f"hidden_states must be BF16 [N, {cfg.hidden}]")
        n = hidden_states.size(0)
        if n > self.n_max:
            raise RuntimeError(f"{n} tokens exceed the {self.n_max} this layer's buffers were sized for")
        if not hidden_states.is_contiguous():
            raise RuntimeError("hidden_states must be contiguous")
        L = self._L
        if router_logits is None:
            if self.router_weight is None:
                raise RuntimeError("router_logits=None needs a layer built with router_weight")
            L.logits = None
        else:
            if router_logits.dtype != torch.float32 or tuple(router_logits.shape) != (n, cfg.n_experts):
                raise RuntimeError(f"router_logits must be FP32 [{n}, {cfg.n_experts}]")
            if not router_logits.is_contiguous():
                raise RuntimeError("router_logits must be contiguous")
            L.logits = ptr(router_logits)
        if (x_fp8 is None) != (x_scale is None):
            raise RuntimeError("x_fp8 and x_scale must be given together; got "
                               f"{'x_scale' if x_fp8 is None else 'x_fp8'} alone")
        if x_fp8 is not None:
            blocks = cfg.hidden // 128
            if x_fp8.dtype not in (torch.float8_e4m3fn, torch.uint8) or tuple(x_fp8.shape) != (n, cfg.hidden):
                raise RuntimeError(f"x_fp8 must be float8_e4m3fn ({n}, {cfg.hidden}), got {x_fp8.dtype} "
                                   f"{tuple(x_fp8.shape)}")
            if not x_fp8.is_contiguous():
                raise RuntimeError("x_fp8 must be contiguous")
            if x_scale.dtype != torch.float32 or tuple(x_scale.shape) != (n, blocks):
                raise RuntimeError(f"x_scale must be fp32 ({n}, {blocks}), got {x_scale.dtype} {tuple(x_scale.shape)}")
            L.x_fp8, L.x_scale = ptr(x_fp8), ptr(x_scale)
            L.x_scale_row_stride, L.x_scale_kb_stride = x_scale.stride(0), x_scale.stride(1)
        else:
            L.x_fp8 = L.x_scale = None
        L.n = n
        L.x = ptr(hidden_states)
        L.routes_given = 0
        check(self._fn(C.byref(L), stream()))
        return self.out[:n]

    def forward_routed(self, hidden_states: torch.Tensor, topk_idx: torch.Tensor,
                       topk_weight: torch.Tensor, distinct_ids: bool = False) -> torch.Tensor:
        """The layer behind an external gate: ``topk_idx`` ``[N, K]`` (global expert ids; ids this rank does not
        hold, and -1, contribute nothing) and ``topk_weight`` ``[N, K]`` fp32 are given, as in
        ``WGMMAMoEBuffers.forward(layer_id, global_x, topk_idx, topk_weight)``
        (batchgen/moe/fp8_wgmma_pipeline.py:294-372): dispatch, quantise, gate_up + SwiGLU + requant, down,
        weighted combine (+ shared expert when the layer has one).

        ``distinct_ids``: the caller vouches that the ids of a row are pairwise different (any top-k gate's are).
        An expert then has at most N rows, and a decode batch runs on the weight-streaming kernels alone, as
        with the layer's own router; without the promise an expert may hold up to N*K rows and batches above
        256 / K tokens also launch the tiled kernel."""
        cfg = self.cfg
        n = hidden_states.size(0)
        if hidden_states.dtype != torch.bfloat16 or tuple(hidden_states.shape) != (n, cfg.hidden) or \
                not hidden_states.is_contiguous() or n > self.n_max:
            raise RuntimeError(f"hidden_states must be contiguous BF16 [N <= {self.n_max}, {cfg.hidden}]")
        if tuple(topk_idx.shape) != (n, cfg.top_k) or tuple(topk_weight.shape) != (n, cfg.top_k):
            raise RuntimeError(f"topk_idx and topk_weight must be [{n}, {cfg.top_k}]")
        self.topk_ids[:n].copy_(topk_idx)                 # any integer dtype -> the layer's int32 buffer
        self.topk_weights[:n].copy_(topk_weight)
        L = self._L
        L.logits = L.x_fp8 = L.x_scale = None
        L.n, L.x, L.routes_given = n, ptr(hidden_states), ROUTES_GIVEN_DISTINCT if distinct_ids else ROUTES_GIVEN
        try:
            check(self._fn(C.byref(L), stream()))
        finally:
            L.routes_given = 0
        return self.out[:n]

    __call__ = forward
