"""MXFP4 (W4A16) MoE layer forward on one GPU's share of the experts.

Host-side counterpart of ``ResidentEPMXFP4MoELayer._expert_path`` / ``forward``
(batchgen/moe/fused_moe_mxfp4_resident.py:709-944) without the latent projections and collectives:
ungrouped sigmoid top-k router -> masked dispatch of bf16 rows -> grouped MXFP4 gate_up + SwiGLU ->
grouped MXFP4 down -> fp32 weighted combine + shared expert.  Weights are repacked once into the
tile-major resident layout (the reference repacks to Marlin at the same point, :13-15).
The shared expert is a plain dense bf16 MLP and runs on the library GEMM (hipBLASLt through torch).
"""
from __future__ import annotations

import ctypes as C

import torch
import torch.nn.functional as F

from .._lib import Mxfp4Weight, check, lib, ptr, stream
from ..kernels import load_extension
from ..workloads import MoEConfig


class Mxfp4MoELayer:
    def __init__(self, cfg: MoEConfig, weights, shared_bf16, bias: torch.Tensor, shared_mode: str = "bf16_add"):
        self.cfg = cfg
        dev = weights["gate_p"].device
        self.device = dev
        with torch.cuda.device(dev):
            check(lib().bgmoe_init())
        mg = load_extension("batchgen_kernels.moe._C_marlin_grouped_gemm")
        self.w = {}
        for name in ("gate", "up", "down"):
            p, s = mg.mxfp4_weight_repack(weights[name + "_p"], weights[name + "_s"])
            self.w[name] = (p, s, Mxfp4Weight(ptr(p), p.size(1) * p.size(2), None, ptr(s), s.size(1) * s.size(2),
                                              None, 1, 0))
        self.shared = shared_bf16
        self.bias = bias.to(dev, torch.float32).contiguous()
        n, h, inter, el, k = cfg.n_tokens, cfg.hidden, cfg.inter, cfg.e_local, cfg.top_k
        if cfg.layout != "masked":
            raise ValueError("the MXFP4 layer uses the masked layout")
        self.rows = el * cfg.max_tokens
        i4, f4, b2 = torch.int32, torch.float32, torch.bfloat16
        self.topk_ids = torch.empty((n, k), dtype=i4, device=dev)
        self.topk_weights = torch.empty((n, k), dtype=f4, device=dev)
        self.expert_counts = torch.zeros(el, dtype=i4, device=dev)
        self.expert_counters = torch.zeros(el, dtype=i4, device=dev)
        self.cu = (torch.arange(el + 1, dtype=i4, device=dev) * cfg.max_tokens).contiguous()
        self.topk_pos = torch.empty(n * k, dtype=i4, device=dev)
        self.act = torch.zeros((self.rows, h), dtype=b2, device=dev)
        self.hmid = torch.zeros((self.rows, inter), dtype=b2, device=dev)
        self.y = torch.zeros((self.rows, h), dtype=b2, device=dev)
        self.out = torch.empty((n, h), dtype=b2, device=dev)
        self.shared_mode = {"bf16_add": 0, "fp32_add": 1}[shared_mode]
        self._routing = load_extension("batchgen_kernels.moe._C_routing")
        self._dispatch = load_extension("batchgen_kernels.moe._C_dispatch_scatter_3d")

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        cfg = self.cfg
        n = hidden_states.size(0)
        if hidden_states.dtype != torch.bfloat16 or tuple(hidden_states.shape) != (n, cfg.hidden) or n > cfg.n_tokens:
            raise RuntimeError(f"hidden_states must be BF16 [N <= {cfg.n_tokens}, {cfg.hidden}]")
        ids, wts, pos = self.topk_ids[:n], self.topk_weights[:n], self.topk_pos[:n * cfg.top_k]
        self._routing.gate_sigmoid_topk(router_logits, self.bias, cfg.top_k, cfg.rsf, ids, wts)
        self._dispatch.dispatch_scatter_3d(hidden_states, ids, self.act, cfg.expert_start, cfg.e_local, cfg.max_tokens,
                                           self.expert_counts, self.expert_counters, pos)
        bound = n * cfg.top_k
        st = stream()
        check(lib().bgmoe_mxfp4_fused_s1(ptr(self.act), C.byref(self.w["gate"][2]), C.byref(self.w["up"][2]),
                                         ptr(self.expert_counts), ptr(self.cu), cfg.e_local, self.rows, cfg.inter,
                                         cfg.hidden, ptr(self.hmid), None, 0, bound, st))
        check(lib().bgmoe_mxfp4_grouped_gemm(ptr(self.hmid), C.byref(self.w["down"][2]), ptr(self.expert_counts),
                                             ptr(self.cu), cfg.e_local, self.rows, cfg.hidden, cfg.inter, ptr(self.y),
                                             None, bound, st))
        sh = None
        if self.shared is not None:
            g = F.linear(hidden_states, self.shared["gate"])
            u = F.linear(hidden_states, self.shared["up"])
            sh = F.linear(F.silu(g) * u, self.shared["down"])
        check(lib().bgmoe_reduce_weighted_scatter(ptr(self.y), ptr(pos), ptr(wts), n, cfg.hidden, cfg.top_k,
                                                  ptr(self.out), -1, ptr(sh), self.shared_mode, st))
        return self.out[:n]

    __call__ = forward
