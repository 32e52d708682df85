"""MXFP4 (W4A16) MoE layer forward on one GPU's share of the experts.

Host-side counterpart of ``ResidentEPMXFP4MoELayer._expert_path`` / ``forward``
(batchgen/moe/fused_moe_mxfp4_resident.py:709-944) without the collectives:
ungrouped sigmoid top-k router -> masked dispatch of bf16 rows -> grouped MXFP4 gate_up + activation ->
grouped MXFP4 down -> fp32 weighted combine + shared expert.  Weights are repacked once into the
tile-major resident layout (the reference repacks to Marlin at the same point, :13-15).
The shared expert is a plain dense bf16 MLP on this library's own bf16 GEMM (``bgmoe_bf16_linear``); the vendor
library through ``torch.mm`` is an explicit option kept for comparison.

With ``latent`` weights the layer is the Kimi-K3 latent MoE (:922-944, kimi_linear/model.py:585-603): the
router sees the hidden rows, ``down_proj`` takes them to the latent width once per token, the experts and
the combine work on latent rows, then RMSNorm (optional) and ``up_proj`` bring the result back, and the
shared expert's output is added.  The two projections are plain bf16 GEMMs (``nn.Linear`` in the reference) on
the same ``bgmoe_bf16_linear``.  ``activation="situ"`` selects the K3 activation for the routed experts
(fused into the stage-1 GEMM) and the shared expert (``situ_and_mul``).
"""
from __future__ import annotations

import os

import ctypes as C

import torch

from .. import _lib
from .._lib import Mxfp4Weight, check, lib, ptr, stream
from ..kernels import load_extension
from .latent import bf16_linear, bf16_linear_workspace_bytes, rmsnorm, silu_and_mul, situ_and_mul
from ..workloads import MoEConfig


i32, i64, f32, vp, sz = C.c_int32, C.c_int64, C.c_float, C.c_void_p, C.c_size_t


class Mxfp4LayerStruct(C.Structure):
    """bgmoe_moe_mxfp4_layer (include/bgmoe.h)"""
    _fields_ = [
        ("n", i32), ("h", i32), ("inter", i32), ("e_total", i32), ("e_local", i32), ("expert_start", i32),
        ("top_k", i32), ("max_tokens", i32), ("rsf", f32), ("shared_mode", i32),
        ("x", vp), ("logits", vp), ("bias", vp),
        ("gate", Mxfp4Weight), ("up", Mxfp4Weight), ("down", Mxfp4Weight),
        ("topk_ids", vp), ("topk_weights", vp), ("expert_counts", vp), ("expert_counters", vp), ("cu_seqlens", vp),
        ("topk_pos", vp), ("act", vp), ("hmid", vp), ("y", vp), ("workspace", vp), ("workspace_bytes", sz),
        ("shared_out", vp), ("out", vp), ("activation", i32), ("row_pair", vp),
    ]


_lib.register("bgmoe_moe_mxfp4_layer_forward", i32, [C.POINTER(Mxfp4LayerStruct), i32, vp])
ROUTED, COMBINE = 1, 2
ACTIVATIONS = {"swiglu": 0, "situ": 1}
K3_SITU_BETA, K3_SITU_LINEAR_BETA = 4.0, 25.0   # the constants the fused stage-1 epilogue compiles in


class Mxfp4MoELayer:
    def __init__(self, cfg: MoEConfig, weights, shared_bf16, bias: torch.Tensor, shared_mode: str = "bf16_add",
                 latent=None, dense_backend: str = "hip", fold_gather: bool = False):
        """``dense_backend``: "hip" (the default) runs the bf16 shared expert and the latent projections on this
        library's own bf16 GEMM, so that the whole layer is this library's kernels and a token's result does not
        depend on its position in the batch; "vendor" runs them on the vendor library through ``torch.mm``, as
        ``nn.Linear`` in the reference does (faster at 512 tokens: measured 45 + 35 us against 2 x 92 us for the
        shared expert; kept for that comparison, never chosen silently).  Either way the results go into buffers
        owned by the layer: ``forward`` allocates no tensor, and what it returns is one of those buffers,
        overwritten by the next call.

        ``fold_gather`` (opt-in): the dispatch only computes indices and stage 1 reads every row from its token
        through a row -> pair map, instead of from a gathered expert-major copy of the rows; same results, one
        launch and one pass over the rows fewer."""
        if dense_backend not in ("hip", "vendor"):
            raise ValueError(f"dense_backend must be 'hip' or 'vendor', got {dense_backend!r}")
        self.dense_backend = dense_backend
        self.cfg = cfg
        dev = weights["gate_p"].device
        self.device = dev
        if cfg.activation not in ACTIVATIONS:
            raise ValueError(f"activation must be one of {sorted(ACTIVATIONS)}, got {cfg.activation!r}")
        if bool(cfg.latent) != (latent is not None):
            raise ValueError("latent weights are needed exactly when cfg.latent is set")
        self.latent = latent
        if latent is not None:
            for name, shape in (("down_proj", (cfg.latent, cfg.hidden)), ("up_proj", (cfg.hidden, cfg.latent))):
                t = latent[name]
                if t.dtype != torch.bfloat16 or tuple(t.shape) != shape or not t.is_contiguous():
                    raise ValueError(f"latent[{name!r}] must be contiguous BF16 {shape}")
            if cfg.latent_norm != (latent.get("norm_weight") is not None):
                raise ValueError("latent['norm_weight'] is needed exactly when cfg.latent_norm is set")
        with torch.cuda.device(dev):
            check(lib().bgmoe_init())
        mg = load_extension("batchgen_kernels.moe._C_marlin_grouped_gemm")
        self.w = {}
        for name in ("gate", "up", "down"):
            p, s = mg.mxfp4_weight_repack(weights[name + "_p"], weights[name + "_s"])
            self.w[name] = (p, s, Mxfp4Weight(ptr(p), p.size(1) * p.size(2), None, ptr(s), s.size(1) * s.size(2),
                                              None, 1, 0))
        self.shared = shared_bf16
        self.overlap_shared = os.environ.get("BGMOE_MXFP4_OVERLAP_SHARED", "1") != "0"
        if shared_bf16 is not None:
            # gate and up as one [2I, H] matrix: one GEMM instead of two
            self._shared_gate_up = torch.cat([shared_bf16["gate"], shared_bf16["up"]], dim=0).contiguous()
            self._side = torch.cuda.Stream(device=dev)
            self._fork, self._join = torch.cuda.Event(), torch.cuda.Event()
        self.bias = bias.to(dev, torch.float32).contiguous()
        n, h, inter, el, k = cfg.n_tokens, cfg.expert_hidden, cfg.inter, cfg.e_local, cfg.top_k
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
        self.fold_gather = bool(fold_gather)
        self.act = None if self.fold_gather else torch.zeros((self.rows, h), dtype=b2, device=dev)
        self.row_pair = torch.zeros(self.rows, dtype=i4, device=dev) if self.fold_gather else None
        self.hmid = torch.zeros((self.rows, inter), dtype=b2, device=dev)
        self.y = torch.zeros((self.rows, h), dtype=b2, device=dev)
        self.out = torch.empty((n, h), dtype=b2, device=dev)
        self.shared_mode = {"bf16_add": 0, "fp32_add": 1}[shared_mode]
        ws_bytes = int(lib().bgmoe_dispatch_workspace_bytes(n * k, el))
        self.workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        L = Mxfp4LayerStruct()
        L.h, L.inter, L.e_total, L.e_local, L.expert_start = h, inter, cfg.n_experts, el, cfg.expert_start
        L.top_k, L.max_tokens, L.rsf, L.shared_mode = k, cfg.max_tokens, cfg.rsf, self.shared_mode
        L.bias = ptr(self.bias)
        L.gate, L.up, L.down = self.w["gate"][2], self.w["up"][2], self.w["down"][2]
        L.topk_ids, L.topk_weights = ptr(self.topk_ids), ptr(self.topk_weights)
        L.expert_counts, L.expert_counters, L.cu_seqlens = ptr(self.expert_counts), ptr(self.expert_counters), ptr(self.cu)
        L.topk_pos, L.hmid, L.y = ptr(self.topk_pos), ptr(self.hmid), ptr(self.y)
        L.act = ptr(self.act) if self.act is not None else None
        L.row_pair = ptr(self.row_pair) if self.row_pair is not None else None
        L.workspace, L.workspace_bytes = ptr(self.workspace), self.workspace.numel()
        L.out = ptr(self.out)
        L.activation = ACTIVATIONS[cfg.activation]
        self._L = L
        self._fn = lib().bgmoe_moe_mxfp4_layer_forward
        # buffers of the dense bf16 parts (shared expert, latent projections): forward() allocates none of them
        hid = cfg.hidden
        use_hip = dense_backend == "hip"

        def ws(nn, hh, ee):
            if not use_hip:
                return None
            return torch.empty(bf16_linear_workspace_bytes(nn, hh, ee), dtype=torch.uint8, device=dev)
        d = {}
        if shared_bf16 is not None:
            si2 = self._shared_gate_up.size(0)
            d["gu"] = torch.empty((n, si2), dtype=b2, device=dev)
            d["hh"] = torch.empty((n, si2 // 2), dtype=b2, device=dev)
            d["sh"] = torch.empty((n, hid), dtype=b2, device=dev)
            d["ws_gu"], d["ws_dn"] = ws(n, hid, si2), ws(n, si2 // 2, hid)
        if latent is not None:
            d["xlat"] = torch.empty((n, cfg.latent), dtype=b2, device=dev)
            d["ynorm"] = torch.empty((n, cfg.latent), dtype=b2, device=dev)
            d["yup"] = torch.empty((n, hid), dtype=b2, device=dev)
            d["ws_lat_dn"], d["ws_lat_up"] = ws(n, hid, cfg.latent), ws(n, cfg.latent, hid)
        self._dense = d

    def _linear(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, workspace) -> torch.Tensor:
        """``x @ w^T`` into ``out``: this library's bf16 GEMM, or the vendor library's through ``torch.mm``."""
        if self.dense_backend == "hip":
            return bf16_linear(x, w, out, workspace)
        return torch.mm(x, w.t(), out=out)

    def forward(self, hidden_states: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        cfg = self.cfg
        n = hidden_states.size(0)
        if hidden_states.dtype != torch.bfloat16 or tuple(hidden_states.shape) != (n, cfg.hidden) or n > cfg.n_tokens:
            raise RuntimeError(f"hidden_states must be BF16 [N <= {cfg.n_tokens}, {cfg.hidden}]")
        if router_logits.dtype != torch.float32 or tuple(router_logits.shape) != (n, cfg.n_experts) or \
                not router_logits.is_contiguous() or not hidden_states.is_contiguous():
            raise RuntimeError(f"router_logits must be contiguous FP32 [{n}, {cfg.n_experts}] and hidden_states contiguous")
        sh = None
        cur = torch.cuda.current_stream(self.device)
        if self.shared is not None:
            # the dense bf16 shared expert runs beside the routed experts on a second stream of
            # the same priority: its GEMMs are MFMA-bound, the routed kernels stream weights from HBM
            side = self._side if self.overlap_shared else cur
            if side is not cur:
                self._fork.record(cur)
                side.wait_event(self._fork)
            with torch.cuda.stream(side):
                d = self._dense
                gu = self._linear(hidden_states, self._shared_gate_up, d["gu"][:n], d["ws_gu"])
                if cfg.activation == "situ":
                    hh = situ_and_mul(gu, K3_SITU_BETA, K3_SITU_LINEAR_BETA, out=d["hh"][:n])
                else:
                    hh = silu_and_mul(gu, out=d["hh"][:n])
                sh = self._linear(hh, self.shared["down"], d["sh"][:n], d["ws_dn"])
                if side is not cur:
                    self._join.record(side)
        x_exp = hidden_states
        if self.latent is not None:                                        # hidden -> latent, once per token
            x_exp = self._linear(hidden_states, self.latent["down_proj"], self._dense["xlat"][:n],
                                 self._dense["ws_lat_dn"])
        L = self._L
        L.n, L.x, L.logits = n, ptr(x_exp), ptr(router_logits)
        # latent: the shared expert's rows are hidden-sized and join after the latent -> hidden projection
        L.shared_out = ptr(sh) if self.latent is None else None
        st = stream()
        joined = False
        if sh is not None and self.overlap_shared and self.latent is None:
            check(self._fn(C.byref(L), ROUTED, st))
            cur.wait_event(self._join)
            joined = True
            check(self._fn(C.byref(L), COMBINE, st))
        else:
            check(self._fn(C.byref(L), ROUTED | COMBINE, st))
        if self.latent is None:
            return self.out[:n]
        y = self.out[:n]
        d = self._dense
        if self.latent.get("norm_weight") is not None:
            y = rmsnorm(y, self.latent["norm_weight"], self.latent["eps"], out=d["ynorm"][:n])
        y = self._linear(y, self.latent["up_proj"], d["yup"][:n], d["ws_lat_up"])     # latent -> hidden
        if sh is not None:
            if self.overlap_shared and not joined:
                cur.wait_event(self._join)
            y = torch.add(y, sh, out=y)
        return y

    __call__ = forward
