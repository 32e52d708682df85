"""The reference's MoE layer template over this build's kernels.

``MoEBufferManager`` and ``MoEBase`` follow ``batchgen/moe/moe_base.py:31-264``: a model file subclasses
``MoEBase`` and fills in ``gate``, ``expert_compute_persistent`` / ``expert_compute_mixed`` and
``shared_expert_forward``; ``forward`` dispatches on ``config.phase`` to the decode template
(all-gather -> gate -> expert compute -> all-reduce -> local slice + shared expert) or to ``_forward_prefill``.
``Fp8BlockwiseMoE`` is the concrete FP8-blockwise layer (what ``Glm5MoE`` is in the reference,
``batchgen/models/glm/glm5/model.py:1624-1700, 2620-2745``): it takes the model's configuration object
(``hidden_size``, ``moe_intermediate_size``, ``n_routed_experts``, ``num_experts_per_tok``, ``n_group``,
``topk_group``, ``routed_scaling_factor``, ``norm_topk_prob``, ``n_shared_experts``, ``phase``) and the weight
stacks, so a model file can instantiate it without knowing this package's own workload description.

This build runs one GPU: with ``world_size == 1`` the all-gather is a copy into the padded buffer and the
all-reduce is the identity; a larger world raises (the exchange is not part of this build).
"""
from __future__ import annotations

from typing import ClassVar, Optional, Tuple

import torch
import torch.nn as nn

from ..workloads import MoEConfig
from .fp8_layer import Fp8MoELayer, repack_tile_major
from .routing.cuda_routing import router_gemm_gate_sigmoid_topk
from .shared_expert import Fp8DenseExpert


class MoEBufferManager:
    """Token buffers of the decode template, shared by every MoE layer of a model (the reference keeps one per
    model as a class attribute of ``MoEBase``, moe_base.py:31-72).  Here both buffers are views of ONE
    allocation of ``(world_size + 1) * num_tokens_per_rank`` rows: the first ``world_size * num_tokens_per_rank``
    are ``all_tokens`` (the gathered batch the experts see), the rest ``padded_hidden_states`` (this rank's
    slice, padded).  Growing replaces the allocation; shrinking never happens, so addresses captured in a graph
    stay valid until a larger batch arrives."""

    def __init__(self, num_tokens_per_rank: int, world_size: int, hidden_size: int, device: torch.device):
        if num_tokens_per_rank <= 0 or world_size <= 0 or hidden_size <= 0:
            raise ValueError("num_tokens_per_rank, world_size and hidden_size must be positive")
        self.world_size = world_size
        self.hidden_size = hidden_size
        self.device = device
        self.num_tokens_per_rank = 0
        self._rows = None
        self._grow(num_tokens_per_rank)

    def _grow(self, num_tokens_per_rank: int) -> None:
        self._rows = torch.zeros(((self.world_size + 1) * num_tokens_per_rank, self.hidden_size),
                                 dtype=torch.bfloat16, device=self.device)
        self.num_tokens_per_rank = num_tokens_per_rank

    @property
    def all_tokens(self) -> torch.Tensor:
        return self._rows[: self.world_size * self.num_tokens_per_rank]

    @property
    def padded_hidden_states(self) -> torch.Tensor:
        return self._rows[self.world_size * self.num_tokens_per_rank:]

    def resize_if_needed(self, num_tokens_per_rank: int) -> None:
        if num_tokens_per_rank > self.num_tokens_per_rank:
            self._grow(num_tokens_per_rank)


def _rank_and_world() -> Tuple[int, int]:
    import torch.distributed as dist
    if dist.is_available() and dist.is_initialized():
        return dist.get_rank(), dist.get_world_size()
    return 0, 1


class MoEBase(nn.Module):
    """Template of the MoE layers (moe_base.py:75-264).  A model file subclasses it and fills in ``gate``,
    ``expert_compute_persistent`` / ``expert_compute_mixed`` and ``shared_expert_forward``; the attribute names
    set here (``experts_per_rank``, ``routed_expert_start_idx``, ``num_persistent_local_experts`` ...) are the
    ones those subclasses read."""

    _buffer_mgr: ClassVar[Optional[MoEBufferManager]] = None

    def __init__(self, config, comm=None):
        super().__init__()
        rank, world = _rank_and_world()
        if world != 1:
            raise NotImplementedError("this build runs one GPU: the expert-parallel exchange (all-gather / "
                                      "all-reduce across ranks) is not part of it")
        per_rank = config.n_routed_experts // world
        self.config, self.comm = config, comm
        self.hidden_size, self.num_experts_per_tok = config.hidden_size, config.num_experts_per_tok
        self.rank, self.world_size = rank, world
        self.experts_per_rank, self.total_experts = per_rank, per_rank * world
        self.routed_expert_start_idx, self.routed_expert_end_idx = rank * per_rank, (rank + 1) * per_rank
        self.device = torch.device("cuda", rank % max(torch.cuda.device_count(), 1))
        self.num_tokens_per_rank: Optional[int] = None
        self.enable_ep_offloading = False
        self.num_persistent_local_experts = per_rank           # every local expert resident unless a subclass says so

    # -- buffers ----------------------------------------------------------------------------------------------
    @classmethod
    def init_buffer_manager(cls, num_tokens_per_rank: int, world_size: int, hidden_size: int, device: torch.device):
        cls._buffer_mgr = MoEBufferManager(num_tokens_per_rank, world_size, hidden_size, device)

    def init_num_tokens(self, num_tokens_per_rank: int):
        self.num_tokens_per_rank = num_tokens_per_rank

    def set_num_tokens_per_rank(self, num_tokens_per_rank: int):
        self.init_num_tokens(num_tokens_per_rank)
        mgr = type(self)._buffer_mgr
        if mgr is not None:
            mgr.resize_if_needed(num_tokens_per_rank)

    # -- what a model fills in --------------------------------------------------------------------------------
    def gate(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """``x [G, H]`` bf16 -> ``(topk_idx [G, K] int32, topk_weight [G, K] fp32)``."""
        raise NotImplementedError

    def expert_compute_persistent(self, global_x: torch.Tensor, topk_idx: torch.Tensor,
                                  topk_weight: torch.Tensor) -> torch.Tensor:
        """Routed experts of this rank on all gathered tokens -> ``[G, H]`` weighted sums, no host synchronisation."""
        raise NotImplementedError

    def expert_compute_mixed(self, global_x: torch.Tensor, topk_idx: torch.Tensor,
                             topk_weight: torch.Tensor) -> torch.Tensor:
        """Same contract; the reference's opt-in path for experts that are not resident."""
        raise NotImplementedError

    def shared_expert_forward(self, identity: torch.Tensor) -> torch.Tensor:
        return torch.zeros_like(identity)

    # -- the template -------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        decode = getattr(self.config, "phase", "decode") == "decode"
        return self._forward_decode(hidden_states) if decode else self._forward_prefill(hidden_states)

    def _gathered_tokens(self, tokens: torch.Tensor) -> torch.Tensor:
        """The batch the experts see: with one rank, this rank's tokens followed by zero rows up to
        ``num_tokens_per_rank`` (what the all-gather of the padded slices delivers), in the shared buffer when
        it is large enough."""
        ntp = self.num_tokens_per_rank
        live, width = tokens.shape
        mgr = type(self)._buffer_mgr
        if mgr is not None and mgr.hidden_size == width and mgr.num_tokens_per_rank >= ntp:
            gathered = mgr.all_tokens[:ntp]
        else:
            gathered = tokens.new_empty((ntp, width), dtype=torch.bfloat16)
        gathered[:live].copy_(tokens)
        gathered[live:].zero_()
        return gathered

    def _run_experts(self, global_x: torch.Tensor, topk_idx: torch.Tensor, topk_weight: torch.Tensor) -> torch.Tensor:
        resident = self.num_persistent_local_experts == self.experts_per_rank and not self.enable_ep_offloading
        compute = self.expert_compute_persistent if resident else self.expert_compute_mixed
        return compute(global_x, topk_idx, topk_weight)

    @torch.inference_mode()
    def _forward_decode(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """The decode template (moe_base.py:188-258) for a world of one rank: gather (= pad) -> gate -> expert
        compute -> (the all-reduce of one rank is the identity) -> this rank's live rows + shared expert."""
        if self.num_tokens_per_rank is None:
            raise RuntimeError("init_num_tokens / set_num_tokens_per_rank must be called before the first forward")
        tokens = hidden_states.view(-1, hidden_states.shape[-1])
        live = tokens.size(0)
        if live > self.num_tokens_per_rank:
            raise RuntimeError(f"MoE buffer overflow: num_tokens={live} > "
                               f"num_tokens_per_rank={self.num_tokens_per_rank}")
        global_x = self._gathered_tokens(tokens)
        global_results = self._run_experts(global_x, *self.gate(global_x))
        first = self.rank * self.num_tokens_per_rank
        routed = global_results[first:first + live].to(tokens.dtype)
        return (routed + self.shared_expert_forward(tokens)).view(hidden_states.shape)

    @torch.inference_mode()
    def _forward_prefill(self, hidden_states: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError("Subclass must implement _forward_prefill for prefill mode")


def _moe_config(config, n_tokens: int, experts_per_rank: int, expert_start: int, with_shared: bool) -> MoEConfig:
    """This package's workload description from a model configuration object."""
    ragged = n_tokens > 1024          # per-expert slot tables of max_tokens rows stop paying beyond decode sizes
    shared_inter = config.moe_intermediate_size * int(getattr(config, "n_shared_experts", 0) or 0)
    return MoEConfig(
        name="model_layer", index=0, n_tokens=n_tokens, hidden=config.hidden_size,
        inter=config.moe_intermediate_size, n_experts=config.n_routed_experts, e_local=experts_per_rank,
        expert_start=expert_start, top_k=config.num_experts_per_tok, n_group=int(getattr(config, "n_group", 1) or 1),
        topk_group=int(getattr(config, "topk_group", 1) or 1), rsf=float(config.routed_scaling_factor),
        shared_inter=shared_inter if with_shared else 0, layout="ragged" if ragged else "masked",
        max_tokens=0 if ragged else n_tokens, row_align=128 if ragged else 64, weight_format="fp8")


class Fp8BlockwiseMoE(MoEBase):
    """FP8-blockwise MoE layer under the template: sigmoid gate with a score-correction bias (group-limited
    when ``config.n_group > 1``), routed experts through the grouped FP8 kernels, FP8 shared expert.

    ``weights``: ``gate_q [E_local, I, H]`` e4m3fn + ``gate_s [E_local, I/128, H/128]`` fp32, likewise ``up_*``
    and ``down_* [E_local, H, I]`` (the stacks ``Glm5MoE._init_fp8_blockwise_weights`` builds,
    model.py:1991-2277); ``shared``: the same keys with one leading group, or None; ``gate_weight [E, H]`` and
    ``e_score_correction_bias [E]`` as in ``Glm5MoEGate`` (model.py:1103-1117).

    ``forward`` runs the template step by step (what a model file's own subclass would do); ``forward_fused``
    runs router GEMM, gate, quantiser, dispatch, both grouped GEMMs, combine and shared expert as ONE call of
    the C library -- same routing, sums that differ in rounding only."""

    def __init__(self, config, weights, shared, gate_weight: torch.Tensor, e_score_correction_bias: torch.Tensor,
                 comm=None, layer_idx: int = 0):
        super().__init__(config, comm)
        if not getattr(config, "norm_topk_prob", True):
            raise NotImplementedError("the gate kernels normalise the top-k weights (norm_topk_prob=True)")
        self.layer_idx = layer_idx
        dev = weights["gate_q"].device
        # one resident copy in the weight-streaming layout, shared by the step-by-step and the fused engine; the
        # caller may drop the row-major stacks
        self._weights = {k: (repack_tile_major(v) if k.endswith("_q") else v) for k, v in weights.items()}
        self._shared = None if shared is None else \
            {k: (repack_tile_major(v) if k.endswith("_q") else v) for k, v in shared.items()}
        self.device = dev
        self.gate_weight = gate_weight.to(dev, torch.bfloat16).contiguous()
        self.e_score_correction_bias = e_score_correction_bias.to(dev, torch.float32).contiguous()
        self.n_group = int(getattr(config, "n_group", 1) or 1)
        self.topk_group = int(getattr(config, "topk_group", 1) or 1)
        self.shared_experts = None
        if shared is not None:
            inter = shared["gate_q"].size(1)
            # gate and up as the row halves of one allocation (the fused gate_up GEMM of the dense chain); bytes are
            # concatenated as uint8: torch has no cat kernel for float8 tensors on every build
            gate_up = torch.cat([shared["gate_q"][0].view(torch.uint8), shared["up_q"][0].view(torch.uint8)],
                                dim=0).contiguous().view(torch.float8_e4m3fn)
            self.shared_experts = Fp8DenseExpert(gate_up[:inter], shared["gate_s"][0].contiguous(), gate_up[inter:],
                                                 shared["up_s"][0].contiguous(), shared["down_q"][0].contiguous(),
                                                 shared["down_s"][0].contiguous(), gate_up=gate_up, layer_idx=layer_idx)
        self._routed: Optional[Fp8MoELayer] = None
        self._fused: Optional[Fp8MoELayer] = None
        # this class's own gate is a top-k: the ids of a row are pairwise different, so no expert can receive more
        # rows than there are tokens and a decode batch keeps the weight-streaming kernels.  A subclass that
        # replaces gate() with something that may repeat an id in a row must clear this.
        self._gate_ids_distinct = True

    # -- engines, built for the current token capacity ------------------------------------------------------------
    def _routed_layer(self, n_tokens: int) -> Fp8MoELayer:
        if self._routed is None or self._routed.n_max < n_tokens:
            cfg = _moe_config(self.config, n_tokens, self.experts_per_rank, self.routed_expert_start_idx, False)
            self._routed = Fp8MoELayer(cfg, self._weights, None, self.e_score_correction_bias, weights_repacked=True)
        return self._routed

    def _fused_layer(self, n_tokens: int) -> Fp8MoELayer:
        if self._fused is None or self._fused.n_max < n_tokens:
            cfg = _moe_config(self.config, n_tokens, self.experts_per_rank, self.routed_expert_start_idx,
                              self._shared is not None)
            self._fused = Fp8MoELayer(cfg, self._weights, self._shared, self.e_score_correction_bias,
                                      router_weight=self.gate_weight, weights_repacked=True)
        return self._fused

    def set_num_tokens_per_rank(self, num_tokens_per_rank: int):
        super().set_num_tokens_per_rank(num_tokens_per_rank)
        self._routed_layer(num_tokens_per_rank * self.world_size)

    # -- the template's pieces -----------------------------------------------------------------------------------
    def gate(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """Router GEMM + sigmoid + (group-limited) top-k + normalise + scale as one op that never writes the
        logits (``glm5_router_gemm_cuda`` then ``gate_sigmoid_topk_cuda`` in the reference, model.py:1119-1161)."""
        return router_gemm_gate_sigmoid_topk(x, self.gate_weight, self.e_score_correction_bias,
                                             k=self.num_experts_per_tok,
                                             routed_scaling_factor=float(self.config.routed_scaling_factor),
                                             n_group=self.n_group if self.n_group > 1 else 0,
                                             topk_group=self.topk_group if self.n_group > 1 else 0)

    def expert_compute_persistent(self, global_x, topk_idx, topk_weight):
        """Dispatch, quantise, gate_up + SwiGLU + requant, down, weighted combine of this rank's experts
        (``WGMMAMoEBuffers.forward``, batchgen/moe/fp8_wgmma_pipeline.py:294-372).  The result is a buffer of
        the layer, overwritten by the next call."""
        return self._routed_layer(global_x.size(0)).forward_routed(global_x, topk_idx, topk_weight,
                                                                   distinct_ids=self._gate_ids_distinct)

    def expert_compute_mixed(self, global_x, topk_idx, topk_weight):
        """Every expert of this build is resident, so the mixed path is the persistent one."""
        return self.expert_compute_persistent(global_x, topk_idx, topk_weight)

    def shared_expert_forward(self, identity, out=None, x_fp8=None, x_scale=None):
        """model.py:2726-2745: optional caller buffer and tokens already quantised by the norm kernel upstream."""
        if self.shared_experts is None:
            return torch.zeros_like(identity)
        return self.shared_experts(identity, out=out, x_fp8=x_fp8, x_scale=x_scale)

    @torch.inference_mode()
    def _forward_prefill(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """Prefill with every expert local: the same three steps on the tokens as they are (no padding)."""
        orig_shape = hidden_states.shape
        x = hidden_states.view(-1, hidden_states.shape[-1])
        if not x.is_contiguous():
            x = x.contiguous()
        topk_idx, topk_weight = self.gate(x)
        out = self.expert_compute_persistent(x, topk_idx, topk_weight)
        out = out + self.shared_expert_forward(x)
        return out.view(*orig_shape)

    @torch.inference_mode()
    def forward_fused(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """The whole layer as one library call (``bgmoe_moe_fp8_layer_forward`` with the router weight)."""
        orig_shape = hidden_states.shape
        x = hidden_states.view(-1, hidden_states.shape[-1])
        if not x.is_contiguous():
            x = x.contiguous()
        return self._fused_layer(x.size(0))(x).view(*orig_shape)
