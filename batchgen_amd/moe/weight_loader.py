"""Checkpoint tensors -> the stacked expert weights the MoE layers take.

What the reference does at load time, restated for this build's layers:

* FP8 block-quantised checkpoints name an expert's three projections
  ``{prefix}.experts.{e}.{gate,up,down}_proj.weight`` (e4m3fn ``[N, K]``) with the dequantisation scales
  next to them as ``...weight_scale_inv`` (fp32 ``[N/128, K/128]``, a multiplier)
  (batchgen/models/deepseek/deepseekv3/Parallel_Strategy_Manager.py:1072-1090,
  batchgen/models/deepseek/deepseekv3/wrappers.py:87-107); the shared expert sits under
  ``{prefix}.shared_experts.``, the router under ``{prefix}.gate.weight`` and
  ``{prefix}.gate.e_score_correction_bias``.
* The per-expert tensors are stacked into ``[E_l, I, H]`` / ``[E_l, H, I]`` blocks plus scale stacks
  (batchgen/models/glm/glm5/model.py:1991-2277).  The stack is allocated once and filled one expert at a
  time, with the source released as soon as it is copied, so that the peak is one stack plus one expert
  rather than two copies of every weight (:2023-2035).  The scale stacks' trailing axis is either exact
  (``K/128``) or padded to a multiple of 4 with zeros (:2003-2006, :2189-2217); the kernels here read
  either through the scale row stride.  ``fuse_gate_up=True`` builds the one ``[E_l, 2I, H]`` block with
  gate in rows ``[0, I)`` and up in ``[I, 2I)`` of each expert (:2104-2137) and hands out the two halves as
  strided views of it.
* MXFP4 checkpoints name a projection's two tensors ``w{1,2,3}.weight_packed`` (uint8 ``[N, K/2]``, low
  nibble = even K) and ``w{1,2,3}.weight_scale`` (uint8 E8M0 ``[N, K/32]``), with w1 = gate, w2 = down,
  w3 = up (batchgen/models/moonshotai/kimi_linear/k3/mxfp4_expert.py:239-303).

``state`` is any mapping from tensor name to tensor: a dict, or :class:`SafetensorsSource` over one or more
``.safetensors`` files (tensors are read one at a time, never the whole file).
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, Mapping, Optional, Sequence

import torch

FP8_PROJ = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}
MXFP4_PROJ = {"gate": "w1", "down": "w2", "up": "w3"}
BLOCK = 128


class WeightLayoutError(RuntimeError):
    pass


class SafetensorsSource(Mapping):
    """Name -> tensor over ``.safetensors`` files, loading one tensor per access."""

    def __init__(self, paths: Iterable[str], device: str = "cpu"):
        from safetensors import safe_open
        self._device = device
        self._handles = []
        self._where: Dict[str, int] = {}
        for p in ([paths] if isinstance(paths, str) else list(paths)):
            h = safe_open(p, framework="pt", device=device)
            for name in h.keys():
                self._where[name] = len(self._handles)
            self._handles.append(h)

    def __getitem__(self, name: str) -> torch.Tensor:
        return self._handles[self._where[name]].get_tensor(name)

    def __iter__(self):
        return iter(self._where)

    def __len__(self):
        return len(self._where)


def _need(state: Mapping, name: str) -> torch.Tensor:
    try:
        return state[name]
    except KeyError:
        raise WeightLayoutError(f"checkpoint has no tensor {name!r}") from None


def _as_bytes(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8)
    if t.dtype != torch.uint8:
        raise WeightLayoutError(f"{name} must be float8_e4m3fn (or its bytes), got {t.dtype}")
    return t


def _pad4(x: int) -> int:
    return (x + 3) // 4 * 4


def stack_fp8_experts(state: Mapping[str, torch.Tensor], prefix: str, expert_ids: Sequence[int], hidden: int,
                      inter: int, device, scale_pad4: bool = False, fuse_gate_up: bool = False,
                      expert_fmt: str = "experts.{e}.", release: Optional[Callable[[str], None]] = None):
    """-> {gate_q, gate_s, up_q, up_s, down_q, down_s} for ``Fp8MoELayer``.

    ``gate_q``/``up_q`` are uint8 ``[E_l, inter, hidden]``, ``down_q`` ``[E_l, hidden, inter]``; the scale stacks
    are fp32 ``[E_l, N/128, K/128]`` (trailing axis padded to a multiple of 4 when ``scale_pad4``: the returned
    tensors are then views ``[..., :K/128]`` of the padded storage, with the padded row stride).
    ``release(name)`` is called after a tensor has been copied into its stack."""
    if hidden % BLOCK or inter % BLOCK:
        raise WeightLayoutError(f"hidden={hidden} and inter={inter} must be multiples of {BLOCK}")
    el = len(expert_ids)
    dev = torch.device(device)
    shapes = {"gate": (inter, hidden), "up": (inter, hidden), "down": (hidden, inter)}
    out: Dict[str, torch.Tensor] = {}
    if fuse_gate_up:
        block = torch.empty((el, 2 * inter, hidden), dtype=torch.uint8, device=dev)
        out["gate_up_q"] = block
        out["gate_q"], out["up_q"] = block[:, :inter, :], block[:, inter:, :]
        kb = hidden // BLOCK
        kbp = _pad4(kb) if scale_pad4 else kb
        sblock = torch.zeros((el, 2 * (inter // BLOCK), kbp), dtype=torch.float32, device=dev)
        out["gate_up_s"] = sblock
        out["gate_s"], out["up_s"] = sblock[:, :inter // BLOCK, :kb], sblock[:, inter // BLOCK:, :kb]
    for name, (n, k) in shapes.items():
        if name + "_q" not in out:
            out[name + "_q"] = torch.empty((el, n, k), dtype=torch.uint8, device=dev)
            kb = k // BLOCK
            kbp = _pad4(kb) if scale_pad4 else kb
            out[name + "_s"] = torch.zeros((el, n // BLOCK, kbp), dtype=torch.float32, device=dev)[:, :, :kb]
        for i, e in enumerate(expert_ids):
            wname = f"{prefix}{expert_fmt.format(e=e)}{FP8_PROJ[name]}.weight"
            sname = wname + "_scale_inv"
            w = _as_bytes(_need(state, wname), wname)
            if tuple(w.shape) != (n, k):
                raise WeightLayoutError(f"{wname} is {tuple(w.shape)}, expected {(n, k)}")
            out[name + "_q"][i].copy_(w)
            s = _need(state, sname)
            if s.dtype != torch.float32 or tuple(s.shape) != (n // BLOCK, k // BLOCK):
                raise WeightLayoutError(f"{sname} must be fp32 {(n // BLOCK, k // BLOCK)}, got {s.dtype} "
                                        f"{tuple(s.shape)}")
            out[name + "_s"][i].copy_(s)
            del w, s
            if release is not None:
                release(wname)
                release(sname)
    return out


def load_fp8_moe_layer_weights(state: Mapping[str, torch.Tensor], prefix: str, e_total: int, expert_start: int,
                               e_local: int, hidden: int, inter: int, device, shared_inter: int = 0,
                               scale_pad4: bool = False, release: Optional[Callable[[str], None]] = None):
    """Everything one FP8 MoE layer needs from a checkpoint: (experts, shared-or-None, bias, router_weight).

    ``prefix`` is the MoE module's name with the trailing dot, e.g. ``"model.layers.3.mlp."``."""
    experts = stack_fp8_experts(state, prefix, range(expert_start, expert_start + e_local), hidden, inter, device,
                                scale_pad4=scale_pad4, release=release)
    shared = None
    if shared_inter:
        shared = stack_fp8_experts(state, prefix, [0], hidden, shared_inter, device, scale_pad4=scale_pad4,
                                   expert_fmt="shared_experts.", release=release)
    bias = _need(state, prefix + "gate.e_score_correction_bias").to(device=device, dtype=torch.float32).contiguous()
    rw = _need(state, prefix + "gate.weight")
    if bias.numel() != e_total or tuple(rw.shape) != (e_total, hidden):
        raise WeightLayoutError(f"router tensors do not match {e_total} experts x {hidden}: bias {tuple(bias.shape)}, "
                                f"weight {tuple(rw.shape)}")
    return experts, shared, bias, rw.to(device=device, dtype=torch.bfloat16).contiguous()


def stack_mxfp4_experts(state: Mapping[str, torch.Tensor], prefix: str, expert_ids: Sequence[int], hidden: int,
                        inter: int, device, expert_fmt: str = "experts.{e}.",
                        release: Optional[Callable[[str], None]] = None):
    """-> {gate_p, gate_s, up_p, up_s, down_p, down_s} (checkpoint byte layout, stacked) for ``Mxfp4MoELayer``."""
    if hidden % 32 or inter % 32:
        raise WeightLayoutError(f"hidden={hidden} and inter={inter} must be multiples of the MXFP4 group size 32")
    el = len(expert_ids)
    dev = torch.device(device)
    shapes = {"gate": (inter, hidden), "up": (inter, hidden), "down": (hidden, inter)}
    out: Dict[str, torch.Tensor] = {}
    for name, (n, k) in shapes.items():
        p = torch.empty((el, n, k // 2), dtype=torch.uint8, device=dev)
        s = torch.empty((el, n, k // 32), dtype=torch.uint8, device=dev)
        for i, e in enumerate(expert_ids):
            base = f"{prefix}{expert_fmt.format(e=e)}{MXFP4_PROJ[name]}."
            for suffix, dst, cols in (("weight_packed", p, k // 2), ("weight_scale", s, k // 32)):
                t = _need(state, base + suffix)
                if t.dtype != torch.uint8 or tuple(t.shape) != (n, cols):
                    raise WeightLayoutError(f"{base + suffix} must be uint8 {(n, cols)}, got {t.dtype} "
                                            f"{tuple(t.shape)}")
                dst[i].copy_(t)
                del t
                if release is not None:
                    release(base + suffix)
        out[name + "_p"], out[name + "_s"] = p, s
    return out


def export_fp8_moe_layer(prefix: str, experts: Mapping[str, torch.Tensor], shared, bias: torch.Tensor,
                         router_weight: torch.Tensor, expert_start: int = 0) -> Dict[str, torch.Tensor]:
    """The inverse of :func:`load_fp8_moe_layer_weights`: per-expert checkpoint tensors from stacks (used to
    write test checkpoints and to round-trip a layer)."""
    out: Dict[str, torch.Tensor] = {}

    def put(base, stacks, i):
        for name, proj in FP8_PROJ.items():
            out[f"{base}{proj}.weight"] = stacks[name + "_q"][i].contiguous().cpu().view(torch.float8_e4m3fn)
            out[f"{base}{proj}.weight_scale_inv"] = stacks[name + "_s"][i].contiguous().cpu()
    for i in range(experts["gate_q"].size(0)):
        put(f"{prefix}experts.{expert_start + i}.", experts, i)
    if shared is not None:
        put(f"{prefix}shared_experts.", shared, 0)
    out[prefix + "gate.e_score_correction_bias"] = bias.detach().float().cpu().contiguous()
    out[prefix + "gate.weight"] = router_weight.detach().cpu().contiguous()
    return out
