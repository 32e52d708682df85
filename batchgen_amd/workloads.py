"""The five benchmark / parity workloads: shapes and seeded synthetic inputs.

Inputs are generated with torch on whatever device is asked for (CPU for the
small parity cases, the GPU for the full-size ones): activations N(0,1) -> bf16,
router logits fp32 N(0,1), correction bias 0.1*N(0,1), weights 0.02*N(0,1)
quantised per 128x128 block to e4m3fn with scale = max(amax,1e-10)/448 (the
reference tests' recipe, tests/test_glm52_deepgemm_masked_parity_gpu.py:80-87).
Seed = 20261125 + config index.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Optional

import torch

SEED0 = 20261125


@dataclass(frozen=True)
class MoEConfig:
    name: str
    index: int
    n_tokens: int
    hidden: int
    inter: int
    n_experts: int
    e_local: int
    expert_start: int
    top_k: int
    n_group: int          # 1 = ungrouped sigmoid top-k
    topk_group: int
    rsf: float
    shared_inter: int     # 0 = no shared expert
    layout: str           # "masked" | "ragged"
    max_tokens: int       # masked: per-expert row stride
    row_align: int        # ragged
    weight_format: str    # "fp8" | "mxfp4"
    zipf_s: float = 0.0
    latent: int = 0       # > 0: routed experts work on rows of this width (hidden -> latent -> hidden projections)
    activation: str = "swiglu"   # "swiglu" | "situ"
    latent_norm: bool = False    # RMSNorm between the combined latent rows and the latent -> hidden projection

    @property
    def seed(self) -> int:
        return SEED0 + self.index

    @property
    def expert_hidden(self) -> int:
        return self.latent or self.hidden


CONFIGS = {
    0: MoEConfig("c0_cpu_plumbing", 0, 64, 1024, 512, 16, 16, 0, 4, 4, 2, 1.0, 512, "masked", 64, 64, "fp8"),
    1: MoEConfig("c1_dsv3_fp8_decode_256tok_ep8_masked", 1, 256, 7168, 2048, 256, 32, 0, 8, 8, 4, 2.5, 2048,
                 "masked", 256, 64, "fp8"),
    2: MoEConfig("c2_dsv3_fp8_prefill_16k_ep8_ragged", 2, 16384, 7168, 2048, 256, 32, 0, 8, 8, 4, 2.5, 2048,
                 "ragged", 0, 128, "fp8"),
    3: MoEConfig("c3_k3_mxfp4_decode_512tok_ep32", 3, 512, 7168, 2048, 896, 28, 0, 16, 1, 1, 1.0, 2048,
                 "masked", 512, 16, "mxfp4"),
    4: MoEConfig("c4_dsv3_fp8_zipf_8k_all_experts", 4, 8192, 7168, 2048, 256, 256, 0, 8, 8, 4, 2.5, 2048,
                 "ragged", 0, 128, "fp8", zipf_s=1.2),
}

# The Kimi-K3 model's own MoE layer (config 3 is its benchmark stand-in with SwiGLU and no latent seam):
# hidden 7168 -> latent 3584 once per token, 896 MXFP4 experts of intermediate size 3072 with the SiTU
# activation on latent rows, fp32 combine, RMSNorm, latent -> hidden, plus one bf16 SiTU shared expert on the
# hidden rows (batchgen/models/moonshotai/kimi_linear/model.py:520-603, k3/mxfp4_expert.py:291-313).
K3_LATENT = MoEConfig("k3_latent_mxfp4_decode_512tok_ep32", 5, 512, 7168, 3072, 896, 28, 0, 16, 1, 1, 1.0, 3072,
                      "masked", 512, 16, "mxfp4", latent=3584, activation="situ", latent_norm=True)


def scaled(cfg: MoEConfig, **kw) -> MoEConfig:
    """A smaller copy of a config for parity runs (same routing structure)."""
    return replace(cfg, **kw)


def block_quant_fp8(w: torch.Tensor):
    """w [..., N, K] fp32 -> (e4m3fn [..., N, K], scale fp32 [..., N/128, K/128])."""
    *lead, n, k = w.shape
    wb = w.reshape(*lead, n // 128, 128, k // 128, 128)
    amax = wb.abs().amax(dim=(-3, -1))
    s = torch.clamp(amax, min=1e-10) / 448.0
    q = (wb / s[..., :, None, :, None]).clamp(-448.0, 448.0)
    return q.reshape(*lead, n, k).to(torch.float8_e4m3fn), s.to(torch.float32)


def _gen_fp8_stack(gen, e, n, k, device, std=0.02, chunk=4):
    q = torch.empty((e, n, k), dtype=torch.float8_e4m3fn, device=device)
    s = torch.empty((e, n // 128, k // 128), dtype=torch.float32, device=device)
    for i in range(0, e, chunk):
        j = min(e, i + chunk)
        w = torch.randn((j - i, n, k), generator=gen, device=device, dtype=torch.float32) * std
        q[i:j], s[i:j] = block_quant_fp8(w)
    return q, s


def zipf_logit_bias(cfg: MoEConfig, c: float, device) -> torch.Tensor:
    """log of the Zipf(s) pmf over a fixed pseudo-random expert ranking, times c."""
    g = torch.Generator().manual_seed(cfg.seed + 7)
    rank = torch.randperm(cfg.n_experts, generator=g).float() + 1.0
    pmf = rank.pow(-cfg.zipf_s)
    pmf = pmf / pmf.sum()
    return (c * pmf.log()).to(device)


ZIPF_C = 0.67   # chosen so that about 30% of the experts get no token and the hottest gets > 2000 (config 4)


def make_inputs(cfg: MoEConfig, device, n_tokens: Optional[int] = None):
    """-> dict(x bf16 [N,H], logits fp32 [N,E], bias fp32 [E])."""
    n = cfg.n_tokens if n_tokens is None else n_tokens
    gen = torch.Generator(device="cpu").manual_seed(cfg.seed)
    x = torch.randn((n, cfg.hidden), generator=gen).to(torch.bfloat16)
    logits = torch.randn((n, cfg.n_experts), generator=gen)
    bias = 0.1 * torch.randn((cfg.n_experts,), generator=gen)
    if cfg.zipf_s > 0:
        logits = logits + zipf_logit_bias(cfg, ZIPF_C, "cpu")[None, :]
    return dict(x=x.to(device), logits=logits.to(device), bias=bias.to(device))


def make_fp8_weights(cfg: MoEConfig, device):
    """Local experts' FP8 weights (+ shared expert), generated on ``device``."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev).manual_seed(cfg.seed + 1)
    w = {}
    w["gate_q"], w["gate_s"] = _gen_fp8_stack(gen, cfg.e_local, cfg.inter, cfg.hidden, dev)
    w["up_q"], w["up_s"] = _gen_fp8_stack(gen, cfg.e_local, cfg.inter, cfg.hidden, dev)
    w["down_q"], w["down_s"] = _gen_fp8_stack(gen, cfg.e_local, cfg.hidden, cfg.inter, dev)
    sh = None
    if cfg.shared_inter:
        sh = {}
        sh["gate_q"], sh["gate_s"] = _gen_fp8_stack(gen, 1, cfg.shared_inter, cfg.hidden, dev)
        sh["up_q"], sh["up_s"] = _gen_fp8_stack(gen, 1, cfg.shared_inter, cfg.hidden, dev)
        sh["down_q"], sh["down_s"] = _gen_fp8_stack(gen, 1, cfg.hidden, cfg.shared_inter, dev)
    return w, sh


def quantize_mxfp4(w: torch.Tensor):
    """w [..., K] fp32 -> (packed uint8 [..., K/2], e8m0 scale bytes [..., K/32]).  OCP MX closed form:
    shared exponent floor(log2(amax)) - 2, elements rounded to nearest-even e2m1, saturating at 6
    (torch restatement of oracle/mxfp4.py::quantize; equality is tested on the CPU)."""
    *lead, k = w.shape
    g = w.reshape(*lead, k // 32, 32)
    amax = g.abs().amax(dim=-1)
    e = torch.frexp(torch.where(amax > 0, amax, torch.ones_like(amax)))[1] - 1
    byte = torch.clamp(e - 2 + 127, 1, 254)
    byte = torch.where(amax > 0, byte, torch.full_like(byte, 127))
    scale = torch.ldexp(torch.ones_like(amax), byte - 127)
    a = (g / scale[..., None]).abs()
    code = torch.zeros_like(a, dtype=torch.uint8)
    for mid, tie_up in ((0.25, False), (0.75, True), (1.25, False), (1.75, True), (2.5, False), (3.5, True),
                        (5.0, False)):
        code += ((a >= mid) if tie_up else (a > mid)).to(torch.uint8)
    code = code | (torch.signbit(g).to(torch.uint8) << 3)
    code = code.reshape(*lead, k)
    packed = code[..., 0::2] | (code[..., 1::2] << 4)
    return packed.contiguous(), byte.to(torch.uint8).contiguous()


def make_mxfp4_weights(cfg: MoEConfig, device):
    """Local experts' MXFP4 weights (checkpoint layout) + a bf16 shared expert."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev).manual_seed(cfg.seed + 1)
    w = {}
    eh = cfg.expert_hidden
    for name, (n, k) in (("gate", (cfg.inter, eh)), ("up", (cfg.inter, eh)), ("down", (eh, cfg.inter))):
        p = torch.empty((cfg.e_local, n, k // 2), dtype=torch.uint8, device=dev)
        s = torch.empty((cfg.e_local, n, k // 32), dtype=torch.uint8, device=dev)
        for i in range(cfg.e_local):
            p[i], s[i] = quantize_mxfp4(torch.randn((n, k), generator=gen, device=dev) * 0.02)
        w[name + "_p"], w[name + "_s"] = p, s
    sh = None
    if cfg.shared_inter:
        sh = {}
        for name, (n, k) in (("gate", (cfg.shared_inter, cfg.hidden)), ("up", (cfg.shared_inter, cfg.hidden)),
                             ("down", (cfg.hidden, cfg.shared_inter))):
            sh[name] = (torch.randn((n, k), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    return w, sh


def make_latent_weights(cfg: MoEConfig, device):
    """The latent seam's bf16 tensors: down_proj [latent, hidden], up_proj [hidden, latent], norm weight [latent]
    (None without ``latent_norm``)."""
    dev = torch.device(device)
    gen = torch.Generator(device=dev).manual_seed(cfg.seed + 2)
    down = (torch.randn((cfg.latent, cfg.hidden), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    up = (torch.randn((cfg.hidden, cfg.latent), generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    norm = None
    if cfg.latent_norm:
        norm = (torch.randn(cfg.latent, generator=gen, device=dev) * 0.2 + 1.0).to(torch.bfloat16)
    return dict(down_proj=down, up_proj=up, norm_weight=norm, eps=1e-5)


def algorithmic_bytes_mxfp4(cfg: MoEConfig, active_experts: int, routed_rows: int) -> int:
    h, i, eh = cfg.hidden, cfg.inter, cfg.expert_hidden
    total = active_experts * (3 * eh * i // 2 + 3 * eh * i // 32)
    if cfg.shared_inter:
        total += 3 * h * cfg.shared_inter * 2
    total += cfg.n_tokens * h * 2 * 2 + routed_rows * (2 * eh + 2 * i) * 2
    if cfg.latent:     # the two projections' weights, and the latent rows written and read around the experts
        total += 2 * h * eh * 2 + cfg.n_tokens * eh * 2 * 4
    return int(total)


def weights_to_numpy(w):
    """torch weight dict -> numpy (bytes as uint8) for the CPU oracle."""
    if w is None:
        return None
    out = {}
    for k, v in w.items():
        v = v.detach().cpu()
        out[k] = (v.view(torch.uint8) if v.dtype == torch.float8_e4m3fn else v).numpy()
    return out


def algorithmic_bytes_fp8(cfg: MoEConfig, active_experts: int, routed_rows: int) -> int:
    """HBM bytes one layer pass must move: weights and scales of the experts that
    have tokens (+ shared expert), activations in and out, quantised rows."""
    h, i = cfg.hidden, cfg.inter
    per_expert = 3 * h * i + 3 * (h // 128) * (i // 128) * 4
    total = active_experts * per_expert
    if cfg.shared_inter:
        total += 3 * h * cfg.shared_inter + 3 * (h // 128) * (cfg.shared_inter // 128) * 4
    total += cfg.n_tokens * h * 2 * 2
    total += routed_rows * (h + i) * 3
    return int(total)


def flops_routed(cfg: MoEConfig, routed_rows: int) -> int:
    return int(routed_rows) * 6 * cfg.expert_hidden * cfg.inter
