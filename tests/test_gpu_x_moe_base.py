"""The reference's layer template (``MoEBase``: gate -> expert compute -> + shared expert) filled in with this
build's FP8 kernels, instantiated from a model configuration object: against the one-call fused layer and
against the CPU oracle run on the same routes."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import layer as ol
from oracle import quant as oq
from tests.util import say

pytestmark = pytest.mark.gpu


def _model_config(phase="decode", n_group=4):
    return SimpleNamespace(hidden_size=512, moe_intermediate_size=256, n_routed_experts=16, num_experts_per_tok=4,
                           n_group=n_group, topk_group=2 if n_group > 1 else 1, routed_scaling_factor=2.5,
                           norm_topk_prob=True, n_shared_experts=1, phase=phase)


def _build(dev, n_group=4, phase="decode"):
    from batchgen_amd import workloads as wl
    from batchgen_amd.moe.moe_base import Fp8BlockwiseMoE
    wcfg = wl.scaled(wl.CONFIGS[0], n_tokens=64, hidden=512, inter=256, shared_inter=256, n_experts=16, e_local=16,
                     expert_start=0, top_k=4, max_tokens=64)
    w, sh = wl.make_fp8_weights(wcfg, "cpu")
    g = torch.Generator().manual_seed(77)
    gate_w = (torch.randn(16, 512, generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(16, generator=g) * 0.1
    layer = Fp8BlockwiseMoE(_model_config(phase, n_group), {k: v.to(dev) for k, v in w.items()},
                            {k: v.to(dev) for k, v in sh.items()}, gate_w.to(dev), bias.to(dev))
    x = (torch.randn(48, 512, generator=g)).to(torch.bfloat16)
    return layer, wcfg, w, sh, x


@pytest.mark.parametrize("n_group", [4, 1])
def test_template_layer_against_fused_layer_and_oracle(dev, n_group):
    from batchgen_amd import workloads as wl
    say("MoEBase template, n_group", n_group)
    layer, wcfg, w, sh, x = _build(dev, n_group)
    assert layer.world_size == 1 and layer.experts_per_rank == 16 and layer.routed_expert_start_idx == 0
    xd = x.to(dev)
    with pytest.raises(RuntimeError):
        layer(xd)                                                    # the token capacity was never announced
    layer.set_num_tokens_per_rank(64)
    out = layer(xd).clone()
    assert out.shape == xd.shape and out.dtype == torch.bfloat16
    ids, wts = layer.gate(xd)
    assert ids.dtype == torch.int32 and wts.dtype == torch.float32 and tuple(ids.shape) == (48, 4)
    fused = layer.forward_fused(xd).clone()
    assert torch.equal(layer._fused.topk_ids[:48], ids), "the fused call routes like gate()"
    a, b = out.float().cpu(), fused.float().cpu()
    # The template's shared expert is the reference's dense per-projection chain: gate and up leave their GEMM as
    # bf16, SiLU and product are bf16 operations (the oracle's variant "iii"), and its sum with the routed part is
    # rounded to bf16 twice.  The fused layer computes SwiGLU on the fp32 sums (variant "i") and adds everything in
    # fp32.  A few percent of the intermediate's e4m3 bytes land on the neighbouring value between the two, so the
    # two outputs differ by about one percent; each is held to the oracle of its own rounding.
    assert float((a - b).norm() / b.norm()) < 3e-2
    routes = (ids.cpu().numpy(), wts.cpu().numpy())
    wn, sn = wl.weights_to_numpy(w), wl.weights_to_numpy(sh)
    ref = ol.moe_layer_fp8(x, None, None, None, wn, 0, 16, layout="masked", max_tokens=64, shared=sn, routes=routes)
    routed = ol.moe_layer_fp8(x, None, None, None, wn, 0, 16, layout="masked", max_tokens=64, shared=None, routes=routes)
    dense = ol.moe_layer_fp8(x, None, None, None, wn, 0, 16, layout="masked", max_tokens=64, shared=sn, routes=routes,
                             variant="iii")["y_shared"]
    want_template = oq.bf16_round(oq.bf16_round(routed["out"]) + np.asarray(dense, dtype=np.float32)[:48])
    assert og.rel_frobenius(a.numpy(), want_template) < 1e-2
    assert og.rel_frobenius(b.numpy(), ref["out"]) < 1e-2
    # the shared buffer manager changes nothing; 3-D input keeps its shape; too many tokens raise
    type(layer).init_buffer_manager(64, 1, 512, torch.device(dev))
    try:
        assert torch.equal(layer(xd), out)
        assert torch.equal(layer(xd.view(4, 12, 512)).view(48, 512), out)
    finally:
        type(layer)._buffer_mgr = None
    with pytest.raises(RuntimeError):
        layer(torch.zeros(65, 512, dtype=torch.bfloat16, device=dev))


def test_template_layer_prefill_phase(dev):
    """``config.phase = 'prefill'``: the same three steps on the tokens as they are; equal to the decode template
    up to the row positions the routed kernels work at (the sums themselves are the same)."""
    layer, wcfg, w, sh, x = _build(dev, phase="prefill")
    xd = x.to(dev)
    pre = layer(xd).clone()
    layer.config.phase = "decode"
    layer.set_num_tokens_per_rank(64)
    dec = layer(xd)
    a, b = pre.float().cpu(), dec.float().cpu()
    assert float((a - b).norm() / b.norm()) < 2e-3
    pieces = layer.expert_compute_persistent(xd, *layer.gate(xd)) + layer.shared_expert_forward(xd)
    assert torch.equal(pieces, pre)
    assert torch.equal(layer.expert_compute_mixed(xd, *layer.gate(xd)), layer.expert_compute_persistent(xd, *layer.gate(xd)))


def test_distinct_ids_promise_changes_the_kernel_choice_not_the_result(dev):
    """``forward_routed(distinct_ids=True)`` (what the template's own top-k gate promises) bounds a group by the
    token count instead of tokens x k, so a decode batch needs no tiled launch; on routes that do keep the
    promise both forms give the same bits (no group here exceeds the rows every form streams)."""
    layer, wcfg, w, sh, x = _build(dev)
    layer.set_num_tokens_per_rank(64)
    xd = x.to(dev)
    ids, wts = layer.gate(xd)
    eng = layer._routed_layer(64)
    a = eng.forward_routed(xd, ids, wts, distinct_ids=False).clone()
    b = eng.forward_routed(xd, ids, wts, distinct_ids=True).clone()
    assert torch.equal(a, b)
    assert layer._gate_ids_distinct and torch.equal(layer.expert_compute_persistent(xd, ids, wts), b)
