"""The third parity bar of the layer: its output is no worse than the reference kernels' own rounding would be.

For configuration 0 and the scaled configurations 1, 2 and 4 the CPU oracle evaluates the layer four times: with
the intermediate rounded as the HIP kernels round it (variant i, the reference's Triton stage 1), as the reference's
fused CuTe stage 1 does (ii), as its DeepGEMM chains do (iii), and with no bf16 rounding at all (the fp32
dequantise-then-matmul yardstick).  Two errors are compared for the HIP output and for the two emulations of the
reference kernels: against the unrounded yardstick, and against the variant-i oracle that the layer's 1e-2 bound
is stated for.  All of them are printed."""
import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from oracle import gemm as og
from oracle import layer as ol
from tests.util import say

pytestmark = pytest.mark.gpu

CASES = {
    "c0": wl.CONFIGS[0],
    "c1_scaled": wl.scaled(wl.CONFIGS[1], hidden=1024, inter=512, shared_inter=512),
    "c2_scaled": wl.scaled(wl.CONFIGS[2], hidden=512, inter=256, shared_inter=256, n_tokens=3000),
    "c4_scaled": wl.scaled(wl.CONFIGS[4], hidden=256, inter=256, shared_inter=256, n_tokens=2048),
}
SLACK = 1.05      # err(HIP) <= max(err(ii), err(iii)) * SLACK


@pytest.mark.parametrize("name", list(CASES))
def test_layer_error_is_no_worse_than_the_reference_kernels_rounding(dev, name):
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = CASES[name]
    say("reference-error", name)
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    layer = Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()},
                        {k: v.to(dev) for k, v in sh.items()} if sh else None, inp["bias"].to(dev))
    hip = layer(inp["x"].to(dev), inp["logits"].to(dev)).float().cpu().numpy()
    rcfg = dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf)
    run = lambda v: ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(), rcfg,
                                     wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local, layout=cfg.layout,
                                     max_tokens=cfg.max_tokens, row_align=cfg.row_align,
                                     shared=wl.weights_to_numpy(sh), variant=v)["out"]
    out = {v: run(v) for v in ("fp32", "i", "ii", "iii")}
    out["hip"] = hip
    vs_fp32 = {v: og.rel_frobenius(out[v], out["fp32"]) for v in ("hip", "i", "ii", "iii")}
    vs_i = {v: og.rel_frobenius(out[v], out["i"]) for v in ("hip", "ii", "iii")}
    say("   rel. Frobenius error against the unrounded fp32 yardstick:", {k: f"{v:.3e}" for k, v in vs_fp32.items()})
    say("   rel. Frobenius error against the variant-i oracle:        ", {k: f"{v:.3e}" for k, v in vs_i.items()})
    assert vs_i["hip"] < 1e-2
    assert vs_fp32["hip"] <= max(vs_fp32["ii"], vs_fp32["iii"]) * SLACK
    assert vs_i["hip"] <= max(vs_i["ii"], vs_i["iii"])
