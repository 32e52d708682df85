"""The SiTU / latent-seam oracle pinned on the CPU: closed forms and limits of the activation, the documented
range of its gate factor, the library's own tanh/sigmoid in fp32, the branch-rounding order of the fused
epilogue, RMSNorm against a textbook evaluation, and the latent layer against a per-token dense evaluation."""
import math

import numpy as np
import torch
import torch.nn.functional as F

from batchgen_amd import workloads as wl
from oracle import gemm as og
from oracle import layer as ol
from oracle import mxfp4 as omx
from oracle import norm_quant as onq
from oracle import quant as oq
from oracle import situ as os_


def _bf16_ulp(v):
    v = np.abs(np.asarray(v, dtype=np.float32))
    e = np.floor(np.log2(np.maximum(v, 2.0 ** -126)))
    return np.exp2(e - 7).astype(np.float32)


def test_known_answers_and_limits():
    # hand evaluation with the math module at a few points (gate and up deliberately different)
    for g, u in ((4.0, 25.0), (1.0, 2.0), (2.0, 1.0), (-1.5, 3.0), (0.5, -40.0)):
        want = 4.0 * math.tanh(g / 4.0) / (1.0 + math.exp(-g)) * 25.0 * math.tanh(u / 25.0)
        assert abs(float(os_.situ_f64(g, u, 4.0, 25.0)) - want) <= 1e-15 * max(1.0, abs(want))
    assert float(os_.situ_f64(1.0, 2.0, 4.0, 25.0)) != float(os_.situ_f64(2.0, 1.0, 4.0, 25.0))   # order matters
    assert float(os_.situ_f64(0.0, 3.0, 4.0, 25.0)) == 0.0
    # saturation: gate -> +inf gives beta * up', gate -> -inf gives 0; up -> +-inf gives +-linear_beta
    assert abs(float(os_.situ_f64(80.0, 1.0, 4.0, None)) - 4.0) < 1e-12
    assert abs(float(os_.situ_f64(-80.0, 1.0, 4.0, None))) < 1e-30
    assert abs(float(os_.situ_f64(80.0, 1e6, 4.0, 25.0)) - 100.0) < 1e-9
    assert abs(float(os_.situ_f64(80.0, -1e6, 4.0, 25.0)) + 100.0) < 1e-9
    # odd in up, with and without the linear beta
    g = np.linspace(-9, 9, 37)
    u = np.linspace(-60, 60, 37)[::-1]
    for lb in (None, 25.0):
        assert np.array_equal(os_.situ_f64(g, -u, 4.0, lb), -os_.situ_f64(g, u, 4.0, lb))


def test_gate_factor_range_documented_by_the_reference_kernel():
    # "situ_a = 4 * tanh(g/4) * sigmoid(g)  in (-0.2698, 4)" (marlin_grouped_gemm.cu:247)
    g = np.linspace(-40.0, 40.0, 800001)
    a = os_.situ_f64(g, 1.0, 4.0, None)
    assert -0.2699 < a.min() < -0.2697 and 3.9999 < a.max() < 4.0
    # "u_c = 25 * tanh(u/25)  in (-25, 25)" (:248)
    uc = os_.situ_f64(80.0, np.linspace(-500, 500, 10001), 4.0, 25.0) / 4.0
    assert -25.0 <= uc.min() < -24.999 and 24.999 < uc.max() <= 25.0


def test_large_beta_reduces_to_swiglu():
    gen = torch.Generator().manual_seed(1)
    g = torch.randn(4096, generator=gen, dtype=torch.float64) * 3
    u = torch.randn(4096, generator=gen, dtype=torch.float64) * 3
    want = (F.silu(g) * u).numpy()
    got = os_.situ_f64(g.numpy(), u.numpy(), 1e9, None)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-15)


def test_module_form_matches_the_librarys_fp32_tanh_and_sigmoid():
    # the eager module's expression (kimi_linear/model.py:109-115) with torch's own fp32 routines
    gen = torch.Generator().manual_seed(2)
    for lb in (None, 25.0):
        x = (torch.randn(64, 2 * 384, generator=gen) * 3).to(torch.bfloat16)
        gate, up = x[:, :384].float(), x[:, 384:].float()
        a = 4.0 * torch.tanh(gate / 4.0) * torch.sigmoid(gate)
        if lb is not None:
            up = lb * torch.tanh(up / lb)
        want = (a * up).to(torch.bfloat16).float().numpy()
        got = os_.situ_and_mul(x, 4.0, lb)
        assert np.all(np.abs(got - want) <= _bf16_ulp(want))
        assert np.mean(got != want) < 5e-3


def test_fused_epilogue_rounds_both_branches_to_bf16_first():
    # 1 + 2^-8 is a tie between bf16 1.0 and 1.0078125 and rounds to even (1.0); 3 + 2^-7 + 2^-12 rounds up
    g = np.array([1.0 + 2.0 ** -8, 3.0 + 2.0 ** -7 + 2.0 ** -12], dtype=np.float32)
    u = np.array([2.0 - 2.0 ** -9, -5.0 - 2.0 ** -7], dtype=np.float32)
    gb = np.array([1.0, 3.015625], dtype=np.float32)
    ub = np.array([2.0, -5.0], dtype=np.float32)
    assert np.array_equal(oq.bf16_round(g), gb) and np.array_equal(oq.bf16_round(u), ub)
    want = oq.bf16_round(os_.situ_f64(gb, ub, 4.0, 25.0).astype(np.float32))
    assert np.array_equal(os_.situ_fused(g, u), want)
    # the order is observable: evaluating on the unrounded products gives other bf16 results somewhere
    gen = np.random.default_rng(4)
    g = gen.normal(0, 2, 4096).astype(np.float32)
    u = gen.normal(0, 2, 4096).astype(np.float32)
    late = oq.bf16_round(os_.situ_f64(g, u, 4.0, 25.0).astype(np.float32))
    assert np.mean(os_.situ_fused(g, u) != late) > 0.05


def test_rmsnorm_textbook_and_fixed_tree():
    gen = torch.Generator().manual_seed(3)
    x = (torch.randn(9, 3584, generator=gen) * 2).to(torch.bfloat16)
    w = (torch.randn(3584, generator=gen) * 0.2 + 1).to(torch.bfloat16)
    xd, wd = x.double(), w.double()
    want = (xd * torch.rsqrt((xd * xd).mean(-1, keepdim=True) + 1e-5) * wd).float().to(torch.bfloat16).float().numpy()
    got = os_.rmsnorm(x, w, 1e-5)
    assert np.array_equal(got, want)
    # constant rows: x = c everywhere -> c / sqrt(c^2 + eps) * w
    c = 3.0
    got_c = os_.rmsnorm(np.full((2, 256), c, dtype=np.float32), np.ones(256, dtype=np.float32), 1e-5)
    assert np.array_equal(got_c, oq.bf16_round(np.full((2, 256), c / math.sqrt(c * c + 1e-5), dtype=np.float32)))
    # the device's summation tree (fp32, fixed order) lands within one bf16 unit in the last place of it
    tree, _ = onq.add_rmsnorm(np.zeros_like(oq.as_f32(x)), x, w, 1e-5)
    assert np.all(np.abs(tree - got) <= _bf16_ulp(got)) and np.mean(tree != got) < 5e-3


def test_latent_layer_equals_dense_per_token_evaluation():
    cfg = wl.scaled(wl.K3_LATENT, n_tokens=12, hidden=256, latent=128, inter=96, n_experts=12, e_local=5,
                    expert_start=3, top_k=4, shared_inter=64, max_tokens=12)
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_mxfp4_weights(cfg, "cpu")
    lat = wl.make_latent_weights(cfg, "cpu")
    wn = wl.weights_to_numpy(w)
    shn = {k: v.float().numpy() for k, v in sh.items()}
    rcfg = dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf)
    ref = ol.moe_layer_mxfp4(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(), rcfg, wn, cfg.expert_start,
                             cfg.e_local, max_tokens=cfg.max_tokens, shared_bf16=shn, activation="situ", latent=lat)
    x = oq.as_f32(inp["x"])
    down, up = oq.as_f32(lat["down_proj"]), oq.as_f32(lat["up_proj"])
    x_lat = oq.bf16_round(x @ down.T)
    assert np.array_equal(ref["x_latent"], x_lat) and ref["x_rows"].shape[1] == cfg.latent
    deq = {n: [omx.dequant(wn[n + "_p"][e], wn[n + "_s"][e]) for e in range(cfg.e_local)] for n in ("gate", "up", "down")}

    def expert(e, row):
        h = os_.situ_fused(row @ deq["gate"][e].T, row @ deq["up"][e].T)
        return oq.bf16_round(h @ deq["down"][e].T)

    y_lat = oq.bf16_round(ol.moe_layer_dense_bruteforce(x_lat, ref["ids"], ref["weights"], expert, cfg.expert_start,
                                                        cfg.e_local))
    assert og.rel_frobenius(ref["y_latent"], y_lat) < 2e-3
    z = os_.rmsnorm(ref["y_latent"], lat["norm_weight"], lat["eps"])
    gu = np.concatenate([oq.bf16_round(x @ shn["gate"].T), oq.bf16_round(x @ shn["up"].T)], axis=-1)
    y_sh = oq.bf16_round(os_.situ_and_mul(gu, 4.0, 25.0) @ shn["down"].T)
    want = oq.bf16_round(oq.bf16_round(z @ up.T) + y_sh)
    assert og.rel_frobenius(ref["out"], want) < 2e-3
    # some routes leave this rank's experts: the layer is a partial sum, not the identity on any token
    assert (ref["pos"] < 0).any() and (ref["pos"] >= 0).any()
