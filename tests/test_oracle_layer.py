"""The oracle's layer composition (CPU only): dense brute force on a tiny layer, the golden fixture of
config 0, and the relation between the quantised-activation oracle and the reference's CPU path."""
import os

import numpy as np
import torch

from batchgen_amd import workloads as wl
from oracle import gemm as og
from oracle import layer as ol
from oracle import quant as oq

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c0_layer.npz")


def _tiny():
    return wl.scaled(wl.CONFIGS[0], n_tokens=24, hidden=256, inter=128, shared_inter=128, max_tokens=24)


def _rcfg(cfg):
    return dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf)


def test_layer_equals_dense_per_token_bruteforce():
    cfg = _tiny()
    inp = wl.make_inputs(cfg, "cpu")
    w, _ = wl.make_fp8_weights(cfg, "cpu")
    wn = {k: v[4:12] for k, v in wl.weights_to_numpy(w).items()}       # this rank holds experts 4..11
    for layout, kw in (("masked", dict(max_tokens=24)), ("ragged", dict(row_align=64))):
        ref = ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(), _rcfg(cfg), wn, 4, 8,
                               layout=layout, shared=None, **kw)

        def expert(le, xrow):
            xq, xs = oq.act_quant(xrow)
            one, zero = np.array([1]), np.array([0, 1])
            y, _, _, _ = og.expert_mlp_fp8(xq, xs, wn["gate_q"][le:le + 1], wn["gate_s"][le:le + 1],
                                           wn["up_q"][le:le + 1], wn["up_s"][le:le + 1], wn["down_q"][le:le + 1],
                                           wn["down_s"][le:le + 1], one, zero)
            return y

        dense = ol.moe_layer_dense_bruteforce(inp["x"], ref["ids"], ref["weights"], expert, 4, 8)
        assert og.rel_frobenius(ref["out"], oq.bf16_round(dense)) < 2e-3
        local = (ref["ids"] >= 4) & (ref["ids"] < 12)
        assert ref["counts"].sum() == local.sum()


def test_config0_matches_golden_fixture():
    from tests.golden.make_c0_golden import compute
    got = compute()
    ref = np.load(GOLDEN)
    for k in ("x_sha", "logits_sha", "gate_q_sha", "down_s_sha", "xq_tok_sha"):
        assert str(got[k]) == str(ref[k]), k
    for k in ("ids", "counts", "pos"):
        assert np.array_equal(got[k], ref[k]), k
    assert np.array_equal(got["weights"].view(np.uint32), ref["weights"].view(np.uint32))
    assert np.array_equal(got["xs_tok"].view(np.uint32), ref["xs_tok"].view(np.uint32))
    assert og.rel_frobenius(got["out"], ref["out"]) < 1e-6          # matmul threading may reorder sums


def test_block_promoted_accumulation_equals_dequantise_then_matmul_up_to_rounding():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(20, 512, generator=g).to(torch.bfloat16)
    xq, xs = oq.act_quant(x)
    wq, ws = oq.weight_block_quant((0.02 * torch.randn(2, 256, 512, generator=g)).numpy())
    counts, cu = np.array([12, 8]), np.array([0, 12, 20])
    a = og.grouped_gemm_fp8(xq, xs, wq, ws, counts, cu, to_bf16=False)
    b = og.grouped_gemm_fp8_blockpromote(xq, xs, wq, ws, counts, cu)
    assert og.rel_frobenius(b, a) < 1e-6


def test_closed_form_constant_gemm():
    k, n = 512, 256
    xq = np.full((4, k), 0x38, dtype=np.uint8)
    xs = np.full((4, k // 128), 0.5, dtype=np.float32)
    wq = np.full((1, n, k), 0x28, dtype=np.uint8)
    ws = np.full((1, n // 128, k // 128), 0.01, dtype=np.float32)
    y = og.grouped_gemm_fp8(xq, xs, wq, ws, [4], [0, 4], to_bf16=False)
    np.testing.assert_allclose(y, k * 0.25 * 0.01 * 0.5, rtol=1e-6)


def test_cpu_reference_path_tracks_the_quantised_oracle():
    """The reference's CPU path (bf16 dequantised weights, unquantised activations) and the FP8-activation
    oracle differ by the activation quantisation noise only (a few percent)."""
    cfg = _tiny()
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    wn, shn = wl.weights_to_numpy(w), wl.weights_to_numpy(sh)
    ref = ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(), _rcfg(cfg), wn, 0, 16,
                           layout="masked", max_tokens=24, shared=shn)
    experts = [tuple(ol.l1_dequant_weights(wn[k + "_q"][e], wn[k + "_s"][e]) for k in ("gate", "up", "down"))
               for e in range(16)]
    shared = tuple(ol.l1_dequant_weights(shn[k + "_q"][0], shn[k + "_s"][0]) for k in ("gate", "up", "down"))
    y = ol.moe_layer_l1_torch(inp["x"], ref["ids"], ref["weights"], experts, 0, shared)
    err = og.rel_frobenius(y.float().numpy(), ref["out"])
    assert 1e-3 < err < 0.08
