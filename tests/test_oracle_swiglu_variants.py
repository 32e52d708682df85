"""The SwiGLU rounding variants of the reference's three stage-1 implementations, pinned by a case worked out
step by step with the ``math`` module (float64) and a bf16 rounding written here with integer arithmetic -- not
by the oracle's own formula.  The case is chosen so that the three variants give three different bf16 results
and every rounding in the hand evaluation is far from its boundary (checked below), so float64 steps stand for
the float32 steps of the kernels without ambiguity."""
import math
import struct

import numpy as np

from oracle import gemm as og
from oracle import layer as ol
from oracle import quant as q
from batchgen_amd import workloads as wl


def bf16(x: float) -> float:
    """float -> nearest bf16 (ties to even), via the float32 bit pattern."""
    bits = struct.unpack("<I", struct.pack("<f", x))[0]
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return struct.unpack("<f", struct.pack("<I", bits))[0]


def margin(x: float) -> float:
    """distance of x from the nearest bf16 rounding boundary, in units of a bf16 ulp (0.5 = on a value)"""
    lo = bf16(x)
    ulp = 2.0 ** (math.floor(math.log2(abs(lo))) - 7)
    return abs(abs(x - lo) / ulp - 0.5)


G, U = 1.3883439302444458, 0.7889391779899597        # both exactly representable in float32


def test_variant_i_fp32_everything_one_round():
    # silu(G) = G / (1 + exp(-G)) = 1.3883439 / 1.2494886 = 1.1111297...; times U = 0.87661...
    p = G / (1.0 + math.exp(-G)) * U
    assert margin(p) > 0.001      # 65 float32 ulps: float64 steps decide like float32 steps
    assert bf16(p) == 0.875
    assert float(q.swiglu_bf16(np.float32([G]), np.float32([U]))[0]) == 0.875


def test_variant_ii_cute_gate_rounded_to_bf16_first():
    gb = bf16(G)
    assert gb == 1.390625                                 # 1.3883439 -> 178/128
    sig = 1.0 / (1.0 + math.exp(-gb))
    p = (gb * sig) * U
    assert margin(p) > 0.001      # 65 float32 ulps: float64 steps decide like float32 steps
    assert bf16(p) == 0.87890625
    assert float(q.swiglu_cute_bf16(np.float32([G]), np.float32([U]))[0]) == 0.87890625


def test_variant_iii_deepgemm_chain_bf16_everywhere():
    gb, ub = bf16(G), bf16(U)
    assert (gb, ub) == (1.390625, 0.7890625)
    s = gb / (1.0 + math.exp(-gb))
    assert margin(s) > 0.001      # 65 float32 ulps: float64 steps decide like float32 steps
    sb = bf16(s)
    assert sb == 1.1171875
    p = sb * ub                                           # exact in float64 (8 x 8 significant bits)
    assert margin(p) > 0.001      # 65 float32 ulps: float64 steps decide like float32 steps
    assert bf16(p) == 0.8828125
    got = q.silu_mul_bf16(q.bf16_round(np.float32([G])), q.bf16_round(np.float32([U])))
    assert float(got[0]) == 0.8828125


def test_fast_exp_argument_rounding_is_modelled():
    """__expf(x) = ex2.approx(x * log2e): the product is rounded to fp32 before the exponential.  At g = -88 the
    rounded product 126.95716 differs from the exact one by 2.4e-6, which moves exp by 1.7e-6 relative: fourteen
    fp32 ulps, and the emulation must show it (a plain expf(-g) would not)."""
    g = np.float32([-88.0])
    t = np.float32(88.0) * np.float32(1.4426950408889634)
    e_fast = np.float32(2.0 ** float(t))
    e_true = np.float32(math.exp(88.0))
    assert e_fast != e_true
    sig = np.float32(1.0) / (np.float32(1.0) + e_fast)
    want = q.bf16_round(np.float32([np.float32(np.float32(-88.0) * sig) * np.float32(3.0)]))
    assert np.array_equal(q.swiglu_cute_bf16(g, np.float32([3.0])), want)


def test_expert_mlp_variants_differ_only_in_the_intermediate():
    """On a tiny expert the four variants share the first GEMM; "iii" alone uses requant form D and bf16 gate/up;
    "fp32" alone leaves h and y unrounded."""
    rng = np.random.default_rng(5)
    m, k, n = 24, 256, 128
    x = q.bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    xq, xs = q.act_quant(x)
    wq = {}
    for name, shape in (("gate", (1, n, k)), ("up", (1, n, k)), ("down", (1, k, n))):
        wq[name] = q.weight_block_quant((rng.standard_normal(shape) * 0.05).astype(np.float32))
    cnt, cu = np.array([m], np.int32), np.array([0, m], np.int32)
    res = {v: og.expert_mlp_fp8(xq, xs, *wq["gate"], *wq["up"], *wq["down"], cnt, cu, variant=v)
           for v in ("i", "ii", "iii", "fp32")}
    g = og.grouped_gemm_fp8(xq, xs, *wq["gate"], cnt, cu, to_bf16=False)
    u = og.grouped_gemm_fp8(xq, xs, *wq["up"], cnt, cu, to_bf16=False)
    assert np.array_equal(res["i"][1], q.swiglu_bf16(g, u))
    assert np.array_equal(res["ii"][1], q.swiglu_cute_bf16(g, u))
    assert np.array_equal(res["iii"][1], q.silu_mul_bf16(q.bf16_round(g), q.bf16_round(u)))
    assert not np.array_equal(res["fp32"][1], q.bf16_round(res["fp32"][1]))     # h kept in fp32
    assert not np.array_equal(res["fp32"][0], q.bf16_round(res["fp32"][0]))     # y kept in fp32
    for v in ("i", "ii", "iii"):
        assert np.array_equal(res[v][0], q.bf16_round(res[v][0]))
        assert og.rel_frobenius(res[v][0], res["fp32"][0]) < 5e-2   # K = 128 in the second product: little averaging
    # form D stores amax/448 with amax floored at 1e-10: equal to form C's scale here, where no block is zero
    hq_d, hs_d, _ = q.silu_mul_group_quant(q.bf16_round(g), q.bf16_round(u), "D")
    assert np.array_equal(res["iii"][2], hq_d) and np.array_equal(res["iii"][3], hs_d)


def test_layer_variants_on_config0():
    """What the reference kernels' own rounding costs at layer level.  Any change of the bf16 intermediate moves
    about one value in a hundred across an FP8 rounding boundary of the requantiser, and one such flip is an
    eighth of the value: every variant sits 1-2e-2 from the unrounded yardstick and from each other, far above
    the 1e-3 that separates two evaluations of the SAME variant (the HIP kernels against variant "i")."""
    cfg = wl.CONFIGS[0]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    rcfg = dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf)
    run = lambda v: ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(), rcfg,
                                     wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local, layout=cfg.layout,
                                     max_tokens=cfg.max_tokens, shared=wl.weights_to_numpy(sh), variant=v)["out"]
    out = {v: run(v) for v in ("fp32", "i", "ii", "iii")}
    errs = {v: og.rel_frobenius(out[v], out["fp32"]) for v in ("i", "ii", "iii")}
    vs_i = {v: og.rel_frobenius(out[v], out["i"]) for v in ("ii", "iii")}
    print("config 0, error of each rounding variant against the unrounded fp32 yardstick:", errs)
    print("config 0, distance of the reference kernels' variants from variant i:", vs_i)
    assert all(3e-3 < e < 3e-2 for e in errs.values())
    assert all(3e-3 < e < 3e-2 for e in vs_i.values())
