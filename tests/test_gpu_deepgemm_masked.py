"""The masked m-grouped chain R1 -> act -> R2 behind the reference's `run_deepgemm_masked_moe`, checked the way the
reference's GPU parity test checks it (tests/test_glm52_deepgemm_masked_parity_gpu.py): every GEMM against the fp32
dequantise-then-matmul of the live rows with DeepGEMM's measure 1 - cosine < 1e-3 (here also rel. Frobenius
< 4e-3), at every tile-edge row count (0, 1, 15, 16, 17, 31, 32, 63, 64, 65, 127, 128) and at a ragged mix; the
activation bit for bit against the oracle applied to the GEMM's own bf16 output; rows at or beyond masked_m keep
their sentinels in every buffer."""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import quant as oq
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu

E, H, I, S = 8, 1024, 512, 128
EDGE_COUNTS = (0, 1, 15, 16, 17, 31, 32, 63, 64, 65, 127, 128)


def calc_diff(x, y) -> float:
    x, y = np.asarray(x, dtype=np.float64), np.asarray(y, dtype=np.float64)
    den = (x * x + y * y).sum()
    return 0.0 if den == 0 else float(1 - 2 * (x * y).sum() / den)


def mn_major(groups, rows, blocks, dev, fill=0.0):
    return torch.full((groups, blocks, rows), fill, dtype=torch.float32, device=dev).transpose(1, 2)


@pytest.fixture(scope="module")
def layer(dev):
    from batchgen_amd.moe.moe_deepgemm_masked import DeepGemmMaskedExpertWeights
    rng = np.random.default_rng(20261021)
    w13, s13 = oq.weight_block_quant((0.03 * rng.standard_normal((E, 2 * I, H))).astype(np.float32))
    w2, s2 = oq.weight_block_quant((0.03 * rng.standard_normal((E, H, I))).astype(np.float32))
    g = torch.Generator().manual_seed(3)
    x = rand_bf16(g, E * S, H)
    xq, xs = oq.act_quant(x, form="A")
    d = lambda a, dt=None: torch.from_numpy(a).to(dev) if dt is None else torch.from_numpy(a).to(dev).view(dt)
    weights = DeepGemmMaskedExpertWeights(d(w13, torch.float8_e4m3fn), d(s13), d(w2, torch.float8_e4m3fn), d(s2))
    weights.validate(num_experts=E, hidden_size=H, intermediate_size=I)
    x_scales = mn_major(E, S, H // 128, dev)
    x_scales.copy_(torch.from_numpy(xs.reshape(E, S, H // 128)))
    return dict(weights=weights, x_fp8=d(xq, torch.float8_e4m3fn).view(E, S, H), x_scales=x_scales, xq=xq, xs=xs,
                w13=oq.weight_block_dequant(w13, s13), w2=oq.weight_block_dequant(w2, s2))


def _run(layer, counts, dev):
    from batchgen_amd.moe.moe_deepgemm_masked import expected_m_per_expert, run_deepgemm_masked_moe
    masked_m = torch.tensor(counts, dtype=torch.int32, device=dev)
    buf = dict(gate_up_out=torch.full((E, S, 2 * I), 7.0, dtype=torch.bfloat16, device=dev),
               act_fp8=torch.full((E, S, I), 0xAB, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn),
               act_scales=mn_major(E, S, I // 128, dev, fill=-7.0),
               out=torch.full((E, S, H), 7.0, dtype=torch.bfloat16, device=dev))
    em = expected_m_per_expert(local_rows=S, world_size=1, topk=1, num_experts_global=E)
    res = run_deepgemm_masked_moe(x_fp8=layer["x_fp8"], x_scales=layer["x_scales"], weights=layer["weights"],
                                  masked_m=masked_m, expected_m=em, **buf)
    assert res is buf["out"]
    return buf


def _check(layer, counts, buf):
    gu = buf["gate_up_out"].float().cpu().numpy()
    aq = buf["act_fp8"].view(torch.uint8).cpu().numpy()
    asc = buf["act_scales"].cpu().numpy()
    out = buf["out"].float().cpu().numpy()
    xdeq = oq.act_dequant(layer["xq"], layer["xs"]).reshape(E, S, H)
    worst = {}
    for e, c in enumerate(counts):
        assert (gu[e, c:] == 7.0).all() and (aq[e, c:] == 0xAB).all() and (asc[e, c:] == -7.0).all() \
            and (out[e, c:] == 7.0).all(), f"expert {e}: a row at or beyond masked_m was written"
        if c == 0:
            continue
        r1 = xdeq[e, :c] @ layer["w13"][e].T
        worst["R1"] = max(worst.get("R1", 0.0), calc_diff(gu[e, :c], r1))
        assert og.rel_frobenius(gu[e, :c], r1) < 4e-3
        y, s, _ = oq.silu_mul_group_quant(gu[e, :c, :I], gu[e, :c, I:], "D")      # on the GEMM's own output
        assert np.array_equal(aq[e, :c], y) and np.array_equal(asc[e, :c], s), f"activation differs, expert {e}"
        r2 = oq.act_dequant(aq[e, :c], asc[e, :c]) @ layer["w2"][e].T
        worst["R2"] = max(worst.get("R2", 0.0), calc_diff(out[e, :c], r2))
        assert og.rel_frobenius(out[e, :c], r2) < 4e-3
    say("   ", counts, {k: f"{v:.2e}" for k, v in worst.items()})
    assert all(v < 1e-3 for v in worst.values())


@pytest.mark.parametrize("rows", EDGE_COUNTS)
def test_chain_at_every_tile_edge(dev, layer, rows):
    counts = [rows] * E
    _check(layer, counts, _run(layer, counts, dev))


def test_chain_with_a_ragged_mix_is_row_count_independent(dev, layer):
    counts = [128, 0, 1, 65, 17, 64, 3, 100]
    buf = _run(layer, counts, dev)
    _check(layer, counts, buf)
    # an expert's live rows do not depend on the other experts' counts: same bits as the uniform run
    full = _run(layer, [128] * E, dev)
    for e, c in enumerate(counts):
        assert torch.equal(buf["out"][e, :c], full["out"][e, :c])
        assert torch.equal(buf["act_fp8"].view(torch.uint8)[e, :c], full["act_fp8"].view(torch.uint8)[e, :c])


def test_layout_contract_is_enforced(dev, layer):
    from batchgen_amd.moe import moe_deepgemm_masked as m
    assert m.is_mn_major_tma_aligned(layer["x_scales"])
    assert not m.is_mn_major_tma_aligned(layer["x_scales"].contiguous())
    assert not m.is_mn_major_tma_aligned(mn_major(E, 6, 8, dev))                   # rows not padded to 4
    with pytest.raises(RuntimeError):
        m.require_mn_major_tma_aligned(layer["x_scales"].contiguous(), "x")
    with pytest.raises(ValueError):
        m.expected_m_per_expert(local_rows=0, world_size=1, topk=1, num_experts_global=8)
    assert m.expected_m_per_expert(local_rows=32, world_size=8, topk=8, num_experts_global=256) == 9
    w = layer["weights"]
    with pytest.raises(RuntimeError):
        w.validate(num_experts=E, hidden_size=H, intermediate_size=I * 2)
    padded = torch.zeros(E, 2 * I // 128, H // 128 + 4, device=dev)[..., :H // 128]
    with pytest.raises(RuntimeError):
        m.DeepGemmMaskedExpertWeights(w.gate_up_w, padded, w.down_w, w.down_scale).validate(
            num_experts=E, hidden_size=H, intermediate_size=I)
    masked_m = torch.zeros(E, dtype=torch.int32, device=dev)
    good = dict(x_fp8=layer["x_fp8"], x_scales=layer["x_scales"], weights=w, masked_m=masked_m, expected_m=16,
                gate_up_out=torch.zeros(E, S, 2 * I, dtype=torch.bfloat16, device=dev),
                act_fp8=torch.zeros(E, S, I, dtype=torch.float8_e4m3fn, device=dev),
                act_scales=mn_major(E, S, I // 128, dev), out=torch.zeros(E, S, H, dtype=torch.bfloat16, device=dev))
    m.run_deepgemm_masked_moe(**good)
    for key, bad in (("expected_m", 16.0), ("gate_up_out", good["gate_up_out"][:, :, :I]),
                     ("x_scales", layer["x_scales"].contiguous()),
                     ("act_scales", torch.zeros(E, S, I // 128, device=dev))):
        with pytest.raises(RuntimeError):
            m.run_deepgemm_masked_moe(**{**good, key: bad})


def test_contiguous_grouped_gemm_by_row_map(dev):
    """`grouped_fp8_deepgemm_gemm` / `m_grouped_fp8_gemm_nt_contiguous`: rows described by a row -> group map
    (128-aligned segment starts, -1 on padding, expert segments mapped to a permuted dense weight stack), both
    activation-scale layouts; padding rows keep their sentinel; a malformed map writes nothing."""
    from batchgen_amd._lib import check, lib, ptr
    from batchgen_amd.moe import grouped_fp8_deepgemm_moe as dg
    counts = np.array([0, 1, 127, 128, 129, 300, 0, 64], dtype=np.int32)
    cu = np.concatenate([[0], np.cumsum((counts + 127) // 128 * 128)]).astype(np.int32)
    g_, n, k = len(counts), 256, 512
    m = int(cu[-1]) + 128
    rng = np.random.default_rng(5)
    wq, ws = oq.weight_block_quant((0.05 * rng.standard_normal((g_, n, k))).astype(np.float32))
    ids = rng.permutation(g_).astype(np.int32)                        # expert segment e uses weight slot ids[e]
    gen = torch.Generator().manual_seed(6)
    x = rand_bf16(gen, m, k)
    xq, xs = oq.act_quant(x, form="A")
    d = lambda a: torch.from_numpy(a).to(dev)
    arena = d(wq).view(torch.float8_e4m3fn)
    stack = dg.dense_group_view([arena[i] for i in range(g_)])
    assert stack.data_ptr() == arena.data_ptr()
    layout = dg.build_grouped_layout(d(counts), d(cu), m, group_ids=d(ids))
    wdeq = oq.weight_block_dequant(wq, ws)
    xdeq = oq.act_dequant(xq, xs)
    live = layout.cpu().numpy() >= 0
    ref = np.zeros((m, n), dtype=np.float32)
    for e, c in enumerate(counts):
        ref[cu[e]:cu[e] + c] = xdeq[cu[e]:cu[e] + c] @ wdeq[ids[e]].T
    for rows_major in (True, False):
        out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
        scale = d(xs) if rows_major else d(np.ascontiguousarray(xs.T))
        res = dg.grouped_fp8_deepgemm_gemm(d(xq).view(torch.float8_e4m3fn), scale, stack, d(ws), output=out,
                                           grouped_layout=layout, x_scale_rows_major=rows_major)
        assert res is out
        o = out.float().cpu().numpy()
        assert (o[~live] == 7.0).all()
        assert calc_diff(o[live], ref[live]) < 1e-3 and og.rel_frobenius(o[live], ref[live]) < 4e-3
    # the map's segments on the device, and a malformed map (group 2 in two runs)
    seg = torch.full((2 * g_ + 2,), -5, dtype=torch.int32, device=dev)
    status = torch.full((1,), -5, dtype=torch.int32, device=dev)
    check(lib().bgmoe_layout_to_segments(ptr(layout), m, g_, ptr(seg), seg.data_ptr() + 4 * g_, ptr(status), None))
    seqs, starts = seg[:g_].cpu().numpy(), seg[g_:].cpu().numpy()
    assert int(status) == 0 and starts[g_] == m
    for e, c in enumerate(counts):
        assert seqs[ids[e]] == c and (c == 0 or starts[ids[e]] == cu[e])
    bad = layout.clone()
    bad[m - 1] = int(ids[2])
    check(lib().bgmoe_layout_to_segments(ptr(bad), m, g_, ptr(seg), seg.data_ptr() + 4 * g_, ptr(status), None))
    assert int(status) == 2 and int(seg[:g_].abs().sum()) == 0
    out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    dg.m_grouped_fp8_gemm_nt_contiguous((d(xq).view(torch.float8_e4m3fn), d(xs)), (stack, d(ws)), out, bad)
    assert (out.float() == 7.0).all()
    with pytest.raises(ValueError):
        dg.grouped_fp8_deepgemm_gemm(d(xq).view(torch.float8_e4m3fn), d(xs), stack, d(ws), output=out,
                                     grouped_layout=layout[:-1], x_scale_rows_major=True)
    with pytest.raises(ValueError):
        dg.m_grouped_fp8_gemm_nt_contiguous((d(xq).view(torch.float8_e4m3fn), d(xs)), (stack[:, :, :256], d(ws)), out, layout)


def test_deepseek_v3_decode_wrappers_with_pointer_arrays(dev):
    """`fused_fp8_moe_stage_1_tma_wrapper` and `fused_dequant_grouped_gemm_fp8_tma_wrapper`: 3-D masked operands,
    one weight tensor per expert behind device pointer arrays, MN-major and row-major activation scales."""
    from batchgen_amd.moe import grouped_gemm_kernel as gk
    e, m_max, k, n = 6, 64, 512, 256
    counts = [0, 1, 17, 64, 33, 5]
    rng = np.random.default_rng(9)
    gen = torch.Generator().manual_seed(10)
    x = rand_bf16(gen, e * m_max, k)
    xq, xs = oq.act_quant(x, form="A")
    d = lambda a: torch.from_numpy(a).to(dev)
    xq_d = d(xq).view(torch.float8_e4m3fn).view(e, m_max, k)
    scales = {"row-major": d(xs).view(e, m_max, k // 128),
              "MN-major": mn_major(e, m_max, k // 128, dev)}
    scales["MN-major"].copy_(scales["row-major"])
    def expert_weights(seed):
        q, s = oq.weight_block_quant((0.05 * np.random.default_rng(seed).standard_normal((e, n, k))).astype(np.float32))
        wl = [d(q[i]).view(torch.float8_e4m3fn) for i in range(e)]
        sl = [d(s[i]) for i in range(e)]
        tbl = lambda ts: torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)
        return wl, tbl(wl), sl, tbl(sl), oq.weight_block_dequant(q, s)
    gw, gp, gs, gsp, gd = expert_weights(1)
    uw, up_, us, usp, ud = expert_weights(2)
    cnt = torch.tensor(counts, dtype=torch.int32, device=dev)
    xdeq = oq.act_dequant(xq, xs).reshape(e, m_max, k)
    for name, sc in scales.items():
        out = torch.full((e, m_max, n), 7.0, dtype=torch.bfloat16, device=dev)
        res = gk.fused_fp8_moe_stage_1_tma_wrapper(xq_d, sc, gw, gp, uw, up_, gs, gsp, us, usp, cnt, e, out=out)
        assert res is out
        y = gk.fused_dequant_grouped_gemm_fp8_tma_wrapper(xq_d, sc, gw, gp, gs, gsp, cnt, e)
        o, yv = out.float().cpu().numpy(), y.float().cpu().numpy()
        for i, c in enumerate(counts):
            assert (o[i, c:] == 7.0).all() and (yv[i, c:] == 0.0).all(), name
            if c:
                g32, u32 = xdeq[i, :c] @ gd[i].T, xdeq[i, :c] @ ud[i].T
                assert og.rel_frobenius(o[i, :c], oq.swiglu_bf16(g32, u32)) < 5e-3, name
                assert og.rel_frobenius(yv[i, :c], g32) < 4e-3, name
    with pytest.raises(RuntimeError):
        gk.fused_dequant_grouped_gemm_fp8_tma_wrapper(xq_d, scales["row-major"], gw, gp.int(), gs, gsp, cnt, e)
    with pytest.raises(RuntimeError):
        gk.fused_dequant_grouped_gemm_fp8_tma_wrapper(xq_d, scales["row-major"], gw, gp, gs, gsp, cnt, e + 1)
