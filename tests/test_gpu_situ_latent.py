"""The Kimi-K3 latent-MoE seam on the GPU: SiTU-and-multiply, RMSNorm, the SiTU epilogue of the MXFP4 stage-1
GEMM, and the latent layer, against the CPU oracle.

Tolerances.  SiTU is compared with its exact (float64) evaluation rounded once to bf16: every element within
one bf16 unit in the last place and fewer than 0.5 % of them different (the reference's own bar for its
Triton kernel is max|diff| <= max|ref| * 2^-7 + 1e-3 and < 2 % different,
tests/test_kimi_k3_situ_triton.py:25-28).  RMSNorm is bit-exact against the fixed-order restatement.  GEMM
outputs carry the accumulation-order freedom of fp32: relative Frobenius error as in the other MXFP4 tests."""
import ctypes as C

import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from oracle import gemm as og
from oracle import layer as ol
from oracle import mxfp4 as mx
from oracle import norm_quant as onq
from oracle import quant as oq
from oracle import situ as os_
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def _ulp(v):
    v = np.abs(np.asarray(v, dtype=np.float32))
    return np.exp2(np.floor(np.log2(np.maximum(v, 2.0 ** -126))) - 7).astype(np.float32)


def _close_bf16(got, want, frac=5e-3):
    assert np.all(np.abs(got - want) <= _ulp(want)), float(np.max(np.abs(got - want) / _ulp(want)))
    assert np.mean(got != want) < frac, float(np.mean(got != want))


@pytest.mark.parametrize("linear_beta", [None, 25.0])
@pytest.mark.parametrize("rows,d", [(1, 2048), (7, 1536), (64, 3072), (301, 1024), (5, 1001), (3, 5), (0, 64)])
def test_situ_and_mul_matches_exact_evaluation(dev, rows, d, linear_beta):
    from batchgen_amd.moe.latent import SituAndMul
    say("situ_and_mul", rows, d, linear_beta)
    g = torch.Generator().manual_seed(rows * 131 + d)
    x = rand_bf16(g, rows, 2 * d, scale=3.0)
    got = SituAndMul(4.0, linear_beta)(x.to(dev))
    assert got.shape == (rows, d) and got.dtype == torch.bfloat16
    if rows:
        _close_bf16(got.float().cpu().numpy(), os_.situ_and_mul(x, 4.0, linear_beta))


def test_situ_and_mul_strided_rows_extremes_and_leading_axes(dev):
    from batchgen_amd.moe.latent import situ_and_mul
    g = torch.Generator().manual_seed(9)
    wide = rand_bf16(g, 33, 4096, scale=3.0).to(dev)
    view = wide[:, 512:512 + 2 * 1024]                     # row stride 4096, 16-byte aligned start
    _close_bf16(situ_and_mul(view, 4.0, 25.0).float().cpu().numpy(), os_.situ_and_mul(view.cpu(), 4.0, 25.0))
    odd = wide[:, 3:3 + 2 * 1024]                          # misaligned start: the one-column path
    _close_bf16(situ_and_mul(odd, 4.0, 25.0).float().cpu().numpy(), os_.situ_and_mul(odd.cpu(), 4.0, 25.0))
    x3 = rand_bf16(g, 2, 5, 2 * 256, scale=2.0)
    y3 = situ_and_mul(x3.to(dev), 2.0, None)
    assert y3.shape == (2, 5, 256)
    _close_bf16(y3.float().cpu().numpy(), os_.situ_and_mul(x3, 2.0, None))
    # saturation and signed zeros: no NaN from exp overflow, gate -> -inf gives (signed) zero
    vals = torch.tensor([0.0, -0.0, 1e-30, 88.0, -88.0, 200.0, -200.0, 3e38, -3e38, 1.0], dtype=torch.float32)
    gate, up = torch.meshgrid(vals, vals, indexing="ij")
    xe = torch.cat([gate.reshape(1, -1), up.reshape(1, -1)], dim=1).to(torch.bfloat16)
    ye = situ_and_mul(xe.to(dev), 4.0, 25.0).float().cpu().numpy()
    want = os_.situ_and_mul(xe, 4.0, 25.0)
    assert np.all(np.isfinite(ye))
    assert np.all(np.abs(ye - want) <= _ulp(want) + 1e-37)


def test_situ_and_mul_rejects_bad_arguments(dev):
    from batchgen_amd._lib import lib, ptr
    from batchgen_amd.moe.latent import situ_and_mul
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        situ_and_mul(x.float(), 4.0, None)
    with pytest.raises(RuntimeError):
        situ_and_mul(x[:, :63], 4.0, None)
    with pytest.raises(RuntimeError, match="beta"):
        situ_and_mul(x, 0.0, None)
    y = torch.zeros(4, 32, dtype=torch.bfloat16, device=dev)
    assert lib().bgmoe_situ_and_mul(ptr(x), 4, 32, 32, 4.0, 0.0, ptr(y), 32, None) != 0    # stride < 2d


@pytest.mark.parametrize("rows,h", [(1, 3584), (37, 3584), (300, 7168), (5, 8), (9, 1000), (4, 8192)])
def test_rmsnorm_bit_exact(dev, rows, h):
    from batchgen_amd._lib import check, lib, ptr
    from batchgen_amd.moe.latent import rmsnorm
    say("rmsnorm", rows, h)
    g = torch.Generator().manual_seed(rows + h)
    x = rand_bf16(g, rows, h, scale=2.0)
    w = (torch.randn(h, generator=g) * 0.2 + 1).to(torch.bfloat16)
    want, _ = onq.add_rmsnorm(np.zeros((rows, h), dtype=np.float32), x, w, 1e-5)
    xd = x.to(dev)
    got = rmsnorm(xd, w.to(dev), 1e-5)
    assert np.array_equal(got.float().cpu().numpy(), want)
    assert np.all(np.abs(want - os_.rmsnorm(x, w, 1e-5)) <= _ulp(want))     # and close to the textbook value
    check(lib().bgmoe_rmsnorm(ptr(xd), ptr(w.to(dev)), rows, h, 1e-5, ptr(xd), None))      # in place
    assert np.array_equal(xd.float().cpu().numpy(), want)


def _mg():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_marlin_grouped_gemm")


def _selection_weight(n, k, cols):
    """MXFP4 weight [1, n, k] whose row r is 1.0 at column cols[r] and 0 elsewhere (e2m1 code 2, scale 2^0)."""
    codes = np.zeros((n, k), dtype=np.uint8)
    codes[np.arange(n), cols] = 2
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    scales = np.full((n, k // 32), 127, dtype=np.uint8)
    assert np.array_equal(mx.dequant(packed, scales), (codes == 2).astype(np.float32))
    return packed[None], scales[None]


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
def test_fused_s1_situ_epilogue_on_exact_products(dev, layout):
    """Selection weights make gate[t, c] = x[t, a(c)] and up[t, c] = x[t, b(c)] exactly, so the output is the
    epilogue alone: SiTU of two known bf16 numbers (gate and up distinguishable: a swap fails)."""
    n, k, m = 256, 512, 48
    rng = np.random.default_rng(11)
    a, b = rng.permutation(k)[:n], rng.permutation(k)[:n]
    g = torch.Generator().manual_seed(12)
    x = rand_bf16(g, m, k, scale=3.0)
    (gp, gs), (up, us) = _selection_weight(n, k, a), _selection_weight(n, k, b)
    d = lambda t: torch.from_numpy(t).to(dev)
    gpd, gsd, upd, usd = d(gp), d(gs), d(up), d(us)
    if layout == "tile_major":
        gpd, gsd = _mg().mxfp4_weight_repack(gpd, gsd)
        upd, usd = _mg().mxfp4_weight_repack(upd, usd)
    cnt, cu = d(np.array([m], dtype=np.int32)), d(np.array([0, m], dtype=np.int32))
    h = _mg().mxfp4_fused_s1(x.to(dev), gpd, gsd, upd, usd, cnt, cu, weight_layout=layout, activation="situ")
    xf = oq.as_f32(x)
    want = os_.situ_fused(xf[:, a], xf[:, b])
    _close_bf16(h.float().cpu().numpy(), want)
    swapped = os_.situ_fused(xf[:, b], xf[:, a])
    assert np.mean(h.float().cpu().numpy() != swapped) > 0.5
    # the same call with the default activation still is SwiGLU
    h0 = _mg().mxfp4_fused_s1(x.to(dev), gpd, gsd, upd, usd, cnt, cu, weight_layout=layout)
    assert og.rel_frobenius(h0.float().cpu().numpy(), oq.silu_f32(xf[:, a]) * xf[:, b]) < 3e-3


@pytest.mark.parametrize("counts,n,k", [((0, 1, 15, 16, 17, 33, 70), 256, 512), ((9, 40, 3), 3072, 3584)])
def test_fused_s1_situ_and_reference_op_name(dev, counts, n, k):
    say("mxfp4 situ", counts, n, k)
    counts = np.asarray(counts, dtype=np.int32)
    cu = np.concatenate([[0], np.cumsum((counts + 15) // 16 * 16)]).astype(np.int32)
    m, e = int(cu[-1]), len(counts)
    g = torch.Generator().manual_seed(n + k)
    x = rand_bf16(g, m, k).to(dev)
    rng = np.random.default_rng(7)
    gp, gs = mx.quantize((0.03 * rng.standard_normal((e, n, k))).astype(np.float32))
    up, us = mx.quantize((0.03 * rng.standard_normal((e, n, k))).astype(np.float32))
    d = lambda t: torch.from_numpy(t).to(dev)
    gpt, gst = _mg().mxfp4_weight_repack(d(gp), d(gs))
    upt, ust = _mg().mxfp4_weight_repack(d(up), d(us))
    cnt_d = d(counts)
    live = np.zeros(m, dtype=bool)
    for i, c in enumerate(counts):
        live[cu[i]:cu[i] + c] = True
    h = _mg().mxfp4_fused_s1(x, gpt, gst, upt, ust, cnt_d, d(cu), weight_layout="tile_major", activation="situ")
    gate = og.grouped_gemm_mxfp4(oq.as_f32(x), gp, gs, counts, cu, to_bf16=False)
    upv = og.grouped_gemm_mxfp4(oq.as_f32(x), up, us, counts, cu, to_bf16=False)
    href = os_.situ_fused(gate, upv)
    err = og.rel_frobenius(h.float().cpu().numpy()[live], href[live])
    say("   rel frobenius", err)
    assert err < 4e-3
    # the reference's op (pointer tables, per-expert output bases) is the same kernel with SiTU selected
    tbl = lambda t: torch.tensor([t[i].data_ptr() for i in range(e)], dtype=torch.int64, device=dev)
    c = torch.zeros((m, n), dtype=torch.bfloat16, device=dev)
    c_ptrs = torch.tensor([c[int(cu[i])].data_ptr() for i in range(e)], dtype=torch.int64, device=dev)
    _mg().grouped_marlin_gemm_m16_s1_mxfp4_situ(x, tbl(gpt), tbl(upt), c_ptrs, tbl(gst), tbl(ust), d(cu[:e].copy()),
                                                cnt_d, e, n, k, None, n // 256, 4)
    lv = torch.from_numpy(live).to(dev)
    assert torch.equal(c[lv], h[lv])


def _latent_case(cfg, dev, sample=None, backend="vendor"):
    from batchgen_amd.moe.mxfp4_layer import Mxfp4MoELayer
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_mxfp4_weights(cfg, dev)
    lat = wl.make_latent_weights(cfg, dev)
    layer = Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat, dense_backend=backend)
    x, logits = inp["x"], inp["logits"]
    out = layer(x, logits).clone()
    assert out.shape == (cfg.n_tokens, cfg.hidden) and torch.isfinite(out.float()).all()
    assert torch.equal(out, layer(x, logits))                      # deterministic
    sub = torch.arange(cfg.n_tokens, device=dev) if sample is None else torch.tensor(sample, device=dev)
    ref = ol.moe_layer_mxfp4(x[sub].cpu(), logits[sub].cpu().numpy(), inp["bias"].cpu().numpy(),
                             dict(top_k=cfg.top_k, n_group=1, topk_group=1, rsf=cfg.rsf),
                             {k: v.cpu().numpy() for k, v in w.items()}, cfg.expert_start, cfg.e_local,
                             layout="masked", max_tokens=cfg.max_tokens,
                             shared_bf16={k: v.float().cpu().numpy() for k, v in sh.items()}, activation="situ",
                             latent={k: (v.cpu() if torch.is_tensor(v) else v) for k, v in lat.items()})
    return layer, out, sub, ref


def check_latent_layer_against_oracle(dev, backend):
    cfg = wl.scaled(wl.K3_LATENT, n_tokens=96, hidden=512, latent=256, inter=384, shared_inter=384, n_experts=224,
                    e_local=28, expert_start=56, max_tokens=96)
    layer, out, sub, ref = _latent_case(cfg, dev, backend=backend)
    assert np.array_equal(layer.topk_ids.cpu().numpy(), ref["ids"])
    assert np.array_equal(layer.topk_pos.cpu().numpy(), ref["pos"])
    assert np.array_equal(layer.expert_counts.cpu().numpy(), ref["counts"])
    e_lat = og.rel_frobenius(layer.out[:cfg.n_tokens].float().cpu().numpy(), ref["y_latent"])
    err = og.rel_frobenius(out.float().cpu().numpy(), ref["out"])
    say("   latent layer rel frobenius: combined latent rows", e_lat, "output", err)
    assert e_lat < 1e-2 and err < 1e-2


def test_latent_situ_layer_matches_oracle(dev):
    """Projections and shared expert on the vendor GEMM here; the layer's default (this library's own bf16 GEMM):
    tests/test_gpu_x_dense_backend.py::test_mxfp4_layers_on_the_default_backend."""
    check_latent_layer_against_oracle(dev, "vendor")


def check_latent_layer_full_size_sample(dev, backend):
    """The Kimi-K3 layer at its real shape (512 tokens, 7168 -> 3584, 28 local experts of 3072, top-16 of 896):
    determinism on the whole batch and a sample of tokens against the oracle."""
    cfg = wl.K3_LATENT
    say("full size", cfg.name)
    inp = wl.make_inputs(cfg, "cpu")
    ids = ol.route(inp["logits"].numpy(), inp["bias"].numpy(), dict(top_k=cfg.top_k, n_group=1, topk_group=1, rsf=cfg.rsf))[0]
    local = (ids >= cfg.expert_start) & (ids < cfg.expert_start + cfg.e_local)
    hit = np.nonzero(local.sum(axis=1) >= 2)[0]
    sample = sorted(set([0, cfg.n_tokens - 1] + hit[:2].tolist()))
    say("   sample tokens", sample)
    layer, out, sub, ref = _latent_case(cfg, dev, sample, backend=backend)
    assert np.array_equal(layer.topk_ids[sub].cpu().numpy(), ref["ids"])
    err = og.rel_frobenius(out[sub].float().cpu().numpy(), ref["out"])
    say("   rel frobenius of the sample vs oracle:", err)
    assert err < 1e-2


def test_latent_situ_layer_full_size_sample(dev):
    check_latent_layer_full_size_sample(dev, "vendor")


def test_new_entry_points_reject_bad_arguments(dev):
    from batchgen_amd._lib import Mxfp4Weight, lib, ptr
    import ctypes as C
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=dev)
    w = torch.ones(64, dtype=torch.bfloat16, device=dev)
    y = torch.zeros_like(x)
    L = lib()
    assert L.bgmoe_rmsnorm(ptr(x), ptr(w), 4, 12, 1e-5, ptr(y), None) != 0                  # h not a multiple of 8
    assert b"multiple of 8" in L.bgmoe_last_error()
    assert L.bgmoe_rmsnorm(ptr(x), ptr(w), 4, 16384, 1e-5, ptr(y), None) != 0               # h too large
    assert L.bgmoe_rmsnorm(x.data_ptr() + 2, ptr(w), 4, 56, 1e-5, ptr(y), None) != 0        # misaligned rows
    assert L.bgmoe_rmsnorm(None, ptr(w), 4, 64, 1e-5, ptr(y), None) != 0
    assert L.bgmoe_rmsnorm(None, None, 0, 64, 1e-5, None, None) == 0                        # nothing to do
    assert L.bgmoe_selfcheck_sigmoid(0, 16, None, None, None) != 0
    assert L.bgmoe_selfcheck_scale_division(1, 16, None, None, None) != 0
    # an unknown activation code is refused before any launch
    cnt = torch.tensor([4], dtype=torch.int32, device=dev)
    cu = torch.tensor([0, 4], dtype=torch.int32, device=dev)
    xk = torch.zeros(4, 128, dtype=torch.bfloat16, device=dev)
    wp = torch.zeros(1, 128, 64, dtype=torch.uint8, device=dev)
    ws = torch.full((1, 128, 4), 127, dtype=torch.uint8, device=dev)
    out = torch.zeros(4, 128, dtype=torch.bfloat16, device=dev)
    desc = Mxfp4Weight(ptr(wp), 128 * 64, None, ptr(ws), 128 * 4, None, 0, 0)
    rc = L.bgmoe_mxfp4_fused_s1(ptr(xk), C.byref(desc), C.byref(desc), ptr(cnt), ptr(cu), 1, 4, 128, 128, ptr(out), None,
                                2, 0, None)
    assert rc != 0 and b"activation" in L.bgmoe_last_error()
    with pytest.raises(RuntimeError):
        _mg().mxfp4_fused_s1(xk, wp, ws, wp, ws, cnt, cu, activation="gelu")
    from batchgen_amd.moe.mxfp4_layer import Mxfp4MoELayer
    cfg = wl.scaled(wl.K3_LATENT, n_tokens=16, hidden=256, latent=128, inter=128, shared_inter=0, n_experts=32, e_local=4,
                    max_tokens=16)
    wts, _ = wl.make_mxfp4_weights(cfg, dev)
    bias = torch.zeros(cfg.n_experts, device=dev)
    with pytest.raises(ValueError):
        Mxfp4MoELayer(cfg, wts, None, bias)                                                 # latent weights missing
    lat = wl.make_latent_weights(cfg, dev)
    with pytest.raises(ValueError):
        Mxfp4MoELayer(cfg, wts, None, bias, latent=dict(lat, norm_weight=None))             # norm weight missing
    with pytest.raises(ValueError):
        Mxfp4MoELayer(wl.scaled(cfg, activation="gelu"), wts, None, bias, latent=lat)
