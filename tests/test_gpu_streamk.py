"""The balanced (stream-K) form of the weight-streaming grouped GEMMs on the GPU: the same results as the
item-per-block form up to the order in which an item's K-chain is summed (an item cut over several blocks is
summed in pieces), for group sizes that make every kind of cut, and bit-for-bit reproducible from run to run."""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import layer as ol
from tests.util import say

pytestmark = pytest.mark.gpu


def gm():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_fp8_blockwise_gemm")


def _pad4(s):
    kb = s.size(2)
    out = torch.zeros(s.size(0), s.size(1), (kb + 3) // 4 * 4, device=s.device)
    out[..., :kb] = s
    return out


def _problem(dev, groups, n, k, cap, seed):
    from batchgen_amd import workloads as wl
    g = torch.Generator(device=dev).manual_seed(seed)
    wq, ws = wl._gen_fp8_stack(g, groups, n, k, dev)
    uq, us = wl._gen_fp8_stack(g, groups, n, k, dev)
    m = groups * cap
    xq = torch.randint(0, 120, (m, k), dtype=torch.uint8, device=dev, generator=g).view(torch.float8_e4m3fn)
    xs = torch.rand(k // 128, m, device=dev, generator=g) * 0.02 + 0.001
    cu = torch.arange(groups + 1, dtype=torch.int32, device=dev) * cap
    return wq, _pad4(ws), uq, _pad4(us), xq, xs, cu, m


COUNTS = [  # groups, rows per group
    [16] * 8,                                  # whole items only when the shares happen to fit
    [1, 0, 17, 64, 0, 3, 33, 65, 130, 256],    # 1..4 row chunks per group, empty groups
    [5] * 31,                                  # every item cut once
    [256],                                     # one group, four chunks: items cut into many parts
    [0, 0, 2, 0],                              # a launch smaller than the grid
    [0, 0, 0],                                 # nothing to do
]


@pytest.mark.parametrize("counts", COUNTS, ids=[f"case{i}" for i in range(len(COUNTS))])
@pytest.mark.parametrize("n,k", [(256, 512), (512, 2048), (384, 1152)])
def test_balanced_ops_match_plain(dev, counts, n, k):
    say("streamk ops", counts, n, k)
    m_ = gm()
    groups, cap = len(counts), 256
    wq, ws, uq, us, xq, xs, cu, m = _problem(dev, groups, n, k, cap, seed=len(counts) * 7 + n)
    wq_t, uq_t = m_.fp8_weight_repack(wq), m_.fp8_weight_repack(uq)
    cnt = torch.tensor(counts, dtype=torch.int32, device=dev)
    wsb = m_.streamk_workspace(dev)
    live = torch.zeros(m, dtype=torch.bool)
    for gi, c in enumerate(counts):
        live[gi * cap: gi * cap + c] = True
    # plain GEMM
    y0 = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    y1 = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    m_.fp8_blockwise_grouped_gemm(xq, wq_t, cnt, cu, xs, ws, 16, y0, weight_layout="tile_major")
    for rep in range(2):
        y1.fill_(7.0)
        m_.fp8_blockwise_grouped_gemm(xq, wq_t, cnt, cu, xs, ws, 16, y1, weight_layout="tile_major",
                                      max_group_rows=256, workspace=wsb)
        torch.cuda.synchronize()
        assert int(wsb[:4096].view(torch.int32).abs().sum()) == 0, "counters must be left at zero"
        a, b = y0.float().cpu(), y1.float().cpu()
        assert torch.equal(a[~live], b[~live]), "rows outside the groups must not be written"
        if live.any():
            err = float((a[live] - b[live]).norm() / a[live].norm().clamp_min(1e-30))
            assert err < 2e-3, err          # bf16 outputs of two fp32 summation orders
            assert float((a[live] - b[live]).abs().max()) <= 2.0 ** -6 * float(a[live].abs().max()) + 1e-6
        if rep == 0:
            first = y1.clone()
        else:
            assert torch.equal(first, y1), "the balanced form must be reproducible bit for bit"
    # fused stage 1 + requant
    hq0 = torch.zeros((m, n), dtype=torch.uint8, device=dev)
    hs0 = torch.zeros((n // 128, m), device=dev)
    hq1, hs1 = torch.zeros_like(hq0), torch.zeros_like(hs0)
    m_.fp8_blockwise_fused_s1_quant(xq, wq_t, uq_t, cnt, cu, xs, ws, us, hq0, hs0, weight_layout="tile_major")
    m_.fp8_blockwise_fused_s1_quant(xq, wq_t, uq_t, cnt, cu, xs, ws, us, hq1, hs1, weight_layout="tile_major",
                                    max_group_rows=256, workspace=wsb)
    torch.cuda.synchronize()
    assert int(wsb[:4096].view(torch.int32).abs().sum()) == 0
    d0 = hq0.view(torch.float8_e4m3fn).float().cpu() * hs0.t().cpu().repeat_interleave(128, dim=1)
    d1 = hq1.view(torch.float8_e4m3fn).float().cpu() * hs1.t().cpu().repeat_interleave(128, dim=1)
    assert torch.equal(d0[~live], d1[~live])
    if live.any():
        err = float((d0[live] - d1[live]).norm() / d0[live].norm().clamp_min(1e-30))
        assert err < 5e-3, err              # one e4m3 step where a bf16 product moved by an ulp
        assert float((hs0.t().cpu()[live] - hs1.t().cpu()[live]).abs().max()) <= 2.0 ** -7 * float(hs0.abs().max())


def test_balanced_falls_back(dev):
    """Row-major weights, no bound on the group size, or too small a workspace: the plain kernels serve the call."""
    m_ = gm()
    counts = [9, 40, 0, 64]
    wq, ws, uq, us, xq, xs, cu, m = _problem(dev, 4, 256, 512, 64, seed=3)
    cnt = torch.tensor(counts, dtype=torch.int32, device=dev)
    y0 = torch.zeros((m, 256), dtype=torch.bfloat16, device=dev)
    m_.fp8_blockwise_grouped_gemm(xq, wq, cnt, cu, xs, ws, 16, y0)
    wsb = m_.streamk_workspace(dev)
    for kw in (dict(max_group_rows=64, workspace=wsb),                        # row-major weights
               dict(max_group_rows=0, workspace=wsb),                         # no bound
               dict(max_group_rows=64, workspace=wsb[:1024])):                # workspace too small
        y1 = torch.zeros_like(y0)
        m_.fp8_blockwise_grouped_gemm(xq, wq, cnt, cu, xs, ws, 16, y1, **kw)
        assert torch.equal(y0, y1)


@pytest.mark.parametrize("ci", [0, 1])
def test_layer_with_balanced_gemms(dev, ci):
    """The whole layer with both grouped GEMMs in the balanced form: configuration 0 against the fp32 oracle, and
    the full-size decode configuration against the layer with the plain kernels."""
    from batchgen_amd import workloads as wl
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = wl.CONFIGS[ci]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    wd, shd = {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()}
    x, logits, bias = inp["x"].to(dev), inp["logits"].to(dev), inp["bias"].to(dev)
    bal = Fp8MoELayer(cfg, wd, shd, bias, balanced_gemm=True)
    assert bal.gemm_workspace is not None
    out = bal(x, logits).clone()
    out2 = bal(x, logits)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    assert int(bal.gemm_workspace[:4096].view(torch.int32).abs().sum()) == 0
    if ci == 0:
        ref = ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(),
                               dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf),
                               wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local, layout=cfg.layout,
                               max_tokens=cfg.max_tokens, shared=wl.weights_to_numpy(sh))
        assert np.array_equal(bal.topk_ids.cpu().numpy(), ref["ids"])
        err = og.rel_frobenius(out.float().cpu().numpy(), ref["out"])
        say("balanced layer c0 rel. Frobenius error", err)
        assert err < 1e-2
    else:
        plain = Fp8MoELayer(cfg, wd, shd, bias, balanced_gemm=False)
        ref = plain(x, logits).float().cpu()
        err = float((out.float().cpu() - ref).norm() / ref.norm())
        say("balanced vs plain layer c1", err)
        assert err < 1e-3
