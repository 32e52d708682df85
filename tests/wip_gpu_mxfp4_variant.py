"""The MXFP4 weight-streaming kernel's second shape (``bgmoe_set_mxfp4_variant(1)``: 32-row work items, six prefetch
stages) against the default shape (64-row items, three stages): every output element is the same chain of
operations, so the plain GEMM, the fused stage 1 with both activations and the whole layer must give the same bits,
rows outside every group untouched.

The second shape has not run on a GPU yet, so this file carries a name pytest does not collect.  Run it by naming
the file (`python -m pytest tests/wip_gpu_mxfp4_variant.py -m gpu`); once green it becomes
tests/test_gpu_y_mxfp4_variant.py."""
import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from tests.test_gpu_mxfp4 import _layout, _weights, mg
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu

CASES = [  # counts, n, k: 1, 2, 5, 6, 7 and 13 K-blocks against the six stages
    ((0, 1, 15, 16, 17, 31, 32, 33, 64, 70, 130), 256, 128),
    ((3, 40, 100), 128, 256),
    ((9,) * 4, 384, 640),
    ((33, 65, 2), 256, 768),
    ((20, 64, 1), 128, 896),
    ((5, 0, 40, 96), 2048, 1664),
]


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
@pytest.mark.parametrize("counts,n,k", CASES, ids=[f"case{i}" for i in range(len(CASES))])
def test_second_shape_gives_the_same_bits(dev, counts, n, k, layout):
    from batchgen_amd._lib import check, lib
    say("mxfp4 variant", counts, n, k, layout)
    counts, cu = _layout(counts)
    m = int(cu[-1])
    x = rand_bf16(torch.Generator().manual_seed(n + k), m, k).to(dev)
    (gp, gs), (up, us) = _weights(1, len(counts), n, k), _weights(2, len(counts), n, k)
    d = lambda a: torch.from_numpy(a).to(dev)
    gpd, gsd, upd, usd = d(gp), d(gs), d(up), d(us)
    if layout == "tile_major":
        gpd, gsd = mg().mxfp4_weight_repack(gpd, gsd)
        upd, usd = mg().mxfp4_weight_repack(upd, usd)
    cnt_d, cu_d = d(counts), d(cu)

    def run():
        out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
        mg().mxfp4_grouped_gemm(x, gpd, gsd, cnt_d, cu_d, out, weight_layout=layout)
        hs = [mg().mxfp4_fused_s1(x, gpd, gsd, upd, usd, cnt_d, cu_d, weight_layout=layout, activation=a)
              for a in ("swiglu", "situ")]
        torch.cuda.synchronize()
        return [out] + hs

    want = run()
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    lv = torch.from_numpy(live).to(dev)
    for variant in (1, 2, 3):
        try:
            check(lib().bgmoe_set_mxfp4_variant(variant))
            got = run()
        finally:
            check(lib().bgmoe_set_mxfp4_variant(0))
        assert torch.equal(got[0], want[0]), f"shape {variant}: plain GEMM (rows outside the groups included)"
        for name, a, b in zip(("swiglu", "situ"), want[1:], got[1:]):
            assert torch.equal(a[lv], b[lv]), f"shape {variant}: fused stage 1 ({name})"


@pytest.mark.parametrize("fold", [False, True], ids=["gathered", "folded_gather"])
def test_layer_on_the_second_shape(dev, fold):
    from batchgen_amd._lib import check, lib
    from batchgen_amd.moe.mxfp4_layer import Mxfp4MoELayer
    cfg = wl.scaled(wl.CONFIGS[3], n_tokens=96, hidden=512, inter=256, shared_inter=256, n_experts=224, e_local=28,
                    expert_start=56, max_tokens=96)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_mxfp4_weights(cfg, dev)
    layer = Mxfp4MoELayer(cfg, w, sh, inp["bias"], fold_gather=fold)
    want = layer(inp["x"], inp["logits"]).clone()
    for variant in (1, 2, 3):
        try:
            check(lib().bgmoe_set_mxfp4_variant(variant))
            got = layer(inp["x"], inp["logits"]).clone()
        finally:
            check(lib().bgmoe_set_mxfp4_variant(0))
        assert torch.equal(got, want), f"shape {variant}"
    assert lib().bgmoe_set_mxfp4_variant(4) != 0 and lib().bgmoe_set_mxfp4_variant(-1) != 0
