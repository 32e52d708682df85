"""Stage 1 of the weight-streaming FP8 kernel with tall work items (``bgmoe_set_skinny_tall_min_rows``): groups above
the row limit are cut into 64-row items, the others into 32-row items, in one launch.  Every output element is
computed by the same chain of operations whatever the item height, so the outputs (bf16 values, e4m3 bytes, scales)
must equal the default kernel's bit for bit, rows outside every group untouched.  The item enumeration behind it is
walked on the CPU in tests/test_hostcheck.py.

The tall path has not run on a GPU yet, so this file carries a name pytest does not collect: a test run that
collects everything must not be the first to launch it.  Run it by naming the file
(`python -m pytest tests/wip_gpu_skinny_tall.py -m gpu`); once green it becomes tests/test_gpu_y_skinny_tall.py."""
import numpy as np
import pytest
import torch

from tests.test_gpu_gemm_fp8 import _dev, _make, gm
from tests.util import say

pytestmark = pytest.mark.gpu

CASES = [  # counts (fewer than eight 256-row tiles above 64 rows: every group streams), n, k
    ((0, 1, 31, 32, 33, 40, 64, 65, 100, 128, 129, 200, 256), 256, 512),
    ((256, 14, 41, 65, 39, 35, 1), 2048, 7168),            # the benchmark layer's stage-1 shape, a folded shared expert
    ((48,) * 9, 384, 128),                                 # one K-block: shorter than the prefetch depth
    ((70, 3), 128, 384),                                   # three K-blocks: an odd count for the two-stage ring
]


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
@pytest.mark.parametrize("counts,n,k", CASES, ids=[f"case{i}" for i in range(len(CASES))])
def test_tall_items_give_the_same_bits(dev, counts, n, k, layout):
    from batchgen_amd._lib import check, lib
    say("tall stage-1 items", counts, n, k, layout)
    counts, cu, m, xq, xs, ws = _make(4100 + n + k, counts, n, k, nmat=2)
    (gq, gs), (uq, us) = ws
    xq_d, xs_t, gq_d, gs_d = _dev(dev, xq, xs, gq, gs)
    _, _, uq_d, us_d = _dev(dev, xq, xs, uq, us)
    if layout == "tile_major":
        gq_d, uq_d = gm().fp8_weight_repack(gq_d), gm().fp8_weight_repack(uq_d)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)

    def run():
        h = torch.full((m, n), 5.0, dtype=torch.bfloat16, device=dev)
        gm().fp8_blockwise_fused_s1(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, 16, h, weight_layout=layout)
        hq = torch.full((m, n), 0x55, dtype=torch.uint8, device=dev)
        hs = torch.full((n // 128, m), -3.0, dtype=torch.float32, device=dev)
        gm().fp8_blockwise_fused_s1_quant(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, hq, hs, weight_layout=layout)
        torch.cuda.synchronize()
        return h, hq, hs

    want = run()
    try:
        for tall_min in (32, 64, 100):
            check(lib().bgmoe_set_skinny_tall_min_rows(tall_min))
            got = run()
            for name, a, b in zip(("bf16 output", "e4m3 bytes", "scales"), want, got):
                assert torch.equal(a, b), f"{name} differ with tall items above {tall_min} rows"
    finally:
        check(lib().bgmoe_set_skinny_tall_min_rows(0))
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    assert torch.all(want[0][torch.from_numpy(~live).to(dev)] == 5.0)


def test_tall_items_in_the_layer(dev):
    """Configuration 1 with smaller matrices (256 tokens, the shared expert folded in as one more group of 256
    rows): the layer's output with tall items equals the default's bit for bit."""
    from batchgen_amd import workloads as wl
    from batchgen_amd._lib import check, lib
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = wl.scaled(wl.CONFIGS[1], hidden=1024, inter=512, shared_inter=512)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_fp8_weights(cfg, dev)
    layer = Fp8MoELayer(cfg, w, sh, inp["bias"])
    want = layer(inp["x"], inp["logits"]).clone()
    counts = layer.expert_counts.cpu().numpy()
    say("   counts", counts.tolist())
    assert counts.max() > 64, "the case is meant to have a group above both limits"
    try:
        for tall_min in (32, 64):
            check(lib().bgmoe_set_skinny_tall_min_rows(tall_min))
            assert torch.equal(layer(inp["x"], inp["logits"]), want)
    finally:
        check(lib().bgmoe_set_skinny_tall_min_rows(0))
