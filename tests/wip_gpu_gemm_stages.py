"""The weight-streaming FP8 kernels with deeper prefetch rings: the plain grouped GEMM (the down projection of a decode
step; ``bgmoe_set_skinny_gemm_stages``: 3 or 4 stages instead of 2) and fused stage 1 (``bgmoe_set_skinny_s1_stages``:
4 instead of 3), with the wait count a deeper ring needs.  Every output
element is computed by the same chain of operations whatever the depth, so the output must equal the default
kernel's bit for bit, rows outside every group untouched.  The rings' wait counts are exercised on the CPU emulator
with every load landing as late as the waits allow (tests/test_emu_kernels.py).

The deeper rings have not run on a GPU yet, so this file carries a name pytest does not collect: a test run that
collects everything must not be the first to launch them.  Run it by naming the file
(`python -m pytest tests/wip_gpu_gemm_stages.py -m gpu`); once green it becomes tests/test_gpu_y_gemm_stages.py."""
import numpy as np
import pytest
import torch

from tests.test_gpu_gemm_fp8 import _dev, _make, gm
from tests.util import say

pytestmark = pytest.mark.gpu

CASES = [  # counts (every group streams), n, k
    ((0, 1, 31, 32, 33, 40, 64, 65, 100, 128, 129, 200, 256), 256, 512),
    ((256, 14, 41, 65, 39, 35, 1), 7168, 2048),            # the benchmark layer's down projection, a folded shared expert
    ((48,) * 9, 384, 128),                                 # one K-block: shorter than every ring
    ((70, 3), 128, 384),                                   # three K-blocks: the four-stage ring never reaches its main loop
    ((8,) * 32, 512, 1152),                                # nine K-blocks: a remainder for every depth
]


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
@pytest.mark.parametrize("counts,n,k", CASES, ids=[f"case{i}" for i in range(len(CASES))])
def test_deeper_rings_give_the_same_bits(dev, counts, n, k, layout):
    from batchgen_amd._lib import check, lib
    say("streaming GEMM prefetch depth", counts, n, k, layout)
    counts, cu, m, xq, xs, ws = _make(5200 + n + k, counts, n, k)
    wq, wsc = ws[0]
    xq_d, xs_t, wq_d, ws_d = _dev(dev, xq, xs, wq, wsc)
    if layout == "tile_major":
        wq_d = gm().fp8_weight_repack(wq_d)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)

    def run():
        out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
        gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, cnt_d, cu_d, xs_t, ws_d, 16, out, weight_layout=layout)
        torch.cuda.synchronize()
        return out

    want = run()
    try:
        for stages in (3, 4, 6):
            check(lib().bgmoe_set_skinny_gemm_stages(stages))
            assert torch.equal(run(), want), f"output differs with {stages} prefetch stages"
    finally:
        check(lib().bgmoe_set_skinny_gemm_stages(2))
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    assert torch.all(want[torch.from_numpy(~live).to(dev)] == 7.0)


def test_deeper_rings_in_the_layer(dev):
    """Configuration 1 with smaller matrices: the layer's output equals the default's bit for bit."""
    from batchgen_amd import workloads as wl
    from batchgen_amd._lib import check, lib
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = wl.scaled(wl.CONFIGS[1], hidden=1024, inter=512, shared_inter=512)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_fp8_weights(cfg, dev)
    layer = Fp8MoELayer(cfg, w, sh, inp["bias"])
    want = layer(inp["x"], inp["logits"]).clone()
    try:
        for stages in (3, 4):
            check(lib().bgmoe_set_skinny_gemm_stages(stages))
            assert torch.equal(layer(inp["x"], inp["logits"]), want)
    finally:
        check(lib().bgmoe_set_skinny_gemm_stages(2))


@pytest.mark.parametrize("m,n,k", [(40, 512, 4224), (100, 1152, 1024), (128, 4096, 7168), (128, 7168, 2048), (200, 512, 4224),
                                    (300, 1152, 1024)])    # the last two: 128-row chunks
def test_deeper_rings_in_the_dense_split_k_gemm(dev, m, n, k):
    """The one-weight GEMM's block-split form with 64-row chunks follows the same switch."""
    from batchgen_amd._lib import check, lib
    from batchgen_amd.moe.shared_expert import fp8_gemm_nt
    from oracle import quant as oq
    from tests.util import rand_bf16
    say("dense split-K prefetch depth", m, n, k)
    g = torch.Generator().manual_seed(m + n + k)
    xq, xs = oq.act_quant(rand_bf16(g, m, k).float().numpy(), form="A")
    wq, ws = oq.weight_block_quant((0.05 * torch.randn(1, n, k, generator=g)).numpy())
    a = torch.from_numpy(xq).to(dev).view(torch.float8_e4m3fn)
    b = torch.from_numpy(wq[0]).to(dev).view(torch.float8_e4m3fn)
    sa, sb = torch.from_numpy(xs).to(dev), torch.from_numpy(ws[0]).to(dev)

    def run():
        d = torch.full((m, n), -7.0, dtype=torch.bfloat16, device=dev)
        fp8_gemm_nt((a, sa), (b, sb), d)
        torch.cuda.synchronize()
        return d

    want = run()
    try:
        for stages in (3, 4):
            check(lib().bgmoe_set_skinny_gemm_stages(stages))
            assert torch.equal(run(), want), f"output differs with {stages} prefetch stages"
    finally:
        check(lib().bgmoe_set_skinny_gemm_stages(2))


S1_CASES = [
    ((0, 1, 31, 32, 33, 40, 64, 65, 100, 128, 129, 200, 256), 256, 512),
    ((256, 14, 41, 65, 39, 35, 1), 2048, 7168),            # the benchmark layer's stage-1 shape, a folded shared expert
    ((48,) * 9, 384, 128),                                 # one K-block
    ((70, 3), 128, 384),                                   # three K-blocks: shorter than the four-stage ring
    ((8,) * 32, 512, 1152),                                # nine K-blocks
]


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
@pytest.mark.parametrize("counts,n,k", S1_CASES, ids=[f"case{i}" for i in range(len(S1_CASES))])
def test_four_stage_fused_stage1_gives_the_same_bits(dev, counts, n, k, layout):
    from batchgen_amd._lib import check, lib
    say("fused stage 1, four prefetch stages", counts, n, k, layout)
    counts, cu, m, xq, xs, ws = _make(6100 + n + k, counts, n, k, nmat=2)
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
        check(lib().bgmoe_set_skinny_s1_stages(4))
        got = run()
    finally:
        check(lib().bgmoe_set_skinny_s1_stages(3))
    for name, a, b in zip(("bf16 output", "e4m3 bytes", "scales"), want, got):
        assert torch.equal(a, b), f"{name} differ with four prefetch stages"


def test_four_stage_stage1_in_the_layer(dev):
    from batchgen_amd import workloads as wl
    from batchgen_amd._lib import check, lib
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = wl.scaled(wl.CONFIGS[1], hidden=1024, inter=512, shared_inter=512)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_fp8_weights(cfg, dev)
    layer = Fp8MoELayer(cfg, w, sh, inp["bias"])
    want = layer(inp["x"], inp["logits"]).clone()
    try:
        check(lib().bgmoe_set_skinny_s1_stages(4))
        check(lib().bgmoe_set_skinny_gemm_stages(3))
        assert torch.equal(layer(inp["x"], inp["logits"]), want)
    finally:
        check(lib().bgmoe_set_skinny_s1_stages(3))
        check(lib().bgmoe_set_skinny_gemm_stages(2))
