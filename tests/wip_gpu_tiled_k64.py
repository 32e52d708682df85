"""The K = 64 variant of the LDS-tiled FP8 grouped GEMM (32x32x64 products accumulated in place, four-slot ring;
``bgmoe_set_tiled_variant(1)``) on the GPU, with every group forced onto the tiled kernel: against the fp32
dequantise-then-matmul oracle at the reference's gates, write sets, the requantisation identity of the fused
epilogue, ragged == uniform placement bit for bit, both weight layouts, and against the K = 128 kernel (the two
differ in rounding only).  The lane maps behind it are walked on the CPU in tests/test_hostcheck.py.

The kernel has not run on a GPU yet, so this file carries a name pytest does not collect: a test run that
collects everything must not be the first to launch a kernel that no GPU has executed.  Run it by naming the
file (`python -m pytest tests/wip_gpu_tiled_k64.py -m gpu`); once it is green it becomes tests/test_gpu_y_tiled_k64.py."""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import quant as oq
from tests.test_gpu_gemm_fp8 import _dev, _make, gm, qops
from tests.util import say

pytestmark = pytest.mark.gpu


@pytest.fixture(params=[2, 1], ids=["plain_stores", "regrouped_stores"])
def k64(request):
    """Every group on the tiled kernel (row limit 0), K = 64 variant with plain per-lane stores (2) or with the
    epilogue regrouped through per-wave LDS patches (1); both settings restored afterwards."""
    from batchgen_amd._lib import check, lib
    check(lib().bgmoe_set_skinny_max_rows(0))
    check(lib().bgmoe_set_tiled_variant(request.param))
    try:
        yield
    finally:
        check(lib().bgmoe_set_tiled_variant(0))
        check(lib().bgmoe_set_skinny_max_rows(256))


def _live(counts, cu, m):
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    return live


CASES = [  # counts, n, k
    ((256, 257, 1, 0, 512), 256, 256),                     # two K-blocks: the shortest K the variant takes
    ((256, 257, 1, 0, 512), 640, 384),                     # an output narrower than the last 256-column tile
    ((0, 1, 15, 16, 17, 31, 32, 63, 64, 65, 127, 128, 129, 255), 384, 640),
    ((300, 44, 700), 128, 1024),                           # one 128-column tile: the plain GEMM's second half past N
    ((130,) * 5, 2048, 7168),                              # the benchmark layer's stage-1 shape
]


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
@pytest.mark.parametrize("counts,n,k", CASES, ids=[f"case{i}" for i in range(len(CASES))])
def test_k64_variant_vs_fp32_oracle(dev, k64, counts, n, k, layout):
    say("tiled K=64", counts, n, k, layout)
    counts, cu, m, xq, xs, ws = _make(1200 + n + k, counts, n, k, nmat=2)
    (gq, gs), (uq, us) = ws
    xq_d, xs_t, gq_d, gs_d = _dev(dev, xq, xs, gq, gs)
    _, _, uq_d, us_d = _dev(dev, xq, xs, uq, us)
    if layout == "tile_major":
        gq_d, uq_d = gm().fp8_weight_repack(gq_d), gm().fp8_weight_repack(uq_d)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)
    live = _live(counts, cu, m)
    out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    gm().fp8_blockwise_grouped_gemm(xq_d, gq_d, cnt_d, cu_d, xs_t, gs_d, 16, out, weight_layout=layout)
    h = torch.full((m, n), 5.0, dtype=torch.bfloat16, device=dev)
    gm().fp8_blockwise_fused_s1(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, 16, h, weight_layout=layout)
    hq = torch.zeros((m, n), dtype=torch.uint8, device=dev)
    hs = torch.zeros((n // 128, m), dtype=torch.float32, device=dev)
    gm().fp8_blockwise_fused_s1_quant(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, hq, hs, weight_layout=layout)
    hq2 = torch.zeros((m, n), dtype=torch.uint8, device=dev)
    hs2 = torch.zeros((n // 128, m), dtype=torch.float32, device=dev)
    qops().act_quant_ragged(h, cnt_d, cu_d, hq2, hs2, 1)
    torch.cuda.synchronize()
    ref = og.grouped_gemm_fp8(xq, xs, gq, gs, counts, cu, to_bf16=False)
    o = out.float().cpu().numpy()
    np.testing.assert_allclose(o[live], ref[live], rtol=2e-2, atol=5e-3)
    assert og.rel_frobenius(o[live], ref[live]) < 3e-3
    assert np.all(o[~live] == 7.0), "rows outside every live range untouched"
    up = og.grouped_gemm_fp8(xq, xs, uq, us, counts, cu, to_bf16=False)
    href = oq.silu_f32(ref) * up
    hh = h.float().cpu().numpy()
    np.testing.assert_allclose(hh[live], href[live], rtol=5e-2, atol=2e-2)
    assert og.rel_frobenius(hh[live], href[live]) < 4e-3 and np.all(hh[~live] == 5.0)
    lv = torch.from_numpy(live).to(dev)
    assert torch.equal(hq[lv], hq2[lv]) and torch.equal(hs[:, lv], hs2[:, lv]), \
        "the fused epilogue's bytes and scales are the quantiser's on the bf16 output"


def test_k64_variant_against_the_k128_kernel_and_placement(dev):
    """The same problem through both tiled kernels: bf16 outputs of two fp32 summation orders; and the K = 64
    variant on the same rows at other offsets (ragged vs uniform placement): bit for bit."""
    from batchgen_amd._lib import check, lib
    counts0 = (300, 0, 257, 70)
    n, k = 256, 512
    counts, cu, m, xq, xs, ws = _make(77, counts0, n, k, align=16)
    wq, wsc = ws[0]
    xq_d, xs_t, wq_d, ws_d = _dev(dev, xq, xs, wq, wsc)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)
    live = _live(counts, cu, m)
    outs = {}
    check(lib().bgmoe_set_skinny_max_rows(0))
    try:
        for variant in (0, 1, 2):
            check(lib().bgmoe_set_tiled_variant(variant))
            outs[variant] = gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, cnt_d, cu_d, xs_t, ws_d, 16).float().cpu().numpy()
        check(lib().bgmoe_set_tiled_variant(1))
        # uniform placement: group e at row 512 e
        cu2 = (np.arange(len(counts) + 1) * 512).astype(np.int32)
        m2 = int(cu2[-1])
        xq2 = np.zeros((m2, k), dtype=np.uint8)
        xs2 = np.ones((m2, k // 128), dtype=np.float32)
        for e, c in enumerate(counts):
            xq2[cu2[e]:cu2[e] + c] = xq[cu[e]:cu[e] + c]
            xs2[cu2[e]:cu2[e] + c] = xs[cu[e]:cu[e] + c]
        xq2_d, xs2_t, _, _ = _dev(dev, xq2, xs2, wq, wsc)
        o2 = gm().fp8_blockwise_grouped_gemm(xq2_d, wq_d, cnt_d, torch.from_numpy(cu2).to(dev), xs2_t, ws_d, 16)
        o2 = o2.float().cpu().numpy()
    finally:
        check(lib().bgmoe_set_tiled_variant(0))
        check(lib().bgmoe_set_skinny_max_rows(256))
    # (live rows only: the op allocates its output, rows outside every group hold whatever the allocation held)
    assert np.array_equal(outs[1][live], outs[2][live]), "the two epilogues of the K = 64 kernel store the same bits"
    a, b = outs[0][live], outs[1][live]
    assert og.rel_frobenius(b, a) < 2e-3
    assert np.abs(a - b).max() <= 2.0 ** -6 * np.abs(a).max() + 1e-6
    for e, c in enumerate(counts):
        assert np.array_equal(o2[cu2[e]:cu2[e] + c], outs[1][cu[e]:cu[e] + c]), "placement must not change a row's bits"


def test_k64_variant_declines_short_k_and_bad_arguments(dev, k64):
    """K = 128 has a single K-block: the variant does not apply and the K = 128 kernel serves the call (same
    results as without the variant); an unknown variant number is refused."""
    from batchgen_amd._lib import lib
    counts, cu, m, xq, xs, ws = _make(5, (256, 3), 128, 128)
    wq, wsc = ws[0]
    xq_d, xs_t, wq_d, ws_d = _dev(dev, xq, xs, wq, wsc)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)
    a = gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, cnt_d, cu_d, xs_t, ws_d, 16)
    assert lib().bgmoe_set_tiled_variant(0) == 0
    b = gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, cnt_d, cu_d, xs_t, ws_d, 16)
    lv = torch.from_numpy(_live(counts, cu, m)).to(dev)          # (rows outside every group are never written)
    assert torch.equal(a[lv], b[lv])
    assert lib().bgmoe_set_tiled_variant(3) != 0 and lib().bgmoe_set_tiled_variant(-1) != 0
