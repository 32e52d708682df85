"""HIP block-scaled FP8 grouped GEMMs vs the fp32 dequantise-then-matmul oracle.

Tolerances are the reference's own gates (tests/test_moe_compact_ragged_fp8.py:370-377):
rtol 2e-2 / atol 5e-3 for a single GEMM, rtol 5e-2 / atol 2e-2 for the fused stage 1, plus a relative
Frobenius bound far below the 1e-2 layer budget.
"""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import quant as oq
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def gm():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_fp8_blockwise_gemm")


def qops():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_fp8_blockwise_ops")


def _layout(counts, align):
    counts = np.asarray(counts, dtype=np.int32)
    al = (counts + align - 1) // align * align
    cu = np.concatenate([[0], np.cumsum(al)]).astype(np.int32)
    return counts, cu


def _make(seed, counts, n, k, align=16, nmat=1):
    g = torch.Generator().manual_seed(seed)
    counts, cu = _layout(counts, align)
    m = max(int(cu[-1]), 1)
    x = rand_bf16(g, m, k)
    xq, xs = oq.act_quant(x)
    ws = []
    for _ in range(nmat):
        w = (0.02 * torch.randn(len(counts), n, k, generator=g)).numpy()
        ws.append(oq.weight_block_quant(w))
    return counts, cu, m, xq, xs, ws


def _dev(dev, xq, xs, wq, wsc, pad4=True):
    kb = xs.shape[1]
    xq_d = torch.from_numpy(xq).to(dev).view(torch.float8_e4m3fn)
    xs_t = torch.from_numpy(np.ascontiguousarray(xs.T)).to(dev)
    wq_d = torch.from_numpy(wq).to(dev).view(torch.float8_e4m3fn)
    kbp = (kb + 3) // 4 * 4 if pad4 else kb
    wsp = np.zeros(wsc.shape[:2] + (kbp,), dtype=np.float32)
    wsp[..., :kb] = wsc
    return xq_d, xs_t, wq_d, torch.from_numpy(wsp).to(dev)


EDGE = (0, 1, 15, 16, 17, 31, 32, 63, 64, 65, 127, 128)


@pytest.mark.parametrize("counts,n,k", [
    (EDGE, 256, 512), ((5, 0, 9, 16), 128, 1024), ((3, 200, 0, 77, 130, 1), 384, 256), ((300,), 256, 384),
    ((8,) * 8, 7168, 2048),
])
def test_grouped_gemm_vs_fp32_oracle(dev, counts, n, k):
    say("grouped_gemm", counts, n, k)
    counts, cu, m, xq, xs, ws = _make(100 + n + k, counts, n, k)
    wq, wsc = ws[0]
    xq_d, xs_t, wq_d, ws_d = _dev(dev, xq, xs, wq, wsc)
    out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev),
                                    xs_t, ws_d, 16, out)
    ref = og.grouped_gemm_fp8(xq, xs, wq, wsc, counts, cu, to_bf16=False)
    o = out.float().cpu().numpy()
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    np.testing.assert_allclose(o[live], ref[live], rtol=2e-2, atol=5e-3)
    assert og.rel_frobenius(o[live], ref[live]) < 3e-3
    assert np.all(o[~live] == 7.0)                       # rows outside every live range untouched


def test_grouped_gemm_closed_form_constant_case(dev):
    """All weights 0.25 (exact in e4m3), scales 0.01, x = 1: y = K * 0.25 * 0.01 * xs."""
    k, n, e = 512, 256, 3
    counts, cu = _layout((7, 0, 40), 16)
    m = int(cu[-1])
    xq = np.full((m, k), 0x38, dtype=np.uint8)            # 1.0
    xs = np.full((m, k // 128), 0.5, dtype=np.float32)
    wq = np.full((e, n, k), 0x28, dtype=np.uint8)         # 0.25
    wsc = np.full((e, n // 128, k // 128), 0.01, dtype=np.float32)
    xq_d, xs_t, wq_d, ws_d = _dev(dev, xq, xs, wq, wsc)
    out = gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, torch.from_numpy(counts).to(dev),
                                          torch.from_numpy(cu).to(dev), xs_t, ws_d, 16)
    expect = torch.tensor(k * 0.25 * 0.01 * 0.5).to(torch.bfloat16)
    assert torch.all(out[:7] == expect.to(dev)) and torch.all(out[cu[2]:cu[2] + 40] == expect.to(dev))


@pytest.mark.parametrize("counts,n,k", [
    (EDGE, 256, 512), ((5, 0, 9, 16), 128, 1024), ((3, 200, 0, 77, 130, 1), 384, 256), ((8,) * 4, 2048, 7168),
])
def test_fused_s1_vs_oracle_and_requant_identity(dev, counts, n, k):
    say("fused_s1", counts, n, k)
    counts, cu, m, xq, xs, ws = _make(200 + n + k, counts, n, k, nmat=2)
    (gq, gs), (uq, us) = ws
    xq_d, xs_t, gq_d, gs_d = _dev(dev, xq, xs, gq, gs)
    _, _, uq_d, us_d = _dev(dev, xq, xs, uq, us)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)
    h = torch.zeros((m, n), dtype=torch.bfloat16, device=dev)
    gm().fp8_blockwise_fused_s1(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, 16, h)
    gate = og.grouped_gemm_fp8(xq, xs, gq, gs, counts, cu, to_bf16=False)
    up = og.grouped_gemm_fp8(xq, xs, uq, us, counts, cu, to_bf16=False)
    ref = oq.silu_f32(gate) * up
    o = h.float().cpu().numpy()
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    np.testing.assert_allclose(o[live], ref[live], rtol=5e-2, atol=2e-2)
    assert og.rel_frobenius(o[live], ref[live]) < 4e-3
    # epilogue requant == separate act_quant_ragged on the bf16 output, bit for bit
    hq = torch.zeros((m, n), dtype=torch.uint8, device=dev)
    hs = torch.zeros((n // 128, m), dtype=torch.float32, device=dev)
    gm().fp8_blockwise_fused_s1_quant(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, hq, hs)
    hq2 = torch.zeros((m, n), dtype=torch.uint8, device=dev)
    hs2 = torch.zeros((n // 128, m), dtype=torch.float32, device=dev)
    qops().act_quant_ragged(h, cnt_d, cu_d, hq2, hs2, 1)
    lv = torch.from_numpy(live).to(dev)
    assert torch.equal(hq[lv], hq2[lv]) and torch.equal(hs[:, lv], hs2[:, lv])


def test_ragged_equals_uniform_layout(dev):
    """The same rows placed at different offsets give bit-identical results."""
    counts = (9, 0, 33, 70)
    n, k = 256, 512
    c1, cu1, m1, xq1, xs1, ws = _make(5, counts, n, k, align=16)
    wq, wsc = ws[0]
    s_ = 128
    cu2 = (np.arange(len(counts) + 1) * s_).astype(np.int32)
    m2 = int(cu2[-1])
    xq2 = np.zeros((m2, k), dtype=np.uint8)
    xs2 = np.ones((m2, k // 128), dtype=np.float32)
    for e, c in enumerate(counts):
        xq2[cu2[e]:cu2[e] + c] = xq1[cu1[e]:cu1[e] + c]
        xs2[cu2[e]:cu2[e] + c] = xs1[cu1[e]:cu1[e] + c]
    outs = []
    for xq, xs, cu, m in ((xq1, xs1, cu1, m1), (xq2, xs2, cu2, m2)):
        xq_d, xs_t, wq_d, ws_d = _dev(dev, xq, xs, wq, wsc)
        o = gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, torch.from_numpy(c1).to(dev), torch.from_numpy(cu).to(dev),
                                            xs_t, ws_d, 16)
        outs.append((o, cu))
    for e, c in enumerate(counts):
        a = outs[0][0][outs[0][1][e]:outs[0][1][e] + c]
        b = outs[1][0][outs[1][1][e]:outs[1][1][e] + c]
        assert torch.equal(a, b)


def test_poisoned_padding_does_not_leak(dev):
    """Rows past a group's count hold NaN bytes / huge scales; live rows must not change."""
    counts = (5, 20, 100)
    n, k = 256, 256
    c, cu, m, xq, xs, ws = _make(6, counts, n, k, align=128)
    wq, wsc = ws[0]
    xq_p, xs_p = xq.copy(), xs.copy()
    for e, cc in enumerate(counts):
        xq_p[cu[e] + cc:cu[e + 1]] = 0x7F
        xs_p[cu[e] + cc:cu[e + 1]] = 1e30
    res = []
    for a, b in ((xq, xs), (xq_p, xs_p)):
        xq_d, xs_t, wq_d, ws_d = _dev(dev, a, b, wq, wsc)
        res.append(gm().fp8_blockwise_grouped_gemm(xq_d, wq_d, torch.from_numpy(c).to(dev),
                                                   torch.from_numpy(cu).to(dev), xs_t, ws_d, 64))
    for e, cc in enumerate(counts):
        assert torch.equal(res[0][cu[e]:cu[e] + cc], res[1][cu[e]:cu[e] + cc])


def test_pointer_table_equals_stacked(dev):
    counts = (4, 0, 18, 90)
    n, k = 256, 384
    c, cu, m, xq, xs, ws = _make(8, counts, n, k, nmat=2)
    (gq, gs), (uq, us) = ws
    xq_d, xs_t, gq_d, gs_d = _dev(dev, xq, xs, gq, gs)
    _, _, uq_d, us_d = _dev(dev, xq, xs, uq, us)
    cnt_d, cu_d = torch.from_numpy(c).to(dev), torch.from_numpy(cu).to(dev)
    ref = gm().fp8_blockwise_grouped_gemm(xq_d, gq_d, cnt_d, cu_d, xs_t, gs_d, 16)
    perm = [2, 0, 3, 1]                                    # tables need not be in memory order
    gparts = [gq_d[i].clone() for i in range(4)]
    sparts = [gs_d[i].clone() for i in range(4)]
    wp = torch.tensor([gparts[i].data_ptr() for i in range(4)], dtype=torch.int64, device=dev)
    sp = torch.tensor([sparts[i].data_ptr() for i in range(4)], dtype=torch.int64, device=dev)
    out = gm().fp8_blockwise_grouped_gemm_ptrs(xq_d, gq_d[0], wp, cnt_d, cu_d, xs_t, gs_d[0], sp, 16)
    live = torch.zeros(m, dtype=torch.bool)
    for e, cc in enumerate(counts):
        live[cu[e]:cu[e] + cc] = True
    assert torch.equal(out[live.to(dev)], ref[live.to(dev)])
    ref1 = gm().fp8_blockwise_fused_s1(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, 16)
    uparts = [uq_d[i].clone() for i in range(4)]
    usparts = [us_d[i].clone() for i in range(4)]
    up = torch.tensor([t.data_ptr() for t in uparts], dtype=torch.int64, device=dev)
    usp = torch.tensor([t.data_ptr() for t in usparts], dtype=torch.int64, device=dev)
    out1 = gm().fp8_blockwise_fused_s1_ptrs(xq_d, gq_d[0], wp, uq_d[0], up, cnt_d, cu_d, xs_t, gs_d[0], sp,
                                            us_d[0], usp, 16)
    assert torch.equal(out1[live.to(dev)], ref1[live.to(dev)])
    del perm


def test_gemm_argument_errors(dev):
    x = torch.zeros((16, 200), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    w = torch.zeros((2, 128, 200), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    sl = torch.zeros(2, dtype=torch.int32, device=dev)
    cu = torch.zeros(3, dtype=torch.int32, device=dev)
    xs = torch.zeros((2, 16), device=dev)
    ws = torch.zeros((2, 1, 4), device=dev)
    with pytest.raises(RuntimeError):
        gm().fp8_blockwise_grouped_gemm(x, w, sl, cu, xs, ws, 16)       # K not a multiple of 128
    w2 = torch.zeros((1025, 128, 128), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    with pytest.raises(RuntimeError):
        gm().fp8_blockwise_grouped_gemm(x, w2, sl, cu, xs, ws, 16)      # too many groups


def _tile_major_numpy(w):
    """[G, N, K] bytes -> tile-major image, written from the layout's definition."""
    g, n, k = w.shape
    t = w.reshape(g, n // 16, 16, k // 128, 2, 4, 16)          # g, nt, r, kb, half, q, j
    return np.ascontiguousarray(t.transpose(0, 1, 3, 4, 5, 2, 6)).reshape(g, n, k)   # g, nt, kb, half, q, r, j


@pytest.mark.parametrize("counts,n,k", [(EDGE, 256, 512), ((3, 200, 0, 77, 130, 1), 384, 256), ((8,) * 6, 2048, 1024)])
def test_tile_major_weights_equal_row_major(dev, counts, n, k):
    say("tile_major", counts, n, k)
    counts, cu, m, xq, xs, ws = _make(300 + n + k, counts, n, k, nmat=2)
    (gq, gs), (uq, us) = ws
    xq_d, xs_t, gq_d, gs_d = _dev(dev, xq, xs, gq, gs)
    _, _, uq_d, us_d = _dev(dev, xq, xs, uq, us)
    gq_t, uq_t = gm().fp8_weight_repack(gq_d), gm().fp8_weight_repack(uq_d)
    assert np.array_equal(gq_t.view(torch.uint8).cpu().numpy(), _tile_major_numpy(gq))
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)
    live = torch.zeros(m, dtype=torch.bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    live = live.to(dev)
    a = gm().fp8_blockwise_grouped_gemm(xq_d, gq_d, cnt_d, cu_d, xs_t, gs_d, 16)
    b = gm().fp8_blockwise_grouped_gemm(xq_d, gq_t, cnt_d, cu_d, xs_t, gs_d, 16, weight_layout="tile_major")
    assert torch.equal(a[live], b[live])
    a = gm().fp8_blockwise_fused_s1(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, 16)
    b = gm().fp8_blockwise_fused_s1(xq_d, gq_t, uq_t, cnt_d, cu_d, xs_t, gs_d, us_d, 16, weight_layout="tile_major")
    assert torch.equal(a[live], b[live])


@pytest.mark.parametrize("limit", [0, 16, 256])
@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
@pytest.mark.parametrize("counts", [
    (0, 1, 15, 16, 17, 127, 128, 129, 260, 5),            # few rows above 64: they stay on the streaming kernel
    (70, 100, 0, 129, 65, 90, 260, 33, 64, 200, 80),      # nine 256-row tiles above 64 rows: those groups are tiled
], ids=["few_big", "many_big"])
def test_kernel_choice_does_not_change_results_beyond_rounding(dev, limit, layout, counts):
    """The same problem through the LDS-tiled kernel only (limit 0), a mix, and the streaming kernel
    (limit 256: groups of 65..256 rows are tiled only when there are at least eight tiles of them)."""
    from batchgen_amd._lib import check, lib
    n, k = 384, 640
    counts, cu, m, xq, xs, ws = _make(400, counts, n, k, nmat=2)
    (gq, gs), (uq, us) = ws
    xq_d, xs_t, gq_d, gs_d = _dev(dev, xq, xs, gq, gs)
    _, _, uq_d, us_d = _dev(dev, xq, xs, uq, us)
    if layout == "tile_major":
        gq_d, uq_d = gm().fp8_weight_repack(gq_d), gm().fp8_weight_repack(uq_d)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    check(lib().bgmoe_set_skinny_max_rows(limit))
    try:
        out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
        gm().fp8_blockwise_grouped_gemm(xq_d, gq_d, cnt_d, cu_d, xs_t, gs_d, 16, out, weight_layout=layout)
        h = gm().fp8_blockwise_fused_s1(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, 16, weight_layout=layout)
        hq = torch.zeros((m, n), dtype=torch.uint8, device=dev)
        hs = torch.zeros((n // 128, m), dtype=torch.float32, device=dev)
        gm().fp8_blockwise_fused_s1_quant(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, hq, hs, weight_layout=layout)
        hq2 = torch.zeros((m, n), dtype=torch.uint8, device=dev)
        hs2 = torch.zeros((n // 128, m), dtype=torch.float32, device=dev)
        qops().act_quant_ragged(h, cnt_d, cu_d, hq2, hs2, 1)
    finally:
        check(lib().bgmoe_set_skinny_max_rows(256))
    ref = og.grouped_gemm_fp8(xq, xs, gq, gs, counts, cu, to_bf16=False)
    o = out.float().cpu().numpy()
    np.testing.assert_allclose(o[live], ref[live], rtol=2e-2, atol=5e-3)
    assert og.rel_frobenius(o[live], ref[live]) < 3e-3 and np.all(o[~live] == 7.0)
    up = og.grouped_gemm_fp8(xq, xs, uq, us, counts, cu, to_bf16=False)
    href = oq.silu_f32(ref) * up
    assert og.rel_frobenius(h.float().cpu().numpy()[live], href[live]) < 4e-3
    lv = torch.from_numpy(live).to(dev)
    assert torch.equal(hq[lv], hq2[lv]) and torch.equal(hs[:, lv], hs2[:, lv])


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
@pytest.mark.parametrize("n,k", [(128, 128), (256, 256), (640, 384)])
def test_tiled_kernel_edge_shapes(dev, n, k, layout):
    """The LDS-tiled kernel alone (row limit 0) on shapes at its edges: one and two K-steps, an output narrower
    than its 256-column tile, groups of exactly one tile, one row more, one row, none, and two tiles."""
    from batchgen_amd._lib import check, lib
    counts = (256, 257, 1, 0, 512)
    say("tiled edges", n, k, layout)
    counts, cu, m, xq, xs, ws = _make(900 + n + k, counts, n, k, nmat=2)
    (gq, gs), (uq, us) = ws
    xq_d, xs_t, gq_d, gs_d = _dev(dev, xq, xs, gq, gs)
    _, _, uq_d, us_d = _dev(dev, xq, xs, uq, us)
    if layout == "tile_major":
        gq_d, uq_d = gm().fp8_weight_repack(gq_d), gm().fp8_weight_repack(uq_d)
    cnt_d, cu_d = torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev)
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    check(lib().bgmoe_set_skinny_max_rows(0))
    try:
        out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
        gm().fp8_blockwise_grouped_gemm(xq_d, gq_d, cnt_d, cu_d, xs_t, gs_d, 16, out, weight_layout=layout)
        h = torch.full((m, n), 5.0, dtype=torch.bfloat16, device=dev)
        gm().fp8_blockwise_fused_s1(xq_d, gq_d, uq_d, cnt_d, cu_d, xs_t, gs_d, us_d, 16, h, weight_layout=layout)
    finally:
        check(lib().bgmoe_set_skinny_max_rows(256))
    ref = og.grouped_gemm_fp8(xq, xs, gq, gs, counts, cu, to_bf16=False)
    o = out.float().cpu().numpy()
    np.testing.assert_allclose(o[live], ref[live], rtol=2e-2, atol=5e-3)
    assert np.all(o[~live] == 7.0)
    up = og.grouped_gemm_fp8(xq, xs, uq, us, counts, cu, to_bf16=False)
    href = oq.silu_f32(ref) * up
    hh = h.float().cpu().numpy()
    assert og.rel_frobenius(hh[live], href[live]) < 4e-3 and np.all(hh[~live] == 5.0)


def test_pointer_tables_slot_permutation_refresh_and_empty_step_under_a_graph(dev):
    """Contract of the reference's tests/test_moe_grouped_fp8_ptrs.py restated: a captured quant -> stage 1 ->
    quant -> down chain over pointer tables follows (a) new device-side counts, (b) a slot permutation written
    into the tables between replays (slot s then holds another expert's weights) and (c) a step in which no
    expert has rows, which must leave the output as it was; every replay equals the eager stacked-weight ops."""
    groups, cap, n, k = 4, 32, 256, 384
    g = torch.Generator().manual_seed(31)
    x = rand_bf16(g, groups * cap, k)
    x_d = x.to(dev)
    mats = []
    for shape in ((groups, n, k), (groups, n, k), (groups, k, n)):
        wq, wsc = oq.weight_block_quant((0.03 * torch.randn(*shape, generator=g)).numpy())
        kb = wsc.shape[2]
        pad = np.zeros(wsc.shape[:2] + ((kb + 3) // 4 * 4,), dtype=np.float32)
        pad[..., :kb] = wsc
        mats.append((torch.from_numpy(wq).to(dev).view(torch.float8_e4m3fn), torch.from_numpy(pad).to(dev)))
    cu = (torch.arange(groups + 1, dtype=torch.int32) * cap).to(dev)
    counts = torch.zeros(groups, dtype=torch.int32, device=dev)
    tables = [torch.zeros(groups, dtype=torch.int64, device=dev) for _ in range(6)]

    def fill_tables(order):
        for j, (w, s_) in enumerate(mats):
            tables[2 * j].copy_(torch.tensor([w[i].data_ptr() for i in order], dtype=torch.int64))
            tables[2 * j + 1].copy_(torch.tensor([s_[i].data_ptr() for i in order], dtype=torch.int64))

    xq = torch.zeros(groups * cap, k, dtype=torch.uint8, device=dev)
    xs = torch.zeros(k // 128, groups * cap, device=dev)
    hq = torch.zeros(groups * cap, n, dtype=torch.uint8, device=dev)
    hs = torch.zeros(n // 128, groups * cap, device=dev)
    h = torch.zeros(groups * cap, n, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(groups * cap, k, dtype=torch.bfloat16, device=dev)
    (gw, gs), (uw, us), (dw, ds) = mats

    def chain(ptrs, order=None):
        qops().act_quant_ragged(x_d, counts, cu, xq, xs, 16)
        a = xq.view(torch.float8_e4m3fn)
        if ptrs:
            gm().fp8_blockwise_fused_s1_ptrs(a, gw[0], tables[0], uw[0], tables[2], counts, cu, xs, gs[0], tables[1],
                                             us[0], tables[3], 16, output=h)
        else:
            o = list(order)
            gm().fp8_blockwise_fused_s1(a, gw[o].contiguous(), uw[o].contiguous(), counts, cu, xs, gs[o].contiguous(),
                                        us[o].contiguous(), 16, output=h)
        qops().act_quant_ragged(h, counts, cu, hq, hs, 16)
        b = hq.view(torch.float8_e4m3fn)
        if ptrs:
            gm().fp8_blockwise_grouped_gemm_ptrs(b, dw[0], tables[4], counts, cu, hs, ds[0], tables[5], 16, output=out)
        else:
            o = list(order)
            gm().fp8_blockwise_grouped_gemm(b, dw[o].contiguous(), counts, cu, hs, ds[o].contiguous(), 16, output=out)

    steps = [((5, 0, 32, 17), (0, 1, 2, 3)), ((1, 31, 2, 0), (2, 0, 3, 1)), ((0, 0, 0, 0), (2, 0, 3, 1)),
             ((32, 32, 32, 32), (3, 2, 1, 0)), ((0, 9, 0, 0), (0, 1, 2, 3))]
    fill_tables(steps[0][1])
    counts.copy_(torch.tensor(steps[0][0], dtype=torch.int32))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain(True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain(True)
    previous = None
    for cnt, order in steps:
        counts.copy_(torch.tensor(cnt, dtype=torch.int32))
        fill_tables(order)
        marker = out.clone() if previous is None else previous.clone()
        out.copy_(marker)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        out.copy_(marker)
        chain(False, order)
        torch.cuda.synchronize()
        say(f"graph step counts={cnt} order={order}")
        assert torch.equal(got, out), (cnt, order)
        if sum(cnt) == 0:
            assert torch.equal(got, marker)
        previous = got
