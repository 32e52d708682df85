"""The library's kernel sources run on the CPU emulator of tests/emu (one fiber per lane; matrix instructions,
shuffles and barriers as rendezvous; asynchronous global -> LDS loads landing either at once or as late as the
kernel's own waits allow).  Kernels a GPU has run are checked here against the oracle first -- that is what says the
emulator executes this code correctly -- and the variants no GPU has run yet are then held to the same oracle and,
where they promise it, to bit equality with the proven form.  Inputs and outputs live in guarded buffers (an
inaccessible page right behind each array): a kernel that reads or writes past an array's end faults on the spot."""
import ctypes as C

import numpy as np
import pytest
import torch

from batchgen_amd._lib import Fp8Act, Fp8Weight
from oracle import fp8 as ofp8
from oracle import gemm as og
from oracle import quant as oq
from tests import emu
from tests.emu import guarded as G
from tests.emu import ok, p
from tests.util import rand_bf16


@pytest.fixture(scope="module")
def h():
    return emu.load()


def test_emulator_e4m3_codec_is_the_oracles(h):
    allb = np.arange(256, dtype=np.uint8)
    dec = ofp8.e4m3fn_decode(allb)
    for b in range(256):
        v = h.emu_e4m3_to_f32(b)
        assert (np.isnan(v) and np.isnan(dec[b])) or v == dec[b], b
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * s for s in (1e-3, 0.02, 1.0, 100.0)])
    x = np.clip(np.concatenate([x, dec[~np.isnan(dec)], [0.0, -0.0, 2.0 ** -10, 2.0 ** -9, 447.9, 448.0]]), -448, 448)
    want = ofp8.e4m3fn_encode(x.astype(np.float32))
    got = np.array([h.emu_f32_to_e4m3(float(v)) for v in x], dtype=np.uint8)
    assert np.array_equal(got, want)


def _layout(counts, align=16):
    counts = np.asarray(counts, dtype=np.int32)
    cu = np.concatenate([[0], np.cumsum((counts + align - 1) // align * align)]).astype(np.int32)
    return counts, cu


def _problem(seed, counts, n, k, nmat=1):
    g = torch.Generator().manual_seed(seed)
    counts, cu = _layout(counts)
    m = max(int(cu[-1]), 1)
    xq, xs = oq.act_quant(rand_bf16(g, m, k))
    ws = [oq.weight_block_quant((0.02 * torch.randn(len(counts), n, k, generator=g)).numpy()) for _ in range(nmat)]
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    ws = [(G(wq), G(wsc.astype(np.float32))) for wq, wsc in ws]
    return G(counts), G(cu), m, G(xq), G(xs), ws, live


def _tile_major(h, wq):
    out = G(np.empty_like(wq))
    g, n, k = wq.shape
    ok(h, h.bgmoe_fp8_weight_repack(p(wq), p(out), g, n, k, None))
    return out


def _weight(wq, wsc, layout):
    g, n, k = wq.shape
    return Fp8Weight(p(wq), n * k, None, p(wsc), wsc.shape[1] * wsc.shape[2], wsc.shape[2], None, layout, 0)


def _act(xq, xs):
    return Fp8Act(p(xq), p(xs), xs.shape[1], 1, 0)


def run_gemm(h, counts, cu, m, xq, xs, w, n, k, layout=0, fill=7.0):
    wq, wsc = w
    wq = G(wq)
    wsc = G(wsc.astype(np.float32))
    out = np.full((m, n), np.float32(fill)).astype(np.float32)
    out16 = G((out.view(np.uint32) >> 16).astype(np.uint16))
    a, b = _act(xq, xs), _weight(wq, wsc, layout)
    ok(h, h.bgmoe_fp8_grouped_gemm(C.byref(a), C.byref(b), p(counts), p(cu), len(counts), m, n, k, p(out16), None))
    return (out16.astype(np.uint32) << 16).view(np.float32)


def test_proven_streaming_gemm_on_the_emulator_matches_the_oracle(h):
    """The weight-streaming grouped GEMM (a GPU has run it) through the emulator: the oracle's gates hold, rows
    outside every group keep their fill value."""
    counts, cu, m, xq, xs, ws, live = _problem(1, (0, 1, 17, 40, 64, 70), 256, 384)
    out = run_gemm(h, counts, cu, m, xq, xs, ws[0], 256, 384)
    ref = og.grouped_gemm_fp8(xq, xs, ws[0][0], ws[0][1], counts, cu, to_bf16=False)
    np.testing.assert_allclose(out[live], ref[live], rtol=2e-2, atol=5e-3)
    assert og.rel_frobenius(out[live], ref[live]) < 3e-3
    assert np.all(out[~live] == 7.0)


def bf16_bits_to_f32(b16):
    return (b16.astype(np.uint32) << 16).view(np.float32)


def run_s1(h, counts, cu, m, xq, xs, wg, wu, n, k, layout=0):
    """Fused stage 1 with both outputs: bf16 h (fill 5.0), e4m3 bytes (fill 0x55) and scales [n/128, m] (fill -3)."""
    arrs = []
    descs = []
    for wq, wsc in (wg, wu):
        wq = G(wq)
        if layout == 1:
            wq = _tile_major(h, wq)
        wsc = G(wsc.astype(np.float32))
        arrs += [wq, wsc]
        descs.append(_weight(wq, wsc, layout))
    a = _act(xq, xs)
    out16 = G(np.full((m, n), 0x40A0, dtype=np.uint16))                   # bf16 5.0
    ok(h, h.bgmoe_fp8_fused_s1(C.byref(a), C.byref(descs[0]), C.byref(descs[1]), p(counts), p(cu), len(counts), m, n, k,
                               p(out16), None, None, 0, 0, None))
    hq = G(np.full((m, n), 0x55, dtype=np.uint8))
    hs = G(np.full((n // 128, m), -3.0, dtype=np.float32))
    ok(h, h.bgmoe_fp8_fused_s1(C.byref(a), C.byref(descs[0]), C.byref(descs[1]), p(counts), p(cu), len(counts), m, n, k,
                               None, p(hq), p(hs), 1, m, None))
    return bf16_bits_to_f32(out16), hq, hs


def check_s1_against_oracle(xq, xs, wg, wu, counts, cu, live, got):
    hh, hq, hs = got
    gate = og.grouped_gemm_fp8(xq, xs, wg[0], wg[1], counts, cu, to_bf16=False)
    up = og.grouped_gemm_fp8(xq, xs, wu[0], wu[1], counts, cu, to_bf16=False)
    href = oq.silu_f32(gate) * up
    np.testing.assert_allclose(hh[live], href[live], rtol=5e-2, atol=2e-2)
    assert og.rel_frobenius(hh[live], href[live]) < 4e-3
    assert np.all(hh[~live] == 5.0) and np.all(hq[~live] == 0x55) and np.all(hs[:, ~live] == -3.0)
    # the fused epilogue's bytes and scales are the quantiser's on the bf16 output
    q2, s2 = oq.act_quant(torch.from_numpy(hh).to(torch.bfloat16))
    assert np.array_equal(hq[live], np.asarray(q2)[live])
    assert np.array_equal(hs.T[live], np.asarray(s2)[live])


S1_COUNTS = (0, 1, 31, 32, 33, 40, 64, 65, 100, 130)


@pytest.mark.parametrize("layout", [0, 1], ids=["row_major", "tile_major"])
def test_streaming_stage1_and_its_tall_items_on_the_emulator(h, layout):
    """Proven form first (32-row items) against the oracle and the requantisation identity; then the tall items
    (no GPU has run them): same bits, for both limits and for groups on either side of them."""
    n, k = 256, 384
    counts, cu, m, xq, xs, ws, live = _problem(2, S1_COUNTS, n, k, nmat=2)
    want = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
    check_s1_against_oracle(xq, xs, ws[0], ws[1], counts, cu, live, want)
    try:
        for tall_min in (32, 64, 100):
            ok(h, h.bgmoe_set_skinny_tall_min_rows(tall_min))
            got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
            for name, a, b in zip(("bf16 output", "e4m3 bytes", "scales"), want, got):
                assert np.array_equal(a, b), f"{name} differ with tall items above {tall_min} rows"
    finally:
        ok(h, h.bgmoe_set_skinny_tall_min_rows(0))


@pytest.mark.parametrize("k", [128, 256, 640])
def test_tall_items_with_short_and_odd_k(h, k):
    """One, two and five K-blocks against the two-stage ring of the tall items."""
    n = 128
    counts, cu, m, xq, xs, ws, live = _problem(3 + k, (70, 3, 48), n, k, nmat=2)
    want = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, 1)
    try:
        ok(h, h.bgmoe_set_skinny_tall_min_rows(32))
        got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, 1)
    finally:
        ok(h, h.bgmoe_set_skinny_tall_min_rows(0))
    for a, b in zip(want, got):
        assert np.array_equal(a, b)


@pytest.fixture
def tiled_only(h):
    """Every group on the LDS-tiled kernels (row limit of the streaming kernel 0); restored afterwards."""
    ok(h, h.bgmoe_set_skinny_max_rows(0))
    try:
        yield
    finally:
        ok(h, h.bgmoe_set_tiled_variant(0))
        ok(h, h.bgmoe_set_skinny_max_rows(256))
        h.emu_set_async_mode(0)
        h.emu_set_schedule(0)


K64_CASES = [  # counts, n, k
    ((256, 257, 1, 0, 300), 256, 256),                 # two K-blocks: the shortest K the variant takes
    ((130, 0, 17), 384, 384),                          # an output narrower than the last 256-column tile of the plain GEMM
    ((40, 520), 128, 512),
]


# asynchronous loads land at once / as late as the waits allow; waves advance together / the first or the last wave
# runs ahead as far as the barriers let it
K64_MODES = [("eager", 0), ("lazy", 0), ("eager", 1), ("eager", 2), ("lazy", 2)]


@pytest.mark.parametrize("mode,schedule", K64_MODES, ids=[f"{m}_sched{s}" for m, s in K64_MODES])
@pytest.mark.parametrize("variant", [2, 1], ids=["plain_stores", "regrouped_stores"])
@pytest.mark.parametrize("layout", [0, 1], ids=["row_major", "tile_major"])
@pytest.mark.parametrize("counts,n,k", K64_CASES, ids=["k256", "k384", "k512"])
def test_k64_tiled_kernel_on_the_emulator(h, tiled_only, counts, n, k, layout, variant, mode, schedule):
    """The K = 64 LDS-tiled kernel (no GPU has run it): plain GEMM and fused stage 1 against the oracle, with the
    asynchronous loads landing at once (a slot refilled too early would corrupt a step still being read -- most
    visibly when one wave runs ahead of the others) and as late as the kernel's wait counts allow (a wait that is
    too lenient would leave a step stale)."""
    counts, cu, m, xq, xs, ws, live = _problem(10 + n + k, counts, n, k, nmat=2)
    ok(h, h.bgmoe_set_tiled_variant(variant))
    h.emu_set_async_mode(1 if mode == "lazy" else 0)
    h.emu_set_schedule(schedule)
    before = emu.stats(h)
    wq = np.ascontiguousarray(ws[0][0])
    out = run_gemm(h, counts, cu, m, xq, xs, (_tile_major(h, wq) if layout else wq, ws[0][1]), n, k, layout)
    ref = og.grouped_gemm_fp8(xq, xs, ws[0][0], ws[0][1], counts, cu, to_bf16=False)
    np.testing.assert_allclose(out[live], ref[live], rtol=2e-2, atol=5e-3)
    assert og.rel_frobenius(out[live], ref[live]) < 3e-3
    assert np.all(out[~live] == 7.0)
    got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
    check_s1_against_oracle(xq, xs, ws[0], ws[1], counts, cu, live, got)
    assert emu.stats(h)["async_loads"] > before["async_loads"]


@pytest.mark.parametrize("mode", ["eager", "lazy"])
def test_k64_split_tail_on_the_emulator(h, tiled_only, mode):
    """24 work items on the emulated device's 16 blocks (two per XCD): every XCD has three items, so its last round
    holds one, which is split into two 128-token halves taken by its two blocks -- including a half whose rows all
    lie past the group's end (the 300-row group's second tile has 44 rows) and a half that starts mid-group."""
    import ctypes
    from batchgen_amd.build import build_hostcheck
    counts0 = (512, 300, 256, 700, 1000)
    n, k = 256, 256
    hc = ctypes.CDLL(build_hostcheck())
    hc.hc_tiled_walk.restype = C.c_int
    hc.hc_tiled_walk.argtypes = [C.POINTER(C.c_int32), C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint, C.POINTER(C.c_int), C.c_int]
    out = (C.c_int * (6 * 128))()
    nv = hc.hc_tiled_walk((C.c_int32 * 5)(*counts0), 5, 0, 2, 8, 16, out, 128)
    visits = np.ctypeslib.as_array(out)[: 6 * nv].reshape(-1, 6)
    assert (visits[:, 5] >= 0).sum() == 16, "the shape is meant to split one item per XCD"
    counts, cu, m, xq, xs, ws, live = _problem(99, counts0, n, k, nmat=2)
    ok(h, h.bgmoe_set_tiled_variant(1))
    h.emu_set_async_mode(1 if mode == "lazy" else 0)
    got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, 1)
    check_s1_against_oracle(xq, xs, ws[0], ws[1], counts, cu, live, got)


# ---- MXFP4 (W4A16) kernels ------------------------------------------------------------------------------------------------
def _mx_problem(seed, counts, n, k, align=16):
    from oracle import mxfp4 as mx
    counts, cu = _layout(counts, align)
    m = max(int(cu[-1]), 1)
    x = rand_bf16(torch.Generator().manual_seed(seed), m, k)
    x16 = G(x.view(torch.int16).numpy().view(np.uint16))
    ws = []
    for s in (seed + 1, seed + 2):
        pk, sc = mx.quantize((0.02 * np.random.default_rng(s).standard_normal((len(counts), n, k))).astype(np.float32))
        ws.append((G(pk), G(sc)))
    live = np.zeros(m, dtype=bool)
    for e, c in enumerate(counts):
        live[cu[e]:cu[e] + c] = True
    return G(counts), G(cu), m, x, x16, ws, live


def _mx_weight(h, pk, sc, layout):
    from batchgen_amd._lib import Mxfp4Weight
    g, n, k2 = pk.shape
    if layout == 1:
        po, so = G(np.empty_like(pk)), G(np.empty_like(sc))
        ok(h, h.bgmoe_mxfp4_weight_repack(p(pk), p(sc), p(po), p(so), g, n, 2 * k2, None))
        pk, sc = po, so
    return (pk, sc), Mxfp4Weight(p(pk), n * k2, None, p(sc), n * sc.shape[2], None, layout, 0)


def run_mx(h, counts, cu, m, x16, ws, n, k, layout, activation=0, row_pair=None, tokens=None, top_k=0):
    keep, descs = [], []
    for pk, sc in ws:
        arrs, d = _mx_weight(h, pk, sc, layout)
        keep.append(arrs)
        descs.append(d)
    out = G(np.full((m, n), 0x40E0, dtype=np.uint16))                     # bf16 7.0
    ok(h, h.bgmoe_mxfp4_grouped_gemm(p(x16), C.byref(descs[0]), p(counts), p(cu), len(counts), m, n, k, p(out), None, 0, None))
    hh = G(np.full((m, n), 0x40A0, dtype=np.uint16))                      # bf16 5.0
    if row_pair is None:
        ok(h, h.bgmoe_mxfp4_fused_s1(p(x16), C.byref(descs[0]), C.byref(descs[1]), p(counts), p(cu), len(counts), m, n, k,
                                     p(hh), None, activation, 0, None))
    else:
        ok(h, h.bgmoe_mxfp4_fused_s1_gather(p(tokens), tokens.shape[0], p(row_pair), top_k, C.byref(descs[0]),
                                            C.byref(descs[1]), p(counts), p(cu), len(counts), m, n, k, p(hh), None,
                                            activation, 0, None))
    return bf16_bits_to_f32(out), bf16_bits_to_f32(hh)


MX_CASES = [((0, 1, 17, 33, 70), 256, 128), ((9, 40, 3), 128, 640), ((65, 2), 256, 896), ((20, 100), 384, 1664)]


@pytest.mark.parametrize("layout", [0, 1], ids=["row_major", "tile_major"])
@pytest.mark.parametrize("counts,n,k", MX_CASES, ids=[f"k{c[2]}" for c in MX_CASES])
def test_mxfp4_kernel_and_its_second_shape_on_the_emulator(h, counts, n, k, layout):
    """The proven shape (64-row items, three prefetch stages) against the oracle; then the second shape (32-row
    items, six stages, a wait count that follows the depth; no GPU has run it): same bits, both activations --
    1, 5, 7 and 13 K-blocks against the six stages."""
    from oracle import situ as osi
    counts, cu, m, x, x16, ws, live = _mx_problem(40 + n + k, counts, n, k)
    want = run_mx(h, counts, cu, m, x16, ws, n, k, layout)
    xf = oq.as_f32(x)
    ref = og.grouped_gemm_mxfp4(xf, ws[0][0], ws[0][1], counts, cu, to_bf16=False)
    np.testing.assert_allclose(want[0][live], ref[live], rtol=1e-2, atol=2e-3)
    assert og.rel_frobenius(want[0][live], ref[live]) < 3e-3 and np.all(want[0][~live] == 7.0)
    upv = og.grouped_gemm_mxfp4(xf, ws[1][0], ws[1][1], counts, cu, to_bf16=False)
    assert og.rel_frobenius(want[1][live], (oq.silu_f32(ref) * upv)[live]) < 4e-3 and np.all(want[1][~live] == 5.0)
    want_situ = run_mx(h, counts, cu, m, x16, ws, n, k, layout, activation=1)[1]
    assert og.rel_frobenius(want_situ[live], osi.situ_fused(ref, upv)[live]) < 6e-3
    for variant in (1, 2, 3):               # 2: the item height per group; 3: the default height with four stages
        try:
            ok(h, h.bgmoe_set_mxfp4_variant(variant))
            got = run_mx(h, counts, cu, m, x16, ws, n, k, layout)
            got_situ = run_mx(h, counts, cu, m, x16, ws, n, k, layout, activation=1)[1]
        finally:
            ok(h, h.bgmoe_set_mxfp4_variant(0))
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]) and np.array_equal(got_situ, want_situ), variant


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
@pytest.mark.parametrize("n_tok,top_k,e_total,start,el,mtp", [(96, 4, 24, 8, 6, 96), (200, 4, 8, 0, 6, 64), (1100, 8, 16, 4, 8, 700)])
def test_index_only_dispatch_and_stage1_through_the_map_on_the_emulator(h, n_tok, top_k, e_total, start, el, mtp, variant):
    """bgmoe_dispatch_index_3d against the oracle (counts, arrivals, positions, the inverse row -> pair map; the
    third case takes the histogram / scan / rank launches), then the fused stage 1 reading its rows through the map
    against the same kernel on the rows gathered by bgmoe_dispatch_scatter_3d: same bits.  No GPU has run either."""
    from oracle import permute as op
    rng = np.random.default_rng(n_tok)
    ids = G(np.stack([rng.permutation(e_total)[:top_k] for _ in range(n_tok)]).astype(np.int32))
    hdim, inter = 256, 128
    nk = n_tok * top_k
    ws_bytes = max(int(h.bgmoe_dispatch_workspace_bytes(nk, el)), 16)
    wsp = G(np.zeros(ws_bytes, dtype=np.uint8))
    counts = G(np.zeros(el, dtype=np.int32))
    counters = G(np.zeros(el, dtype=np.int32))
    pos = G(np.full(nk, -7, dtype=np.int32))
    row_pair = G(np.full(el * mtp, 2 ** 30, dtype=np.int32))
    ok(h, h.bgmoe_dispatch_index_3d(p(ids), n_tok, top_k, start, el, mtp, p(counts), p(counters), p(pos), p(row_pair), p(wsp),
                                    ws_bytes, None))
    want_counts, want_pos, arrivals = op.dispatch_masked_arrivals(ids, start, el, mtp)
    want_pos = np.asarray(want_pos).reshape(-1)
    assert np.array_equal(counts, want_counts) and np.array_equal(counters, arrivals) and np.array_equal(pos, want_pos)
    want_rp = np.full(el * mtp, 2 ** 30, dtype=np.int32)
    placed = np.nonzero(want_pos >= 0)[0]
    want_rp[want_pos[placed]] = placed
    assert np.array_equal(row_pair, want_rp)
    if n_tok > 500:
        return                                                  # the GEMM part at the two smaller sizes only
    x = rand_bf16(torch.Generator().manual_seed(5), n_tok, hdim)
    x16 = G(x.view(torch.int16).numpy().view(np.uint16))
    act = G(np.zeros((el * mtp, hdim), dtype=np.uint16))
    counts2, counters2, pos2 = np.zeros_like(counts), np.zeros_like(counters), np.zeros_like(pos)
    ok(h, h.bgmoe_dispatch_scatter_3d(p(x16), p(ids), n_tok, top_k, hdim, p(act), start, el, mtp, p(counts2), p(counters2),
                                      p(pos2), p(wsp), ws_bytes, None))
    assert np.array_equal(counts2, counts) and np.array_equal(pos2, pos)
    from oracle import mxfp4 as mx
    ws = []
    for s in (1, 2):
        pk, sc = mx.quantize((0.02 * np.random.default_rng(s).standard_normal((el, inter, hdim))).astype(np.float32))
        ws.append((G(pk), G(sc)))
    cu = G((np.arange(el + 1) * mtp).astype(np.int32))
    try:
        ok(h, h.bgmoe_set_mxfp4_variant(variant))
        want = run_mx(h, counts, cu, el * mtp, act, ws, inter, hdim, 1)[1]
        got = run_mx(h, counts, cu, el * mtp, act, ws, inter, hdim, 1, row_pair=row_pair, tokens=x16, top_k=top_k)[1]
    finally:
        ok(h, h.bgmoe_set_mxfp4_variant(0))
    assert np.array_equal(got, want)


# ---- bf16 GEMM (router GEMM / linear layers) --------------------------------------------------------------------------------
RG_PLANS = [(-1, -1), (-1, 0), (-1, 1), (-1, 2), (-1, 3), (-1, 4), (-1, 5)]      # chosen from the sizes; forced shapes; 5 = 128 x 64 tiles


@pytest.mark.parametrize("mode", ["eager", "lazy"])
@pytest.mark.parametrize("n,hd,e", [(129, 64, 64), (300, 1024, 100), (70, 512, 257), (256, 1536, 192)])
def test_bf16_gemm_shapes_agree_bit_for_bit_on_the_emulator(h, n, hd, e, mode):
    """Every launch shape of the bf16 GEMM computes the same chain per logit, so fp32 logits and bf16 outputs must be
    the same bits whichever shape runs -- the proven ones among themselves (which is what says the emulator runs
    this file correctly) and the 128-token x 64-output block tile that no GPU has run; and all of them the float64
    product to 1e-5.  Shapes that a size does not admit fall back to the automatic choice inside the library."""
    g = torch.Generator().manual_seed(n + hd + e)
    x = rand_bf16(g, n, hd)
    w = rand_bf16(g, e, hd, scale=0.05)
    x16 = G(x.view(torch.int16).numpy().view(np.uint16))
    w16 = G(w.view(torch.int16).numpy().view(np.uint16))
    ws_bytes = max(int(h.bgmoe_router_gemm_workspace_bytes(n, hd, e)), 16)
    ref = x.double().numpy() @ w.double().numpy().T
    h.emu_set_async_mode(1 if mode == "lazy" else 0)
    results = {}
    try:
        for plan in RG_PLANS:
            ok(h, h.bgmoe_set_router_gemm_plan(*plan))
            wsp = G(np.zeros(ws_bytes, dtype=np.uint8))
            logits = G(np.full((n, e), 9.0, dtype=np.float32))
            ok(h, h.bgmoe_router_gemm(p(x16), p(w16), n, hd, e, None, 0, 0, p(logits), p(wsp), ws_bytes, None))
            out16 = G(np.zeros((n, e), dtype=np.uint16))
            ok(h, h.bgmoe_bf16_linear(p(x16), p(w16), n, hd, e, p(out16), p(wsp), ws_bytes, None))
            results[plan] = (logits, out16)
    finally:
        ok(h, h.bgmoe_set_router_gemm_plan(-1, -1))
        h.emu_set_async_mode(0)
    base = results[(-1, -1)]
    assert np.linalg.norm(base[0] - ref) / np.linalg.norm(ref) < 1e-5
    for plan, (lg, o16) in results.items():
        assert np.array_equal(lg, base[0]), f"fp32 logits of plan {plan} differ"
        assert np.array_equal(o16, base[1]), f"bf16 outputs of plan {plan} differ"


def test_guarded_buffers_catch_an_overrun():
    """The guard is real: a kernel given an output buffer one tile short dies on the spot with a message that names
    the overrun (run in a child process: the emulator aborts)."""
    import subprocess
    import sys
    code = (
        "import numpy as np\n"
        "from tests import emu\n"
        "from tests.emu import guarded as G, p\n"
        "h = emu.load()\n"
        "src = G(np.zeros((1, 32, 128), dtype=np.uint8))\n"
        "dst = G(np.zeros((1, 16, 128), dtype=np.uint8))\n"          # half of what the repack writes
        "h.bgmoe_fp8_weight_repack(p(src), p(dst), 1, 32, 128, None)\n"
        "print('not reached')\n")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=emu.os.path.dirname(emu.os.path.dirname(emu.os.path.dirname(emu.os.path.abspath(emu.__file__)))))
    assert r.returncode != 0 and "not reached" not in r.stdout
    assert "past the end of a guarded buffer" in r.stderr, r.stderr[-500:]


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_through_the_new_variants(h, seed):
    """Seeded random group sizes, widths, depths, layouts, load models and schedules through the three variants of the
    FP8 / MXFP4 grouped kernels that no GPU has run (a longer private soak of the same generator found nothing)."""
    rng = np.random.default_rng(4242 + seed)
    kind = ("k64", "tall", "mx")[seed % 3]
    try:
        if kind == "k64":
            counts = tuple(int(rng.choice([0, 1, 5, 127, 128, 129, 255, 256, 257, 300, 511, 513])) for _ in range(int(rng.integers(1, 5)))) + (3,)
            n, k = int(rng.choice([128, 256, 384, 512])), int(rng.choice([256, 384, 512, 768]))
            layout = int(rng.integers(0, 2))
            counts, cu, m, xq, xs, ws, live = _problem(seed, counts, n, k, nmat=2)
            ok(h, h.bgmoe_set_skinny_max_rows(0))
            ok(h, h.bgmoe_set_tiled_variant(int(rng.choice([1, 2]))))
            h.emu_set_async_mode(int(rng.integers(0, 2)))
            h.emu_set_schedule(int(rng.integers(0, 3)))
            got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
            check_s1_against_oracle(xq, xs, ws[0], ws[1], counts, cu, live, got)
        elif kind == "tall":
            counts = tuple(int(rng.choice([0, 1, 16, 31, 32, 33, 47, 64, 65, 96, 100, 128, 130, 200])) for _ in range(int(rng.integers(1, 7)))) + (40,)
            n, k = int(rng.choice([128, 256, 384])), int(rng.choice([128, 256, 384, 640]))
            layout = int(rng.integers(0, 2))
            counts, cu, m, xq, xs, ws, live = _problem(seed, counts, n, k, nmat=2)
            h.emu_set_schedule(int(rng.integers(0, 3)))
            want = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
            ok(h, h.bgmoe_set_skinny_tall_min_rows(int(rng.choice([32, 40, 64, 100]))))
            got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
            for a, b in zip(want, got):
                assert np.array_equal(a, b)
        else:
            counts = tuple(int(rng.choice([0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 130])) for _ in range(int(rng.integers(1, 6)))) + (9,)
            n, k = int(rng.choice([128, 256, 384])), int(rng.choice([128, 256, 640, 768, 896, 1152]))
            layout = int(rng.integers(0, 2))
            counts, cu, m, x, x16, ws, live = _mx_problem(seed, counts, n, k)
            want = run_mx(h, counts, cu, m, x16, ws, n, k, layout)
            ok(h, h.bgmoe_set_mxfp4_variant(1))
            got = run_mx(h, counts, cu, m, x16, ws, n, k, layout)
            assert np.array_equal(got[0], want[0]) and np.array_equal(got[1][live], want[1][live])
    finally:
        ok(h, h.bgmoe_set_mxfp4_variant(0))
        ok(h, h.bgmoe_set_skinny_tall_min_rows(0))
        ok(h, h.bgmoe_set_tiled_variant(0))
        ok(h, h.bgmoe_set_skinny_max_rows(256))
        h.emu_set_async_mode(0)
        h.emu_set_schedule(0)


def run_plain_gemm(h, counts, cu, m, xq, xs, w, n, k, layout):
    wq, wsc = w
    if layout == 1:
        wq = _tile_major(h, wq)
    out16 = G(np.full((m, n), 0x40E0, dtype=np.uint16))                   # bf16 7.0
    a, b = _act(xq, xs), _weight(wq, wsc, layout)
    ok(h, h.bgmoe_fp8_grouped_gemm(C.byref(a), C.byref(b), p(counts), p(cu), len(counts), m, n, k, p(out16), None))
    return np.array(out16)


@pytest.fixture
def streaming_knobs(h):
    yield
    ok(h, h.bgmoe_set_skinny_s1_stages(3))
    ok(h, h.bgmoe_set_skinny_gemm_stages(2))
    ok(h, h.bgmoe_set_mxfp4_variant(0))
    ok(h, h.bgmoe_set_skinny_tall_min_rows(0))
    h.emu_set_async_mode(0)
    h.emu_set_schedule(0)
    h.emu_set_wait_slack(0)


@pytest.mark.parametrize("layout", [0, 1], ids=["row_major", "tile_major"])
@pytest.mark.parametrize("k", [128, 256, 384, 640, 1152])
def test_plain_streaming_gemm_at_every_prefetch_depth(h, streaming_knobs, k, layout):
    """The down projection's kernel with two (a GPU has run it), three, four and six prefetch stages; 1 to 9 K-blocks, so
    shorter than, equal to and longer than every ring.  Loads land at once, or as late as the kernel's hand-placed
    waits allow with every global load of the item counted the way the hardware counts them (the deeper rings wait
    for a different count than the proven one); three wave schedules.  One set of bits throughout."""
    n = 256
    counts, cu, m, xq, xs, ws, live = _problem(40 + k, (0, 1, 17, 40, 64, 70, 130), n, k)
    want = run_plain_gemm(h, counts, cu, m, xq, xs, ws[0], n, k, layout)
    ref = og.grouped_gemm_fp8(xq, xs, ws[0][0], ws[0][1], counts, cu, to_bf16=False)
    got = bf16_bits_to_f32(want)
    assert og.rel_frobenius(got[live], ref[live]) < 3e-3 and np.all(got[~live] == 7.0)
    for stages in (2, 3, 4, 6):
        ok(h, h.bgmoe_set_skinny_gemm_stages(stages))
        for mode, schedule in ((0, 1), (2, 0), (2, 2)):
            h.emu_set_async_mode(mode)
            h.emu_set_schedule(schedule)
            out = run_plain_gemm(h, counts, cu, m, xq, xs, ws[0], n, k, layout)
            assert np.array_equal(out, want), f"{stages} stages, load model {mode}, schedule {schedule}"


@pytest.mark.parametrize("stages,slack", [(2, 16), (3, 16), (4, 16), (6, 24)])
def test_counted_load_model_catches_a_wait_that_is_too_lenient(h, streaming_knobs, stages, slack):
    """The negative control of the test above: the same kernels with every hand-placed wait loosened by `slack`
    loads (in the emulator, not in the source) compute on token bytes that have not landed, and the result shows it."""
    n, k = 128, 1152
    counts, cu, m, xq, xs, ws, live = _problem(77, (64, 33), n, k)
    want = run_plain_gemm(h, counts, cu, m, xq, xs, ws[0], n, k, 1)
    ok(h, h.bgmoe_set_skinny_gemm_stages(stages))
    h.emu_set_async_mode(2)
    out = run_plain_gemm(h, counts, cu, m, xq, xs, ws[0], n, k, 1)
    assert np.array_equal(out, want)
    h.emu_set_wait_slack(slack)
    out = run_plain_gemm(h, counts, cu, m, xq, xs, ws[0], n, k, 1)
    assert not np.array_equal(out, want)


@pytest.mark.parametrize("layout", [0, 1], ids=["row_major", "tile_major"])
def test_streaming_kernels_with_loads_as_late_as_their_waits_allow(h, streaming_knobs, layout):
    """Stage 1 (32-row and tall items) and the MXFP4 kernel (both shapes), whose hand-placed waits count their
    ordinary weight loads as well: every global load of an item takes its place in the lane's queue, a token load
    lands only when a wait leaves it no other choice.  Same bits as with loads that land at once."""
    n, k = 256, 640
    counts, cu, m, xq, xs, ws, live = _problem(91, (1, 31, 33, 64, 100), n, k, nmat=2)
    want = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
    mxc, mxcu, mxm, x, x16, mws, mlive = _mx_problem(92, (17, 33, 70), n, 1152)
    mwant = run_mx(h, mxc, mxcu, mxm, x16, mws, n, 1152, layout)
    for schedule in (0, 2):
        h.emu_set_async_mode(2)
        h.emu_set_schedule(schedule)
        for tall_min in (0, 32):
            ok(h, h.bgmoe_set_skinny_tall_min_rows(tall_min))
            got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
            for a, b in zip(want, got):
                assert np.array_equal(a, b), f"stage 1, tall_min {tall_min}, schedule {schedule}"
        for variant in (0, 1, 2, 3):
            ok(h, h.bgmoe_set_mxfp4_variant(variant))
            got = run_mx(h, mxc, mxcu, mxm, x16, mws, n, 1152, layout)
            assert np.array_equal(got[0], mwant[0]) and np.array_equal(got[1], mwant[1]), f"MXFP4 shape {variant}"


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
def test_counted_load_model_catches_a_lenient_wait_in_the_mxfp4_kernel(h, streaming_knobs, variant):
    n, k = 128, 1664
    counts, cu, m, x, x16, ws, live = _mx_problem(93, (64, 20), n, k)
    want = run_mx(h, counts, cu, m, x16, ws, n, k, 1)
    ok(h, h.bgmoe_set_mxfp4_variant(variant))
    h.emu_set_async_mode(2)
    got = run_mx(h, counts, cu, m, x16, ws, n, k, 1)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    h.emu_set_wait_slack(24)
    got = run_mx(h, counts, cu, m, x16, ws, n, k, 1)
    assert not (np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]))


@pytest.mark.parametrize("layout", [0, 1], ids=["row_major", "tile_major"])
@pytest.mark.parametrize("m,n,k", [(70, 256, 1024), (100, 128, 2688), (40, 128, 4096), (150, 128, 4096), (300, 128, 1024)])
def test_dense_split_k_gemm_at_every_prefetch_depth(h, streaming_knobs, m, n, k, layout):
    """The one-weight GEMM's block-split form (K-slices of 8 blocks over blocks, fp32 partial sums, ordered sum): the
    proven two-stage kernel against the oracle, then three and four stages under the counted late-load model -- slices
    of 8, 5 and 8 K-blocks against rings of 2, 3 and 4."""
    g = torch.Generator().manual_seed(300 + m + k)
    xq, xs = oq.act_quant(rand_bf16(g, m, k))
    wq, wsc = oq.weight_block_quant((0.02 * torch.randn(1, n, k, generator=g)).numpy())
    xq, xs, wq, wsc = G(xq), G(xs), G(wq), G(wsc.astype(np.float32))
    ref = og.grouped_gemm_fp8(xq, xs, wq, wsc, np.array([m], np.int32), np.array([0, m], np.int32), to_bf16=False)
    wdev = _tile_major(h, wq) if layout == 1 else wq
    need = int(h.bgmoe_fp8_dense_gemm_workspace(m, n, k, layout))
    if need == 0:
        pytest.skip("this shape is served by the wave-split kernel")
    a = _act(xq, xs)

    def run():
        out = G(np.full((m, n), 0x40E0, dtype=np.uint16))
        ws = G(np.full(need // 4, np.nan, dtype=np.float32))
        ok(h, h.bgmoe_fp8_dense_gemm(C.byref(a), p(wdev), p(wsc), wsc.shape[2], layout, m, n, k, p(out), p(ws), need, None))
        return np.array(out)

    want = run()
    assert og.rel_frobenius(bf16_bits_to_f32(want), ref) < 3e-3
    for stages in (3, 4):
        ok(h, h.bgmoe_set_skinny_gemm_stages(stages))
        for mode, schedule in ((0, 1), (2, 0), (2, 2)):
            h.emu_set_async_mode(mode)
            h.emu_set_schedule(schedule)
            assert np.array_equal(run(), want), f"{stages} stages, load model {mode}, schedule {schedule}"


@pytest.mark.parametrize("layout", [0, 1], ids=["row_major", "tile_major"])
@pytest.mark.parametrize("k", [128, 384, 512, 640, 1152])
def test_fused_stage1_with_four_prefetch_stages(h, streaming_knobs, k, layout):
    """Fused stage 1 with a four-stage ring (no GPU has run it) against the proven three-stage form: bf16 output, e4m3
    bytes and scales bit for bit; 1 to 9 K-blocks; loads at once and as late as the waits allow with every global load
    counted; then the negative control -- the same run with every wait loosened by 24 loads must differ."""
    n = 256
    counts, cu, m, xq, xs, ws, live = _problem(500 + k, (0, 1, 31, 33, 64, 100), n, k, nmat=2)
    want = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
    if k == 384:
        check_s1_against_oracle(xq, xs, ws[0], ws[1], counts, cu, live, want)
    ok(h, h.bgmoe_set_skinny_s1_stages(4))
    for mode, schedule in ((0, 1), (2, 0), (2, 2)):
        h.emu_set_async_mode(mode)
        h.emu_set_schedule(schedule)
        got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
        for name, a, b in zip(("bf16 output", "e4m3 bytes", "scales"), want, got):
            assert np.array_equal(a, b), f"{name}: load model {mode}, schedule {schedule}"
    if k >= 640:                             # long enough for the main loop of the four-stage ring
        h.emu_set_wait_slack(24)
        got = run_s1(h, counts, cu, m, xq, xs, ws[0], ws[1], n, k, layout)
        assert not all(np.array_equal(a, b) for a, b in zip(want, got))
