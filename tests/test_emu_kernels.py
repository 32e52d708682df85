"""The library's kernel sources run on the CPU emulator of tests/emu (one fiber per lane; matrix instructions,
shuffles and barriers as rendezvous; asynchronous global -> LDS loads landing either at once or as late as the
kernel's own waits allow).  Kernels a GPU has run are checked here against the oracle first -- that is what says the
emulator executes this code correctly -- and the variants no GPU has run yet are then held to the same oracle and,
where they promise it, to bit equality with the proven form."""
import ctypes as C

import numpy as np
import pytest
import torch

from batchgen_amd._lib import Fp8Act, Fp8Weight
from oracle import fp8 as ofp8
from oracle import gemm as og
from oracle import quant as oq
from tests import emu
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
    return counts, cu, m, np.ascontiguousarray(xq), np.ascontiguousarray(xs), ws, live


def _tile_major(h, wq):
    out = np.empty_like(wq)
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
    wq = np.ascontiguousarray(wq)
    wsc = np.ascontiguousarray(wsc.astype(np.float32))
    out = np.full((m, n), np.float32(fill)).astype(np.float32)
    out16 = (out.view(np.uint32) >> 16).astype(np.uint16)
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
        wq = np.ascontiguousarray(wq)
        if layout == 1:
            wq = _tile_major(h, wq)
        wsc = np.ascontiguousarray(wsc.astype(np.float32))
        arrs += [wq, wsc]
        descs.append(_weight(wq, wsc, layout))
    a = _act(xq, xs)
    out16 = np.full((m, n), 0x40A0, dtype=np.uint16)                      # bf16 5.0
    ok(h, h.bgmoe_fp8_fused_s1(C.byref(a), C.byref(descs[0]), C.byref(descs[1]), p(counts), p(cu), len(counts), m, n, k,
                               p(out16), None, None, 0, 0, None))
    hq = np.full((m, n), 0x55, dtype=np.uint8)
    hs = np.full((n // 128, m), -3.0, dtype=np.float32)
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
