"""CPU checks of the arithmetic the kernels share with the host (csrc/bgmoe_hostdev.h, csrc/bgmoe_tilemap.h),
through the g++-built lib/libbgmoe_hostcheck.so: the text the GPU runs, walked on the CPU.

* pointer halves: a wave builtin's `int` low half with bit 31 set must not sign-extend into the high half;
* launch ranges: lowest / highest byte a strided access touches against its allocation;
* the balanced (stream-K) GEMM's share walk over random launches: no share without a unit, every unit of work
  owned exactly once, a cut item's parts in consecutive shares with the first / last share the kernel computes;
* the K = 64 tile images: a wave's asynchronous loads followed by its operand reads deliver, to every lane, the
  bytes the 32x32x64 matrix instruction expects from it, without LDS bank conflicts.
"""
import ctypes as C
import os
import random

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "batchgen_amd", "lib", "libbgmoe_hostcheck.so")


@pytest.fixture(scope="module")
def hc():
    if not os.path.exists(LIB):                       # nothing built yet: build it (g++, seconds)
        from batchgen_amd import build as b
        b.build_hostcheck(verbose=False)
    lib = C.CDLL(LIB)
    lib.hc_compose_from_int_halves.restype = C.c_uint64
    lib.hc_compose_from_int_halves.argtypes = [C.c_int, C.c_int]
    lib.hc_rows_range_inside.restype = C.c_int
    lib.hc_rows_range_inside.argtypes = [C.c_uint64] * 6 + [C.POINTER(C.c_uint64)] * 2
    lib.hc_sk_weights_ok.restype = C.c_int
    lib.hc_sk_weights_ok.argtypes = [C.POINTER(C.c_int)]
    lib.hc_sk_walk.restype = C.c_int
    lib.hc_sk_walk.argtypes = [C.POINTER(C.c_int32), C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                               C.c_int, C.POINTER(C.c_int), C.c_uint, C.c_uint, C.POINTER(C.c_int), C.c_int,
                               C.POINTER(C.c_uint32)]
    lib.hc_k64_tile_roundtrip.restype = None
    lib.hc_k64_tile_roundtrip.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p]
    lib.hc_k64_tm_tile_roundtrip.restype = None
    lib.hc_k64_tm_tile_roundtrip.argtypes = [C.c_void_p, C.c_void_p]
    lib.hc_k64_operand_offsets.restype = None
    lib.hc_k64_operand_offsets.argtypes = [C.c_void_p, C.c_int]
    lib.hc_k64_acc_coord.restype = None
    lib.hc_k64_acc_coord.argtypes = [C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
    return lib


def _as_int32(v):
    return v - (1 << 32) if v >= (1 << 31) else v


def test_pointer_halves_do_not_sign_extend(hc):
    """The device address 0x00007f12_8000_0040 split into halves and handed over as `int` (bit 31 of the low half
    set: a negative int) comes back whole; so do random 64-bit values."""
    for v in [0x00007F1280000040, 0x00007FFFFFFFFFF0, 0x0000000080000000, 0xFFFFFFFFFFFFFFFF, 0x00000000FFFFFFFF]:
        assert hc.hc_compose_from_int_halves(_as_int32(v & 0xFFFFFFFF), _as_int32(v >> 32)) == v
    rng = random.Random(3)
    for _ in range(2000):
        v = rng.getrandbits(64) | (1 << 31)
        assert hc.hc_compose_from_int_halves(_as_int32(v & 0xFFFFFFFF), _as_int32(v >> 32)) == v


def test_launch_byte_range_against_the_allocation(hc):
    lo, hi = C.c_uint64(), C.c_uint64()
    base = 0x7F0000000000
    # 256 rows of 7168 bytes at a pitch of 7168: exactly the allocation
    assert hc.hc_rows_range_inside(base, 256, 7168, 7168, base, 256 * 7168, lo, hi) == 1
    assert (lo.value, hi.value) == (base, base + 256 * 7168)
    # one row too many, one byte too wide, a base in front of the allocation, an empty launch
    assert hc.hc_rows_range_inside(base, 257, 7168, 7168, base, 256 * 7168, lo, hi) == 0
    assert hc.hc_rows_range_inside(base, 256, 7169, 7168, base, 256 * 7168, lo, hi) == 0
    assert hc.hc_rows_range_inside(base - 16, 1, 16, 16, base, 4096, lo, hi) == 0
    assert hc.hc_rows_range_inside(base + 4096, 0, 64, 64, base, 4096, lo, hi) == 1 and lo.value == hi.value
    # a pitch larger than the row: the last row ends before the pitch does
    assert hc.hc_rows_range_inside(base, 4, 64, 1024, base, 3 * 1024 + 64, lo, hi) == 1
    assert hc.hc_rows_range_inside(base, 4, 64, 1024, base, 3 * 1024 + 63, lo, hi) == 0


# ---- the balanced GEMM's share walk ---------------------------------------------------------------------------
DEFAULT_W = [23, 21, 23, 21, 23, 21, 23, 21]
COST = (4, 2, 2)
# local token counts of benchmark configuration 1's routing draw (32 experts) and the shared expert's 256 rows
CONFIG1_DRAW = [14, 0, 4, 41, 0, 0, 0, 14, 0, 11, 0, 15, 0, 0, 0, 65, 0, 1, 0, 1, 13, 39, 0, 9, 3, 1, 2, 35, 0, 16, 2, 11, 256]


def walk(hc, counts, hi, tt, wc, ntiles, kb, grid, w=DEFAULT_W, cost=COST, min_units=8):
    arr = (C.c_int32 * len(counts))(*counts)
    w8 = (C.c_int * 8)(*w)
    cap = 1 << 18
    out = (C.c_int * (10 * cap))()
    info = (C.c_uint32 * 4)()
    n = hc.hc_sk_walk(arr, len(counts), hi, ntiles, kb, tt, wc, cost[0], cost[1], cost[2], w8, grid, min_units, out, cap, info)
    parts = np.ctypeslib.as_array(out)[: 10 * max(n, 0)].reshape(-1, 10).copy()
    return n, parts, tuple(info)


def check_walk(counts, hi, tt, ntiles, kb, n, parts, info):
    """Every (group, chunk, slab, K-block) owned exactly once; cut items consistent with first / last share."""
    c_total, shares, _, _ = info
    live = [c if 0 <= c <= hi else 0 for c in counts]
    if not any(live):
        assert n == 0
        return
    assert n > 0, f"share {-n - 1} owns no unit"
    assert set(parts[:, 0]) == set(range(shares)), "every share owns at least one part"
    owned = {}
    per_item = {}
    for share, grp, ntile, chunk, cnt, kb_lo, kb_hi, first, last, cpk in parts.tolist():
        assert cnt == live[grp] and 0 <= ntile < ntiles and 0 <= kb_lo < kb_hi <= kb and chunk * 16 * tt < cnt
        for k in range(kb_lo, kb_hi):
            assert (grp, chunk, ntile, k) not in owned
            owned[(grp, chunk, ntile, k)] = share
        per_item.setdefault((grp, chunk, ntile), []).append((share, kb_lo, kb_hi, first, last))
    want = sum(((c + 16 * tt - 1) // (16 * tt)) * ntiles * kb for c in live if c)
    assert len(owned) == want, "units of work missing"
    heads = set()
    for item, ps in per_item.items():
        ps.sort(key=lambda p: p[1])
        assert ps[0][1] == 0 and ps[-1][2] == kb and all(a[2] == b[1] for a, b in zip(ps, ps[1:]))
        first, last = ps[0][3], ps[0][4]
        assert all(p[3] == first and p[4] == last for p in ps), "every part computes the same first / last share"
        assert [p[0] for p in ps] == list(range(first, last + 1)), "one part in each share from first to last"
        if len(ps) > 1:                               # the counter of a cut item lives at its first share: one item each
            assert first not in heads
            heads.add(first)


@pytest.mark.parametrize("shape", [(4, 16, 16, 56, 512), (4, 8, 56, 16, 768)])
def test_share_walk_of_config_1(hc, shape):
    """Stage 1 (2048 gate+up columns = 16 slabs, K = 7168) and the down projection (7168 columns = 56 slabs,
    K = 2048) on configuration 1's draw."""
    tt, wc, ntiles, kb, grid = shape
    n, parts, info = walk(hc, CONFIG1_DRAW, 256, tt, wc, ntiles, kb, grid)
    check_walk(CONFIG1_DRAW, 256, tt, ntiles, kb, n, parts, info)
    assert info[1] == grid                            # enough work for every resident block


def test_share_walk_random_launches(hc):
    rng = random.Random(1)
    for _ in range(300):
        ng = rng.choice([1, 2, 5, 33, 100, 257])
        hi = rng.choice([16, 64, 256])
        counts = [rng.choice([0, 0, 1, 3, 16, 17, 64, 65, 200, 256, 300, -1]) for _ in range(ng)]
        tt, wc = rng.choice([2, 4, 8]), rng.choice([8, 16])
        ntiles, kb = rng.choice([1, 2, 16, 56]), rng.choice([1, 2, 3, 16, 56])
        grid = rng.choice([8, 64, 512, 768, 1024])
        n, parts, info = walk(hc, counts, hi, tt, wc, ntiles, kb, grid)
        check_walk(counts, hi, tt, ntiles, kb, n, parts, info)


def test_share_walk_with_every_accepted_xcd_weighting(hc):
    """Weights the setter accepts (each in [1, 64], sum <= 32 x the smallest) never leave a share without a unit,
    however skewed; the weighting the setter now rejects ({1, 64, 64, ...}) does, which is why it is rejected."""
    rng = random.Random(7)
    tried = 0
    while tried < 150:
        w = [rng.choice([1, 2, 3, 8, 21, 23, 40, 64]) for _ in range(8)]
        if not hc.hc_sk_weights_ok((C.c_int * 8)(*w)):
            continue
        tried += 1
        counts = [rng.choice([0, 1, 8, 16, 33, 64, 100, 256]) for _ in range(rng.choice([3, 20, 33]))]
        tt, wc, ntiles, kb, grid = rng.choice([(4, 16, 16, 56, 512), (4, 8, 56, 16, 768), (2, 8, 4, 8, 64)])
        n, parts, info = walk(hc, counts, 256, tt, wc, ntiles, kb, grid, w=w)
        check_walk(counts, 256, tt, ntiles, kb, n, parts, info)
    for w in ([1] + [64] * 7, [64] * 7 + [1], [0] + [8] * 7, [65] + [8] * 7):
        assert not hc.hc_sk_weights_ok((C.c_int * 8)(*w))
    assert hc.hc_sk_weights_ok((C.c_int * 8)(*DEFAULT_W))
    bad = [1] + [64] * 7
    starved = False
    for counts in ([16] * 32, CONFIG1_DRAW, [1] * 8, [64] * 20):
        for tt, wc, ntiles, kb, grid in [(4, 16, 16, 56, 512), (4, 8, 56, 16, 768)]:
            n, _, _ = walk(hc, counts, 256, tt, wc, ntiles, kb, grid, w=bad)
            starved = starved or n < 0
    assert starved, "the rejected weighting was expected to starve a share on at least one of these launches"


# ---- predicted weight traffic of the two work orders --------------------------------------------------------------
def restream_model(hc, counts, tt, wc, ntiles, kb, grid, tile_bytes=2048, window_bytes=4 << 20):
    """Weight bytes the balanced launch takes from HBM, under a simple L2 model: shares advance through their cost at
    the same rate; a re-stream (chunk > 0) of a slab's K-block is an L2 hit when the same (group, slab, K-block) is
    streamed by a share of the SAME XCD at a time (= cost offset inside the share) no further away than the time
    the XCD needs to replace its 4 MiB L2.  Returns (first-stream bytes, re-stream bytes from HBM, from L2)."""
    n, parts, info = walk(hc, counts, 256, tt, wc, ntiles, kb, grid)
    assert n > 0
    _, shares, n8, _ = info
    # time of every unit = running cost inside its share (every share advances one cost unit per unit of time)
    clock = {s: 0 for s in range(shares)}
    when = {}
    for share, grp, ntile, chunk, cnt, kb_lo, kb_hi, first, last, cpk in parts.tolist():
        for k in range(kb_lo, kb_hi):
            when[(grp, chunk, ntile, k)] = (share // n8 if shares >= 8 else 0, clock[share])
            clock[share] += cpk
    # an XCD's n8 shares move n8 cost units per unit of time; a first-stream weight tile is COST[0] cost units
    window = window_bytes / (n8 * tile_bytes / COST[0])
    first_b = hbm_b = l2_b = 0
    for (grp, chunk, ntile, k), (xcd, t) in when.items():
        nbytes = wc * tile_bytes
        if chunk == 0:
            first_b += nbytes
            continue
        hit = any((grp, c2, ntile, k) in when and when[(grp, c2, ntile, k)][0] == xcd and
                  abs(when[(grp, c2, ntile, k)][1] - t) <= window for c2 in range(chunk))
        if hit:
            l2_b += nbytes
        else:
            hbm_b += nbytes
    return first_b, hbm_b, l2_b


def test_restream_model_of_the_current_cut(hc):
    """What the chunk-by-chunk work order of the balanced launch costs in weight traffic on configuration 1's
    draw (64-row chunks: the group of 65 rows has two, the shared expert's 256 rows four) and on 32 groups of 16
    rows (none): with
    single-chunk groups nothing is streamed twice; with multi-chunk groups the later chunks of a slab run a whole
    chunk's cost later than the first, far outside one L2's reach, so every re-stream comes from HBM.  This is
    the traffic that the item walk of the default kernel avoids by running a slab's chunks side by side."""
    first_b, hbm_b, l2_b = restream_model(hc, [16] * 32, 4, 16, 16, 56, 512)
    assert hbm_b == 0 and l2_b == 0 and first_b == 32 * 2 * 2048 * 7168          # every gate+up byte once
    first_b, hbm_b, l2_b = restream_model(hc, CONFIG1_DRAW, 4, 16, 16, 56, 512)
    active = sum(1 for c in CONFIG1_DRAW if c)
    assert first_b == active * 2 * 2048 * 7168
    chunks_more = sum((c + 63) // 64 - 1 for c in CONFIG1_DRAW if c)
    assert hbm_b + l2_b == chunks_more * 2 * 2048 * 7168
    # 4 more chunks (65 rows: 1, the shared expert's 256 rows: 3) on 21 active groups: 19% more weight bytes, and
    # nine tenths of them come from HBM again
    assert hbm_b / (hbm_b + l2_b) > 0.85 and hbm_b / first_b > 0.15, "the chunk-major order re-streams from HBM"


# ---- K = 64 tile images ----------------------------------------------------------------------------------------------
def test_k64_row_major_tile_image(hc):
    """32 rows x 64 bytes at a pitch of 7168: after the two half-image loads, lane l's operand is row l % 32,
    bytes 32 * (l / 32) .. + 32 of the row's 64."""
    rng = np.random.default_rng(5)
    pitch = 7168
    src = rng.integers(0, 256, size=(32, pitch), dtype=np.uint8)
    got = np.zeros((64, 32), dtype=np.uint8)
    hc.hc_k64_tile_roundtrip(src.ctypes.data, pitch, got.ctypes.data)
    for lane in range(64):
        row, h = lane % 32, lane // 32
        assert np.array_equal(got[lane], src[row, 32 * h: 32 * h + 32]), lane


def test_k64_tile_major_tile_image(hc):
    """Two 16-row tiles in the resident tile-major order ([K half][16-byte piece][row] per 2 KiB tile): the K half
    that the step uses is one contiguous KiB per tile, copied linearly; lane l's operand is again row l % 32, bytes
    32 * (l / 32) .. + 32 of the step's 64."""
    rng = np.random.default_rng(6)
    rows = rng.integers(0, 256, size=(32, 128), dtype=np.uint8)          # 32 weight rows x one 128-wide K-block
    tiles = np.zeros((2, 2, 4, 16, 16), dtype=np.uint8)                   # [tile][K half][piece][row][byte]
    for t in range(2):
        for kh in range(2):
            for q in range(4):
                for r in range(16):
                    tiles[t, kh, q, r] = rows[16 * t + r, 64 * kh + 16 * q: 64 * kh + 16 * q + 16]
    for kh in range(2):
        halves = np.ascontiguousarray(tiles[:, kh]).reshape(2, 1024)      # the two KiB the step loads
        got = np.zeros((64, 32), dtype=np.uint8)
        hc.hc_k64_tm_tile_roundtrip(halves.ctypes.data, got.ctypes.data)
        for lane in range(64):
            row, h = lane % 32, lane // 32
            assert np.array_equal(got[lane], rows[row, 64 * kh + 32 * h: 64 * kh + 32 * h + 32]), (kh, lane)


@pytest.mark.parametrize("tile_major", [0, 1])
def test_k64_operand_reads_have_no_bank_conflicts(hc, tile_major):
    """A 16-byte read occupies 4 of the 64 four-byte banks; any 8 consecutive lanes of one read instruction (what
    the LDS serves per clock at 128 B/clk) must fall into 8 different 16-byte groups of the 256-byte bank row."""
    offs = np.zeros(128, dtype=np.uint32)
    hc.hc_k64_operand_offsets(offs.ctypes.data, tile_major)
    for which in (offs[:64], offs[64:]):
        assert np.all(which % 16 == 0) and which.max() < 2048
        for g0 in range(0, 64, 8):
            groups = (which[g0: g0 + 8] // 16) % 16
            assert len(set(groups.tolist())) == 8, (tile_major, g0, groups)
    assert len(set(offs.tolist())) == 128, "the 64 lanes' two pieces are 128 different pieces of the image"


def test_accumulator_coordinates_cover_the_32x32_product(hc):
    a, b = C.c_uint32(), C.c_uint32()
    seen = set()
    for lane in range(64):
        for v in range(16):
            hc.hc_k64_acc_coord(lane, v, a, b)
            assert b.value == lane % 32 and a.value == 8 * (v // 4) + 4 * (lane // 32) + v % 4
            seen.add((a.value, b.value))
    assert len(seen) == 1024


# ---- the K = 64 kernel's dataflow on one macro tile, against a plain block-scaled GEMM -------------------------------
def _e4m3_table():
    t = np.zeros(256, dtype=np.float64)
    for b in range(256):
        sign, e, m = b >> 7, (b >> 3) & 15, b & 7
        v = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        t[b] = -v if sign else v
    return t


def _tile_major(w):
    """[n, K] bytes -> the resident layout: 16-row x 128-column tiles, byte half*1024 + (q*16 + r)*16 + j of tile
    (nt, kb) = row 16 nt + r, column 128 kb + 64 half + 16 q + j."""
    n, k = w.shape
    t = w.reshape(n // 16, 16, k // 128, 2, 4, 16)            # [nt][r][kb][half][q][j]
    return np.ascontiguousarray(t.transpose(0, 2, 3, 4, 1, 5)).reshape(-1)


@pytest.mark.parametrize("regroup", [0, 1])
@pytest.mark.parametrize("fused,tile_major,cnt,m0,n,n0", [
    (0, 0, 256, 0, 256, 0), (0, 1, 256, 0, 256, 0),            # a full tile, both weight layouts
    (0, 0, 300, 256, 384, 256),                                 # 44 live rows (one token half dead), images past N
    (0, 1, 130, 0, 384, 256), (1, 0, 256, 0, 256, 128), (1, 1, 300, 256, 128, 0), (1, 1, 1, 0, 256, 0),
    (0, 1, 256, 128, 256, 0), (1, 0, 200, 128, 128, 0),        # second halves of split items (count clipped to m0 + 128)
])
def test_k64_kernel_dataflow_on_one_macro_tile(hc, fused, tile_major, cnt, m0, n, n0, regroup):
    """The K = 64 kernel's loads, operand reads, in-place accumulation with the scale change per 128-K block and its
    epilogue coordinates, walked on the CPU with the kernel's own maps: equal (up to fp32 summation order) to
    out[t, c] = sum_kb (sum_k x[t, k] w[c, k]) xs[t, kb] ws[c / 128, kb] on exactly the elements of the macro tile
    that lie inside the group and inside N; nothing else is written; no address leaves its buffer.  `regroup`: the
    epilogue through the per-wave LDS patches (whole row segments per store) instead of per-lane stores."""
    rng = np.random.default_rng(fused * 100 + tile_major * 10 + cnt + n0)
    K, KB = 512, 4
    dec = _e4m3_table()
    codes = np.array([b for b in range(256) if (b & 0x7F) != 0x7F and (b & 0x7F) < 0x60], dtype=np.uint8)   # |v| <= 15
    x = codes[rng.integers(0, len(codes), size=(cnt, K))]
    w0 = codes[rng.integers(0, len(codes), size=(n, K))]
    w1 = codes[rng.integers(0, len(codes), size=(n, K))]
    xs = (rng.random((cnt, KB)) * 0.02 + 0.001).astype(np.float32)
    xs[0, 1] = np.float32(1e-12) / np.float32(448.0)            # a token block that was all zeros: the scale floor
    x[0, 128:256] = 0
    ws0 = (rng.random((n // 128, KB)) * 1e-3 + 1e-5).astype(np.float32)
    ws1 = (rng.random((n // 128, KB)) * 1e-3 + 1e-5).astype(np.float32)
    a0 = _tile_major(w0) if tile_major else np.ascontiguousarray(w0).reshape(-1)
    a1 = _tile_major(w1) if tile_major else np.ascontiguousarray(w1).reshape(-1)
    out = np.zeros((cnt, n), dtype=np.float32)
    written = np.zeros((cnt, n), dtype=np.uint8)
    hc.hc_k64_emulate_item.restype = C.c_int
    hc.hc_k64_emulate_item.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    rc = hc.hc_k64_emulate_item(x.ctypes.data, xs.ctypes.data, cnt, K, a0.ctypes.data, a1.ctypes.data, ws0.ctypes.data,
                                ws1.ctypes.data, n, fused, tile_major, regroup, m0, n0, out.ctypes.data, written.ctypes.data)
    assert rc == 0, rc
    ncols = 128 if fused else 256
    want_mask = np.zeros((cnt, n), dtype=np.uint8)
    want_mask[m0: min(cnt, m0 + 256), n0: min(n, n0 + ncols)] = 1
    assert np.array_equal(written, want_mask), "the write set is the live part of the macro tile"
    xf, rows = dec[x], slice(m0, min(cnt, m0 + 256))
    cols = slice(n0, min(n, n0 + ncols))

    def gemm(wq, ws):
        wf = dec[wq]
        ref = np.zeros((cnt, n))
        for kb in range(KB):
            part = xf[:, 128 * kb: 128 * kb + 128] @ wf[:, 128 * kb: 128 * kb + 128].T
            ref += part * xs[:, kb: kb + 1].astype(np.float64) * np.repeat(ws[:, kb], 128)[None, :]
        return ref

    ref = gemm(w0, ws0)
    if fused:
        up = gemm(w1, ws1)
        ref = ref / (1.0 + np.exp(-ref)) * up
    got, want = out[rows, cols].astype(np.float64), ref[rows, cols]
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max() + 1e-30


# ---- the tiled kernels' walk over work items ---------------------------------------------------------------------------
@pytest.mark.parametrize("counts,lo,ntn,grid", [
    ([512] * 32, 64, 16, 256),                                       # benchmark configuration 2's shape, uniform
    ([130, 0, 700, 65, 64, 3000, 1, 257, 256, 90], 64, 16, 256),     # ragged: empty, below the limit, one row over a tile
    ([300], 0, 1, 8), ([2100, 5, 9000] + [0] * 253, 64, 28, 256), ([257] * 7, 256, 3, 24),
    ([512] * 4, 64, 16, 256),                                        # 16 items on an XCD's 32 blocks: every item split
])
def test_tiled_walk_visits_every_item_once(hc, counts, lo, ntn, grid):
    """Blocks x rounds of the persistent walk cover every (group, m-tile, n-tile) of the groups above the row limit
    exactly once -- whole, or as two 128-token halves taken by two different blocks when the XCD's last round is at
    most half full (a half is then the last thing its block does); and the items one XCD holds in one round form a
    compact patch (few distinct m-tiles and n-tiles: the streams its L2 has to hold)."""
    hc.hc_tiled_walk.restype = C.c_int
    hc.hc_tiled_walk.argtypes = [C.POINTER(C.c_int32), C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint, C.POINTER(C.c_int), C.c_int]
    want = {(g, m, n) for g, c in enumerate(counts) if c > lo for m in range((c + 255) // 256) for n in range(ntn)}
    cap = 2 * len(want) + 16
    out = (C.c_int * (6 * cap))()
    n = hc.hc_tiled_walk((C.c_int32 * len(counts))(*counts), len(counts), lo, ntn, 8, grid, out, cap)
    assert n >= len(want)
    visits = np.ctypeslib.as_array(out)[: 6 * n].reshape(-1, 6)
    whole = [tuple(v[2:5]) for v in visits.tolist() if v[5] == -1]
    halves = {}
    for b, rnd, g, m, nn, half in visits.tolist():
        if half >= 0:
            halves.setdefault((g, m, nn), []).append((half, b))
    assert len(whole) == len(set(whole)) and not (set(whole) & set(halves))
    for item, hs in halves.items():                                  # both halves, taken by two different blocks
        assert sorted(h for h, _ in hs) == [0, 1] and hs[0][1] != hs[1][1], (item, hs)
    assert set(whole) | set(halves) == want
    if counts == [512] * 4:
        assert len(halves) == len(want) and not whole
    last_round = {}
    for b, rnd, g, m, nn, half in visits.tolist():
        last_round[b] = max(last_round.get(b, -1), rnd)
    for b, rnd, g, m, nn, half in visits.tolist():                   # a split item is the last thing its block does
        assert half == -1 or rnd == last_round[b]
    visits = visits[:, :5]
    per_x = -(-len(want) // 8)
    flat = sorted(want)                                              # the list order is group-major
    first_of_group = {}
    for (g, m, nn) in flat:
        first_of_group.setdefault(g, len(first_of_group))
    by_round = {}
    for b, rnd, g, m, nn in visits.tolist():
        by_round.setdefault((b % 8, rnd), []).append((g, m, nn))
    for (xcd, rnd), items in by_round.items():
        assert len(items) <= (grid + 7 - xcd) // 8
        if len({g for g, _, _ in items}) == 1 and len(items) >= 16:  # a round inside one group: a patch, not a line
            ms, ns = {m for _, m, _ in items}, {nn for _, _, nn in items}
            assert len(ms) + len(ns) <= len(items) // 2 + 9, (xcd, rnd, len(ms), len(ns), len(items))


def test_in_place_block_scaling_keeps_fp32_accuracy():
    """The K = 64 kernel's arithmetic in a float32 model: accumulators kept in units of the current 128-K block's
    scale (acc *= s[kb-1] / s[kb], then the block's products are added unscaled; out = acc * s[last]) against the
    promotion form (acc += product * s[kb]) and the float64 sum, with a token block that was all zeros (its scale is
    the quantiser's floor 1e-12 / 448, fourteen orders of magnitude below its neighbours): both stay within a few
    fp32 ulps of the exact sum, also on that row, and nothing leaves the fp32 range."""
    rng = np.random.default_rng(0)
    kb_n, m, n = 56, 64, 64
    f32 = np.float32
    prod = rng.standard_normal((kb_n, m, n)) * 300.0
    xs = (np.abs(rng.standard_normal((kb_n, m))) * 0.01 + 1e-4).astype(f32)
    xs[3, 5] = f32(1e-12) / f32(448)
    prod[3, 5, :] = 0.0
    ws = (np.abs(rng.standard_normal(kb_n)) * 1e-4 + 1e-5).astype(f32)
    exact = sum(prod[k] * xs[k][:, None].astype(np.float64) * float(ws[k]) for k in range(kb_n))
    promoted = np.zeros((m, n), f32)
    in_place = np.zeros((m, n), f32)
    prev, peak = None, 0.0
    for k in range(kb_n):
        c = (xs[k] * ws[k]).astype(f32)
        promoted = (prod[k].astype(f32) * c[:, None] + promoted).astype(f32)
        if prev is not None:
            in_place = (in_place * (prev * (f32(1) / c)).astype(f32)[:, None]).astype(f32)
        in_place = (in_place + prod[k].astype(f32)).astype(f32)
        peak = max(peak, float(np.abs(in_place).max()))
        prev = c
    out = (in_place * prev[:, None]).astype(f32)
    err = lambda a: np.linalg.norm(a - exact) / np.linalg.norm(exact)
    assert err(promoted) < 1e-6 and err(out) < 1e-6
    assert np.abs(out[5] - exact[5]).max() <= 4e-6 * np.abs(exact[5]).max()
    assert np.isfinite(out).all() and peak < 1e30


def test_narrow_bf16_gemm_tile_loads_and_reads(hc):
    """The 128-token x 64-output block tile of the bf16 GEMM: the 24 issues of a K step fill the stage's 192 rows
    exactly once, and lane (r, q) of a wave reads, for output tile tn and its token tile, K elements 16 q .. 16 q + 15
    (two 16-byte pieces) of output row 16 tn + r and of token 16 wt + r -- the operand layout of the 16x16x32 bf16
    matrix instruction as the wide kernel feeds it."""
    rng = np.random.default_rng(11)
    experts = rng.integers(0, 1 << 16, size=(64, 64), dtype=np.uint16)
    tokens = rng.integers(0, 1 << 16, size=(128, 64), dtype=np.uint16)
    got_e = np.zeros((4, 64, 2, 8), dtype=np.uint16)
    got_t = np.zeros((8, 64, 2, 8), dtype=np.uint16)
    hc.hc_rg64_step.restype = C.c_int
    hc.hc_rg64_step.argtypes = [C.c_void_p] * 4
    assert hc.hc_rg64_step(experts.ctypes.data, tokens.ctypes.data, got_e.ctypes.data, got_t.ctypes.data) == 0
    for lane in range(64):
        r, q = lane % 16, lane // 16
        for jj in range(2):
            k0 = 8 * (2 * q + jj)
            for tn in range(4):
                assert np.array_equal(got_e[tn, lane, jj], experts[16 * tn + r, k0: k0 + 8]), (tn, lane, jj)
            for wt in range(8):
                assert np.array_equal(got_t[wt, lane, jj], tokens[16 * wt + r, k0: k0 + 8]), (wt, lane, jj)


def item_walk(hc, counts, lo, hi, chunk_rows, tall_min, tall_rows, ntiles):
    arr = (C.c_int32 * len(counts))(*counts)
    cap = 1 << 16
    out = (C.c_int32 * (5 * cap))()
    hc.hc_item_walk.restype = C.c_int64
    hc.hc_item_walk.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                C.c_int64]
    n = hc.hc_item_walk(arr, len(counts), lo, hi, chunk_rows, tall_min, tall_rows, ntiles, out, cap)
    assert n >= 0
    return [tuple(out[5 * b: 5 * b + 5]) for b in range(n)]


def check_item_walk(hc, counts, lo, hi, chunk_rows, tall_min, tall_rows, ntiles, row_bound=None):
    """Every (group, n-tile, chunk) of the served groups is some virtual block's item exactly once; the chunks
    partition the group's rows; all chunks of one weight tile sit on one XCD (block % 8); the host's bound on the
    virtual blocks covers the list."""
    items = item_walk(hc, counts, lo, hi, chunk_rows, tall_min, tall_rows, ntiles)
    seen = {}
    for b, (grp, ntile, chunk, rows, cnt) in enumerate(items):
        if grp < 0:
            assert ntile >= ntiles
            continue
        assert cnt == counts[grp] and lo < cnt <= hi
        want_rows = tall_rows if tall_min > 0 and cnt > tall_min else chunk_rows
        assert rows == want_rows
        assert 0 <= ntile < ntiles and 0 <= chunk * rows < cnt
        assert (grp, ntile, chunk) not in seen
        seen[(grp, ntile, chunk)] = b
    for g, c in enumerate(counts):
        if not lo < c <= hi:
            continue
        rows = tall_rows if tall_min > 0 and c > tall_min else chunk_rows
        chunks = -(-c // rows)
        for t in range(ntiles):
            blocks = [seen[(g, t, ch)] for ch in range(chunks)]          # KeyError = an item nobody works on
            assert len({b % 8 for b in blocks}) == 1, "the chunks of one weight tile are spread over several XCDs"
    served = [c for c in counts if lo < c <= hi]
    assert len(seen) == sum(-(-c // (tall_rows if tall_min > 0 and c > tall_min else chunk_rows)) for c in served) * ntiles
    hc.hc_item_grid.restype = C.c_uint
    hc.hc_item_grid.argtypes = [C.c_int, C.c_int, C.c_int64, C.c_int, C.c_int]
    bound = sum(counts) if row_bound is None else row_bound
    assert hc.hc_item_grid(ntiles, len(counts), bound, hi, chunk_rows) >= len(items)
    return len(seen)


def test_streaming_items_with_and_without_tall_groups(hc):
    """Work items of the weight-streaming kernels (32-row chunks for the fused stage 1), with the opt-in tall items
    (groups above a row count in 64-row chunks): configuration 1's draw, the shapes of the kernel tests, random
    launches.  Tall items only lower the item count, so the host's grid bound holds unchanged."""
    n32 = check_item_walk(hc, CONFIG1_DRAW, 0, 256, 32, 0, 0, 16)
    n_tall32 = check_item_walk(hc, CONFIG1_DRAW, 0, 256, 32, 32, 64, 16)
    n_tall64 = check_item_walk(hc, CONFIG1_DRAW, 0, 256, 32, 64, 64, 16)
    # passes over a weight tile, by hand: 15 groups of at most 32 rows, then 41 / 65 / 39 / 35 / 256 rows
    assert (n32, n_tall32, n_tall64) == ((15 + 2 + 3 + 2 + 2 + 8) * 16, (15 + 1 + 2 + 1 + 1 + 4) * 16, (15 + 2 + 2 + 2 + 2 + 4) * 16)
    rng = random.Random(5)
    for _ in range(200):
        groups = rng.randint(1, 70)
        counts = [rng.choice([0, 0, 1, 5, 16, 31, 32, 33, 63, 64, 65, 100, 128, 129, 200, 256, 300]) for _ in range(groups)]
        ntiles = rng.choice([1, 3, 8, 9, 16, 56])
        lo, hi = rng.choice([(0, 256), (0, 64), (64, 256), (0, 1 << 30)])
        tall_min = rng.choice([0, 32, 40, 64, 128])
        check_item_walk(hc, counts, lo, hi, rng.choice([16, 32, 64]) if tall_min == 0 else 32, tall_min, 64, ntiles,
                        row_bound=sum(counts))
