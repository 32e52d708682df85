"""Pins for the oracle's permute, combine and MXFP4 codec (CPU only)."""
import numpy as np
import torch

from oracle import combine as oc
from oracle import mxfp4 as mx
from oracle import permute as op_
from oracle.quant import bf16_round


def _ids(rng, n, k, e):
    return np.stack([rng.permutation(e)[:k] for _ in range(n)]).astype(np.int32)


def test_vectorised_dispatch_equals_the_sequential_loop():
    rng = np.random.default_rng(0)
    for n, k, et, es, el in [(1, 4, 16, 0, 16), (50, 4, 64, 16, 8), (200, 8, 256, 32, 32), (33, 2, 8, 0, 8)]:
        ids = _ids(rng, n, k, et)
        ids.reshape(-1)[:3] = [-1, es - 1, es + el]
        c0, off0, pos0 = op_.dispatch_sequential(ids, es, el)
        c1, cu1, pos1 = op_.dispatch_ragged(ids, es, el, 1)
        assert np.array_equal(c0, c1) and np.array_equal(off0, cu1) and np.array_equal(pos0, pos1)
        for align in (64, 128):
            c2, cu2, pos2 = op_.dispatch_ragged(ids, es, el, align)
            assert np.array_equal(c2, c0) and np.all(cu2 % align == 0)
            assert np.array_equal(np.diff(cu2), (c0 + align - 1) // align * align)
            live = pos0 >= 0
            loc = ids.reshape(-1)[live] - es
            assert np.array_equal(pos2[live] - cu2[loc], pos0[live] - off0[loc])
            assert cu2[-1] <= op_.ragged_capacity_rows(n, k, el, align)
        mtp = max(int(c0.max()), 1)
        c3, pos3 = op_.dispatch_masked(ids, es, el, mtp)
        live = pos0 >= 0
        loc = ids.reshape(-1)[live] - es
        assert np.array_equal(pos3[live], loc * mtp + (pos0[live] - off0[loc])) and np.all(pos3[~live] == -1)


def test_masked_dispatch_drops_overflow():
    ids = np.zeros((10, 1), dtype=np.int32)
    c, pos = op_.dispatch_masked(ids, 0, 2, 4)
    assert c.tolist() == [4, 0] and pos.tolist() == [0, 1, 2, 3] + [-1] * 6


def test_masked_arrivals_equal_the_sequential_running_counter():
    """Arrivals before clipping = the final value of the per-expert running counter of the sequential loop
    (every local pair counts, kept or dropped); counts = the same clipped; a dropped pair has pos -1 and the
    kept pairs of an expert are exactly its first max_tokens arrivals in (token, k) order."""
    rng = np.random.default_rng(7)
    for n, k, et, es, el, mtp in [(10, 2, 2, 0, 2, 4), (40, 4, 16, 4, 8, 3), (64, 8, 32, 0, 32, 1), (9, 3, 8, 2, 4, 100)]:
        ids = rng.integers(es - 2, es + el + 2, size=(n, k)).astype(np.int32)       # repeats and non-local ids
        counts, pos, arrivals = op_.dispatch_masked_arrivals(ids, es, el, mtp)
        ctr = np.zeros(el, dtype=np.int64)
        for i, eid in enumerate(ids.reshape(-1)):
            le = int(eid) - es
            if 0 <= le < el:
                want = le * mtp + ctr[le] if ctr[le] < mtp else -1
                assert pos[i] == want
                ctr[le] += 1
            else:
                assert pos[i] == -1
        assert np.array_equal(arrivals, ctr) and np.array_equal(counts, np.minimum(ctr, mtp))
    ids = np.zeros((10, 2), dtype=np.int32)
    ids[:, 1] = 1
    counts, pos, arrivals = op_.dispatch_masked_arrivals(ids, 0, 2, 4)
    assert counts.tolist() == [4, 4] and arrivals.tolist() == [10, 10]


def test_gather_rows_places_tokens():
    rng = np.random.default_rng(1)
    ids = _ids(rng, 20, 4, 16)
    x = rng.standard_normal((20, 8)).astype(np.float32)
    c, cu, pos = op_.dispatch_ragged(ids, 0, 16, 1)
    act = op_.gather_rows(x, pos, 4, int(cu[-1]))
    for i, p in enumerate(pos):
        assert np.array_equal(act[p], x[i // 4])


def test_combine_matches_the_per_token_loop_and_handles_no_local_routes():
    rng = np.random.default_rng(2)
    n, k, h = 30, 8, 64
    y = bf16_round(rng.standard_normal((n * k, h)).astype(np.float32))
    pos = rng.permutation(n * k).astype(np.int32)
    pos[rng.random(n * k) < 0.4] = -1
    pos.reshape(n, k)[3] = -1
    w = rng.random((n, k)).astype(np.float32)
    a = oc.reduce_weighted_scatter(y, pos, w, n, k)
    assert np.array_equal(a, oc.reduce_loop(y, pos, w, n, k)) and np.all(a[3] == 0)
    f = oc.reduce_weighted_scatter_fp32(y, pos, w, n, k)
    assert np.array_equal(bf16_round(f), a)
    sh = bf16_round(rng.standard_normal((n, h)).astype(np.float32))
    b = oc.reduce_weighted_scatter(y, pos, w, n, k, shared=sh, shared_mode="bf16_add")
    assert np.array_equal(b, bf16_round(a + sh))
    c = oc.reduce_weighted_scatter(y, pos, w, n, k, shared=sh, shared_mode="fp32_add")
    assert np.array_equal(c, bf16_round(f + sh))


def test_ordered_bf16_combine_is_slot_order_independent():
    rng = np.random.default_rng(3)
    n, k, h = 12, 4, 16
    y = bf16_round(rng.standard_normal((n * k, h)).astype(np.float32))
    pos = rng.permutation(n * k).astype(np.int32)
    ids = _ids(rng, n, k, 32)
    w = rng.random((n, k)).astype(np.float32)
    a = oc.reduce_weighted_scatter_bf16_ordered(y, pos, ids, w, n, k)
    perm = rng.permutation(k)
    b = oc.reduce_weighted_scatter_bf16_ordered(y, pos.reshape(n, k)[:, perm], ids[:, perm], w[:, perm], n, k)
    assert np.array_equal(a, b)
    # literal definition: acc = bf16(acc + bf16(x * bf16(w))) in ascending expert id
    t = 5
    order = np.argsort(ids[t], kind="stable")
    acc = np.zeros(h, dtype=np.float32)
    for j in order:
        acc = bf16_round(acc + bf16_round(y[pos.reshape(n, k)[t, j]] * bf16_round(w[t, j:j + 1])))
    assert np.array_equal(a[t], acc)


# frozen vector of the reference: batchgen/moe/mxfp4_oracle_vector.py:62-70 (16 packed bytes + scale 0x79
# -> 32 bf16 bit patterns; real checkpoint data, oracle compressed-tensors 0.17.1)
VEC_PACKED = bytes([0xAB, 0x4C, 0x18, 0x65, 0x2C, 0x91, 0x04, 0x39, 0x48, 0x94, 0x58, 0x33, 0x94, 0xB5, 0x5B, 0x30])
VEC_SCALE = 0x79
VEC_BF16 = (0xBCC0, 0xBC80, 0xBD00, 0x3D00, 0x8000, 0x3C00, 0x3D40, 0x3D80, 0xBD00, 0x3C80, 0x3C00, 0xBC00, 0x3D00,
            0x0000, 0xBC00, 0x3CC0, 0x8000, 0x3D00, 0x3D00, 0xBC00, 0x8000, 0x3D40, 0x3CC0, 0x3CC0, 0x3D00, 0xBC00,
            0x3D40, 0xBCC0, 0xBCC0, 0x3D40, 0x0000, 0x3CC0)


def test_mxfp4_dequant_frozen_vector():
    out = mx.dequant(np.frombuffer(VEC_PACKED, dtype=np.uint8)[None, :], np.array([[VEC_SCALE]], dtype=np.uint8))
    bits = (out.view(np.uint32) >> 16).astype(np.uint16).reshape(-1)
    assert np.array_equal(bits, np.array(VEC_BF16, dtype=np.uint16))
    assert np.all((out.view(np.uint32) & 0xFFFF) == 0)      # exactly representable in bf16


def test_mxfp4_dequant_unit_cases():
    # the reference's tests/unit/test_mxfp4_dequant_reference.py:36-148
    d = lambda p, s: mx.dequant(np.array(p, dtype=np.uint8), np.array(s, dtype=np.uint8))
    assert d([0x12, 0x34] + [0] * 14, [127])[:4].tolist() == [1.0, 0.5, 2.0, 1.5]
    assert np.all(d([0x22] * 16, [128]) == 2.0) and np.all(d([0x44] * 16, [126]) == 1.0)
    assert d([0x9A] * 16, [127]).tolist() == [-1.0, -0.5] * 16
    two = d([0x22] * 32, [128, 126])
    assert np.all(two[:32] == 2.0) and np.all(two[32:] == 0.5)
    m = mx.dequant(np.array([[0x22] * 16, [0x44] * 16], dtype=np.uint8), np.array([[127], [128]], dtype=np.uint8))
    assert np.all(m[0] == 1.0) and np.all(m[1] == 4.0)
    assert mx.LUT16.tolist() == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def test_mxfp4_quantize_closed_form():
    # representable values round-trip exactly; the shared scale is 2^(floor(log2 amax) - 2)
    vals = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], dtype=np.float32)
    w = np.concatenate([vals, -vals, vals, -vals])[None, :] * np.float32(2.0 ** -5)
    p, s = mx.quantize(w)
    assert s[0, 0] == 127 - 5 and np.array_equal(mx.dequant(p, s), w)
    rng = np.random.default_rng(0)
    w = (0.02 * rng.standard_normal((8, 128))).astype(np.float32)
    p, s = mx.quantize(w)
    amax = np.abs(w.reshape(8, 4, 32)).max(-1)
    assert np.array_equal(s.astype(np.int32) - 127, np.floor(np.log2(amax)).astype(np.int32) - 2)
    d = mx.dequant(p, s)
    step = np.repeat(np.ldexp(1.0, s.astype(np.int32) - 127), 32, axis=1)
    # amax/scale lies in [4, 8): values above 6 saturate, so the error is below 2 scale units
    assert np.all(np.abs(d - w) <= 2.0 * step)
    p2, s2 = mx.quantize(d)
    assert np.array_equal(p, p2) and np.array_equal(s, s2)  # idempotent
    # ties go to the even code: 0.25 -> 0, 0.75 -> 1.0, 2.5 -> 2.0, 5.0 -> 4.0 (scale 1: amax = 6)
    t = np.array([[0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] + [0.0] * 24], dtype=np.float32)
    pt, st = mx.quantize(t)
    assert st[0, 0] == 127 and mx.dequant(pt, st)[0, :8].tolist() == [0.0, 1.0, 1.0, 2.0, 2.0, 4.0, 4.0, 6.0]


def test_torch_mxfp4_quantiser_of_the_workloads_equals_the_oracle():
    from batchgen_amd.workloads import quantize_mxfp4
    g = torch.Generator().manual_seed(5)
    w = torch.randn(64, 256, generator=g) * 0.02
    w[0, :32] = 0
    w[1, 0] = 5.0 * 2.0 ** -7
    p, s = quantize_mxfp4(w)
    po, so = mx.quantize(w.numpy())
    assert np.array_equal(p.numpy(), po) and np.array_equal(s.numpy(), so)
