"""The add + RMSNorm + FP8-cast oracle pinned without a GPU: the fma emulation against exact rational
arithmetic (adversarial ties included), one row against a scalar walk of the reference kernel's loops, and
the contract the reference's own tests state (tests/test_glm52_norm_quant_fuse.py:283-355)."""
from fractions import Fraction

import numpy as np
import torch

from oracle import norm_quant as onq
from oracle.quant import act_quant, bf16_round
from tests.util import rand_bf16

F32 = np.float32


def _round_f32(fr: Fraction) -> np.float32:
    """Correct rounding of a rational to float32 (ties to even) by brute force on its neighbours."""
    approx = F32(float(fr))
    cands = {approx, np.nextafter(approx, F32(np.inf)), np.nextafter(approx, F32(-np.inf))}
    best = None
    for c in cands:
        d = abs(Fraction(float(c)) - fr)
        even = (int(np.array(c, dtype=F32).view(np.uint32)) & 1) == 0
        key = (d, 0 if even else 1)
        if best is None or key < best[0]:
            best = (key, c)
    return best[1]


def test_fma_emulation_against_rational_arithmetic():
    rng = np.random.default_rng(0)
    a = rng.standard_normal(4000).astype(F32) * F32(3.0)
    c = (rng.standard_normal(4000) ** 2).astype(F32) * F32(50.0)
    # adversarial: a*a + c exactly halfway between two float32, and a hair to either side
    base = F32(1.0) + F32(2.0 ** -23) * F32(5)
    half = F32(2.0 ** -24)
    a_adv = np.array([F32(2.0 ** -12)] * 3 + [F32(2.0 ** -13)] * 2, dtype=F32)     # a*a = 2^-24 / 2^-26
    c_adv = np.array([base, np.nextafter(base, F32(2)), F32(4) + F32(2.0 ** -21), base, F32(2.0)], dtype=F32)
    a = np.concatenate([a, a_adv])
    c = np.concatenate([c, c_adv])
    got = onq.fma_f32(a, a, c)
    for i in range(len(a)):
        exact = Fraction(float(a[i])) * Fraction(float(a[i])) + Fraction(float(c[i]))
        assert got[i] == _round_f32(exact), (i, a[i], c[i])
    assert half > 0
    # a tie that only the exact error term resolves: a*b = 2^-4 -+ 2^-50 is lost when added to c in float64,
    # which lands on the float32 midpoint above c = 2^20 + 5*2^-3
    c1 = F32(2.0 ** 20) + F32(5 * 2.0 ** -3)
    one_up, one_dn = F32(1) + F32(2.0 ** -23), F32(1) - F32(2.0 ** -24)
    cases = [(one_up, F32(2.0 ** -4) * (F32(1) - F32(2.0 ** -23)), c1),      # exact sum just below the tie
             (one_up, F32(2.0 ** -4) * one_up, c1),                          # just above
             (one_dn, F32(2.0 ** -4) * one_dn, c1)]
    for x, y2, z in cases:
        exact = Fraction(float(x)) * Fraction(float(y2)) + Fraction(float(z))
        assert onq.fma_f32(np.array([x]), np.array([y2]), np.array([z]))[0] == _round_f32(exact)
    below = onq.fma_f32(np.array([cases[0][0]]), np.array([cases[0][1]]), np.array([c1]))[0]
    assert below == c1                                                       # plain float64 + RNE would say c1 + 2^-3


def _row_walk(res, hid, w, eps):
    """add_rmsnorm_fp8_quant.cu:296-327 for one row, one scalar at a time."""
    h = len(res)
    threads = h // 8
    sums = [F32(res[i]) + F32(hid[i]) for i in range(h)]
    sq = []
    for t in range(threads):
        acc = F32(0)
        for i in range(8):
            s = sums[8 * t + i]
            acc = _round_f32(Fraction(float(s)) * Fraction(float(s)) + Fraction(float(acc)))
        sq.append(acc)

    def tree(v):
        v = list(v) + [F32(0)] * (32 - len(v))
        off = 16
        while off:
            for lane in range(off):
                v[lane] = F32(v[lane] + v[lane + off])
            off //= 2
        return v[0]
    warp_sums = [tree(sq[i:i + 32]) for i in range(0, threads, 32)]
    total = tree(warp_sums)
    inv = F32(1.0 / np.sqrt(np.float64(F32(F32(total / F32(h)) + F32(eps)))))
    rounded = bf16_round(np.array(sums, dtype=F32))
    normed = bf16_round((rounded * inv).astype(F32) * w)
    return normed, rounded


def test_one_row_against_a_scalar_walk_of_the_kernel():
    g = torch.Generator().manual_seed(3)
    h = 1152                                   # 144 threads: four full warps and a half one
    res, hid = rand_bf16(g, 2, h, scale=0.9), rand_bf16(g, 2, h, scale=0.4)
    w = (torch.randn(h, generator=g) * 0.3 + 1.0).to(torch.bfloat16)
    normed, new_res = onq.add_rmsnorm(res, hid, w, 1e-5)
    for r in range(2):
        n_ref, r_ref = _row_walk(res[r].float().numpy(), hid[r].float().numpy(), w.float().numpy(), 1e-5)
        assert np.array_equal(new_res[r], r_ref) and np.array_equal(normed[r], n_ref)


def test_norm_matches_the_textbook_formula_closely():
    g = torch.Generator().manual_seed(4)
    res, hid = rand_bf16(g, 8, 6144), rand_bf16(g, 8, 6144)
    w = (torch.randn(6144, generator=g) * 0.3 + 1.0).to(torch.bfloat16)
    normed, new_res = onq.add_rmsnorm(res, hid, w, 1e-5)
    s = res.double().numpy() + hid.double().numpy()
    ref = bf16_round(s.astype(F32)).astype(np.float64)
    ref = ref / np.sqrt((s ** 2).mean(axis=1, keepdims=True) + 1e-5) * w.double().numpy()
    np.testing.assert_allclose(normed, ref, rtol=2 ** -7, atol=1e-6)      # one bf16 rounding


def test_quantising_from_registers_equals_quantising_the_stored_bf16_and_gates():
    g = torch.Generator().manual_seed(5)
    res, hid = rand_bf16(g, 16, 1024, scale=0.9), rand_bf16(g, 16, 1024, scale=0.4)
    w = (torch.randn(1024, generator=g) * 0.3 + 1.0).to(torch.bfloat16)
    mask = torch.ones(16, dtype=torch.bfloat16)
    mask[3] = 0
    hid_nan = hid.clone()
    hid_nan[3] = float("nan")
    normed, new_res, y, s = onq.add_rmsnorm_fp8_quant(res, hid_nan, w, 1e-5, quant_num_valid_tokens=10,
                                                       row_valid_mask=mask)
    assert np.isfinite(normed).all() and np.array_equal(new_res[3], res[3].float().numpy())
    ya, sa = act_quant(normed, form="A")
    yc, sc = act_quant(normed, form="C")
    assert np.array_equal(y[:10], ya[:10]) and np.array_equal(s[:10], sa[:10])
    assert np.array_equal(ya, yc) and np.array_equal(sa, sc)             # amax >= 2^-16 everywhere
    assert np.all(y[10:] == 0) and np.all(s[10:] == F32(1e-12))
    # the norm gate leaves the residual of skipped rows alone
    _, res2, _, _ = onq.add_rmsnorm_fp8_quant(res, hid, w, 1e-5, norm_num_valid_tokens=4, quant_num_valid_tokens=4)
    assert np.array_equal(res2[4:], res[4:].float().numpy())
