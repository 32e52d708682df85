"""The router-GEMM oracle pinned without a GPU: the exact product against exact rational arithmetic,
the reference-order restatement against a scalar walk of the reference kernel's loops, and the structural
properties the reference's own tests check (tests/test_glm5_router_gemm_cuda.py:63-113)."""
from fractions import Fraction

import numpy as np
import torch

from oracle import router_gemm as org
from tests.util import rand_bf16


def _ops(seed, n, h, e, scale=0.1):
    g = torch.Generator().manual_seed(seed)
    return rand_bf16(g, n, h, scale=scale), rand_bf16(g, e, h, scale=scale)


def test_bf16_decode_matches_torch():
    x, _ = _ops(1, 5, 64, 3)
    assert np.array_equal(org.bf16_to_f32(x), x.float().numpy())


def test_exact_product_against_rational_arithmetic():
    x, w = _ops(2, 3, 200, 4)
    out = org.router_gemm_exact(x, w)
    xf, wf = x.float().numpy(), w.float().numpy()
    for i in range(3):
        for j in range(4):
            exact = sum(Fraction(float(a)) * Fraction(float(b)) for a, b in zip(xf[i], wf[j]))
            assert out[i, j] == np.float32(float(exact))       # float(Fraction) rounds correctly to double


def _kernel_walk(xrow, wrow, threads=256, warp=32):
    """glm5_router_gemm.cu:82-104 for one output, one scalar at a time."""
    f32 = np.float32
    acc = [f32(0)] * threads
    for tid in range(threads):
        for k in range(tid, len(xrow), threads):
            acc[tid] = f32(np.float64(xrow[k]) * np.float64(wrow[k]) + np.float64(acc[tid]))   # fmaf: one rounding
    def tree(v):                                   # __shfl_down_sync tree as seen from lane 0
        v = list(v)
        off = warp // 2
        while off:
            for lane in range(off):
                v[lane] = f32(v[lane] + v[lane + off])
            off //= 2
        return v[0]
    sums = [tree(acc[wi * warp:(wi + 1) * warp]) for wi in range(threads // warp)]
    return tree(sums + [f32(0)] * (warp - len(sums)))


def test_reference_order_against_a_scalar_walk_of_the_kernel():
    x, w = _ops(3, 2, 600, 3, scale=1.0)           # 600: the third sweep touches 88 of the 256 threads
    out = org.router_gemm_ref_order(x, w)
    xf, wf = x.float().numpy(), w.float().numpy()
    for i in range(2):
        for j in range(3):
            assert out[i, j] == _kernel_walk(xf[i], wf[j])


def test_orders_agree_within_fp32_summation_error():
    x, w = _ops(4, 16, 7168, 32)
    exact = org.router_gemm_exact(x, w)
    scale = org.abs_product_sum(x, w)
    for other in (org.router_gemm_ref_order(x, w), org.router_gemm_segmented(x, w)):
        assert np.all(np.abs(other.astype(np.float64) - exact) <= 1e-6 * scale)
    # a dropped term would not pass: the typical single term is 1/h of the scale
    assert 1.0 / 7168 > 50 * 1e-6


def test_padding_rows_are_zero_and_valid_rows_do_not_depend_on_the_bucket():
    world, bucket = 3, 7
    x, w = _ops(5, world * bucket, 96, 48)
    counts = np.array([7, 3, 5], dtype=np.int64)
    pad = org.padding_rows(world * bucket, counts, bucket, world)
    assert pad.sum() == world * bucket - counts.sum()
    poisoned = x.clone()
    poisoned[torch.from_numpy(pad)] = float("nan")
    for fn in (org.router_gemm_exact, org.router_gemm_ref_order, org.router_gemm_segmented):
        padded = fn(poisoned, w, counts, bucket, world)
        assert np.all(padded[pad] == 0)
        compact = fn(x[torch.from_numpy(~pad)].contiguous(), w)
        assert np.array_equal(padded[~pad], compact)
    # a rank index past world_size is padding too
    assert org.padding_rows(10, np.array([5], dtype=np.int64), 5, 1).tolist() == [False] * 5 + [True] * 5
