"""HIP router GEMM (bf16 x bf16 -> fp32 logits) against the CPU oracle, and the fused GEMM + top-k against the
two-op sequence.  The cases follow the reference's tests/test_glm5_router_gemm_cuda.py.

Floating-point bar: |logit - exact| <= 1e-6 * sum_k |x_k w_k|, where `exact` is the float64 product rounded
to fp32 (the fp32 summation error of a 7168-term MFMA chain stays an order of magnitude below that, and one
dropped term of a 7168-term row is two orders above it).  The reference holds its kernel to
1e-5 + 1.6e-2*|ref| against a bf16 matmul.  Everything structural is bit-exact: padding rows, independence
of a row from the batch it sits in, independence from the launch shape, fused == unfused.
"""
import numpy as np
import pytest
import torch

from oracle import router as orr
from oracle import router_gemm as org
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu
TOL = 1e-6


def routing():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_routing")


def _ops(seed, n, h, e, scale=0.1):
    g = torch.Generator().manual_seed(seed)
    return rand_bf16(g, n, h, scale=scale), rand_bf16(g, e, h, scale=scale)


def _check_close(actual, x, w, counts=None, bucket=0, world=1):
    exact = org.router_gemm_exact(x, w, counts, bucket, world)
    scale = org.abs_product_sum(x, w)
    err = np.abs(actual.astype(np.float64) - exact)
    worst = float((err / np.maximum(scale, 1e-30)).max()) if err.size else 0.0
    say("   max |err| / sum|xw| =", worst)
    assert np.all(err <= TOL * scale + 1e-37)


@pytest.mark.parametrize("m", [1, 3, 7, 8, 11, 16, 32, 61, 64, 128, 256, 512, 1024])
def test_shape_sweep_matches_oracle(dev, m):
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    say("router_gemm sweep", m)
    x, w = _ops(1234 + m, m, 64, 32)
    out = glm5_router_gemm_cuda(x.to(dev), w.to(dev))
    assert out.dtype == torch.float32 and tuple(out.shape) == (m, 32)
    _check_close(out.cpu().numpy(), x, w)


@pytest.mark.parametrize("n,h,e", [(4, 6144, 256), (256, 7168, 256), (37, 2880, 128), (5, 4096, 896),
                                   (19, 1000, 20), (70, 72, 5), (300, 520, 130)])
def test_model_shapes_match_both_oracles(dev, n, h, e):
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    say("router_gemm", n, h, e)
    x, w = _ops(n + h + e, n, h, e)
    out = glm5_router_gemm_cuda(x.to(dev), w.to(dev)).cpu().numpy()
    _check_close(out, x, w)
    if n * e <= 4096:
        # the reference kernel's own summation order is another fp32 evaluation of the same sums
        ref = org.router_gemm_ref_order(x, w)
        assert np.all(np.abs(out.astype(np.float64) - ref) <= 2 * TOL * org.abs_product_sum(x, w))
    seg = org.router_gemm_segmented(x, w)
    assert np.all(np.abs(out.astype(np.float64) - seg) <= 0.5 * TOL * org.abs_product_sum(x, w))


def test_rank_counts_zero_invalid_rows(dev):
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    world, bucket = 4, 8
    x, w = _ops(99, world * bucket, 128, 64)
    counts = torch.tensor([3, 8, 0, 5], dtype=torch.int64)
    pad = torch.from_numpy(org.padding_rows(world * bucket, counts.numpy(), bucket, world))
    poisoned = x.clone()
    poisoned[pad] = float("nan")
    out = glm5_router_gemm_cuda(poisoned.to(dev), w.to(dev), rank_token_counts=counts.to(dev),
                                bucket_size=bucket, world_size=world).cpu()
    assert torch.all(out[pad] == 0)
    _check_close(out.numpy(), poisoned, w, counts.numpy(), bucket, world)


def test_valid_rows_are_bucket_stable(dev):
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    world, bucket = 3, 7
    x, w = _ops(100, world * bucket, 96, 48)
    counts = torch.tensor([7, 3, 5], dtype=torch.int64)
    valid = torch.from_numpy(~org.padding_rows(world * bucket, counts.numpy(), bucket, world))
    padded = glm5_router_gemm_cuda(x.to(dev), w.to(dev), rank_token_counts=counts.to(dev), bucket_size=bucket,
                                   world_size=world).cpu()
    compact = glm5_router_gemm_cuda(x[valid].contiguous().to(dev), w.to(dev)).cpu()
    assert torch.equal(padded[valid], compact)


@pytest.mark.parametrize("world,bucket", [(16, 1), (16, 8), (16, 32)])
def test_production_graph_envelope_rank_counts(dev, world, bucket):
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    x, w = _ops(20260511 + bucket, world * bucket, 6144, 256)
    counts = (torch.arange(world, dtype=torch.int64) * 7) % (bucket + 1)
    counts[0] = bucket
    counts[1] = 0
    pad = torch.from_numpy(org.padding_rows(world * bucket, counts.numpy(), bucket, world))
    poisoned = x.clone()
    poisoned[pad] = float("nan")
    out = glm5_router_gemm_cuda(poisoned.to(dev), w.to(dev), rank_token_counts=counts.to(dev),
                                bucket_size=bucket, world_size=world).cpu()
    assert torch.all(out[pad] == 0)
    _check_close(out.numpy(), poisoned, w, counts.numpy(), bucket, world)
    compact = glm5_router_gemm_cuda(x[~pad].contiguous().to(dev), w.to(dev)).cpu()
    assert torch.equal(out[~pad], compact)


@pytest.mark.parametrize("n,h,e", [(50, 7168, 256), (200, 1096, 72), (1, 512, 256), (130, 64, 16), (300, 1088, 200)])
def test_every_launch_shape_gives_the_same_bits(dev, n, h, e):
    """Whole-K and split-K, 1/2/4 token tiles and 2/4 expert tiles per wave: one summation order, so one
    result."""
    from batchgen_amd._lib import check, lib
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    x, w = _ops(7 * n + h, n, h, e)
    xd, wd = x.to(dev), w.to(dev)
    outs = {}
    try:
        for tm in (1, 2, 4):
            for split in (0, 1, 2, 3, 4):
                check(lib().bgmoe_set_router_gemm_plan(tm, split))
                outs[(tm, split)] = glm5_router_gemm_cuda(xd, wd).clone()
    finally:
        check(lib().bgmoe_set_router_gemm_plan(-1, -1))
    base = glm5_router_gemm_cuda(xd, wd)
    for key, o in outs.items():
        assert torch.equal(o, base), f"launch shape {key} changes the logits"
    # ... and a row does not care which rows surround it
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(3))
    assert torch.equal(glm5_router_gemm_cuda(xd[perm.to(dev)].contiguous(), wd), base[perm.to(dev)])


GATES = [  # n, h, e, n_group, topk_group, k, rsf     (n_group 0 = ungrouped)
    (256, 7168, 256, 8, 4, 8, 2.5),
    (33, 1024, 64, 4, 2, 2, 1.5),
    (512, 2880, 128, 0, 0, 4, 1.0),
    (40, 7168, 896, 0, 0, 16, 1.0),
    (7, 520, 256, 1, 1, 8, 2.5),
    (64, 512, 64, 0, 0, 4, 1.0),        # one K segment: the whole-K shape feeds the gate a single plane
]


@pytest.mark.parametrize("n,h,e,ng,tg,k,rsf", GATES)
def test_fused_gemm_gate_equals_gemm_then_gate(dev, n, h, e, ng, tg, k, rsf):
    from batchgen_amd.kernels import load_extension
    from batchgen_amd.moe.routing import (gate_sigmoid_topk_cuda, glm5_router_gemm_cuda,
                                          router_gemm_gate_sigmoid_topk)
    say("router_gemm_gate", n, h, e, ng, tg, k)
    x, w = _ops(n + e + k, n, h, e)
    g = torch.Generator().manual_seed(5)
    bias = (0.1 * torch.randn(e, generator=g)).to(dev)
    xd, wd = x.to(dev), w.to(dev)
    logits = glm5_router_gemm_cuda(xd, wd)
    ids_f, w_f = router_gemm_gate_sigmoid_topk(xd, wd, bias, k, rsf, n_group=ng, topk_group=tg)
    if ng:
        mgn = load_extension("batchgen_kernels.common._C_mgn_ops")
        ids_u, w_u = mgn.moe_fused_gate_logits(logits, bias, ng, tg, e, k, rsf)
        ido, wo = orr.grouped_router(logits.cpu().numpy(), bias.cpu().numpy(), ng, tg, k, rsf)
    else:
        ids_u, w_u = gate_sigmoid_topk_cuda(logits, bias, k, rsf)
        ido, wo = orr.gate_sigmoid_topk(logits.cpu().numpy(), bias.cpu().numpy(), k, rsf)
    assert torch.equal(ids_f, ids_u) and torch.equal(w_f, w_u)
    # and the routes are the oracle's routes for these logits
    assert np.array_equal(ids_f.cpu().numpy(), ido)
    np.testing.assert_allclose(w_f.cpu().numpy(), wo, rtol=2e-7, atol=0)


def test_fused_gemm_gate_padding_rows(dev):
    from batchgen_amd.moe.routing import (gate_sigmoid_topk_cuda, glm5_router_gemm_cuda,
                                          router_gemm_gate_sigmoid_topk)
    world, bucket, h, e, k = 4, 8, 1024, 128, 4
    x, w = _ops(41, world * bucket, h, e)
    counts = torch.tensor([3, 8, 0, 5], dtype=torch.int64)
    pad = torch.from_numpy(org.padding_rows(world * bucket, counts.numpy(), bucket, world))
    x[pad] = float("nan")
    bias = torch.zeros(e, device=dev)
    xd, wd, cd = x.to(dev), w.to(dev), counts.to(dev)
    logits = glm5_router_gemm_cuda(xd, wd, rank_token_counts=cd, bucket_size=bucket, world_size=world)
    ids_u, w_u = gate_sigmoid_topk_cuda(logits, bias, k, 1.0, rank_token_counts=cd, rows_per_rank=bucket)
    ids_f, w_f = router_gemm_gate_sigmoid_topk(xd, wd, bias, k, 1.0, rank_token_counts=cd, rows_per_rank=bucket)
    assert torch.equal(ids_f, ids_u) and torch.equal(w_f, w_u)
    assert torch.all(ids_f[pad.to(dev)] == -1) and torch.all(w_f[pad.to(dev)] == 0)


def test_argument_errors(dev):
    from batchgen_amd._lib import check, lib, ptr, stream
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    x = torch.zeros((4, 64), dtype=torch.bfloat16, device=dev)
    w = torch.zeros((8, 64), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        glm5_router_gemm_cuda(x, torch.zeros((8, 32), dtype=torch.bfloat16, device=dev))       # hidden dim mismatch
    with pytest.raises(RuntimeError):
        glm5_router_gemm_cuda(x, w, router_logits=torch.zeros((4, 9), device=dev))             # output shape
    with pytest.raises(RuntimeError):
        glm5_router_gemm_cuda(x, w, rank_token_counts=torch.ones(2, dtype=torch.int64, device=dev),
                              bucket_size=0, world_size=2)                                      # bucket_size
    with pytest.raises(RuntimeError):
        glm5_router_gemm_cuda(x[:, :60].contiguous(), w[:, :60].contiguous())                   # H % 8
    ids = torch.empty((4, 2), dtype=torch.int32, device=dev)
    wt = torch.empty((4, 2), dtype=torch.float32, device=dev)
    bias = torch.zeros(8, device=dev)
    with pytest.raises(RuntimeError, match="workspace"):
        check(lib().bgmoe_router_gemm_gate(ptr(x), ptr(w), ptr(bias), 4, 64, 8, 0, 0, 2, 1.0, ptr(ids), ptr(wt),
                                           None, 0, None, 0, stream()))
    assert glm5_router_gemm_cuda(x[:0], w).shape == (0, 8)


@pytest.mark.parametrize("n,e,ng,tg,k", [(256, 256, 8, 4, 8), (16384, 256, 8, 4, 8), (512, 896, 0, 0, 16)])
def test_full_size_router_gemm_properties(dev, n, e, ng, tg, k):
    """The benchmark configurations' router shapes (H = 7168): rows do not depend on their position in the
    batch (bit-exact under a permutation of the tokens), a sample of rows meets the oracle's bar, and the
    fused GEMM + gate returns the routes of the two-op sequence."""
    from batchgen_amd.kernels import load_extension
    from batchgen_amd.moe.routing import (gate_sigmoid_topk_cuda, glm5_router_gemm_cuda,
                                          router_gemm_gate_sigmoid_topk)
    h = 7168
    say("router_gemm full size", n, h, e)
    g = torch.Generator().manual_seed(n + e)
    x = rand_bf16(g, n, h, scale=0.1).to(dev)
    w = rand_bf16(g, e, h, scale=0.1).to(dev)
    bias = (0.1 * torch.randn(e, generator=g)).to(dev)
    logits = glm5_router_gemm_cuda(x, w)
    assert torch.equal(logits, glm5_router_gemm_cuda(x, w))
    perm = torch.randperm(n, generator=g).to(dev)
    assert torch.equal(glm5_router_gemm_cuda(x[perm].contiguous(), w), logits[perm])
    sample = torch.tensor(sorted({0, 1, n // 2, n - 1}), device=dev)
    _check_close(logits[sample].cpu().numpy(), x[sample].cpu(), w.cpu())
    ids_f, w_f = router_gemm_gate_sigmoid_topk(x, w, bias, k, 2.5, n_group=ng, topk_group=tg)
    if ng:
        ids_u, w_u = load_extension("batchgen_kernels.common._C_mgn_ops").moe_fused_gate_logits(
            logits, bias, ng, tg, e, k, 2.5)
    else:
        ids_u, w_u = gate_sigmoid_topk_cuda(logits, bias, k, 2.5)
    assert torch.equal(ids_f, ids_u) and torch.equal(w_f, w_u)
