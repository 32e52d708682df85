"""HIP routers vs the CPU oracle: ids bit-exact, weights bit-exact (same fp32 op sequence)."""
import numpy as np
import pytest
import torch

from oracle import router as orr
from tests.util import say

pytestmark = pytest.mark.gpu


def mgn():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.common._C_mgn_ops")


def routing():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_routing")


GROUPED = [  # n, e, n_group, topk_group, top_k, rsf
    (64, 16, 4, 2, 4, 1.0),
    (256, 256, 8, 4, 8, 2.5),
    (1000, 256, 8, 4, 8, 2.5),
    (37, 64, 4, 2, 2, 1.5),
    (19, 128, 8, 4, 6, 2.0),
    (5, 512, 8, 4, 8, 1.0),
    (40, 96, 4, 2, 4, 1.0),      # 24 experts per group: not a power of two, the LDS scan
    (20, 256, 1, 1, 8, 2.5),     # one group of 256: whole register slots per group
    (9, 384, 2, 1, 4, 1.0),      # 192 per group
    (12, 512, 2, 2, 8, 1.0),
    (6, 1024, 4, 3, 16, 1.0),
]


@pytest.mark.parametrize("n,e,ng,tg,k,rsf", GROUPED)
def test_fused_gate_scores_bit_exact(dev, n, e, ng, tg, k, rsf):
    say("fused_gate", n, e, ng, tg, k)
    g = torch.Generator().manual_seed(n * 31 + e)
    scores = torch.sigmoid(torch.randn(n, e, generator=g))
    bias = 0.1 * torch.randn(e, generator=g)
    ids, w = mgn().moe_fused_gate(scores.to(dev), bias.to(dev), ng, tg, e, k, rsf)
    ido, wo = orr.fused_gate(scores.numpy(), bias.numpy(), ng, tg, k, rsf)
    assert ids.dtype == torch.int32 and w.dtype == torch.float32
    assert np.array_equal(ids.cpu().numpy(), ido)
    assert np.array_equal(w.cpu().numpy().view(np.uint32), wo.view(np.uint32))


@pytest.mark.parametrize("n,e,ng,tg,k,rsf", GROUPED[:3])
def test_fused_gate_logits_sigmoid_inside(dev, n, e, ng, tg, k, rsf):
    g = torch.Generator().manual_seed(n + 7 * e)
    logits = torch.randn(n, e, generator=g)
    bias = 0.1 * torch.randn(e, generator=g)
    ids, w = mgn().moe_fused_gate_logits(logits.to(dev), bias.to(dev), ng, tg, e, k, rsf)
    ido, wo = orr.grouped_router(logits.numpy(), bias.numpy(), ng, tg, k, rsf)
    assert np.array_equal(ids.cpu().numpy(), ido)
    # the device evaluates exp in fp64 like the oracle; allow one fp32 ulp on the weights
    np.testing.assert_allclose(w.cpu().numpy(), wo, rtol=2e-7, atol=0)


def test_fused_gate_ties_lowest_index(dev):
    e, ng, tg, k = 32, 4, 2, 4
    scores = torch.full((3, e), 0.5)
    scores[1, 20] = 0.75
    scores[2, :] = torch.linspace(0.1, 0.9, e).flip(0)
    bias = torch.zeros(e)
    ids, w = mgn().moe_fused_gate(scores.to(dev), bias.to(dev), ng, tg, e, k, 1.0)
    ido, wo = orr.fused_gate(scores.numpy(), bias.numpy(), ng, tg, k, 1.0)
    assert np.array_equal(ids.cpu().numpy(), ido)
    assert ids[0].tolist() == [0, 1, 2, 3]           # all equal: lowest groups, lowest ids


UNGROUPED = [(512, 896, 16, 1.0), (64, 384, 8, 2.5), (33, 256, 8, 2.5), (7, 64, 4, 1.0), (3, 1024, 2, 1.0)]


@pytest.mark.parametrize("n,e,k,rsf", UNGROUPED)
def test_gate_sigmoid_topk(dev, n, e, k, rsf):
    say("gate_sigmoid_topk", n, e, k)
    g = torch.Generator().manual_seed(n + e + k)
    logits = torch.randn(n, e, generator=g)
    bias = 0.1 * torch.randn(e, generator=g)
    ids = torch.empty((n, k), dtype=torch.int32, device=dev)
    w = torch.empty((n, k), dtype=torch.float32, device=dev)
    routing().gate_sigmoid_topk(logits.to(dev), bias.to(dev), k, rsf, ids, w)
    ido, wo = orr.gate_sigmoid_topk(logits.numpy(), bias.numpy(), k, rsf)
    assert np.array_equal(ids.cpu().numpy(), ido)
    np.testing.assert_allclose(w.cpu().numpy(), wo, rtol=2e-7, atol=0)
    # invariants of the reference tests: distinct ids, weights sum to rsf
    assert all(len(set(r)) == k for r in ids.cpu().tolist())
    np.testing.assert_allclose(w.sum(1).cpu().numpy(), rsf, rtol=1e-5)


def test_gate_sigmoid_topk_tie_cases_and_nan(dev):
    e, k = 64, 8
    logits = torch.zeros(5, e)
    logits[1, :] = 40.0                               # saturated sigmoids -> ascending ids
    logits[2, :k - 1] = 3.0
    logits[2, k - 1:k + 3] = 1.0                      # duplicates across the k-th boundary
    logits[3, ::2] = float("nan")                     # NaN logits are never selected
    logits[3, 1::2] = torch.linspace(-1, 1, e // 2)
    logits[4, 10] = 2.0
    bias = torch.zeros(e)
    ids = torch.empty((5, k), dtype=torch.int64, device=dev)
    w = torch.empty((5, k), dtype=torch.float32, device=dev)
    routing().gate_sigmoid_topk_warp(logits.to(dev), bias.to(dev), k, 1.0, ids, w)
    ido, wo = orr.gate_sigmoid_topk(logits.numpy(), bias.numpy(), k, 1.0)
    assert np.array_equal(ids.cpu().numpy(), ido.astype(np.int64))
    assert ids[0].tolist() == list(range(k)) and ids[1].tolist() == list(range(k))
    assert ids[2].tolist() == list(range(k))
    assert all(i % 2 == 1 for i in ids[3].tolist())


def test_gate_sigmoid_topk_padding_and_strided_rows(dev):
    n, e, k = 24, 128, 4
    g = torch.Generator().manual_seed(9)
    wide = torch.randn(n, e + 64, generator=g).to(dev)
    logits = wide[:, :e]                              # strided rows
    bias = (0.1 * torch.randn(e, generator=g)).to(dev)
    ids = torch.full((n, k), 77, dtype=torch.int32, device=dev)
    w = torch.full((n, k), 5.0, dtype=torch.float32, device=dev)
    nv = torch.tensor([10], dtype=torch.int32, device=dev)
    lat = torch.empty((n, 64), dtype=torch.bfloat16, device=dev)
    routing().gate_sigmoid_topk(logits, bias, k, 2.0, ids, w, nv, lat, e)
    ido, wo = orr.gate_sigmoid_topk(logits.cpu().numpy(), bias.cpu().numpy(), k, 2.0, num_valid_tokens=10)
    assert np.array_equal(ids.cpu().numpy(), ido)
    np.testing.assert_allclose(w.cpu().numpy(), wo, rtol=2e-7)
    assert torch.equal(lat[:10], wide[:10, e:].to(torch.bfloat16)) and torch.all(lat[10:] == 0)
    # per-rank live prefixes
    rc = torch.tensor([3, 0, 8], dtype=torch.int64, device=dev)
    routing().gate_sigmoid_topk(logits, bias, k, 2.0, ids, w, None, None, None, rc, 8)
    ido, wo = orr.gate_sigmoid_topk(logits.cpu().numpy(), bias.cpu().numpy(), k, 2.0,
                                    rank_token_counts=[3, 0, 8], rows_per_rank=8)
    assert np.array_equal(ids.cpu().numpy(), ido)


def test_router_argument_errors(dev):
    logits = torch.zeros(4, 16, device=dev)
    bias = torch.zeros(16, device=dev)
    ids = torch.empty((4, 3), dtype=torch.int32, device=dev)
    w = torch.empty((4, 3), dtype=torch.float32, device=dev)
    with pytest.raises(RuntimeError):
        routing().gate_sigmoid_topk(logits, bias, 3, 1.0, ids, w)      # k not in {2,4,8,16}
    with pytest.raises(RuntimeError):
        mgn().moe_fused_gate(logits, bias, 3, 2, 16, 4, 1.0)           # 16 % 3 != 0
