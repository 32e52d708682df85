"""Pins for the oracle's routers (CPU only): an independent torch.topk transcription of the PyTorch gate,
brute force on tiny inputs, and the tie / NaN / padding cases the reference tests spell out."""
import itertools

import numpy as np
import torch

from oracle import router as orr


def _r1_torch(scores, bias, ng, tg, k, rsf):
    """MoEGate.forward recipe (modeling_deepseek_v3.py:793-845) with sorted top-k."""
    n, e = scores.shape
    sfc = scores + bias
    gs = sfc.view(n, ng, -1).topk(2, dim=-1)[0].sum(-1)
    gi = gs.topk(tg, dim=-1)[1]
    gm = torch.zeros_like(gs).scatter_(1, gi, 1.0)
    sm = gm.unsqueeze(-1).expand(n, ng, e // ng).reshape(n, -1)
    tmp = sfc.masked_fill(~sm.bool(), float("-inf"))
    ti = tmp.topk(k, dim=-1, sorted=True)[1]
    tw = scores.gather(1, ti)
    return ti, tw / (tw.sum(-1, keepdim=True) + 1e-20) * rsf


def test_fused_gate_equals_torch_topk_transcription():
    g = torch.Generator().manual_seed(0)
    for n, e, ng, tg, k, rsf in [(500, 256, 8, 4, 8, 2.5), (64, 16, 4, 2, 4, 1.0), (100, 64, 4, 2, 2, 1.5)]:
        logits = torch.randn(n, e, generator=g)
        bias = 0.1 * torch.randn(e, generator=g)
        scores = torch.sigmoid(logits)
        ids, w = orr.fused_gate(scores.numpy(), bias.numpy(), ng, tg, k, rsf)
        ti, tw = _r1_torch(scores, bias, ng, tg, k, rsf)
        assert np.array_equal(ids, ti.numpy().astype(np.int32))
        np.testing.assert_allclose(w, tw.numpy(), rtol=3e-7)
        np.testing.assert_allclose(w.sum(1), rsf, rtol=1e-6)


def test_fused_gate_brute_force_tiny():
    rng = np.random.default_rng(1)
    e, ng, tg, k = 8, 4, 2, 3
    for _ in range(200):
        scores = rng.random((1, e)).astype(np.float32)
        bias = (0.3 * rng.standard_normal(e)).astype(np.float32)
        ids, _ = orr.fused_gate(scores, bias, ng, tg, k, 1.0)
        s = (scores[0] + bias).astype(np.float32)
        gsum = [np.float32(np.sort(s[2 * g:2 * g + 2])[::-1].sum(dtype=np.float32)) for g in range(ng)]
        best = max(itertools.combinations(range(ng), tg), key=lambda c: (sum(float(gsum[i]) for i in c)))
        allowed = [i for i in range(e) if i // 2 in best]
        expect = sorted(allowed, key=lambda i: (-s[i], i))[:k]
        assert ids[0].tolist() == expect


def test_fused_gate_tie_rules():
    e, ng, tg, k = 32, 4, 2, 4
    scores = np.full((2, e), 0.5, dtype=np.float32)
    scores[1, 20] = 0.75
    ids, w = orr.fused_gate(scores, np.zeros(e, np.float32), ng, tg, k, 1.0)
    assert ids[0].tolist() == [0, 1, 2, 3]                 # equal everywhere: lowest groups, lowest ids
    assert ids[1, 0] == 20 and set(ids[1, 1:].tolist()) <= set(range(0, 8)) | set(range(16, 24))
    np.testing.assert_allclose(w.sum(1), 1.0, rtol=1e-6)


def test_sigmoid_is_correctly_rounded_and_close_to_torch():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(100000, generator=g) * 4
    s = orr.sigmoid_f32(x.numpy())
    t = torch.sigmoid(x).numpy()
    ulp = np.spacing(np.abs(s))
    assert np.all(np.abs(s - t) <= 2 * ulp)                # torch's vectorised fp32 sigmoid is within 2 ulp of it
    exact = 1.0 / (1.0 + np.exp(-x.double().numpy()))
    assert np.all(np.abs(s.astype(np.float64) - exact) <= 0.5 * np.spacing(s).astype(np.float64) * (1 + 1e-9))


def test_gate_sigmoid_topk_against_torch_topk():
    g = torch.Generator().manual_seed(3)
    for n, e, k, rsf in [(300, 896, 16, 1.0), (64, 384, 8, 2.5), (10, 64, 2, 1.0)]:
        logits = torch.randn(n, e, generator=g)
        bias = 0.1 * torch.randn(e, generator=g)
        ids, w = orr.gate_sigmoid_topk(logits.numpy(), bias.numpy(), k, rsf)
        sc = torch.from_numpy(orr.sigmoid_f32(logits.numpy()))
        ti = (sc + bias).topk(k, dim=-1, sorted=True)[1]
        assert np.array_equal(ids, ti.numpy().astype(np.int32))
        raw = sc.gather(1, ti)
        np.testing.assert_allclose(w, (raw / (raw.sum(-1, keepdim=True) + 1e-20) * rsf).numpy(), rtol=3e-7, atol=2e-6)
        assert all(len(set(r)) == k for r in ids.tolist())


def test_gate_sigmoid_topk_ties_nan_padding():
    e, k = 64, 8
    logits = np.zeros((4, e), dtype=np.float32)
    logits[1] = 40.0
    logits[2, :k - 1] = 3.0
    logits[2, k - 1:k + 3] = 1.0
    logits[3, ::2] = np.nan
    logits[3, 1::2] = np.linspace(-1, 1, e // 2)
    ids, w = orr.gate_sigmoid_topk(logits, np.zeros(e, np.float32), k, 1.0)
    assert ids[0].tolist() == list(range(k)) and ids[1].tolist() == list(range(k)) and ids[2].tolist() == list(range(k))
    assert all(i % 2 == 1 for i in ids[3].tolist())
    ids, w = orr.gate_sigmoid_topk(logits, np.zeros(e, np.float32), k, 1.0, num_valid_tokens=2)
    assert np.all(ids[2:] == -1) and np.all(w[2:] == 0) and np.all(ids[:2] >= 0)
    ids, w = orr.gate_sigmoid_topk(logits, np.zeros(e, np.float32), k, 1.0, rank_token_counts=[1, 0], rows_per_rank=2)
    assert np.all(ids[0] >= 0) and np.all(ids[1:] == -1)
    allnan = np.full((1, e), np.nan, dtype=np.float32)
    ids, w = orr.gate_sigmoid_topk(allnan, np.zeros(e, np.float32), k, 1.0)
    assert np.all(ids == -1) and np.all(w == 0)
