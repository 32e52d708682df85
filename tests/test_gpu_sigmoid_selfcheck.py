"""Device self-checks of two exact short cuts.  The routers' short sigmoid evaluation against the library
evaluation, over EVERY float bit pattern: the two must agree in all bits (NaN with NaN), and the short path
must decide almost always.  The quantisers' division by the block scale against the IEEE division, on 2^34
pseudo-random pairs from the quantisers' domain: identical e4m3 bytes and identical quotient bits."""
import numpy as np
import pytest
import torch

from oracle import router as orr
from tests.util import say

pytestmark = pytest.mark.gpu


def test_short_sigmoid_equals_fp64_evaluation_for_all_floats(dev):
    from batchgen_amd._lib import check, lib, ptr
    counters = torch.zeros(2, dtype=torch.int64, device=dev)
    step = 1 << 30
    for part in range(4):
        say("sigmoid self-check, bit patterns from", hex(part * step))
        check(lib().bgmoe_selfcheck_sigmoid(part * step, step, ptr(counters[0:1]), ptr(counters[1:2]), None))
        torch.cuda.synchronize()
    bad, slow = counters.cpu().tolist()
    in_range = 2 * (np.float32(80.0).view(np.uint32).item() + 1)       # |x| <= 80, both signs
    say("   mismatches", bad, "handed to the library evaluation", slow, "of", in_range)
    assert bad == 0
    assert slow / in_range < 1e-3


def test_router_scores_still_match_the_oracle_on_awkward_logits(dev):
    """Logits whose sigmoid lies close to a float rounding boundary are the ones a wrong error bound would
    break: take the inputs with the smallest distance to a boundary from a dense sample and run the gate."""
    from batchgen_amd.moe.routing import gate_sigmoid_topk_cuda
    x = np.linspace(-30, 30, 4_000_001).astype(np.float32)
    y = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    f = y.astype(np.float32)
    nxt = np.where(f.astype(np.float64) <= y, np.nextafter(f, np.float32(2)), np.nextafter(f, np.float32(-1)))
    mid = (f.astype(np.float64) + nxt.astype(np.float64)) / 2
    order = np.argsort(np.abs(y - mid) / y)[:4096]
    logits = torch.from_numpy(x[order].reshape(512, 8).copy())        # k = E = 8: every score reaches the output
    bias = torch.zeros(8)
    ids = torch.empty((512, 8), dtype=torch.int32, device=dev)
    w = torch.empty((512, 8), dtype=torch.float32, device=dev)
    gate_sigmoid_topk_cuda(logits.to(dev), bias.to(dev), 8, 1.0, ids, w)
    rid, rw = orr.gate_sigmoid_topk(logits.numpy(), bias.numpy(), 8, 1.0)
    assert np.array_equal(ids.cpu().numpy(), rid) and np.array_equal(w.cpu().numpy(), rw)


def test_scale_division_equals_ieee_division(dev):
    from batchgen_amd._lib import check, lib, ptr
    counters = torch.zeros(2, dtype=torch.int64, device=dev)
    for part in range(4):
        say("scale-division self-check, part", part)
        check(lib().bgmoe_selfcheck_scale_division(20261125 + part * (1 << 40), 1 << 32, ptr(counters[0:1]),
                                                   ptr(counters[1:2]), None))
        torch.cuda.synchronize()
    bad_bytes, bad_bits = counters.cpu().tolist()
    say("   e4m3 byte mismatches", bad_bytes, "quotient bit mismatches", bad_bits)
    assert bad_bytes == 0 and bad_bits == 0
