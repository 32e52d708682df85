"""The ragged workspace module driven as the GLM-5 prefill path drives it: sizes from its own helpers, every op
through its wrappers, each step against the oracle (indices and bytes bit-exact, the ordered combine bit-exact)."""
import numpy as np
import pytest
import torch

from oracle import combine as oc
from oracle import permute as op
from oracle import quant as oq
from tests.util import rand_bf16

pytestmark = pytest.mark.gpu


def test_ragged_pipeline_through_the_module(dev):
    from batchgen_amd.moe import moe_ragged as mr
    n, k, e_l, start, h, inter = 96, 8, 8, 16, 256, 128
    g = torch.Generator().manual_seed(77)
    x = rand_bf16(g, n, h)
    ids = torch.stack([torch.randperm(32, generator=g)[:k] for _ in range(n)]).to(torch.int32)
    wts = torch.rand(n, k, generator=g)
    rows = mr.ragged_row_capacity(n, k, e_l)
    assert rows % 128 == 0 and rows >= op.ragged_capacity_rows(n, k, e_l, mr.ROW_ALIGN)
    act = torch.zeros(rows, h, dtype=torch.bfloat16, device=dev)
    counts = torch.zeros(e_l, dtype=torch.int32, device=dev)
    counters = torch.zeros(e_l, dtype=torch.int32, device=dev)
    cu = torch.zeros(e_l + 1, dtype=torch.int32, device=dev)
    pos = torch.full((n * k,), -7, dtype=torch.int32, device=dev)
    mr.dispatch_scatter_ragged(x.to(dev), ids.to(dev), act, start, e_l, counts, counters, cu, pos)
    want_counts, want_cu, want_pos = op.dispatch_ragged(ids.numpy(), start, e_l, mr.ROW_ALIGN)
    assert np.array_equal(counts.cpu().numpy(), want_counts) and np.array_equal(cu.cpu().numpy(), want_cu)
    assert np.array_equal(pos.cpu().numpy(), want_pos)
    live = want_pos[want_pos >= 0]
    assert torch.equal(act.cpu()[live], x[np.nonzero(want_pos >= 0)[0] // k])

    xq, xs = mr.make_quant_buffers(rows, h, dev)
    mr.act_quant_ragged(act, counts, cu, xq, xs)
    ref_q, ref_s = oq.act_quant(act.cpu().float().numpy())
    assert np.array_equal(xq.cpu().numpy()[live], ref_q[live])
    assert np.array_equal(xs.cpu().numpy().T[live], ref_s[live])

    gate = rand_bf16(g, rows, inter).to(dev)
    up = rand_bf16(g, rows, inter).to(dev)
    hq = torch.zeros(rows, inter, dtype=torch.float8_e4m3fn, device=dev)
    hs = torch.zeros(rows, inter // 128, device=dev)
    mr.silu_mul_quant_ragged(gate, up, hq, hs, counts, cu)
    ref_hq, ref_hs, _ = oq.silu_mul_group_quant(gate.cpu().float().numpy(), up.cpu().float().numpy(), "D")
    assert np.array_equal(hq.cpu().view(torch.uint8).numpy()[live], ref_hq[live])
    assert np.array_equal(hs.cpu().numpy()[live], ref_hs[live])
    dead = np.setdiff1d(np.arange(rows), live)
    assert not hq.cpu().view(torch.uint8).numpy()[dead].any()          # rows outside the live set untouched

    y = rand_bf16(g, rows, h)
    out = torch.zeros(n, h, dtype=torch.bfloat16, device=dev)
    got = mr.reduce_weighted_scatter_bf16_ordered(y.to(dev), pos, ids.to(dev), wts.to(dev), n, h, k, output=out)
    want = oc.reduce_weighted_scatter_bf16_ordered(y.float().numpy(), want_pos, ids.numpy(), wts.numpy(), n, k)
    assert got.data_ptr() == out.data_ptr()
    assert np.array_equal(out.cpu().float().numpy(), np.asarray(want, dtype=np.float32))
    assert mr.require_ragged_kernels()[0] is not None
