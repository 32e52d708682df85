"""The tight (align 1) dispatch ops on the GPU against the sequential CPU oracle, bit for bit:
``dispatch_count_gather`` (batchgen_kernels/src/moe/routing/dispatch_count_gather.cu:145-251),
``fused_moe_token_dispatch`` (batchgen_kernels/src/moe/mgn/fused_moe_token_dispatch.cu:172-292) and
``expert_bincount`` (batchgen_kernels/src/moe/mgn/expert_bin_count.cu:155-231), with the non-local ids the
reference's own tests inject (-1, 0, start - 1, start + E, 10**6)."""
import numpy as np
import pytest
import torch

from oracle import permute as op_
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def routing():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_routing")


def mgn():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.common._C_mgn_ops")


def _ids(g, n, k, e_total, es, el):
    ids = torch.stack([torch.randperm(e_total, generator=g)[:k] for _ in range(n)]).to(torch.int32)
    extra = [-1, 0, es - 1, es + el, 10 ** 6]
    if n * k >= 4 * len(extra):
        where = torch.randperm(n * k, generator=g)[: len(extra)]
        ids.view(-1)[where] = torch.tensor(extra, dtype=torch.int32)
    return ids


CASES = [  # n, k, h, e_total, expert_start, e_local
    (1, 4, 256, 16, 0, 16), (64, 4, 1024, 16, 4, 8), (256, 8, 7168, 256, 32, 32), (100, 2, 131, 64, 32, 8),
    (700, 8, 256, 256, 0, 256), (4096, 8, 128, 256, 64, 32), (513, 16, 64, 896, 28, 28), (37, 6, 2880, 128, 16, 16),
]


def _sequential(ids, es, el):
    counts, offs, pos = op_.dispatch_sequential(ids.numpy(), es, el)
    return counts, offs, pos


@pytest.mark.parametrize("n,k,h,et,es,el", CASES)
@pytest.mark.parametrize("valid", [-1, 0.5])
def test_dispatch_count_gather(dev, n, k, h, et, es, el, valid):
    nv = -1 if valid == -1 else max(1, int(n * valid))
    if nv == n:
        pytest.skip("same as the untruncated case")
    say("dispatch_count_gather", n, k, h, et, es, el, nv)
    g = torch.Generator().manual_seed(n * 7 + k + 1000 * (nv > 0))
    ids = _ids(g, n, k, et, es, el)
    x = rand_bf16(g, n, h)
    n_eff = n if nv < 0 else nv
    counts_o, offs_o, pos_o = _sequential(ids[:n_eff], es, el)
    total = int(offs_o[-1])
    cap = n * k
    counts = torch.full((el,), -3, dtype=torch.int32, device=dev)
    offs = torch.full((el + 1,), -3, dtype=torch.int32, device=dev)
    counters = torch.full((el,), -3, dtype=torch.int32, device=dev)
    pos = torch.full((n * k,), -9, dtype=torch.int32, device=dev)
    out = torch.full((cap, h), 7.0, dtype=torch.bfloat16, device=dev)
    got = routing().dispatch_count_gather(x.to(dev), ids.to(dev), es, el, counts, offs, counters, out, pos, nv)
    assert got[0] is counts and got[1] is offs and got[2] is pos
    assert np.array_equal(counts.cpu().numpy(), counts_o)
    assert np.array_equal(counters.cpu().numpy(), counts_o)
    assert np.array_equal(offs.cpu().numpy(), offs_o)
    assert np.array_equal(pos.cpu().numpy()[: n_eff * k], pos_o)
    assert (pos.cpu().numpy()[n_eff * k:] == -9).all(), "pairs of tokens past num_valid_tokens must not be touched"
    ref = op_.gather_rows(x[:n_eff].view(torch.int16).numpy(), pos_o, k, total)
    o = out.view(torch.int16).cpu().numpy()
    assert np.array_equal(o[:total], ref)
    seven = torch.tensor([7.0], dtype=torch.bfloat16).view(torch.int16).item()
    assert (o[total:] == seven).all(), "rows past the last offset must not be written"


@pytest.mark.parametrize("n,k,h,et,es,el", CASES)
def test_fused_moe_token_dispatch(dev, n, k, h, et, es, el):
    say("fused_moe_token_dispatch", n, k, h, et, es, el)
    g = torch.Generator().manual_seed(n * 11 + k)
    ids = _ids(g, n, k, et, es, el)
    x = rand_bf16(g, n, h)
    counts_o, offs_o, pos_o = _sequential(ids, es, el)
    total = int(offs_o[-1])
    # the reference passes (and ignores) token_idx / topk_pos tensors
    tok_in = torch.arange(n, dtype=torch.int32, device=dev)
    pos_in = torch.arange(k, dtype=torch.int32, device=dev).repeat(n, 1)
    out_x, out_eids, out_tok, out_pos, counts, offs = mgn().fused_moe_token_dispatch(
        x.to(dev), ids.to(dev), tok_in, pos_in, es, es + el)
    assert out_x.shape == (n * k, h) and out_x.dtype == torch.bfloat16
    for t in (out_eids, out_tok, out_pos):
        assert t.shape == (n * k,) and t.dtype == torch.int32
    assert counts.shape == (el,) and offs.shape == (el + 1,)
    assert np.array_equal(counts.cpu().numpy(), counts_o)
    assert np.array_equal(offs.cpu().numpy(), offs_o)
    ref = op_.gather_rows(x.view(torch.int16).numpy(), pos_o, k, total)
    assert np.array_equal(out_x.view(torch.int16).cpu().numpy()[:total], ref)
    # the three per-row arrays: row pos_o[i] belongs to pair i
    eids_o = np.full(n * k, -1, np.int32)
    tok_o = np.full(n * k, -1, np.int32)
    slot_o = np.full(n * k, -1, np.int32)
    flat = ids.numpy().reshape(-1)
    for i in np.nonzero(pos_o >= 0)[0]:
        eids_o[pos_o[i]] = flat[i]
        tok_o[pos_o[i]] = i // k
        slot_o[pos_o[i]] = i % k
    assert np.array_equal(out_eids.cpu().numpy(), eids_o)
    assert np.array_equal(out_tok.cpu().numpy(), tok_o)
    assert np.array_equal(out_pos.cpu().numpy(), slot_o)
    # an expert's rows are its segment, in ascending (token, slot) order
    for e in range(el):
        seg = slice(int(offs_o[e]), int(offs_o[e + 1]))
        assert (eids_o[seg] == es + e).all()
        key = tok_o[seg].astype(np.int64) * k + slot_o[seg]
        assert (np.diff(key) > 0).all()


def test_fused_moe_token_dispatch_is_graph_capturable(dev):
    """No device -> host read anywhere in the op: with its allocations made by a warm-up call on the capture
    stream's pool, the whole op records into a HIP graph and a replay on new ids gives the new answer."""
    n, k, h, et, es, el = 128, 8, 512, 256, 32, 32
    g = torch.Generator().manual_seed(5)
    x = rand_bf16(g, n, h).to(dev)
    ids_a = _ids(g, n, k, et, es, el)
    ids_b = _ids(g, n, k, et, es, el)
    ids_dev = ids_a.to(dev)
    m = mgn()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        m.fused_moe_token_dispatch(x, ids_dev, None, None, es, es + el)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = m.fused_moe_token_dispatch(x, ids_dev, None, None, es, es + el)
    for ids in (ids_b, ids_a, ids_b):
        ids_dev.copy_(ids.to(dev))
        graph.replay()
        torch.cuda.synchronize()
        counts_o, offs_o, pos_o = _sequential(ids, es, el)
        total = int(offs_o[-1])
        assert np.array_equal(outs[4].cpu().numpy(), counts_o)
        assert np.array_equal(outs[5].cpu().numpy(), offs_o)
        ref = op_.gather_rows(x.cpu().view(torch.int16).numpy(), pos_o, k, total)
        assert np.array_equal(outs[0].view(torch.int16).cpu().numpy()[:total], ref)
        tok = outs[2].cpu().numpy()
        assert (tok[total:] == -1).all() and (tok[:total] >= 0).all()


def test_fused_moe_token_dispatch_errors(dev):
    x = torch.zeros((4, 64), dtype=torch.bfloat16, device=dev)
    ids = torch.zeros((4, 2), dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        mgn().fused_moe_token_dispatch(x.cpu(), ids, None, None, 0, 4)
    with pytest.raises(RuntimeError):
        mgn().fused_moe_token_dispatch(x, ids, None, None, 4, 4)
    with pytest.raises(RuntimeError):
        mgn().fused_moe_token_dispatch(x.float(), ids, None, None, 0, 4)


@pytest.mark.parametrize("n,et,es,el", [(1, 16, 0, 16), (77, 64, 8, 8), (2048, 256, 32, 32), (50000, 256, 0, 256),
                                         (300, 896, 28, 28), (5, 16, 0, 600)])
def test_expert_bincount(dev, n, et, es, el):
    say("expert_bincount", n, et, es, el)
    g = torch.Generator().manual_seed(n + el)
    eids = torch.randint(0, et, (n,), generator=g, dtype=torch.int32)
    extra = torch.tensor([-1, 0, es - 1, es + el, 10 ** 6], dtype=torch.int32)
    if n >= 20:
        eids[torch.randperm(n, generator=g)[:5]] = extra
    counts_o = np.zeros(el, np.int64)
    for e in eids.tolist():
        if es <= e < es + el:
            counts_o[e - es] += 1
    size, idx, start, num = mgn().expert_bincount(eids.to(dev), es, el, torch.device(dev))
    for t in (size, idx, start):
        assert t.shape == (el,) and t.dtype == torch.int32
    na = int(num.item())
    nz = np.nonzero(counts_o)[0]
    assert na == len(nz)
    assert np.array_equal(idx.cpu().numpy()[:na], nz)
    assert np.array_equal(size.cpu().numpy()[:na], counts_o[nz])
    assert np.array_equal(start.cpu().numpy()[:na], np.cumsum(counts_o[nz]) - counts_o[nz])
