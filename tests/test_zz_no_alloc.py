"""bgmoe_dispatch_scatter_ragged_static (the entry point that allocates nothing: its chunk histograms live in a
device array inside the library) against bgmoe_dispatch_scatter_ragged with a caller workspace, through the C
ABI: counts, cu_seqlens, positions and the scattered rows bit for bit, on two calls in a row, the second one
smaller (fewer chunks, so stale histogram entries of the first call lie behind it), and against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import permute as op_
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def _ids(g, n, k, e_total):
    # k distinct experts per token without a Python loop over tokens
    return torch.rand(n, e_total, generator=g).argsort(dim=1)[:, :k].to(torch.int32).contiguous()


def _run(dev, static, x, ids, es, el, align):
    from batchgen_amd import _lib
    L = _lib.lib()
    n, k = ids.shape
    h = x.shape[1]
    nk = n * k
    cap = (nk + (align - 1) * min(nk, el)) // align * align
    act = torch.full((cap, h), -1.0, dtype=torch.bfloat16, device=dev)
    counts = torch.full((el,), -3, dtype=torch.int32, device=dev)
    counters = torch.full((el,), -3, dtype=torch.int32, device=dev)
    pos = torch.full((nk,), -9, dtype=torch.int32, device=dev)
    cu = torch.full((el + 1,), -5, dtype=torch.int32, device=dev)
    xd, idd = x.to(dev), ids.to(dev)
    if static:
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(dev)
        _lib.check(L.bgmoe_dispatch_scatter_ragged_static(
            xd.data_ptr(), idd.data_ptr(), n, k, h, act.data_ptr(), cap, es, el, counts.data_ptr(),
            counters.data_ptr(), pos.data_ptr(), cu.data_ptr(), align, _lib.stream()))
        assert torch.cuda.memory_allocated(dev) == before
    else:
        need = L.bgmoe_dispatch_workspace_bytes(nk, el)
        assert need > 0, "the case must be large enough to use the histogram workspace"
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        _lib.check(L.bgmoe_dispatch_scatter_ragged(
            xd.data_ptr(), idd.data_ptr(), n, k, h, act.data_ptr(), cap, es, el, counts.data_ptr(),
            counters.data_ptr(), pos.data_ptr(), cu.data_ptr(), align, ws.data_ptr(), need, _lib.stream()))
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (counts, counters, pos, cu)] + [act.view(torch.int16).cpu().numpy()]


def test_static_dispatch_equals_workspace_dispatch_twice(dev):
    from batchgen_amd import _lib
    L = _lib.lib()
    assert L.bgmoe_dispatch_static_max_pairs(256) == 1024 * 2048
    g = torch.Generator().manual_seed(77)
    # (n, k, h, e_total, expert_start, e_local, row_align): 32768 pairs in 16 chunks, then 12000 pairs in 6
    for n, k, h, et, es, el, align in [(4096, 8, 128, 256, 32, 32, 64), (1500, 8, 128, 256, 32, 32, 64)]:
        say("dispatch_ragged_static", n, k, h, et, es, el, align)
        ids = _ids(g, n, k, et)
        ids.view(-1)[:5] = torch.tensor([-1, 0, es - 1, es + el, 10 ** 6], dtype=torch.int32)
        x = rand_bf16(g, n, h)
        got = _run(dev, True, x, ids, es, el, align)
        want = _run(dev, False, x, ids, es, el, align)
        for a, b, name in zip(got, want, ("counts", "counters", "pos", "cu_seqlens", "rows")):
            assert np.array_equal(a, b), f"{name} differ between the static and the workspace entry point"
        counts_o, cu_o, pos_o = op_.dispatch_ragged(ids.numpy(), es, el, align)
        assert np.array_equal(got[0], counts_o) and np.array_equal(got[3], cu_o) and np.array_equal(got[2], pos_o)


def test_static_dispatch_rejects_sizes_beyond_its_buffer(dev):
    from batchgen_amd import _lib
    L = _lib.lib()
    el = 1024
    n = L.bgmoe_dispatch_static_max_pairs(el) // 8 + 2048      # one chunk more than the buffer holds
    rc = L.bgmoe_dispatch_scatter_ragged_static(None, None, n, 8, 64, None, 0, 0, el, 16, None, 16, 16, 1, None)
    assert rc == 3
    assert b"static buffer holds" in L.bgmoe_last_error()
