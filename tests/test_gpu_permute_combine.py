"""HIP permute / combine vs the CPU oracle: indices and outputs bit-exact."""
import numpy as np
import pytest
import torch

from oracle import combine as oc
from oracle import permute as op_
from oracle.quant import act_quant
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def ds3d():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_dispatch_scatter_3d")


def _ids(g, n, k, e_total, extra=None):
    ids = torch.stack([torch.randperm(e_total, generator=g)[:k] for _ in range(n)]).to(torch.int32)
    if extra is not None and n * k >= len(extra):
        ids.view(-1)[: len(extra)] = torch.tensor(extra, dtype=torch.int32)
    return ids


CASES = [  # n, k, h, e_total, expert_start, e_local
    (1, 4, 256, 16, 0, 16), (64, 4, 1024, 16, 0, 16), (256, 8, 7168, 256, 0, 32), (256, 8, 512, 256, 64, 32),
    (100, 2, 131, 64, 32, 8), (700, 8, 256, 256, 0, 256), (4096, 8, 128, 256, 32, 32), (513, 16, 64, 896, 28, 28),
    (200, 8, 128, 256, 0, 256),      # <= 2048 pairs, 256 local experts: the one-block kernel at its limit
    (250, 8, 64, 600, 100, 300),     # <= 2048 pairs, more than 256 local experts: the four-wave one-launch kernel
    (512, 16, 64, 896, 28, 28),      # 8192 pairs: the one-block kernel's eight sub-steps, at its limit
    (1000, 8, 64, 256, 0, 256),      # 8000 pairs, 256 local experts
]


@pytest.mark.parametrize("n,k,h,et,es,el", CASES)
def test_dispatch_masked(dev, n, k, h, et, es, el):
    say("dispatch_3d", n, k, h, et, es, el)
    g = torch.Generator().manual_seed(n * 13 + k)
    ids = _ids(g, n, k, et, extra=[-1, 0, es - 1, es + el, 10 ** 6])
    x = rand_bf16(g, n, h)
    counts_o, pos_o = op_.dispatch_masked(ids.numpy(), es, el, 10 ** 9)
    mtp = max(int(counts_o.max()), 1)
    counts_o, pos_o = op_.dispatch_masked(ids.numpy(), es, el, mtp)
    act = torch.zeros((el * mtp, h), dtype=torch.bfloat16, device=dev)
    counts = torch.full((el,), -3, dtype=torch.int32, device=dev)
    counters = torch.full((el,), -3, dtype=torch.int32, device=dev)
    pos = torch.full((n * k,), -9, dtype=torch.int32, device=dev)
    ds3d().dispatch_scatter_3d(x.to(dev), ids.to(dev), act, es, el, mtp, counts, counters, pos)
    assert np.array_equal(counts.cpu().numpy(), counts_o)
    assert np.array_equal(counters.cpu().numpy(), counts_o)
    assert np.array_equal(pos.cpu().numpy(), pos_o)
    ref = op_.gather_rows(x.view(torch.int16).numpy(), pos_o, k, el * mtp)
    assert np.array_equal(act.view(torch.int16).cpu().numpy(), ref)


@pytest.mark.parametrize("row_align", [1, 64, 128])
@pytest.mark.parametrize("n,k,h,et,es,el", CASES)
def test_dispatch_ragged(dev, n, k, h, et, es, el, row_align):
    say("dispatch_ragged", n, k, h, et, es, el, row_align)
    g = torch.Generator().manual_seed(n * 17 + k + row_align)
    ids = _ids(g, n, k, et, extra=[-1, 0, es - 1, es + el, 10 ** 6])
    x = rand_bf16(g, n, h)
    cap = op_.ragged_capacity_rows(n, k, el, row_align)
    counts_o, cu_o, pos_o = op_.dispatch_ragged(ids.numpy(), es, el, row_align)
    assert cu_o[-1] <= cap
    act = torch.zeros((max(cap, 1), h), dtype=torch.bfloat16, device=dev)
    counts = torch.empty(el, dtype=torch.int32, device=dev)
    counters = torch.empty(el, dtype=torch.int32, device=dev)
    cu = torch.empty(el + 1, dtype=torch.int32, device=dev)
    pos = torch.empty(n * k, dtype=torch.int32, device=dev)
    if cap == 0:
        pytest.skip("empty capacity")
    r = ds3d().dispatch_scatter_ragged(x.to(dev), ids.to(dev), act, es, el, counts, counters, pos, cu, row_align)
    assert r[0] is counts and r[1] is cu and r[2] is pos          # caller-owned tensors come back
    assert np.array_equal(counts.cpu().numpy(), counts_o)
    assert np.array_equal(cu.cpu().numpy(), cu_o)
    assert np.array_equal(pos.cpu().numpy(), pos_o)
    ref = op_.gather_rows(x.view(torch.int16).numpy(), pos_o, k, max(cap, 1))
    assert np.array_equal(act.view(torch.int16).cpu().numpy(), ref)
    # invariants the reference tests check: rows of expert e are exactly [cu[e], cu[e]+count)
    pn = pos.cpu().numpy()
    flat = ids.view(-1).numpy().astype(np.int64) - es
    for e in range(el):
        rows = np.sort(pn[(flat == e)])
        assert np.array_equal(rows, np.arange(cu_o[e], cu_o[e] + counts_o[e]))


def test_dispatch_ragged_rejects_small_buffer_and_bad_align(dev):
    x = torch.zeros((8, 64), dtype=torch.bfloat16, device=dev)
    ids = torch.zeros((8, 2), dtype=torch.int32, device=dev)
    mk = lambda n: torch.empty(n, dtype=torch.int32, device=dev)
    act = torch.zeros((64, 64), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        ds3d().dispatch_scatter_ragged(x, ids, act, 0, 4, mk(4), mk(4), mk(16), mk(5), 64)   # needs 256 rows
    with pytest.raises(RuntimeError):
        ds3d().dispatch_scatter_ragged(x, ids, act, 0, 4, mk(4), mk(4), mk(16), mk(5), 48)


def test_scatter_quant_equals_scatter_then_quant(dev):
    from batchgen_amd._lib import check, lib, ptr, stream
    g = torch.Generator().manual_seed(21)
    n, k, h, el = 50, 4, 1024, 8
    ids = _ids(g, n, k, 16)
    x = rand_bf16(g, n, h)
    counts_o, cu_o, pos_o = op_.dispatch_ragged(ids.numpy(), 0, el, 16)
    rows = int(cu_o[-1])
    pos = torch.from_numpy(pos_o).to(dev)
    y = torch.zeros((rows, h), dtype=torch.uint8, device=dev)
    s = torch.zeros((rows, h // 128), dtype=torch.float32, device=dev)
    x_d = x.to(dev)                                   # keep every device tensor alive across the raw call
    check(lib().bgmoe_scatter_quant(ptr(x_d), ptr(pos), n, k, h, ptr(y), ptr(s), h // 128, 1, stream()))
    torch.cuda.synchronize()
    yq, sq = act_quant(x)
    assert np.array_equal(y.cpu().numpy(), op_.gather_rows(yq, pos_o, k, rows))
    assert np.array_equal(s.cpu().numpy(), op_.gather_rows(sq, pos_o, k, rows))


@pytest.mark.parametrize("h,mn_major", [(1024, False), (7168, True), (400 * 16, False), (144, True)])
def test_scatter_of_prequantised_rows_equals_scatter_quant(dev, h, mn_major):
    from batchgen_amd._lib import check, lib, ptr, stream
    g = torch.Generator().manual_seed(h)
    n, k, el = 70, 8, 32
    ids = _ids(g, n, k, 64, extra=[-1, 70])
    x = rand_bf16(g, n, h)
    counts_o, cu_o, pos_o = op_.dispatch_ragged(ids.numpy(), 0, el, 16)
    rows = int(cu_o[-1])
    pos = torch.from_numpy(pos_o).to(dev)
    kb = (h + 127) // 128
    yq, sq = act_quant(x)
    xq_d = torch.from_numpy(yq).to(dev)
    xs_d = torch.from_numpy(sq).to(dev)
    if mn_major:                                      # [kb, align4(n)] storage viewed as [n, kb]
        store = torch.zeros((kb, (n + 3) // 4 * 4), dtype=torch.float32, device=dev)
        store[:, :n] = xs_d.t()
        xs_d = store.t()[:n]
    y = torch.zeros((rows, h), dtype=torch.uint8, device=dev)
    s = torch.zeros((rows, kb), dtype=torch.float32, device=dev)
    check(lib().bgmoe_scatter_fp8_rows(ptr(xq_d), ptr(xs_d), xs_d.stride(0), xs_d.stride(1), ptr(pos), n, k, h,
                                       ptr(y), ptr(s), kb, 1, stream()))
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), op_.gather_rows(yq, pos_o, k, rows))
    assert np.array_equal(s.cpu().numpy(), op_.gather_rows(sq, pos_o, k, rows))


@pytest.mark.parametrize("n,k,h", [(1, 2, 256), (64, 4, 1024), (256, 8, 7168), (33, 8, 131), (17, 4, 2880)])
def test_reduce_weighted_scatter(dev, n, k, h):
    say("reduce", n, k, h)
    g = torch.Generator().manual_seed(n + k + h)
    rows = n * k + 5
    y = rand_bf16(g, rows, h)
    pos = torch.randperm(rows, generator=g)[: n * k].to(torch.int32)
    pos[torch.rand(n * k, generator=g) < 0.3] = -1
    if n > 1:
        pos.view(n, k)[1] = -1                                        # a token with no local expert
    w = torch.rand(n, k, generator=g)
    out = torch.full((n, h), 3.0, dtype=torch.bfloat16, device=dev)
    ds3d().reduce_weighted_scatter(y.to(dev), pos.to(dev), w.to(dev), n, h, k, out)
    ref = oc.reduce_weighted_scatter(y, pos.numpy(), w.numpy(), n, k)
    assert np.array_equal(out.float().cpu().numpy(), ref)
    if n > 1:
        assert torch.all(out[1] == 0)
    if n * k * h <= 70000:                                            # the literal loop evaluates every fma exactly
        assert np.array_equal(ref, oc.reduce_loop(y, pos.numpy(), w.numpy(), n, k))
    if h % 8 == 0:
        ids = torch.stack([torch.randperm(64, generator=g)[:k] for _ in range(n)]).to(torch.int32)
        out2 = torch.empty((n, h), dtype=torch.bfloat16, device=dev)
        ds3d().reduce_weighted_scatter_bf16_ordered(y.to(dev), pos.to(dev), ids.to(dev), w.to(dev), n, h, k, out2)
        ref2 = oc.reduce_weighted_scatter_bf16_ordered(y, pos.numpy(), ids.numpy(), w.numpy(), n, k)
        assert np.array_equal(out2.float().cpu().numpy(), ref2)


def test_reduce_fp32_k16_and_shared(dev):
    from batchgen_amd._lib import check, lib, ptr, stream
    g = torch.Generator().manual_seed(4)
    n, k, h = 40, 16, 3584
    rows = n * k
    y = rand_bf16(g, rows, h)
    pos = torch.randperm(rows, generator=g).to(torch.int32)
    pos[torch.rand(rows, generator=g) < 0.5] = -1
    w = torch.rand(n, k, generator=g)
    out = torch.empty((n, h), dtype=torch.float32, device=dev)
    ds3d().reduce_weighted_scatter_fp32(y.to(dev), pos.to(dev), w.to(dev), n, h, k, out)
    ref = oc.reduce_weighted_scatter_fp32(y, pos.numpy(), w.numpy(), n, k)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref.view(np.uint32))
    sh = rand_bf16(g, n, h)
    y_d, pos_d, w_d, sh_d = y.to(dev), pos.to(dev), w.to(dev), sh.to(dev)   # alive across the raw calls
    for mode, name in ((0, "bf16_add"), (1, "fp32_add")):
        ob = torch.empty((n, h), dtype=torch.bfloat16, device=dev)
        check(lib().bgmoe_reduce_weighted_scatter(ptr(y_d), ptr(pos_d), ptr(w_d), n, h, k,
                                                  ptr(ob), -1, ptr(sh_d), mode, stream()))
        refb = oc.reduce_weighted_scatter(y, pos.numpy(), w.numpy(), n, k, shared=sh, shared_mode=name)
        assert np.array_equal(ob.float().cpu().numpy(), refb)


def test_compact_expert_data(dev):
    from batchgen_amd.kernels import load_extension
    m = load_extension("batchgen_kernels.common._C_mgn_ops")
    counts = torch.tensor([0, 3, 0, 0, 5, 1] + [0] * 70 + [2], dtype=torch.int32)
    size, idx, start, num = m.compact_expert_data(counts.to(dev))
    nz = torch.nonzero(counts).view(-1)
    na = int(num.item())
    assert na == len(nz)
    assert idx[:na].cpu().tolist() == nz.tolist()
    assert size[:na].cpu().tolist() == counts[nz].tolist()
    assert start[:na].cpu().tolist() == (torch.cumsum(counts[nz], 0) - counts[nz]).tolist()


def test_legacy_combine_helpers(dev):
    """`moe_weighted_sum_*` (dense [T, K, H]) and `scatter_weight_reduce_optimized` (sparse rows + inverse mapping)
    against the fp32 fma chain in ascending k: bit-exact (the same arithmetic as reduce_weighted_scatter)."""
    from oracle.norm_quant import fma_f32
    from batchgen_amd.moe import combine_variants as cv
    g = torch.Generator().manual_seed(21)
    t, k, h = 37, 8, 520
    res3 = (torch.randn(t, k, h, generator=g)).to(torch.bfloat16)
    w = torch.rand(t, k, generator=g)
    want = torch.from_numpy(sum_k(res3, w)).to(torch.bfloat16)
    for fn in (cv.moe_weighted_sum_triton, cv.moe_weighted_sum_triton_v2, cv.moe_weighted_sum_v3):
        got = fn(res3.to(dev), w.to(dev))
        assert got.dtype == torch.bfloat16 and torch.equal(got.cpu(), want)
    assert torch.equal(cv.moe_weighted_sum_v3(res3.to(dev), w.to(torch.bfloat16).to(dev)).cpu(),
                       torch.from_numpy(sum_k(res3, w.to(torch.bfloat16).float())).to(torch.bfloat16))
    # sparse form: only some (token, slot) pairs have a row, in a shuffled order, buffers oversized
    keep = torch.rand(t, k, generator=g) < 0.6
    tok, slot = torch.nonzero(keep, as_tuple=True)
    order = torch.randperm(tok.numel(), generator=g)
    tok, slot = tok[order], slot[order]
    rows = res3[tok, slot]
    pad = torch.zeros(50, dtype=torch.int64)
    out = cv.scatter_weight_reduce_optimized(rows.to(dev), torch.cat([tok, pad]).to(dev), torch.cat([slot, pad]).to(dev),
                                             w.to(dev), t, k)
    acc = np.zeros((t, h), dtype=np.float32)
    for j in range(k):
        x = res3[:, j].float().numpy()
        acc = np.where(keep[:, j:j + 1].numpy(), fma_f32(x, np.broadcast_to(w[:, j:j + 1].numpy(), x.shape), acc), acc)
    assert out.dtype == torch.float32 and np.array_equal(out.cpu().numpy(), acc)
    m = cv.build_inverse_mapping(tok.to(dev), slot.to(dev), t, k).cpu()
    assert m.dtype == torch.int64 and (m >= 0).sum() == tok.numel() and torch.equal(m[tok, slot], torch.arange(tok.numel()))
    assert cv.scatter_weight_reduce_optimized(rows[:0].to(dev), tok.to(dev), slot.to(dev), w.to(dev), t, k).abs().sum() == 0
    with pytest.raises(ValueError):
        cv.moe_weighted_sum_triton(res3.to(dev), w[:, :4].to(dev))
    # expert-sorted rows + the sorting permutation (the prefill path's combine)
    ids = torch.randint(0, 16, (t * k,), generator=g)
    idxs = ids.argsort(stable=True)
    sorted_rows = res3.view(t * k, h)[idxs]
    got = cv.moe_fp32_accum_triton_v2(sorted_rows.to(dev), idxs.to(dev), w.to(dev))
    assert got.dtype == torch.bfloat16 and torch.equal(got.cpu(), want)


def sum_k(res3, w):
    from oracle.norm_quant import fma_f32
    acc = np.zeros((res3.shape[0], res3.shape[2]), dtype=np.float32)
    for j in range(res3.shape[1]):
        x = res3[:, j].float().numpy()
        acc = fma_f32(x, np.broadcast_to(w[:, j:j + 1].numpy(), x.shape), acc)
    return acc
