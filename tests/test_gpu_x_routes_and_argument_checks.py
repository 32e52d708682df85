"""Op-entry argument checks and routes handed in from outside, on the GPU: wrong dtypes and short tensors raise
before a launch; a group fed by repeated expert ids may hold more rows than there are tokens."""
import numpy as np
import pytest
import torch

from tests.util import say

pytestmark = pytest.mark.gpu


def ds3d():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_dispatch_scatter_3d")


def test_given_routes_may_repeat_an_expert(dev):
    """Routes from outside may name one expert several times in a token's row: a group can then hold more rows
    than there are tokens (here 4 x 96 = 384 rows of one expert, more than the streaming kernel's 256-row limit),
    and every row must still be computed: against the oracle on the same routes."""
    from batchgen_amd import workloads as wl
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    from oracle import gemm as og
    from oracle import layer as ol
    cfg = wl.scaled(wl.CONFIGS[0], n_tokens=96, hidden=512, inter=256, shared_inter=256, n_experts=32, e_local=8,
                    expert_start=8, n_group=4, topk_group=2, top_k=4, max_tokens=0, layout="ragged", row_align=64)
    say("given routes with repeats", cfg.name)
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    layer = Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()},
                        inp["bias"].to(dev))
    x = inp["x"].to(dev)
    layer(x, inp["logits"].to(dev))                                   # leaves other values in the row buffers
    rid = torch.full((cfg.n_tokens, cfg.top_k), 9, dtype=torch.int32)
    rid[7, 2] = 11
    rw = torch.rand(cfg.n_tokens, cfg.top_k, generator=torch.Generator().manual_seed(9)) + 0.25
    got = layer.forward_routed(x, rid.to(dev), rw.to(dev)).float().cpu().numpy()
    ref = ol.moe_layer_fp8(inp["x"], None, None, None, wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local,
                           layout=cfg.layout, max_tokens=cfg.max_tokens, row_align=cfg.row_align, shared=wl.weights_to_numpy(sh),
                           routes=(rid.numpy(), rw.numpy()))
    assert np.array_equal(layer.expert_counts[:cfg.e_local].cpu().numpy(), ref["counts"])
    assert int(ref["counts"].max()) == 383
    assert np.array_equal(layer.topk_pos.cpu().numpy(), ref["pos"])
    assert og.rel_frobenius(got, ref["out"]) < 1e-2


@pytest.mark.parametrize("n,k,et,es,el,mtp", [(10, 2, 2, 0, 2, 4), (300, 8, 64, 8, 16, 7), (2000, 8, 64, 0, 64, 100),
                                              (40, 4, 600, 100, 300, 1)])
def test_dispatch_masked_overflow_rows_are_dropped(dev, n, k, et, es, el, mtp):
    """More arrivals than max_tokens_padded: the extra pairs get pos -1, the count is clipped and
    expert_counters holds the arrivals before clipping (the overflow signal), all as the oracle says; the three
    sizes take the one-block, the multi-chunk and the four-wave index kernels."""
    from oracle import permute as op_
    say("dispatch_3d overflow", n, k, et, es, el, mtp)
    g = torch.Generator().manual_seed(n + mtp)
    ids = torch.randint(0, et, (n, k), generator=g).to(torch.int32)
    if n == 10:
        ids[:, 0], ids[:, 1] = 0, 1
    x = torch.randn((n, 64), generator=g).to(torch.bfloat16)
    act = torch.zeros((el * mtp, 64), dtype=torch.bfloat16, device=dev)
    counts = torch.full((el,), -3, dtype=torch.int32, device=dev)
    counters = torch.full((el,), -3, dtype=torch.int32, device=dev)
    pos = torch.full((n * k,), -9, dtype=torch.int32, device=dev)
    ds3d().dispatch_scatter_3d(x.to(dev), ids.to(dev), act, es, el, mtp, counts, counters, pos)
    co, po, arrivals = op_.dispatch_masked_arrivals(ids.numpy(), es, el, mtp)
    assert int(arrivals.max()) > mtp, "the case must overflow"
    assert np.array_equal(counts.cpu().numpy(), co)
    assert np.array_equal(pos.cpu().numpy(), po)
    assert np.array_equal(counters.cpu().numpy(), arrivals)
    ref = op_.gather_rows(x.view(torch.int16).numpy(), po, k, el * mtp)
    assert np.array_equal(act.view(torch.int16).cpu().numpy(), ref)


@pytest.mark.parametrize("mod", ["ds3d", "routing", "ds3d_compiled", "routing_compiled"])
def test_combine_and_dispatch_reject_wrong_arguments(dev, mod):
    """Wrong dtypes and short tensors raise before anything is launched (no raw pointer of the wrong type or
    size reaches the kernel): the ctypes modules and the compiled extension modules, same table."""
    from batchgen_amd.kernels import load_extension
    name = "batchgen_kernels.moe._C_dispatch_scatter_3d" if mod.startswith("ds3d") else "batchgen_kernels.moe._C_routing"
    if mod.endswith("_compiled"):
        if dev.type != "cuda":
            pytest.skip("the compiled extension takes CUDA tensors only (rehearsal on the CPU emulator)")
        from tests.test_torch_extension_modules import load
        m = load(name)
    else:
        m = load_extension(name)
    n, k, h = 8, 4, 256
    y = torch.zeros((n * k, h), dtype=torch.bfloat16, device=dev)
    pos = torch.arange(n * k, dtype=torch.int32, device=dev)
    w = torch.ones((n, k), dtype=torch.float32, device=dev)
    out = torch.zeros((n, h), dtype=torch.bfloat16, device=dev)
    m.reduce_weighted_scatter(y, pos, w, n, h, k, out)                                    # the good call
    for bad in (dict(w=w.bfloat16()), dict(pos=pos.long()), dict(pos=pos[:-1]), dict(w=w[:, :-1].contiguous()),
                dict(out=out[:-1]), dict(out=out.float()), dict(y=y.float()), dict(y=y.view(n * k * 2, h // 2))) + \
            ((dict(w=w.cpu()),) if dev.type == "cuda" else ()):       # (one device only when rehearsed on the emulator)
        a = dict(y=y, pos=pos, w=w, out=out)
        a.update(bad)
        with pytest.raises(RuntimeError):
            m.reduce_weighted_scatter(a["y"], a["pos"], a["w"], n, h, k, a["out"])
    if mod.startswith("ds3d"):
        x = torch.zeros((n, h), dtype=torch.bfloat16, device=dev)
        ids = torch.zeros((n, k), dtype=torch.int32, device=dev)
        act = torch.zeros((2 * 16, h), dtype=torch.bfloat16, device=dev)
        cnt = torch.zeros(2, dtype=torch.int32, device=dev)
        ctr = torch.zeros(2, dtype=torch.int32, device=dev)
        tp = torch.zeros(n * k, dtype=torch.int32, device=dev)
        m.dispatch_scatter_3d(x, ids, act, 0, 2, 16, cnt, ctr, tp)                        # the good call
        for bad in (dict(cnt=cnt[:1]), dict(ctr=ctr[:1]), dict(tp=tp[:-1]), dict(ids=ids[:-1]), dict(ids=ids.view(-1)),
                    dict(act=act[:-1])):
            a = dict(ids=ids, act=act, cnt=cnt, ctr=ctr, tp=tp)
            a.update(bad)
            with pytest.raises(RuntimeError):
                m.dispatch_scatter_3d(x, a["ids"], a["act"], 0, 2, 16, a["cnt"], a["ctr"], a["tp"])
