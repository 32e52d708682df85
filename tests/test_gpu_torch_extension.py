"""The PyTorch C++ extension modules on the GPU: every op called by its reference module name gives the same bits
as the same op through the ctypes mirror (both are argument marshalling over the one C ABI), and the router and
the quantiser are checked against the CPU oracle as well."""
import numpy as np
import pytest
import torch

from oracle import router as orr
from tests.test_torch_extension_modules import load
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def mirror(name):
    from batchgen_amd.kernels import load_extension
    return load_extension(name)


def test_routing_module(dev):
    ext, py = load("batchgen_kernels.moe._C_routing"), mirror("batchgen_kernels.moe._C_routing")
    g = torch.Generator().manual_seed(1)
    n, e, k = 97, 256, 8
    logits = torch.randn(n, e, generator=g)
    bias = torch.randn(e, generator=g) * 0.1
    ids, w = ext.gate_sigmoid_topk(logits.to(dev), bias.to(dev), k, 2.5, torch.empty(0, device=dev), torch.empty(0, device=dev))
    ids_o, w_o = orr.gate_sigmoid_topk(logits.numpy(), bias.numpy(), k, 2.5)
    assert np.array_equal(ids.cpu().numpy(), ids_o) and np.array_equal(w.cpu().numpy(), w_o)
    ids64 = torch.empty((n, k), dtype=torch.int64, device=dev)
    w2 = torch.empty((n, k), device=dev)
    ext.gate_sigmoid_topk_warp(logits.to(dev), bias.to(dev), k, 2.5, ids64, w2, num_valid_tokens=None)
    assert torch.equal(ids64.int(), ids) and torch.equal(w2, w)
    h = 1024
    hid, wt = rand_bf16(g, n, h).to(dev), (torch.randn(e, h, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    a = ext.glm5_router_gemm(hid, wt, None, None, 0, 1)
    b = py.glm5_router_gemm(hid, wt, None, None, 0, 1)
    assert torch.equal(a, b)
    # tight dispatch + combine
    x = rand_bf16(g, n, 256).to(dev)
    ids_l = ids.clone()
    outs = []
    for m in (ext, py):
        counts, offs, ctr = (torch.empty(32, dtype=torch.int32, device=dev), torch.empty(33, dtype=torch.int32, device=dev),
                             torch.empty(32, dtype=torch.int32, device=dev))
        disp = torch.zeros((n * k, 256), dtype=torch.bfloat16, device=dev)
        pos = torch.empty(n * k, dtype=torch.int32, device=dev)
        m.dispatch_count_gather(x, ids_l, 64, 32, counts, offs, ctr, disp, pos)
        out = m.reduce_weighted_scatter(disp, pos, w, n, 256, k, torch.empty(0, device=dev))
        outs.append((counts, offs, pos, disp, out))
    for s, t in zip(*outs):
        assert torch.equal(s, t)


def test_mgn_module(dev):
    ext, py = load("batchgen_kernels.common._C_mgn_ops"), mirror("batchgen_kernels.common._C_mgn_ops")
    g = torch.Generator().manual_seed(2)
    n, e, k = 64, 256, 8
    scores = torch.sigmoid(torch.randn(n, e, generator=g)).to(dev)
    bias = (torch.randn(e, generator=g) * 0.1).to(dev)
    a = ext.moe_fused_gate(scores, bias, 8, 4, e, k, 2.5)
    b = py.moe_fused_gate(scores, bias, 8, 4, e, k, 2.5)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    x = rand_bf16(g, n, 512).to(dev)
    fa = ext.fused_moe_token_dispatch(x, a[0], torch.empty(0, device=dev), torch.empty(0, device=dev), 32, 64)
    fb = py.fused_moe_token_dispatch(x, a[0], None, None, 32, 64)
    total = int(fb[5][-1])
    assert torch.equal(fa[0][:total], fb[0][:total])
    for i in (1, 2, 3, 4, 5):
        assert torch.equal(fa[i], fb[i])
    eids = a[0].reshape(-1).contiguous()
    ba = ext.expert_bincount(eids, 32, 32, torch.device(dev))
    bb = py.expert_bincount(eids, 32, 32, torch.device(dev))
    nb = int(bb[3].item())
    assert int(ba[3].item()) == nb
    for i in range(3):
        assert torch.equal(ba[i][:nb], bb[i][:nb])
    ca = ext.compact_expert_data(fb[4])
    cb = py.compact_expert_data(fb[4])
    na = int(cb[3].item())
    assert int(ca[3].item()) == na
    for i in range(3):
        assert torch.equal(ca[i][:na], cb[i][:na])


def test_dispatch_scatter_module(dev):
    ext, py = load("batchgen_kernels.moe._C_dispatch_scatter_3d"), mirror("batchgen_kernels.moe._C_dispatch_scatter_3d")
    g = torch.Generator().manual_seed(3)
    n, k, h, el, es, mtp = 300, 8, 256, 32, 64, 128
    ids = torch.stack([torch.randperm(256, generator=g)[:k] for _ in range(n)]).to(torch.int32).to(dev)
    x = rand_bf16(g, n, h).to(dev)
    w = torch.rand(n, k, generator=g).to(dev)
    res = []
    for m in (ext, py):
        act = torch.zeros((el * mtp, h), dtype=torch.bfloat16, device=dev)
        counts, ctr = torch.empty(el, dtype=torch.int32, device=dev), torch.empty(el, dtype=torch.int32, device=dev)
        pos = torch.empty(n * k, dtype=torch.int32, device=dev)
        m.dispatch_scatter_3d(x, ids, act, es, el, mtp, counts, ctr, pos)
        out = m.reduce_weighted_scatter(act, pos, w, n, h, k, torch.empty(0, device=dev))
        ordered = torch.empty((n, h), dtype=torch.bfloat16, device=dev)
        m.reduce_weighted_scatter_bf16_ordered(act, pos, ids, w, n, h, k, ordered)
        cap = (n * k + 63 * el) // 64 * 64
        ract = torch.zeros((cap, h), dtype=torch.bfloat16, device=dev)
        rcounts, rctr = torch.empty(el, dtype=torch.int32, device=dev), torch.empty(el, dtype=torch.int32, device=dev)
        rpos, cu = torch.empty(n * k, dtype=torch.int32, device=dev), torch.empty(el + 1, dtype=torch.int32, device=dev)
        m.dispatch_scatter_ragged(x, ids, ract, es, el, rcounts, rctr, rpos, cu, 64)
        res.append((act, counts, pos, out, ordered, ract, rcounts, rpos, cu))
    for s, t in zip(*res):
        assert torch.equal(s, t)
    with pytest.raises(RuntimeError):
        ext.dispatch_scatter_ragged(x, ids, res[0][5], es, el, res[0][6], res[0][6], res[0][7], res[0][8], 48)


def test_fp8_modules(dev):
    gx, gp = load("batchgen_kernels.moe._C_fp8_blockwise_gemm"), mirror("batchgen_kernels.moe._C_fp8_blockwise_gemm")
    ox, op = load("batchgen_kernels.moe._C_fp8_blockwise_ops"), mirror("batchgen_kernels.moe._C_fp8_blockwise_ops")
    from batchgen_amd import workloads as wl
    g = torch.Generator(device=dev).manual_seed(4)
    groups, n, k, cap = 4, 256, 512, 64
    wq, ws = wl._gen_fp8_stack(g, groups, n, k, dev)
    uq, us = wl._gen_fp8_stack(g, groups, n, k, dev)
    pad = lambda s: torch.nn.functional.pad(s, (0, (-s.size(2)) % 4)).contiguous()
    ws, us = pad(ws), pad(us)
    m = groups * cap
    xb = (torch.randn(m, k, generator=g, device=dev)).to(torch.bfloat16)
    cnt = torch.tensor([9, 0, 64, 33], dtype=torch.int32, device=dev)
    cu = torch.arange(groups + 1, dtype=torch.int32, device=dev) * cap
    res = []
    for q, o in ((ox, gx), (op, gp)):
        y = torch.zeros((m, k), dtype=torch.uint8, device=dev)
        s = torch.zeros((k // 128, m), device=dev)
        q.act_quant_ragged(xb, cnt, cu, y, s, 1)
        out = o.fp8_blockwise_grouped_gemm(y.view(torch.float8_e4m3fn), wq, cnt, cu, s, ws, 16)
        h = o.fp8_blockwise_fused_s1(y.view(torch.float8_e4m3fn), wq, uq, cnt, cu, s, ws, us, 16,
                                     output=torch.zeros((m, n), dtype=torch.bfloat16, device=dev))
        x3 = xb.view(groups, cap, k)
        y3, s3 = q.act_quant_3d(x3, cnt)
        sm = q.silu_mul_3d(x3, x3.flip(1).contiguous(), cnt)
        fq, fs = q.fused_silu_quant_3d(x3, x3.flip(1).contiguous(), cnt)
        res.append((y, s, out, h, sm, fq, fs))
    live = torch.zeros(m, dtype=torch.bool, device=dev)
    for gi, c in enumerate(cnt.tolist()):
        live[gi * cap: gi * cap + c] = True
    for i, (s, t) in enumerate(zip(*res)):
        if i in (2, 3):
            assert torch.equal(s[live], t[live]), i            # rows outside the groups are whatever `empty` held
        elif i in (4, 5, 6):
            assert torch.equal(s.reshape(m, -1)[live], t.reshape(m, -1)[live]), i
        else:
            assert torch.equal(s, t), i


def test_add_rmsnorm_module(dev):
    ext = load("batchgen_kernels.attention._C_add_rmsnorm_fp8_quant")
    py = mirror("batchgen_kernels.attention._C_add_rmsnorm_fp8_quant")
    g = torch.Generator().manual_seed(5)
    rows, h = 37, 1024
    res0, hid, wt = rand_bf16(g, rows, h), rand_bf16(g, rows, h), rand_bf16(g, h)
    a = ext.add_rmsnorm_fp8_quant_forward(res0.clone().to(dev), hid.to(dev), wt.to(dev), 1e-6, scale_tma_aligned=True)
    b = py.add_rmsnorm_fp8_quant_forward(res0.clone().to(dev), hid.to(dev), wt.to(dev), 1e-6, scale_tma_aligned=True)
    assert a[3].stride() == b[3].stride()
    for s, t in zip(a, b):
        assert torch.equal(s.view(torch.uint8) if s.dtype == torch.float8_e4m3fn else s,
                           t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t)
    say("extension modules: add_rmsnorm ok")
