"""The MXFP4 layer with the row gather folded into stage 1 (``Mxfp4MoELayer(fold_gather=True)``): the dispatch
computes indices only (``bgmoe_dispatch_index_3d``: counts, positions and the row -> pair map), and
``bgmoe_mxfp4_fused_s1_gather`` reads every row from its token through the map.  Same rows, same arithmetic: all
results must equal the gathered form's bit for bit; the index entry must equal the masked dispatch's indices and the
oracle's (``oracle.permute``).

Neither entry point has run on a GPU yet, so this file carries a name pytest does not collect.  Run it by naming
the file (`python -m pytest tests/wip_gpu_mxfp4_fold_gather.py -m gpu`); once green it becomes
tests/test_gpu_y_mxfp4_fold_gather.py."""
import ctypes as C

import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from oracle import permute as op
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,k,e_total,start,el,mtp", [
    (96, 8, 64, 16, 8, 96), (512, 16, 384, 96, 12, 512), (7, 2, 8, 4, 4, 8),
    (300, 4, 16, 0, 16, 40),            # groups overflow: dropped pairs have no row
    (4096, 8, 64, 0, 64, 640),          # more pairs than one block ranks: histogram / scan / rank launches
    (64, 8, 512, 0, 512, 8),            # more local experts than the one-block kernel takes
])
def test_index_only_dispatch_and_its_inverse_map(dev, n, k, e_total, start, el, mtp):
    from batchgen_amd._lib import check, lib, ptr, stream
    say("dispatch_index_3d", n, k, e_total, start, el, mtp)
    rng = np.random.default_rng(n + k)
    ids = np.stack([rng.permutation(e_total)[:k] for _ in range(n)]).astype(np.int32)
    ids_d = torch.from_numpy(ids).to(dev)
    ws = torch.empty(max(int(lib().bgmoe_dispatch_workspace_bytes(n * k, el)), 16), dtype=torch.uint8, device=dev)
    counts = torch.zeros(el, dtype=torch.int32, device=dev)
    counters = torch.zeros(el, dtype=torch.int32, device=dev)
    pos = torch.full((n * k,), -7, dtype=torch.int32, device=dev)
    row_pair = torch.full((el * mtp,), -5, dtype=torch.int32, device=dev)
    check(lib().bgmoe_dispatch_index_3d(ptr(ids_d), n, k, start, el, mtp, ptr(counts), ptr(counters), ptr(pos),
                                        ptr(row_pair), ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    want_counts, want_pos, arrivals = op.dispatch_masked_arrivals(ids, start, el, mtp)
    assert np.array_equal(counts.cpu().numpy(), want_counts)
    assert np.array_equal(counters.cpu().numpy(), arrivals)
    assert np.array_equal(pos.cpu().numpy(), want_pos.reshape(-1))
    rp = row_pair.cpu().numpy()
    want_rp = np.full(el * mtp, -5, dtype=np.int32)                 # rows without a pair keep what they held
    placed = np.nonzero(want_pos.reshape(-1) >= 0)[0]
    want_rp[want_pos.reshape(-1)[placed]] = placed
    assert np.array_equal(rp, want_rp)


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
def test_stage1_through_the_map_equals_stage1_on_gathered_rows(dev, layout):
    from batchgen_amd._lib import Mxfp4Weight, check, lib, ptr, stream
    from batchgen_amd.kernels import load_extension
    from oracle import mxfp4 as mx
    mg = load_extension("batchgen_kernels.moe._C_marlin_grouped_gemm")
    n, k, el, mtp, h, inter = 200, 4, 6, 64, 512, 256
    rng = np.random.default_rng(9)
    ids = np.stack([rng.permutation(el + 2)[:k] for _ in range(n)]).astype(np.int32)    # some pairs go elsewhere
    gen = torch.Generator().manual_seed(3)
    x = rand_bf16(gen, n, h).to(dev)
    wts = []
    for seed in (1, 2):
        p, s = mx.quantize((0.02 * np.random.default_rng(seed).standard_normal((el, inter, h))).astype(np.float32))
        p, s = torch.from_numpy(p).to(dev), torch.from_numpy(s).to(dev)
        if layout == "tile_major":
            p, s = mg.mxfp4_weight_repack(p, s)
        wts.append((p, s))
    lay = 1 if layout == "tile_major" else 0
    desc = [Mxfp4Weight(ptr(p), p.size(1) * p.size(2), None, ptr(s), s.size(1) * s.size(2), None, lay, 0) for p, s in wts]
    ids_d = torch.from_numpy(ids).to(dev)
    ws = torch.empty(max(int(lib().bgmoe_dispatch_workspace_bytes(n * k, el)), 16), dtype=torch.uint8, device=dev)
    counts = torch.zeros(el, dtype=torch.int32, device=dev)
    counters = torch.zeros(el, dtype=torch.int32, device=dev)
    pos = torch.zeros(n * k, dtype=torch.int32, device=dev)
    cu = (torch.arange(el + 1, dtype=torch.int32, device=dev) * mtp).contiguous()
    rows = el * mtp
    act = torch.zeros((rows, h), dtype=torch.bfloat16, device=dev)
    check(lib().bgmoe_dispatch_scatter_3d(ptr(x), ptr(ids_d), n, k, h, ptr(act), 0, el, mtp, ptr(counts), ptr(counters),
                                          ptr(pos), ptr(ws), ws.numel(), stream()))
    want = torch.full((rows, inter), 3.0, dtype=torch.bfloat16, device=dev)
    check(lib().bgmoe_mxfp4_fused_s1(ptr(act), C.byref(desc[0]), C.byref(desc[1]), ptr(counts), ptr(cu), el, rows, inter, h,
                                     ptr(want), None, 0, n * k, stream()))
    row_pair = torch.full((rows,), 2 ** 30, dtype=torch.int32, device=dev)     # unplaced rows: an index far outside
    counts2 = torch.zeros_like(counts)
    check(lib().bgmoe_dispatch_index_3d(ptr(ids_d), n, k, 0, el, mtp, ptr(counts2), ptr(counters), ptr(pos),
                                        ptr(row_pair), ptr(ws), ws.numel(), stream()))
    got = torch.full((rows, inter), 3.0, dtype=torch.bfloat16, device=dev)
    check(lib().bgmoe_mxfp4_fused_s1_gather(ptr(x), n, ptr(row_pair), k, C.byref(desc[0]), C.byref(desc[1]), ptr(counts2),
                                            ptr(cu), el, rows, inter, h, ptr(got), None, 0, n * k, stream()))
    torch.cuda.synchronize()
    assert torch.equal(counts, counts2) and int(counts.max()) == mtp, "the case is meant to fill a group to its limit"
    assert torch.equal(got, want), "rows read through the map give other bits than the gathered rows"
    # argument checks of the new entry points
    assert lib().bgmoe_mxfp4_fused_s1_gather(ptr(x), n, None, k, C.byref(desc[0]), C.byref(desc[1]), ptr(counts2), ptr(cu),
                                             el, rows, inter, h, ptr(got), None, 0, n * k, stream()) != 0
    assert b"row_pair" in lib().bgmoe_last_error()
    assert lib().bgmoe_mxfp4_fused_s1_gather(ptr(x), n, ptr(row_pair), 0, C.byref(desc[0]), C.byref(desc[1]), ptr(counts2),
                                             ptr(cu), el, rows, inter, h, ptr(got), None, 0, n * k, stream()) != 0
    assert lib().bgmoe_dispatch_index_3d(ptr(ids_d), n, k, 0, el, mtp, ptr(counts2), ptr(counters), ptr(pos), None,
                                         ptr(ws), ws.numel(), stream()) != 0


@pytest.mark.parametrize("which", ["config3_small", "k3_latent_small"])
def test_layer_with_folded_gather_equals_the_gathered_layer(dev, which):
    from batchgen_amd.moe.mxfp4_layer import Mxfp4MoELayer
    if which == "config3_small":
        cfg = wl.scaled(wl.CONFIGS[3], n_tokens=96, hidden=512, inter=256, shared_inter=256, n_experts=224, e_local=28,
                        expert_start=56, max_tokens=96)
    else:
        cfg = wl.scaled(wl.K3_LATENT, n_tokens=96, hidden=512, latent=256, inter=384, shared_inter=384, n_experts=224,
                        e_local=28, expert_start=56, max_tokens=96)
    say("fold_gather", cfg.name, which)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_mxfp4_weights(cfg, dev)
    lat = wl.make_latent_weights(cfg, dev) if cfg.latent else None
    plain = Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat)
    folded = Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat, fold_gather=True)
    a = plain(inp["x"], inp["logits"]).clone()
    b = folded(inp["x"], inp["logits"]).clone()
    assert torch.equal(plain.topk_pos, folded.topk_pos) and torch.equal(plain.expert_counts, folded.expert_counts)
    assert torch.equal(a, b)
    # a second step with fewer tokens: stale map entries of the first step lie in rows no group reaches now
    m = cfg.n_tokens // 3
    a2 = plain(inp["x"][:m].contiguous(), inp["logits"][:m].contiguous()).clone()
    b2 = folded(inp["x"][:m].contiguous(), inp["logits"][:m].contiguous()).clone()
    assert torch.equal(a2, b2)
