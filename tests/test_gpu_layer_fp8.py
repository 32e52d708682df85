"""Whole FP8 MoE layer on the GPU vs the CPU oracle.

Integer / byte results (router ids, counts, cu_seqlens, topk_pos, quantised activation bytes and scales) are
bit-exact; the layer output is within 1e-2 relative Frobenius error of the fp32 dequantise-then-matmul oracle
(the bound the benchmark definition states), in practice ~1e-3.
"""
import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from oracle import gemm as og
from oracle import layer as ol
from tests.util import say

pytestmark = pytest.mark.gpu

SMALL = {
    "c0": wl.CONFIGS[0],
    "c1_small": wl.scaled(wl.CONFIGS[1], hidden=1024, inter=512, shared_inter=512),
    "c1_unfolded_shared": wl.scaled(wl.CONFIGS[1], hidden=512, inter=512, shared_inter=256, n_tokens=100),
    "c2_small": wl.scaled(wl.CONFIGS[2], hidden=512, inter=256, shared_inter=256, n_tokens=3000),
    "c4_small": wl.scaled(wl.CONFIGS[4], hidden=256, inter=256, shared_inter=256, n_tokens=2048),
    "ungrouped_fp8": wl.scaled(wl.CONFIGS[1], hidden=512, inter=256, shared_inter=0, n_group=1, topk_group=1,
                               n_experts=384, e_local=48, expert_start=96, n_tokens=77, max_tokens=128),
}


def _rcfg(cfg):
    return dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf)


@pytest.mark.parametrize("name", list(SMALL))
def test_layer_matches_oracle(dev, name):
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = SMALL[name]
    say("layer", name)
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    wd = {k: v.to(dev) for k, v in w.items()}
    shd = {k: v.to(dev) for k, v in sh.items()} if sh else None
    layer = Fp8MoELayer(cfg, wd, shd, inp["bias"].to(dev))
    out = layer(inp["x"].to(dev), inp["logits"].to(dev))
    torch.cuda.synchronize()
    ref = ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(), _rcfg(cfg),
                           wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local, layout=cfg.layout,
                           max_tokens=cfg.max_tokens, row_align=cfg.row_align, shared=wl.weights_to_numpy(sh))
    el = cfg.e_local
    assert np.array_equal(layer.topk_ids.cpu().numpy(), ref["ids"])
    np.testing.assert_allclose(layer.topk_weights.cpu().numpy(), ref["weights"], rtol=2e-7, atol=0)
    assert np.array_equal(layer.expert_counts[:el].cpu().numpy(), ref["counts"])
    assert np.array_equal(layer.cu_seqlens[:el].cpu().numpy(), ref["cu"][:el])
    assert np.array_equal(layer.topk_pos.cpu().numpy(), ref["pos"])
    live = np.zeros(layer.cap_rows, dtype=bool)
    for e in range(el):
        live[ref["cu"][e]:ref["cu"][e] + ref["counts"][e]] = True
    xq = layer.xq[:layer.cap_rows].cpu().numpy()
    xs = layer.xs[:layer.cap_rows].cpu().numpy()
    nrows = ref["xq"].shape[0]
    assert np.array_equal(xq[:nrows][live[:nrows]], ref["xq"][live[:nrows]])
    assert np.array_equal(xs[:nrows][live[:nrows]].view(np.uint32), ref["xs"][live[:nrows]].view(np.uint32))
    if sh is not None:   # shared expert rows = quantised tokens
        assert np.array_equal(layer.xq[layer.cap_rows:].cpu().numpy(), ref["xq_tok"])
    err = og.rel_frobenius(out.float().cpu().numpy(), ref["out"])
    say("   rel frobenius vs fp32 oracle:", err)
    assert err < 1e-2
    # intermediate requant: bytes may differ where fp32 accumulation order moves a value across a rounding
    # boundary; they must agree almost everywhere
    hq = layer.hq[:nrows].cpu().numpy()[live[:nrows]]
    agree = (hq == ref["hq"][live[:nrows]]).mean() if hq.size else 1.0
    say("   requant byte agreement:", agree)
    assert agree > 0.97


def test_layer_is_deterministic_and_reusable(dev):
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = SMALL["c1_small"]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    layer = Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()},
                        inp["bias"].to(dev))
    x, lg = inp["x"].to(dev), inp["logits"].to(dev)
    a = layer(x, lg).clone()
    other = layer(x[:50].contiguous(), lg[:50].contiguous()).clone()      # fewer tokens, same buffers
    b = layer(x, lg).clone()
    assert torch.equal(a, b)
    assert torch.equal(other, a[:50])                                     # tokens are independent


def test_layer_rejects_bad_arguments(dev):
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = SMALL["c0"]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    layer = Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()},
                        inp["bias"].to(dev))
    with pytest.raises(RuntimeError):
        layer(inp["x"].to(dev).float(), inp["logits"].to(dev))
    with pytest.raises(RuntimeError):
        layer(torch.zeros((65, cfg.hidden), dtype=torch.bfloat16, device=dev),
              torch.zeros((65, cfg.n_experts), device=dev))


def test_config0_against_the_committed_golden_fixture(dev):
    """Same check from files only: tests/golden/c0_layer.npz (written by tests/golden/make_c0_golden.py)."""
    import os
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c0_layer.npz"))
    cfg = wl.CONFIGS[0]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    layer = Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()},
                        inp["bias"].to(dev))
    out = layer(inp["x"].to(dev), inp["logits"].to(dev))
    assert np.array_equal(layer.topk_ids.cpu().numpy(), gold["ids"])
    assert np.array_equal(layer.topk_pos.cpu().numpy(), gold["pos"])
    assert np.array_equal(layer.expert_counts[:cfg.e_local].cpu().numpy(), gold["counts"])
    assert np.array_equal(layer.xs[layer.cap_rows:].cpu().numpy().view(np.uint32), gold["xs_tok"].view(np.uint32))
    assert og.rel_frobenius(out.float().cpu().numpy(), gold["out"]) < 1e-2


@pytest.mark.parametrize("layout", ["row_major", "tile_major"])
def test_weight_layouts_give_identical_layers(dev, layout):
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = SMALL["c1_small"]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    mk = lambda lay: Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()},
                                 inp["bias"].to(dev), weight_layout=lay)
    a = mk("row_major")(inp["x"].to(dev), inp["logits"].to(dev)).clone()
    b = mk(layout)(inp["x"].to(dev), inp["logits"].to(dev)).clone()
    assert torch.equal(a, b)


def test_layer_forward_replays_from_a_hip_graph(dev):
    """One captured forward pass, replayed over changing inputs (the device-side counts change with them),
    with eager work and synchronisations between the replays: every replay equals the eager result bit for
    bit.  Launch geometry depends on host shapes only and the library allocates nothing, which is what makes
    the capture legal."""
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = wl.scaled(wl.CONFIGS[1], hidden=1024, inter=512, shared_inter=512)
    w, sh = wl.make_fp8_weights(cfg, dev)
    bias = wl.make_inputs(cfg, dev)["bias"]
    layer = Fp8MoELayer(cfg, w, sh, bias)
    gen = torch.Generator(device="cpu").manual_seed(7)
    xs = [torch.randn((cfg.n_tokens, cfg.hidden), generator=gen).to(torch.bfloat16).to(dev) for _ in range(3)]
    ls = [(torch.randn((cfg.n_tokens, cfg.n_experts), generator=gen) * (1.0 + i)).to(dev) for i in range(3)]
    eager = []
    for x, lg in zip(xs, ls):
        eager.append(layer(x, lg).clone())
    torch.cuda.synchronize()
    x_in, l_in = xs[0].clone(), ls[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer(x_in, l_in)                       # warm-up on the capture stream (first-launch attribute queries)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = layer(x_in, l_in)
    for rnd in range(2):
        for i in (2, 0, 1):
            x_in.copy_(xs[i])
            l_in.copy_(ls[i])
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_static, eager[i]), f"replay of input {i} (round {rnd}) differs from eager"
            scratch = layer(xs[(i + 1) % 3], ls[(i + 1) % 3])   # eager work between replays
            assert torch.equal(scratch, eager[(i + 1) % 3])


@pytest.mark.parametrize("name", ["c1_small", "c2_small", "ungrouped_fp8"])
def test_layer_fed_by_the_fused_producer_and_its_own_router_gemm(dev, name):
    """residual + hidden -> add + RMSNorm + FP8 cast -> (normed, x_fp8, x_scale) -> layer with router_weight.
    The same layer fed the bf16 `normed` and the logits of the standalone router GEMM gives the same bits:
    the producer's cast is the layer's own quantiser, and the fused router sums the same planes."""
    from batchgen_amd.attention import cuda_add_rmsnorm_fp8_quant
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    from batchgen_amd.moe.routing import glm5_router_gemm_cuda
    cfg = SMALL[name]
    g = torch.Generator().manual_seed(31)
    n, h = cfg.n_tokens, cfg.hidden
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    wd = {k: v.to(dev) for k, v in w.items()}
    shd = {k: v.to(dev) for k, v in sh.items()} if sh else None
    rw = (torch.randn(cfg.n_experts, h, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    residual = (torch.randn(n, h, generator=g) * 0.9).to(torch.bfloat16).to(dev)
    hidden = (torch.randn(n, h, generator=g) * 0.4).to(torch.bfloat16).to(dev)
    gamma = (torch.randn(h, generator=g) * 0.3 + 1.0).to(torch.bfloat16).to(dev)
    normed, _, x_fp8, x_scale = cuda_add_rmsnorm_fp8_quant(residual, hidden, gamma, 1e-5, scale_tma_aligned=True)
    layer = Fp8MoELayer(cfg, wd, shd, inp["bias"].to(dev), router_weight=rw)
    fused = layer(normed, None, x_fp8=x_fp8, x_scale=x_scale).clone()
    ids_f, xq_f = layer.topk_ids.clone(), layer.xq.clone()
    logits = glm5_router_gemm_cuda(normed, rw)
    plain = layer(normed, logits).clone()
    assert torch.equal(layer.topk_ids, ids_f)
    assert torch.equal(layer.xq, xq_f)
    assert torch.equal(fused, plain)
    with pytest.raises(RuntimeError, match="together"):
        layer(normed, logits, x_fp8=x_fp8)
    with pytest.raises(RuntimeError, match="router_weight"):
        Fp8MoELayer(cfg, wd, shd, inp["bias"].to(dev))(normed, None)


@pytest.mark.parametrize("weight_layout", ["tile_major", "row_major"])
@pytest.mark.parametrize("name,fold", [("c1_small", True), ("c1_unfolded_shared", False)])
def test_layer_built_from_a_checkpoint(dev, tmp_path, name, fold, weight_layout):
    """Per-expert checkpoint tensors (safetensors, HF names) -> loader (scale axis padded to 4, gate/up in one
    fused block) -> layer.  Same bits as the layer built from the original stacks."""
    from safetensors.torch import save_file
    from batchgen_amd.moe import weight_loader as wld
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = SMALL[name]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    g = torch.Generator().manual_seed(9)
    rw = (torch.randn(cfg.n_experts, cfg.hidden, generator=g) * 0.05).to(torch.bfloat16)
    prefix = "model.layers.5.mlp."
    ck = wld.export_fp8_moe_layer(prefix, {k: v.view(torch.uint8) if v.dtype != torch.float32 else v for k, v in w.items()},
                                  {k: v.view(torch.uint8) if v.dtype != torch.float32 else v for k, v in sh.items()},
                                  inp["bias"], rw, expert_start=cfg.expert_start)
    path = str(tmp_path / "layer.safetensors")
    save_file(ck, path)
    src = wld.SafetensorsSource(path)
    experts = wld.stack_fp8_experts(src, prefix, range(cfg.expert_start, cfg.expert_start + cfg.e_local), cfg.hidden,
                                    cfg.inter, dev, scale_pad4=True, fuse_gate_up=True)
    shared = wld.stack_fp8_experts(src, prefix, [0], cfg.hidden, cfg.shared_inter, dev, scale_pad4=fold,
                                   expert_fmt="shared_experts.")
    bias = src[prefix + "gate.e_score_correction_bias"].to(dev)
    a = Fp8MoELayer(cfg, experts, shared, bias, fold_shared=fold, weight_layout=weight_layout,
                    router_weight=src[prefix + "gate.weight"].to(dev))
    b = Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()},
                    inp["bias"].to(dev), fold_shared=fold, weight_layout=weight_layout, router_weight=rw.to(dev))
    assert a.folded == fold
    x = inp["x"].to(dev)
    assert torch.equal(a(x, None), b(x, None))
    assert torch.equal(a(x, inp["logits"].to(dev)), b(x, inp["logits"].to(dev)))


def test_producer_chain_replays_from_a_hip_graph(dev):
    """add + RMSNorm + FP8 cast -> layer (router GEMM + gate inside, pre-quantised tokens) captured as one graph
    and replayed over changing inputs, eager work in between: every replay equals the eager chain bit for bit."""
    from batchgen_amd._lib import check, lib, ptr, stream
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = wl.scaled(wl.CONFIGS[1], hidden=1024, inter=512, shared_inter=512)
    n, h = cfg.n_tokens, cfg.hidden
    w, sh = wl.make_fp8_weights(cfg, dev)
    bias = wl.make_inputs(cfg, dev)["bias"]
    gen = torch.Generator(device="cpu").manual_seed(11)
    rw = (torch.randn(cfg.n_experts, h, generator=gen) * 0.05).to(torch.bfloat16).to(dev)
    gamma = (torch.randn(h, generator=gen) * 0.3 + 1.0).to(torch.bfloat16).to(dev)
    layer = Fp8MoELayer(cfg, w, sh, bias, router_weight=rw)
    res = [(torch.randn(n, h, generator=gen) * (0.5 + i)).to(torch.bfloat16).to(dev) for i in range(3)]
    hid = [(torch.randn(n, h, generator=gen) * 0.4).to(torch.bfloat16).to(dev) for _ in range(3)]
    normed = torch.empty((n, h), dtype=torch.bfloat16, device=dev)
    xq = torch.empty((n, h), dtype=torch.uint8, device=dev)
    xs = torch.empty((n, h // 128), dtype=torch.float32, device=dev)
    r_in, h_in = res[0].clone(), hid[0].clone()

    def chain(r, hd):
        check(lib().bgmoe_add_rmsnorm_fp8_quant(ptr(r), ptr(hd), ptr(gamma), n, h, 1e-5, ptr(normed), ptr(xq),
                                                ptr(xs), h // 128, 1, None, None, None, stream()))
        return layer(normed, None, x_fp8=xq, x_scale=xs)

    eager = [chain(res[i].clone(), hid[i]).clone() for i in range(3)]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain(r_in.clone(), h_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = chain(r_in, h_in)
    for rnd in range(2):
        for i in (1, 2, 0):
            r_in.copy_(res[i])                   # the captured kernel updates the residual in place
            h_in.copy_(hid[i])
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out_static, eager[i]), f"replay of input {i} (round {rnd}) differs from eager"
            j = (i + 1) % 3
            assert torch.equal(chain(res[j].clone(), hid[j]), eager[j])      # eager work between replays


def test_layer_with_given_routes(dev):
    """`forward_routed`: the layer behind an external gate.  Routes taken from the layer's own router reproduce
    its output bit for bit; arbitrary routes (int64 ids, ids of other ranks, -1 padding, unnormalised weights)
    match the oracle run on the same routes."""
    from batchgen_amd import workloads as wl
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    from oracle import gemm as og
    from oracle import layer as ol
    cfg = wl.scaled(wl.CONFIGS[0], n_tokens=48, hidden=512, inter=256, shared_inter=256, n_experts=32, e_local=8,
                    expert_start=8, n_group=4, topk_group=2, top_k=4, max_tokens=48)
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    layer = Fp8MoELayer(cfg, {k: v.to(dev) for k, v in w.items()}, {k: v.to(dev) for k, v in sh.items()},
                        inp["bias"].to(dev))
    x = inp["x"].to(dev)
    out = layer(x, inp["logits"].to(dev)).clone()
    ids, wts = layer.topk_ids.clone(), layer.topk_weights.clone()
    assert torch.equal(layer.forward_routed(x, ids, wts), out)
    assert torch.equal(layer.forward_routed(x, ids.long(), wts), out)
    g = torch.Generator().manual_seed(4)
    rid = torch.stack([torch.randperm(cfg.n_experts, generator=g)[:cfg.top_k] for _ in range(cfg.n_tokens)])
    rid[5] = -1                                                        # a padding row
    rw = torch.rand(cfg.n_tokens, cfg.top_k, generator=g) * 2
    got = layer.forward_routed(x, rid.to(dev), rw.to(dev)).float().cpu().numpy()
    ref = ol.moe_layer_fp8(inp["x"], None, None, None, wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local,
                           layout=cfg.layout, max_tokens=cfg.max_tokens, shared=wl.weights_to_numpy(sh),
                           routes=(rid.numpy(), rw.numpy()))
    assert np.array_equal(layer.topk_pos.cpu().numpy(), ref["pos"])
    assert np.array_equal(layer.expert_counts[:cfg.e_local].cpu().numpy(), ref["counts"])
    assert og.rel_frobenius(got, ref["out"]) < 1e-2
    assert torch.equal(layer(x, inp["logits"].to(dev)), out)          # the routed call leaves the layer as it was
    with pytest.raises(RuntimeError):
        layer.forward_routed(x, rid[:, :2].to(dev), rw[:, :2].to(dev))
