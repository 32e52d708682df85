"""The dense FP8 expert chains (shared expert / dense MLP) and the exact 1-D quantiser behind them.  Restates the
contracts of the reference's tests/test_glm5_shared_expert_fused_gate_up.py (fused == unfused, eagerly and under
graph replay; pre-quantised input and caller buffer accepted by the fused chain only) and
tests/test_act_quant_1d_vs_3d.py (quantiser entry points agree)."""
import numpy as np
import pytest
import torch

from oracle import gemm as og
from oracle import quant as oq
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def _bf16_np(t):
    return t.float().numpy()


@pytest.mark.parametrize("m,k,aligned", [(1, 128, False), (7, 6144, True), (33, 2048, True), (64, 7168, False),
                                         (5, 200, False), (3, 72, True)])
def test_1d_quantiser_bit_exact_including_tiny_blocks(dev, m, k, aligned):
    from batchgen_amd.kernels.triton.fp8_quantize import per_token_blocked_quantize_bf16_to_fp8_1d as q1d
    g = torch.Generator().manual_seed(m * 7 + k)
    x = rand_bf16(g, m, k)
    x[0, :min(k, 128)] *= 1e-7                    # amax below 2^-16: the floor decides the scale
    if m > 2:
        x[2] = 0
        x[1, :min(k, 128)] = torch.tensor(3e-6).to(torch.bfloat16)
    y, s = q1d(x.to(dev), scale_tma_aligned=aligned)
    want_y, want_s = oq.act_quant(_bf16_np(x), form="A")
    nb = (k + 127) // 128
    assert tuple(s.shape) == (m, nb)
    assert s.stride() == ((1, (m + 3) // 4 * 4) if aligned else (nb, 1))
    assert np.array_equal(y.cpu().view(torch.uint8).numpy(), want_y)
    assert np.array_equal(s.cpu().numpy().view(np.int32), want_s.view(np.int32))


def test_1d_quantiser_valid_token_gate_and_act_quant_shapes(dev):
    from batchgen_amd.kernels.triton.fp8_quantize import per_token_blocked_quantize_bf16_to_fp8_1d as q1d
    from batchgen_amd.quantization import act_quant
    g = torch.Generator().manual_seed(3)
    x = rand_bf16(g, 12, 512)
    nv = torch.tensor([5], dtype=torch.int32, device=dev)
    y, s = q1d(x.to(dev), num_valid_tokens=nv)
    want_y, want_s = oq.act_quant(_bf16_np(x), form="A")
    want_y[5:] = 0
    want_s[5:] = np.float32(1e-12)
    assert np.array_equal(y.cpu().view(torch.uint8).numpy(), want_y)
    assert np.array_equal(s.cpu().numpy(), want_s)
    y3, s3 = act_quant(x.view(3, 4, 512).to(dev))
    assert tuple(y3.shape) == (3, 4, 512) and tuple(s3.shape) == (3, 4, 4)
    full_y, full_s = oq.act_quant(_bf16_np(x), form="A")
    assert np.array_equal(y3.cpu().view(torch.uint8).numpy().reshape(12, 512), full_y)
    assert np.array_equal(s3.cpu().numpy().reshape(12, 4), full_s)
    with pytest.raises(TypeError):
        q1d(x.to(dev), num_valid_tokens=nv.long())
    with pytest.raises(ValueError):
        act_quant(x.view(3, 4, 512).to(dev), scale_tma_aligned=True)
    with pytest.raises(NotImplementedError):
        act_quant(x.float().to(dev))


def _expert(dev, seed, hidden, inter):
    from batchgen_amd.moe.shared_expert import Fp8DenseExpert
    g = torch.Generator().manual_seed(seed)
    gu_q, gu_s = oq.weight_block_quant((0.03 * torch.randn(1, 2 * inter, hidden, generator=g)).numpy())
    d_q, d_s = oq.weight_block_quant((0.03 * torch.randn(1, hidden, inter, generator=g)).numpy())
    gate_up = torch.from_numpy(gu_q[0]).to(dev).view(torch.float8_e4m3fn)
    gs = torch.from_numpy(np.ascontiguousarray(gu_s[0][:inter // 128])).to(dev)
    us = torch.from_numpy(np.ascontiguousarray(gu_s[0][inter // 128:])).to(dev)
    down = torch.from_numpy(d_q[0]).to(dev).view(torch.float8_e4m3fn)
    ds = torch.from_numpy(d_s[0]).to(dev)
    make = lambda fused: Fp8DenseExpert(gate_up[:inter], gs, gate_up[inter:], us, down, ds,
                                        gate_up=gate_up if fused else None, layer_idx=3)
    return make, (gu_q[0], gu_s[0], d_q[0], d_s[0])


@pytest.mark.parametrize("rows,hidden,inter", [(1, 512, 256), (37, 1024, 384), (300, 512, 256)])
def test_fused_chain_equals_unfused_chain_and_the_oracle(dev, rows, hidden, inter):
    make, (gu_q, gu_s, d_q, d_s) = _expert(dev, rows, hidden, inter)
    fused, unfused = make(True), make(False)
    g = torch.Generator().manual_seed(rows + 1)
    x = rand_bf16(g, rows, hidden)
    got_f = fused(x.to(dev))
    got_u = unfused(x.to(dev))
    # the two chains differ in one place only: the unfused one takes SiLU from torch's bf16 kernel, the fused one
    # from this library's evaluation of the same formula; both then round to bf16
    diff = (got_f.float() - got_u.float()).abs().max().item()
    say(f"fused vs unfused rows={rows}: max abs diff {diff:.3e}, equal={torch.equal(got_f, got_u)}")
    assert torch.allclose(got_f.float(), got_u.float(), rtol=2e-2, atol=2e-3)
    assert (got_f != got_u).float().mean().item() < 1e-3
    # oracle: the fused chain, stage by stage, in fp32 (bytes of the intermediate quantisation exact by construction)
    xq, xs = oq.act_quant(_bf16_np(x), form="A")
    gu = og.grouped_gemm_fp8(xq, xs, gu_q[None], gu_s[None], np.array([rows], np.int32), np.array([0, rows], np.int32))
    gu = torch.from_numpy(gu).to(torch.bfloat16)          # already bf16-valued
    hq, hs, _ = oq.silu_mul_group_quant(_bf16_np(gu[:, :inter]), _bf16_np(gu[:, inter:]), "A")
    want = og.grouped_gemm_fp8(hq, hs, d_q[None], d_s[None], np.array([rows], np.int32), np.array([0, rows], np.int32))
    want = torch.from_numpy(want)
    rel = (got_f.cpu().float() - want).norm() / want.norm()
    say(f"fused vs oracle rel-Frobenius {rel:.3e}")
    assert rel < 5e-3
    # 3-D input keeps its leading shape; caller buffer is written in place
    buf = torch.zeros(rows, hidden, dtype=torch.bfloat16, device=dev)
    again = fused(x.view(1, rows, hidden).to(dev), out=buf)
    assert tuple(again.shape) == (1, rows, hidden) and again.data_ptr() == buf.data_ptr() and torch.equal(buf, got_f)


def test_prequantised_input_from_the_norm_kernel_and_graph_replay(dev):
    from batchgen_amd.attention.add_rmsnorm_fp8_quant import cuda_add_rmsnorm_fp8_quant
    rows, hidden, inter = 48, 1024, 256
    make, _ = _expert(dev, 11, hidden, inter)
    fused = make(True)
    g = torch.Generator().manual_seed(12)
    res = rand_bf16(g, rows, hidden).to(dev)
    hid = rand_bf16(g, rows, hidden).to(dev)
    gamma = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16).to(dev)
    normed, _, x_fp8, x_scale = cuda_add_rmsnorm_fp8_quant(res.clone(), hid, gamma, 1e-6, scale_tma_aligned=True)
    plain = fused(normed)
    handed = fused(normed, x_fp8=x_fp8, x_scale=x_scale)
    assert torch.equal(plain, handed)
    out = torch.zeros(rows, hidden, dtype=torch.bfloat16, device=dev)
    static_x = normed.clone()
    fused(static_x, out=out)                                 # warm-up: scratch tables exist before capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fused(static_x, out=out)
    for seed in (1, 2, 3):
        fresh = rand_bf16(torch.Generator().manual_seed(seed), rows, hidden).to(dev)
        static_x.copy_(fresh)
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, fused(fresh)), seed


def test_argument_policy(dev):
    make, _ = _expert(dev, 5, 512, 256)
    fused, unfused = make(True), make(False)
    x = rand_bf16(torch.Generator().manual_seed(1), 4, 512).to(dev)
    with pytest.raises(ValueError, match="out= requires"):
        unfused(x, out=torch.zeros(4, 512, dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError, match="x_fp8/x_scale require"):
        unfused(x, x_fp8=torch.zeros(4, 512, device=dev).to(torch.float8_e4m3fn))
    with pytest.raises(ValueError, match="together"):
        fused(x, x_fp8=torch.zeros(4, 512, device=dev).to(torch.float8_e4m3fn))
    with pytest.raises(ValueError, match="MN-major"):
        fused(x, x_fp8=torch.zeros(4, 512, device=dev).to(torch.float8_e4m3fn), x_scale=torch.ones(4, 4, device=dev))
    with pytest.raises(TypeError):
        fused(x.float())
    with pytest.raises(ValueError, match="shared-expert out"):
        fused(x, out=torch.zeros(4, 256, dtype=torch.bfloat16, device=dev))
    assert tuple(fused(x[:0]).shape) == (0, 512)
    scales = {"gate_proj.weight_scale_inv": fused.gate_scale, "up_proj.weight_scale_inv": fused.up_scale,
              "down_proj.weight_scale_inv": fused.down_scale}
    assert torch.equal(unfused.deepgemm_forward(x, scales), unfused(x))
    assert torch.equal(unfused.deepgemm_forward(x), unfused(x))
    from batchgen_amd.moe.shared_expert import Fp8DenseExpert
    with pytest.raises(RuntimeError, match="row halves"):
        Fp8DenseExpert(fused.gate.clone(), fused.gate_scale, fused.up, fused.up_scale, fused.down, fused.down_scale,
                       gate_up=fused.gate_up)
    with pytest.raises(RuntimeError, match="block scales"):
        Fp8DenseExpert(fused.gate, fused.gate_scale[:1], fused.up, fused.up_scale, fused.down, fused.down_scale,
                       gate_up=fused.gate_up)


@pytest.mark.parametrize("m", [1, 4, 15, 16, 17, 32, 33, 63, 64, 65, 130, 257, 512])
@pytest.mark.parametrize("n,k", [(128, 128), (256, 384), (1152, 1024), (8320, 256), (512, 7168), (16512, 128), (6272, 256), (256, 1152),
                                  (384, 2176), (256, 4224)])
def test_dense_k_split_gemm_vs_oracle_and_stacked_halves(dev, m, n, k):
    """The K-split dense GEMM (both of its forms: wave split, block split with a workspace) against the fp32 dequantise-then-matmul oracle at the
    reference's single-GEMM gate (rtol 2e-2 / atol 5e-3, tests/test_moe_compact_ragged_fp8.py:370-377), with
    row-major and MN-major activation scales; the two halves of the weight give the bytes of the whole."""
    from batchgen_amd.moe.shared_expert import DENSE_MAX_ROWS, DENSE_MAX_ROWS_NARROW, DENSE_NARROW_N, fp8_gemm_nt
    if m > DENSE_MAX_ROWS and n > DENSE_NARROW_N:
        pytest.skip("served by the grouped GEMM")
    assert m <= DENSE_MAX_ROWS_NARROW
    g = torch.Generator().manual_seed(m * 31 + n + k)
    x = rand_bf16(g, m, k)
    xq, xs = oq.act_quant(_bf16_np(x), form="A")
    wq, ws = oq.weight_block_quant((0.05 * torch.randn(1, n, k, generator=g)).numpy())
    want = og.grouped_gemm_fp8(xq, xs, wq, ws, np.array([m], np.int32), np.array([0, m], np.int32), to_bf16=False)
    a = torch.from_numpy(xq).to(dev).view(torch.float8_e4m3fn)
    b = torch.from_numpy(wq[0]).to(dev).view(torch.float8_e4m3fn)
    sb = torch.from_numpy(ws[0]).to(dev)
    sa_row = torch.from_numpy(xs).to(dev)
    sa_mn = torch.empty(k // 128, (m + 3) // 4 * 4, device=dev).transpose(0, 1)[:m]
    sa_mn.copy_(sa_row)
    outs = []
    for sa in (sa_row, sa_mn):
        d = torch.full((m, n), -7.0, dtype=torch.bfloat16, device=dev)
        fp8_gemm_nt((a, sa), (b, sb), d)
        outs.append(d)
    assert torch.equal(outs[0], outs[1])
    got = outs[0].cpu().float().numpy()
    np.testing.assert_allclose(got, want, rtol=2e-2, atol=5e-3)
    rel = np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30)
    assert rel < 4e-3, rel
    if n >= 256:
        half = n // 2 // 128 * 128
        lo = torch.empty(m, half, dtype=torch.bfloat16, device=dev)
        hi = torch.empty(m, n - half, dtype=torch.bfloat16, device=dev)
        fp8_gemm_nt((a, sa_row), (b[:half], sb[:half // 128]), lo)
        fp8_gemm_nt((a, sa_row), (b[half:], sb[half // 128:]), hi)
        assert torch.equal(torch.cat([lo, hi], dim=1), outs[0])


@pytest.mark.parametrize("m", [3, 16, 40, 64, 200, 700])
def test_dense_gemm_on_tile_major_weights(dev, m):
    from batchgen_amd.kernels import load_extension
    from batchgen_amd.moe.shared_expert import fp8_gemm_nt
    n, k = 512, 1024
    g = torch.Generator().manual_seed(m)
    xq, xs = oq.act_quant(_bf16_np(rand_bf16(g, m, k)), form="A")
    wq, ws = oq.weight_block_quant((0.05 * torch.randn(1, n, k, generator=g)).numpy())
    want = og.grouped_gemm_fp8(xq, xs, wq, ws, np.array([m], np.int32), np.array([0, m], np.int32), to_bf16=False)
    a = torch.from_numpy(xq).to(dev).view(torch.float8_e4m3fn)
    b = torch.from_numpy(wq[0]).to(dev).view(torch.float8_e4m3fn)
    tiled = load_extension("batchgen_kernels.moe._C_fp8_blockwise_gemm").fp8_weight_repack(b)
    sa, sb = torch.from_numpy(xs).to(dev), torch.from_numpy(ws[0]).to(dev)
    d_row = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    d_tile = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    fp8_gemm_nt((a, sa), (b, sb), d_row)
    fp8_gemm_nt((a, sa), (tiled, sb), d_tile, weight_layout="tile_major")
    np.testing.assert_allclose(d_tile.cpu().float().numpy(), want, rtol=2e-2, atol=5e-3)
    np.testing.assert_allclose(d_row.cpu().float().numpy(), want, rtol=2e-2, atol=5e-3)
    if m > 64:                                        # both layouts take the block-split form with equal slices
        assert torch.equal(d_row, d_tile)


@pytest.mark.parametrize("rows,hidden,inter", [(48, 4224, 256), (200, 2176, 384), (300, 512, 256), (512, 1152, 128)])
def test_activation_fed_by_partial_sums_equals_gemm_then_activation(dev, rows, hidden, inter):
    """The fused chain's shortcut (the activation kernel adds the [gate; up] GEMM's K-slices itself) against the
    plain sequence GEMM -> bf16 -> SiLU * up + cast: identical bytes and scales."""
    from batchgen_amd.kernels.triton.fp8_quantize import (per_token_blocked_quantize_bf16_to_fp8_1d,
                                                          silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d)
    from batchgen_amd.moe.shared_expert import fp8_gemm_nt
    make, _ = _expert(dev, rows + hidden, hidden, inter)
    fused = make(True)
    x = rand_bf16(torch.Generator().manual_seed(rows), rows, hidden).to(dev)
    x_fp8, x_scale = per_token_blocked_quantize_bf16_to_fp8_1d(x, scale_tma_aligned=True)
    short = fused._gate_up_activation_from_partials(x_fp8, x_scale, rows, hidden)
    assert short is not None, "this shape is meant to take the block-split GEMM"
    gate_up = torch.empty(rows, 2 * inter, dtype=torch.bfloat16, device=dev)
    fp8_gemm_nt((x_fp8, x_scale), (fused.gate_up, fused.gate_up_scale), gate_up)
    h_fp8, h_scale = silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d(gate_up, scale_tma_aligned=True)
    assert torch.equal(short[0].view(torch.uint8), h_fp8.view(torch.uint8))
    assert torch.equal(short[1], h_scale) and short[1].stride() == h_scale.stride()
    small = fused._gate_up_activation_from_partials(x_fp8[:8], x_scale[:8], 8, hidden)
    assert small is None                                   # a handful of rows: no partial sums exist


def test_scratch_pool_survives_growth_after_capture(dev):
    """A graph captured while the pool's buffer was small keeps giving the right answer after an eager call has
    made the pool allocate a larger one (the old buffer is retired, not freed), and two streams get two buffers."""
    from batchgen_amd.kernels import _workspace as wsp
    from batchgen_amd.kernels import load_extension
    rt = load_extension("batchgen_kernels.moe._C_routing")
    g = torch.Generator().manual_seed(11)
    e, h = 64, 1024
    w = (torch.randn(e, h, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    small = torch.randn(8, h, generator=g).to(torch.bfloat16).to(dev)
    big = torch.randn(4096, h, generator=g).to(torch.bfloat16).to(dev)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        out_small = torch.empty((8, e), dtype=torch.float32, device=dev)
        rt.glm5_router_gemm(small, w, None, out_small, 0, 1)          # warm-up on the capture stream
        s.synchronize()
        key = ("router_gemm", dev.index or 0, s.cuda_stream)
        first = wsp._LIVE.get(key)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            rt.glm5_router_gemm(small, w, None, out_small, 0, 1)
        want = out_small.clone()
        from batchgen_amd._lib import lib
        need_big = int(lib().bgmoe_router_gemm_workspace_bytes(4096, h, e))
        out_big = torch.empty((4096, e), dtype=torch.float32, device=dev)
        rt.glm5_router_gemm(big, w, None, out_big, 0, 1)               # may grow the pool on this stream
        torch.zeros(1 << 22, device=dev).fill_(3.0)                   # churn the allocator
        out_small.zero_()
        graph.replay()
        s.synchronize()
        assert torch.equal(out_small, want)
        if first is not None and need_big > first.numel():
            assert wsp._LIVE[key] is not first and any(b is first for b in wsp._RETIRED)
    other = wsp.scratch("router_gemm", dev, 1024)
    with torch.cuda.stream(s):
        mine = wsp.scratch("router_gemm", dev, 1024)
    assert other.data_ptr() != mine.data_ptr()
