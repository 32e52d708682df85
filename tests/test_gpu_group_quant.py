"""SiLU * up + per-128-group FP8 cast in one pass (the activation between the two grouped GEMMs of the DeepGEMM
chains and of the dense shared expert) against the CPU oracle: the bf16 product, the FP8 bytes and the scales
are compared BIT FOR BIT (the device evaluates SiLU as the oracle does: correctly rounded exp, fp32 add, IEEE
division); rows outside the live counts keep their sentinels."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def _mod():
    from batchgen_amd.kernels.triton import moe_masked_act_quant as m
    return m


def _special(gate, up):
    """Edge values of the reference's fused-quantiser test (tests/test_silu_mul_fp8_quantize.py:43-73), written
    into views of one tensor."""
    first = gate[(0,) * (gate.dim() - 1)]
    first[:6] = torch.tensor([90.0, -90.0, 30.0, -30.0, 1e-30, 0.0]).to(torch.bfloat16)
    second = up[(0,) * (up.dim() - 2) + (min(1, up.shape[-2] - 1),)]
    second[:128] = 0                                             # a whole zero group


@pytest.mark.parametrize("scale", [1.0, 8.0, 0.02])
def test_masked_group_quant_bit_exact_and_masked_rows_untouched(dev, scale):
    from batchgen_amd._lib import check, lib, ptr
    e, s_, n = 3, 20, 640
    g = torch.Generator().manual_seed(int(scale * 100))
    r1 = rand_bf16(g, e, s_, 2 * n, scale=scale)                 # one GEMM output [E, S, 2I]: gate | up
    _special(r1[..., :n], r1[..., n:])
    counts = [20, 7, 0]
    masked_m = torch.tensor(counts, dtype=torch.int32, device=dev)
    r1d = r1.to(dev)
    gate, up = r1d[..., :n], r1d[..., n:]
    out = torch.full((e, s_, n), 0xAB, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    sc = torch.full((e, n // 128, s_), -7.0, dtype=torch.float32, device=dev).transpose(1, 2)     # MN-major view
    _mod().silu_mul_masked_group_quant(gate, up, out, sc, masked_m)
    ob, sb = out.view(torch.uint8).cpu().numpy(), sc.cpu().numpy()
    prod = torch.full((e, s_, n), 7.0, dtype=torch.bfloat16, device=dev)
    check(lib().bgmoe_silu_mul_group_quant(ptr(r1d), gate.data_ptr() + 2 * n, s_ * 2 * n, 2 * n, ptr(masked_m), None, e,
                                           s_, n, 1, ptr(out), s_ * n, n, ptr(sc), sc.stride(0), sc.stride(1),
                                           sc.stride(2), ptr(prod), None))
    pb = prod.float().cpu().numpy()
    for i, c in enumerate(counts):
        y, s, p = oq.silu_mul_group_quant(r1[i, :c, :n], r1[i, :c, n:], "D")
        assert np.array_equal(pb[i, :c], p), f"bf16 product differs, expert {i}"
        assert np.array_equal(ob[i, :c], y) and np.array_equal(sb[i, :c], s)
        assert (ob[i, c:] == 0xAB).all() and (sb[i, c:] == -7.0).all() and (pb[i, c:] == 7.0).all()


def test_ragged_group_quant_bit_exact_and_holes_untouched(dev):
    counts = np.array([0, 1, 63, 64, 65, 2, 0], dtype=np.int32)
    cu = np.concatenate([[0], np.cumsum((counts + 63) // 64 * 64)]).astype(np.int32)
    m, n = int(cu[-1]) + 64, 256
    g = torch.Generator().manual_seed(5)
    gate, up = rand_bf16(g, m, n, scale=2.0), rand_bf16(g, m, n, scale=2.0)
    out = torch.full((m, n), 0xAB, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    sc = torch.full((m, n // 128), -7.0, dtype=torch.float32, device=dev)
    _mod().silu_mul_ragged_group_quant(gate.to(dev), up.to(dev), out, sc, torch.from_numpy(counts).to(dev),
                                       torch.from_numpy(cu).to(dev))
    ob, sb = out.view(torch.uint8).cpu().numpy(), sc.cpu().numpy()
    live = np.zeros(m, dtype=bool)
    for i, c in enumerate(counts):
        live[cu[i]:cu[i] + c] = True
    y, s, _ = oq.silu_mul_group_quant(gate[torch.from_numpy(live)], up[torch.from_numpy(live)], "D")
    assert np.array_equal(ob[live], y) and np.array_equal(sb[live], s)
    assert (ob[~live] == 0xAB).all() and (sb[~live] == -7.0).all()


@pytest.mark.parametrize("m,dim,aligned", [(1, 128, False), (37, 2048, False), (37, 2048, True), (256, 1536, True)])
def test_one_dimensional_form_matches_the_1d_quantiser_of_the_product(dev, m, dim, aligned):
    from batchgen_amd.kernels import load_extension
    from batchgen_amd.kernels.triton.fp8_quantize import silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d as fused
    say("silu_mul 1-D", m, dim, aligned)
    g = torch.Generator().manual_seed(m + dim)
    x = rand_bf16(g, m, 2 * dim, scale=3.0)
    _special(x[:, :dim], x[:, dim:])
    out, sc = fused(x.to(dev), scale_tma_aligned=aligned)
    assert out.shape == (m, dim) and sc.shape == (m, dim // 128)
    if aligned:
        assert sc.stride() == (1, (m + 3) // 4 * 4)
    y, s, p = oq.silu_mul_group_quant(x[:, :dim], x[:, dim:], "A")
    assert np.array_equal(out.view(torch.uint8).cpu().numpy(), y) and np.array_equal(sc.cpu().numpy(), s)
    # ... which is the standalone 1-D quantiser applied to the bf16 product (the reference's contract)
    ops = load_extension("batchgen_kernels.moe._C_fp8_blockwise_ops")
    assert hasattr(ops, "act_quant_rows")
    yq, sq = oq.act_quant(p, form="A")
    assert np.array_equal(y, yq) and np.array_equal(s, sq)


def test_group_quant_argument_policy(dev):
    m = _mod()
    e, s_, n = 2, 4, 128
    gate = torch.zeros(e, s_, n, dtype=torch.bfloat16, device=dev)
    out = torch.zeros(e, s_, n, dtype=torch.float8_e4m3fn, device=dev)
    sc = torch.zeros(e, s_, 1, dtype=torch.float32, device=dev)
    mm = torch.zeros(e, dtype=torch.int32, device=dev)
    m.silu_mul_masked_group_quant(gate, gate, out, sc, mm)            # nothing live: a no-op
    for bad in (lambda: m.silu_mul_masked_group_quant(gate[0], gate[0], out[0], sc[0], mm),
                lambda: m.silu_mul_masked_group_quant(gate, gate.float(), out, sc, mm),
                lambda: m.silu_mul_masked_group_quant(gate, gate, out.view(torch.uint8), sc, mm),
                lambda: m.silu_mul_masked_group_quant(gate, gate, out, sc.double(), mm),
                lambda: m.silu_mul_masked_group_quant(gate, gate, out, sc[:, :3], mm),
                lambda: m.silu_mul_masked_group_quant(gate, gate, out, sc, mm.long()),
                lambda: m.silu_mul_masked_group_quant(gate[..., :100], gate[..., :100], out[..., :100], sc, mm),
                lambda: m.silu_mul_ragged_group_quant(gate[0], gate[0], out[0], sc[0].t().contiguous().t(), mm, mm),
                lambda: m.silu_mul_ragged_group_quant(gate[0], gate[0], out[0], sc[0], mm, mm)):
        with pytest.raises(ValueError):
            bad()
    from batchgen_amd.kernels.triton.fp8_quantize import silu_mul_per_token_blocked_quantize_bf16_to_fp8_1d as fused
    with pytest.raises(TypeError):
        fused(torch.zeros(4, 256, device=dev))
    for bad in (torch.zeros(4, 255, dtype=torch.bfloat16, device=dev), torch.zeros(4, 200, dtype=torch.bfloat16, device=dev),
                torch.zeros(0, 256, dtype=torch.bfloat16, device=dev), torch.zeros(2, 4, 256, dtype=torch.bfloat16, device=dev)):
        with pytest.raises(ValueError):
            fused(bad)


def test_silu_of_every_bf16_value_equals_the_oracle(dev):
    """All 65536 bf16 gates against the oracle, bit for bit: with up = 1 the bf16 product the kernel can hand
    out IS bf16(silu(gate)).  Covers the short evaluation, its hand-over to the exact one, +-0, +-inf, NaN and
    the denormals."""
    from batchgen_amd._lib import check, lib, ptr
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = torch.cat([bits.view(512, 128), torch.ones(512, 128, dtype=torch.bfloat16)], dim=1).contiguous().to(dev)
    out = torch.empty(512, 128, dtype=torch.uint8, device=dev)
    sc = torch.empty(512, 1, dtype=torch.float32, device=dev)
    prod = torch.empty(512, 128, dtype=torch.bfloat16, device=dev)
    check(lib().bgmoe_silu_mul_group_quant(ptr(x), x.data_ptr() + 256, 0, 256, None, None, 1, 512, 128, 0, ptr(out), 0,
                                           128, ptr(sc), 0, 1, 1, ptr(prod), None))
    got = prod.view(torch.int16).cpu().numpy().reshape(-1).view(np.uint16)
    with np.errstate(invalid="ignore", over="ignore"):
        want = oq.bf16_round(oq.silu_torch_f32(bits.float().numpy()))
    wb = (want.view(np.uint32) >> 16).astype(np.uint16)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan], wb[~nan])
    assert np.all((got[nan] & 0x7F80) == 0x7F80) and np.all((got[nan] & 0x7F) != 0)      # NaN stays NaN
