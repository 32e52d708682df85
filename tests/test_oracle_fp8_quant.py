"""Pins for the oracle's FP8 codec and quantisers (CPU only)."""
import numpy as np
import torch

from oracle import quant as oq
from oracle.fp8 import e4m3fn_decode, e4m3fn_encode


def _all_bf16_in_range():
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    return bits[torch.isfinite(bits) & (bits.abs() <= 448)]


def test_encode_matches_torch_cast_on_every_bf16_value_and_random_fp32():
    v = _all_bf16_in_range()
    assert np.array_equal(e4m3fn_encode(v.numpy()), v.to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    g = torch.Generator().manual_seed(0)
    for scale in (1e-3, 1.0, 50.0, 400.0):
        x = (torch.randn(200000, generator=g) * scale).clamp(-448, 448)
        assert np.array_equal(e4m3fn_encode(x.numpy()), x.to(torch.float8_e4m3fn).view(torch.uint8).numpy())


def test_encode_ties_go_to_even_and_saturate():
    # 17 and 19 are halfway between e4m3 neighbours (16,18,20): ties to even mantissa -> 16 and 20
    assert e4m3fn_decode(e4m3fn_encode(np.float32([17.0, 19.0, 1000.0, -1000.0]))).tolist() == [16.0, 20.0, 448.0, -448.0]
    assert e4m3fn_encode(np.float32([np.nan]))[0] == 0x7F
    # subnormals: 2^-9 is the smallest step; 2^-10 is a tie with 0 -> 0; 1.5*2^-9 ties to even -> 2 * 2^-9
    assert e4m3fn_encode(np.float32([2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9])).tolist() == [1, 0, 2]


def test_decode_is_the_closed_form_and_inverts_encode():
    d = e4m3fn_decode(np.arange(256, dtype=np.uint8))
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(d, nan=7.0), np.nan_to_num(t, nan=7.0))
    codes = np.array([c for c in range(256) if c not in (0x7F, 0xFF)], dtype=np.uint8)
    back = e4m3fn_encode(e4m3fn_decode(codes))
    keep = codes != 0x80                                    # -0.0 encodes as 0x80 too
    assert np.array_equal(back[keep], codes[keep])


def test_act_quant_special_cases():
    x = np.zeros((3, 256), dtype=np.float32)
    x[1, :128] = np.linspace(-3, 3, 128)
    x[2, 5] = np.float32(3e38)
    y, s = oq.act_quant(x)
    assert np.all(y[0] == 0) and np.all(s[0] == np.float32(1e-12) * (np.float32(1) / np.float32(448)))
    assert s[1, 0] == np.float32(3.0) * (np.float32(1) / np.float32(448))
    assert y[1, 0] == 0xFE and y[1, 127] == 0x7E           # -448 and +448: the extremes map to +-max
    assert y[2, 5] == 0x7E and np.all(np.delete(y[2, :128], 5) == 0)
    xn = np.full((1, 128), 1.0, dtype=np.float32)
    xn[0, 3] = np.nan
    yn, sn = oq.act_quant(xn)
    assert yn[0, 3] == 0x7E                                 # fminf/fmaxf clamp turns NaN into +448
    assert sn[0, 0] == np.float32(1.0) * (np.float32(1) / np.float32(448))   # NaN is ignored by the amax


def test_dequantised_value_is_within_half_an_fp8_step():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(64, 1024, generator=g).to(torch.bfloat16).float().numpy()
    y, s = oq.act_quant(x)
    d = oq.act_dequant(y, s)
    q = x / np.repeat(s, 128, axis=1)
    step = np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(q), 2.0 ** -6))) - 3), 2.0 ** -9)
    assert np.all(np.abs(d - x) <= 0.5 * step * np.repeat(s, 128, axis=1) * (1 + 1e-6))


def test_form_a_equals_form_c_when_amax_is_not_tiny():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(50, 640, generator=g).to(torch.bfloat16)
    ya, sa = oq.act_quant(x, "A")
    yc, sc = oq.act_quant(x, "C")
    assert np.array_equal(ya, yc) and np.array_equal(sa.view(np.uint32), sc.view(np.uint32))
    z = torch.zeros(2, 128)
    yza, sza = oq.act_quant(z, "A")
    yzc, szc = oq.act_quant(z, "C")
    assert np.array_equal(yza, yzc) and not np.array_equal(sza, szc)  # only the stored scale differs
    # forms B and D differ from C in few bytes
    yb, _ = oq.act_quant(x, "B")
    yd, _ = oq.act_quant(x, "D")
    assert (yb != yc).mean() < 5e-3 and (yd != yc).mean() < 5e-3


def test_ragged_write_set_model():
    counts = np.array([0, 1, 63, 64, 65, 2, 0])
    cu = np.concatenate([[0], np.cumsum((counts + 63) // 64 * 64)])
    x = np.random.default_rng(0).standard_normal((int(cu[-1]) + 10, 256)).astype(np.float32)
    y, st, written, valid = oq.act_quant_ragged_model(x, counts, cu, 64)
    assert written.sum() == ((counts + 63) // 64 * 64).sum() and valid.sum() == counts.sum()
    assert not written[int(cu[-1]):].any()
    yv, sv = oq.act_quant(x[valid])
    assert np.array_equal(y[valid], yv) and np.array_equal(st[:, valid], sv.T)
    pad = written & ~valid
    assert np.all(y[pad] == 0) and np.all(st[:, pad] == oq.pad_row_scale())


def test_weight_block_quant_matches_the_torch_recipe_and_dequantises():
    from batchgen_amd.workloads import block_quant_fp8
    g = torch.Generator().manual_seed(3)
    w = torch.randn(2, 256, 384, generator=g) * 0.02
    q, s = block_quant_fp8(w)
    qo, so = oq.weight_block_quant(w.numpy())
    assert np.array_equal(q.view(torch.uint8).numpy(), qo) and np.array_equal(s.numpy(), so)
    d = oq.weight_block_dequant(qo, so)
    assert np.linalg.norm(d - w.numpy()) / np.linalg.norm(w.numpy()) < 0.04
    db = oq.weight_block_dequant(qo, so, to_bf16=True)
    ref = (q.float().view(2, 2, 128, 3, 128) * s[:, :, None, :, None]).view(2, 256, 384).to(torch.bfloat16).float()
    assert np.array_equal(db, ref.numpy())


def test_bf16_round_matches_torch():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(100000, generator=g) * 3
    assert np.array_equal(oq.bf16_round(x.numpy()), x.to(torch.bfloat16).float().numpy())


def test_short_scale_division_model_equals_ieee_division():
    """The device quantisers compute x / s as q0 = x*r, e = fma(-q0, s, x), q = fma(e, r, q0) with r = 1/s.
    Modelled here with a correctly rounded float32 fma, the step gives the IEEE quotient for scales and
    values from the quantisers' domain (the device repeats the comparison on 2^34 pairs)."""
    from oracle.norm_quant import fma_f32
    rng = np.random.default_rng(77)
    n = 1_000_000
    s = (np.exp2(rng.uniform(-99, 99, n)) * rng.uniform(1, 2, n)).astype(np.float32)
    x = (rng.uniform(-448.5, 448.5, n) * s.astype(np.float64)).astype(np.float32)
    half = n // 2
    x[:half] = (x[:half].view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)      # bf16 values
    r = (np.float32(1.0) / s).astype(np.float32)
    q0 = (x * r).astype(np.float32)
    e = fma_f32(-q0, s, x)
    q = np.where(e == 0, q0, fma_f32(e, r, q0))
    assert np.array_equal(q.view(np.uint32), (x / s).astype(np.float32).view(np.uint32))


def test_silu_in_the_reference_precision_and_the_group_quantiser_of_the_deepgemm_chain():
    """``silu_torch_f32`` against the library's own fp32 SiLU and closed forms; ``silu_mul_group_quant`` form D
    against the reference test's ``act_reference`` written with torch CPU operations
    (tests/test_glm52_deepgemm_masked_parity_gpu.py:128-149)."""
    import torch.nn.functional as F
    gen = torch.Generator().manual_seed(11)
    g = (torch.randn(300_000, generator=gen) * 5).to(torch.bfloat16).float()
    mine = oq.silu_torch_f32(g.numpy())
    lib = F.silu(g).numpy()
    assert np.max(np.abs(mine.view(np.int32).astype(np.int64) - lib.view(np.int32).astype(np.int64))) <= 2
    assert np.mean(oq.bf16_round(mine) != oq.bf16_round(lib)) < 1e-4
    x64 = g.double()
    np.testing.assert_allclose(mine, (x64 * torch.sigmoid(x64)).numpy(), rtol=3e-7, atol=1e-37)
    special = oq.silu_torch_f32(np.array([0.0, 200.0, -200.0, 90.0, -90.0, 1e-30], dtype=np.float32))
    assert special[0] == 0 and special[1] == 200.0 and special[2] == 0 and np.signbit(special[2])
    assert special[3] == 90.0 and abs(special[4]) < 1e-36 and special[5] == np.float32(5e-31)

    gate = (torch.randn(37, 384, generator=gen) * 3).to(torch.bfloat16)
    up = (torch.randn(37, 384, generator=gen) * 3).to(torch.bfloat16)
    up[3, :128] = 0                                                   # a whole zero group: floor 1e-10
    gf = gate.float()
    sg = (gf / (1 + torch.exp(-gf))).to(torch.bfloat16)
    prod = (up * sg).reshape(37, 3, 128)
    amax = prod.abs().amax(-1).float().clamp_min(1e-10)
    s_ref = amax / 448.0
    q_ref = (prod.float() / s_ref.unsqueeze(-1)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).reshape(37, 384)
    y, s, p = oq.silu_mul_group_quant(gate, up, "D")
    assert np.mean(p != prod.reshape(37, 384).float().numpy()) < 1e-3  # torch's exp vs the correctly rounded one
    same = (p == prod.reshape(37, 384).float().numpy()).reshape(37, 3, 128).all(-1)
    assert np.array_equal(s[same], s_ref.numpy()[same])
    yb = q_ref.view(torch.uint8).numpy().reshape(37, 3, 128)
    assert np.array_equal(y.reshape(37, 3, 128)[same], yb[same])
    assert s[3, 0] == np.float32(1e-10) / np.float32(448.0) and not (y[3, :128] & 0x7F).any()    # signed zeros
