"""HIP act-quant entry points vs the CPU oracle: bytes and scales bit-exact."""
import numpy as np
import pytest
import torch

from oracle import quant as oq
from oracle.fp8 import e4m3fn_encode
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


def ops():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_fp8_blockwise_ops")


@pytest.mark.parametrize("m,k", [(1, 128), (7, 256), (5, 300), (33, 7168), (64, 2048), (3, 6144), (2, 8)])
def test_act_quant_rows_bit_exact(dev, m, k):
    say("act_quant_rows", m, k)
    g = torch.Generator().manual_seed(1000 + m + k)
    x = rand_bf16(g, m, k)
    x[0, : min(k, 128)] = 0                       # an all-zero block
    if m > 1:
        x[1] *= 1e-3
        x[1, 0] = 3.0e38                          # huge value saturates its block
    y, s = ops().act_quant_rows(x.to(dev))
    yo, so = oq.act_quant(x)
    assert np.array_equal(y.view(torch.uint8).cpu().numpy(), yo)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), so.view(np.uint32))
    # transposed scale layout
    y2, s2 = ops().act_quant_rows(x.to(dev), scale_transposed=True)
    assert np.array_equal(s2.cpu().numpy().T.copy().view(np.uint32), so.view(np.uint32))
    assert torch.equal(y2.view(torch.uint8), y.view(torch.uint8))


def test_hardware_e4m3_convert_matches_oracle_on_every_bf16_value(dev):
    """All bf16 bit patterns in one row-block each, scale forced to 1 by a 448 in the block."""
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    vals = bits.float()
    ok = torch.isfinite(vals) & (vals.abs() <= 448)
    v = vals[ok]
    pad = (-len(v)) % 127
    v = torch.cat([v, torch.zeros(pad)])
    rows = v.view(-1, 127)
    x = torch.cat([torch.full((rows.size(0), 1), 448.0), rows], dim=1).to(torch.bfloat16)  # amax = 448 -> s = 1
    y, s = ops().act_quant_rows(x.to(dev))
    yo, so = oq.act_quant(x)
    assert np.all(so == np.float32(448.0) * (np.float32(1.0) / np.float32(448.0)))
    assert np.array_equal(y.view(torch.uint8).cpu().numpy(), yo)


def test_act_quant_3d_masked_rows_untouched(dev):
    g = torch.Generator().manual_seed(7)
    e, mtp, k = 5, 9, 384
    x = rand_bf16(g, e, mtp, k)
    cnt = torch.tensor([0, 1, 9, 4, 8], dtype=torch.int32)
    x[1, 1:] = float("nan")                       # rows past the count are never read
    y, s = ops().act_quant_3d(x.to(dev), cnt.to(dev))
    yo, so, written = oq.act_quant_masked(x, cnt.numpy())
    y = y.cpu().numpy()
    s = s.cpu().numpy()
    assert np.array_equal(y[written], yo[written])
    assert np.array_equal(s[written].view(np.uint32), so[written].view(np.uint32))


@pytest.mark.parametrize("k", [256, 300, 6144])
@pytest.mark.parametrize("row_align", [64, 128])
def test_act_quant_ragged_write_set(dev, k, row_align):
    say("act_quant_ragged", k, row_align)
    g = torch.Generator().manual_seed(11 + k)
    counts = np.array([0, 1, 63, 64, 65, 2, 0], dtype=np.int32)
    aligned = (counts + row_align - 1) // row_align * row_align
    cu = np.concatenate([[0], np.cumsum(aligned)]).astype(np.int32)
    max_rows = int(cu[-1]) + 70
    x = rand_bf16(g, max_rows, k)
    kb = (k + 127) // 128
    y = torch.full((max_rows, k), 0xAB, dtype=torch.uint8)
    s = torch.full((kb, max_rows), -7.0)
    yo, so, written, valid = oq.act_quant_ragged_model(x, counts, cu, row_align)
    x_dev = x.clone()
    x_dev[~torch.from_numpy(valid)] = float("inf")     # unread inputs may hold anything
    yd, sd = ops().act_quant_ragged(x_dev.to(dev), torch.from_numpy(counts).to(dev), torch.from_numpy(cu).to(dev),
                                    y.to(dev), s.to(dev), row_align)
    yd = yd.cpu().numpy()
    sd = sd.cpu().numpy()
    assert np.array_equal(yd[written], yo[written])
    assert np.array_equal(sd[:, written].view(np.uint32), so[:, written].view(np.uint32))
    assert np.all(yd[~written] == 0xAB) and np.all(sd[:, ~written] == -7.0)
    pad = written & ~valid
    assert np.all(yd[pad] == 0) and np.all(sd[:, pad] == oq.pad_row_scale())


def test_uniform_stride_ragged_equals_masked(dev):
    """cu[e] = e*S describes the masked layout; both entry points give the same bytes."""
    g = torch.Generator().manual_seed(5)
    e, s_, k = 4, 64, 512
    x = rand_bf16(g, e * s_, k)
    cnt = torch.tensor([3, 0, 64, 17], dtype=torch.int32)
    cu = (torch.arange(e + 1, dtype=torch.int32) * s_)
    y3, s3 = ops().act_quant_3d(x.view(e, s_, k).to(dev), cnt.to(dev))
    yr = torch.zeros((e * s_, k), dtype=torch.uint8, device=dev)
    sr = torch.zeros((k // 128, e * s_), dtype=torch.float32, device=dev)
    ops().act_quant_ragged(x.to(dev), cnt.to(dev), cu.to(dev), yr, sr, 1)
    for i in range(e):
        c = int(cnt[i])
        assert torch.equal(y3[i, :c], yr.view(e, s_, k)[i, :c])
        assert torch.equal(s3[i, :c], sr.t().reshape(e, s_, -1)[i, :c])


@pytest.mark.parametrize("scale", [1.0, 8.0, 0.02])
def test_fused_silu_quant_equals_unfused(dev, scale):
    g = torch.Generator().manual_seed(3)
    e, mtp, n = 3, 20, 640
    gate = rand_bf16(g, e, mtp, n, scale=scale)
    up = rand_bf16(g, e, mtp, n, scale=scale)
    gate[0, 0, :5] = torch.tensor([90.0, -90.0, 30.0, -30.0, 1e-30]).to(torch.bfloat16)
    up[0, 1, :128] = 0                                  # a whole zero block
    cnt = torch.tensor([20, 7, 0], dtype=torch.int32).to(dev)
    h = ops().silu_mul_3d(gate.to(dev), up.to(dev), cnt)
    y1, s1 = ops().act_quant_3d(h, cnt)
    y2, s2 = ops().fused_silu_quant_3d(gate.to(dev), up.to(dev), cnt)
    for i, c in enumerate([20, 7, 0]):
        assert torch.equal(y1[i, :c], y2[i, :c]) and torch.equal(s1[i, :c], s2[i, :c])
    # against the oracle's SwiGLU within one bf16 ulp (device exp is not the oracle's exp)
    ho = oq.swiglu_bf16(gate[0, :20].float().numpy(), up[0, :20].float().numpy())
    hd = h[0, :20].float().cpu().numpy()
    assert np.all(np.abs(hd - ho) <= np.abs(ho) * 2 ** -7 + 1e-30)
