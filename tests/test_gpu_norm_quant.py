"""HIP add + RMSNorm + FP8 cast against the CPU oracle, bit for bit, with the cases of the reference's
bitwise gate (tests/test_glm52_norm_quant_fuse_bitwise_gpu.py:238-440): plain / gated / masked rows, the
num_valid edges, both scale layouts, the 3-D layer shape, and fused == norm followed by the standalone
quantiser."""
import numpy as np
import pytest
import torch

from oracle import norm_quant as onq
from tests.util import say

pytestmark = pytest.mark.gpu


def fused(*a, **k):
    from batchgen_amd.attention import cuda_add_rmsnorm_fp8_quant
    return cuda_add_rmsnorm_fp8_quant(*a, **k)


def _inputs(seed, rows, dim, rs=0.9, hs=0.4, ws=0.3, wb=1.0):
    g = torch.Generator().manual_seed(seed)
    res = (torch.randn(rows, dim, generator=g) * rs).to(torch.bfloat16)
    hid = (torch.randn(rows, dim, generator=g) * hs).to(torch.bfloat16)
    w = (torch.randn(dim, generator=g) * ws + wb).to(torch.bfloat16)
    return res, hid, w


def _bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy()


def _check(dev, res, hid, w, eps, gated_at=None, norm_gated=False, mask=None, tma=True):
    rows = res.shape[0]
    nvt = torch.tensor([gated_at], dtype=torch.int32, device=dev) if gated_at is not None else None
    res_d = res.clone().to(dev)
    stale = torch.full_like(res_d, 7.0)
    normed, res_out, q, s = fused(res_d, hid.to(dev), w.to(dev), eps,
                                  norm_num_valid_tokens=nvt if norm_gated else None,
                                  quant_num_valid_tokens=nvt, row_valid_mask=None if mask is None else mask.to(dev),
                                  scale_tma_aligned=tma)
    assert res_out.data_ptr() == res_d.data_ptr()                 # in place
    assert q.dtype == torch.float8_e4m3fn and tuple(q.shape) == (rows, res.shape[1])
    blocks = res.shape[1] // 128
    assert tuple(s.shape) == (rows, blocks)
    assert s.stride() == ((1, (rows + 3) // 4 * 4) if tma else (blocks, 1))
    n_o, r_o, y_o, s_o = onq.add_rmsnorm_fp8_quant(res, hid, w, eps,
                                                   norm_num_valid_tokens=gated_at if norm_gated else None,
                                                   quant_num_valid_tokens=gated_at, row_valid_mask=mask)
    live = rows if not norm_gated else min(gated_at, rows)
    assert np.array_equal(res_out.float().cpu().numpy(), r_o)
    assert np.array_equal(normed.float().cpu().numpy()[:live], n_o[:live])
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), y_o)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), s_o.view(np.uint32))
    del stale
    return normed, q, s


@pytest.mark.parametrize("rows", [1, 4, 64, 257])
@pytest.mark.parametrize("gated,masked", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("dim", [6144, 7168])
def test_fused_add_norm_quant_is_bitwise_the_oracle(dev, rows, gated, masked, dim):
    say("add_rmsnorm_fp8_quant", rows, dim, gated, masked)
    res, hid, w = _inputs(rows * 3 + dim + gated + 2 * masked, rows, dim)
    mask = None
    if masked:
        mask = torch.ones(rows, dtype=torch.bfloat16)
        mask[::3] = 0
        hid[::3] = float("nan")                                    # dropped rows may hold anything
    _check(dev, res, hid, w, 1e-5, gated_at=max(1, rows // 2) if gated else None, mask=mask)


@pytest.mark.parametrize("valid", [0, 1, 3, 4, 63, 64, 65])
def test_num_valid_edges_with_large_values(dev, valid):
    res, hid, w = _inputs(valid, 64, 6144, rs=40.0, hs=40.0, ws=3.0, wb=0.0)
    _check(dev, res, hid, w, 1e-5, gated_at=valid)
    _check(dev, res, hid, w, 1e-6, gated_at=valid, norm_gated=True)


@pytest.mark.parametrize("dim", [128, 1152, 2880 // 128 * 128, 8192])
def test_other_widths_and_contiguous_scales(dev, dim):
    res, hid, w = _inputs(dim, 37, dim, rs=1.0, hs=1.0, ws=0.5)
    _check(dev, res, hid, w, 1e-5, tma=False)


def test_fused_equals_norm_then_standalone_quantiser(dev):
    """The reference's contract for the fused op, with this build's own unfused pair."""
    from batchgen_amd._lib import check, lib, ptr, stream
    res, hid, w = _inputs(11, 200, 7168)
    normed, q, s = _check(dev, res, hid, w, 1e-5, tma=False)
    rows, h = normed.shape
    # (a) the same entry point without the cast is the unfused add + RMSNorm
    res2 = res.clone().to(dev)
    normed2 = torch.empty_like(res2)
    hid_d, w_d = hid.to(dev), w.to(dev)
    check(lib().bgmoe_add_rmsnorm_fp8_quant(ptr(res2), ptr(hid_d), ptr(w_d), rows, h, 1e-5, ptr(normed2), None,
                                            None, 0, 0, None, None, None, stream()))
    assert torch.equal(normed2, normed)
    # (b) the standalone row quantiser on that output gives the fused bytes and scales
    y = torch.empty((rows, h), dtype=torch.uint8, device=dev)
    sc = torch.empty((rows, h // 128), dtype=torch.float32, device=dev)
    check(lib().bgmoe_act_quant_rows(ptr(normed2), rows, h, ptr(y), ptr(sc), h // 128, 1, stream()))
    assert torch.equal(y, q.view(torch.uint8)) and torch.equal(sc, s)


def test_3d_layer_shape_and_argument_errors(dev):
    res, hid, w = _inputs(5, 6, 6144)
    normed, r, q, s = fused(res.view(6, 1, 6144).to(dev), hid.view(6, 1, 6144).to(dev), w.to(dev), 1e-5,
                            scale_tma_aligned=True)
    n_o, r_o, y_o, s_o = onq.add_rmsnorm_fp8_quant(res, hid, w, 1e-5)
    assert tuple(normed.shape) == (6, 1, 6144) and tuple(q.shape) == (6, 6144)
    assert np.array_equal(normed.float().cpu().numpy().reshape(6, 6144), n_o)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), y_o)
    d = lambda t: t.to(dev)
    nv = torch.tensor([4], dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError):
        fused(d(res), d(hid), d(w), 1e-5, norm_num_valid_tokens=nv)                       # norm gate alone
    with pytest.raises(RuntimeError):
        fused(d(res), d(hid), d(w), 1e-5, norm_num_valid_tokens=nv, quant_num_valid_tokens=nv.clone())
    with pytest.raises(RuntimeError):
        fused(d(res[:, :1000]), d(hid[:, :1000]), d(w[:1000]), 1e-5)                      # width not a 128 multiple
    with pytest.raises(RuntimeError):
        fused(d(res).float(), d(hid), d(w), 1e-5)                                         # dtype
    with pytest.raises(RuntimeError):
        fused(d(res), d(hid), d(w), 1e-5, row_valid_mask=torch.ones(5, dtype=torch.bfloat16, device=dev))
    out = fused(d(res[:0]), d(hid[:0]), d(w), 1e-5)
    assert out[2].shape == (0, 6144)


def test_full_size_prefill_rows(dev):
    """16384 rows of 7168: determinism, row-position independence, and a sample of rows against the oracle."""
    rows, dim = 16384, 7168
    g = torch.Generator().manual_seed(77)
    res = (torch.randn(rows, dim, generator=g) * 0.9).to(torch.bfloat16)
    hid = (torch.randn(rows, dim, generator=g) * 0.4).to(torch.bfloat16)
    w = (torch.randn(dim, generator=g) * 0.3 + 1.0).to(torch.bfloat16)
    res_d, hid_d, w_d = res.to(dev), hid.to(dev), w.to(dev)
    n1, r1, q1, s1 = fused(res_d.clone(), hid_d, w_d, 1e-5)
    n2, r2, q2, s2 = fused(res_d.clone(), hid_d, w_d, 1e-5)
    assert torch.equal(n1, n2) and torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s1, s2)
    perm = torch.randperm(rows, generator=g).to(dev)
    n3, r3, q3, s3 = fused(res_d[perm].contiguous(), hid_d[perm].contiguous(), w_d, 1e-5)
    assert torch.equal(n3, n1[perm]) and torch.equal(r3, r1[perm]) and torch.equal(s3, s1[perm])
    assert torch.equal(q3.view(torch.uint8), q1.view(torch.uint8)[perm])
    sample = [0, 1, rows // 2, rows - 1]
    n_o, r_o, y_o, s_o = onq.add_rmsnorm_fp8_quant(res[sample], hid[sample], w, 1e-5)
    idx = torch.tensor(sample, device=dev)
    assert np.array_equal(n1[idx].float().cpu().numpy(), n_o) and np.array_equal(r1[idx].float().cpu().numpy(), r_o)
    assert np.array_equal(q1.view(torch.uint8)[idx].cpu().numpy(), y_o)
    assert np.array_equal(s1[idx].cpu().numpy(), s_o)
