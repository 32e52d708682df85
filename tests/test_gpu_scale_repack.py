"""`deepep_ll_scale_repack`: exchange scale block [E, KB, S] -> the grouped GEMM's [KB, E*S] matrix, live span
only.  Contract restated from the reference's tests/test_deepep_ll_scale_repack.py: bit-identical inside each
expert's span, `out` untouched outside it, an impossible count does not copy (here: raises a device flag
instead of trapping), argument checks raise before any launch."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_fp8_blockwise_ops")


def _block(e, kb, s, dev, seed):
    g = torch.Generator().manual_seed(seed)
    bits = torch.randint(-2**31, 2**31 - 1, (e, kb, s), generator=g, dtype=torch.int64).to(torch.int32)
    return bits.view(torch.float32).to(dev)          # arbitrary bit patterns, NaNs included: the copy is bit for bit


@pytest.mark.parametrize("e,kb,s,align", [(32, 48, 128, 64), (8, 56, 256, 128), (3, 1, 4, 4), (16, 16, 192, 64),
                                          (1, 7, 1024, 4)])
def test_span_copied_rest_untouched(dev, ops, e, kb, s, align):
    block = _block(e, kb, s, dev, seed=e * 1000 + kb)
    rng = np.random.default_rng(s)
    counts = rng.integers(0, s + 1, size=e).astype(np.int32)
    counts[0] = s
    if e > 1:
        counts[1] = 0
    out = torch.full((kb, e * s), -123.0, device=dev)
    got = ops.deepep_ll_scale_repack(block.transpose(1, 2), torch.from_numpy(counts).to(dev), out, align)
    assert got is out
    want = np.full((kb, e * s), -123.0, dtype=np.float32).view(np.int32)
    src = block.cpu().numpy().view(np.int32)
    for i in range(e):
        span = -(-int(counts[i]) // align) * align
        want[:, i * s:i * s + span] = src[i, :, :span]
    assert np.array_equal(out.cpu().numpy().view(np.int32), want)
    assert int(ops.deepep_ll_scale_repack_status(dev).item()) == 0


def test_impossible_count_raises_flag_and_copies_nothing(dev, ops):
    e, kb, s = 4, 8, 64
    block = _block(e, kb, s, dev, seed=5)
    flag = ops.deepep_ll_scale_repack_status(dev)
    flag.zero_()
    out = torch.zeros((kb, e * s), device=dev)
    counts = torch.tensor([3, s + 1, -1, s], dtype=torch.int32, device=dev)
    ops.deepep_ll_scale_repack(block.transpose(1, 2), counts, out, 4)
    o = out.cpu().numpy().view(np.int32).reshape(kb, e, s)
    src = block.cpu().numpy().view(np.int32)
    assert np.array_equal(o[:, 0, :4], src[0, :, :4]) and not o[:, 0, 4:].any()
    assert not o[:, 1].any() and not o[:, 2].any()
    assert np.array_equal(o[:, 3], src[3])
    assert int(flag.item()) == 1
    flag.zero_()


def test_argument_checks(dev, ops):
    e, kb, s = 4, 8, 64
    block = _block(e, kb, s, dev, seed=6)
    counts = torch.zeros(e, dtype=torch.int32, device=dev)
    out = torch.zeros((kb, e * s), device=dev)
    view = block.transpose(1, 2)
    with pytest.raises(RuntimeError, match="transposed view"):
        ops.deepep_ll_scale_repack(view.contiguous(), counts, out, 4)
    with pytest.raises(RuntimeError, match="recv_count"):
        ops.deepep_ll_scale_repack(view, counts[:3], out, 4)
    with pytest.raises(RuntimeError, match="recv_count"):
        ops.deepep_ll_scale_repack(view, counts.long(), out, 4)
    with pytest.raises(RuntimeError, match="out must be"):
        ops.deepep_ll_scale_repack(view, counts, out[:, :-4].contiguous(), 4)
    for bad in (0, 6, 48, 128):
        with pytest.raises(RuntimeError, match="span_align"):
            ops.deepep_ll_scale_repack(view, counts, out, bad)
    with pytest.raises(RuntimeError, match="overlap"):
        flat = torch.zeros(2 * e * kb * s, device=dev)
        src = flat[:e * kb * s].view(e, kb, s).transpose(1, 2)
        ops.deepep_ll_scale_repack(src, counts, flat[16:16 + e * kb * s].view(kb, e * s), 4)


def test_repacked_scales_feed_the_grouped_gemm_like_the_block_read_in_place(dev, ops):
    """The [KB, E*S] matrix is the transposed activation-scale layout of the grouped GEMM op; the same GEMM reading
    the exchange's block in place (per-group scale stride) gives identical bytes."""
    from batchgen_amd.moe.moe_deepgemm_masked import fp8_m_grouped_gemm_nt_masked
    from batchgen_amd.kernels import load_extension
    gemm = load_extension("batchgen_kernels.moe._C_fp8_blockwise_gemm")
    e, s, k, n = 4, 64, 512, 256
    g = torch.Generator().manual_seed(9)
    a = torch.randint(0, 256, (e, s, k), generator=g, dtype=torch.int32).to(torch.uint8)
    a[(a & 0x7F) == 0x7F] = 0                            # no NaN bytes
    b = torch.randint(0, 256, (e, n, k), generator=g, dtype=torch.int32).to(torch.uint8)
    b[(b & 0x7F) == 0x7F] = 0
    sa_block = (torch.rand(e, k // 128, s, generator=g) * 0.01 + 1e-3).to(dev)
    sb = (torch.rand(e, n // 128, k // 128, generator=g) * 0.01 + 1e-3).to(dev)
    counts = torch.tensor([64, 0, 17, 33], dtype=torch.int32, device=dev)
    a, b = a.to(dev).view(torch.float8_e4m3fn), b.to(dev).view(torch.float8_e4m3fn)
    d_place = torch.zeros(e, s, n, dtype=torch.bfloat16, device=dev)
    fp8_m_grouped_gemm_nt_masked((a, sa_block.transpose(1, 2)), (b, sb), d_place, counts, 16)
    packed = torch.zeros(k // 128, e * s, device=dev)
    ops.deepep_ll_scale_repack(sa_block.transpose(1, 2), counts, packed, 64)
    d_packed = torch.zeros(e * s, n, dtype=torch.bfloat16, device=dev)
    cu = (torch.arange(e + 1, dtype=torch.int32, device=dev) * s).contiguous()
    gemm.fp8_blockwise_grouped_gemm(a.view(e * s, k), b, counts, cu, packed, sb, 16, output=d_packed)
    assert torch.equal(d_packed.view(e, s, n), d_place)
