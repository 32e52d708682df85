"""Host helpers of the two DeepGEMM-shaped chains (CPU only): the row -> group map against a literal loop, the
dense stack view and its refusals, the scale transpose shim, the masked kernel's row-count hint."""
import numpy as np
import pytest
import torch

from batchgen_amd.moe import grouped_fp8_deepgemm_moe as dg
from batchgen_amd.moe import moe_deepgemm_masked as mk


def _loop_layout(seq, cu, total, ids=None):
    ref = np.full(total, -1, dtype=np.int32)
    for g in range(len(seq)):
        ref[cu[g]:cu[g] + seq[g]] = g if ids is None else ids[g]
    return ref


@pytest.mark.parametrize("align", [64, 128])
def test_build_grouped_layout_equals_a_literal_loop(align):
    rng = np.random.default_rng(align)
    for _ in range(20):
        groups = int(rng.integers(1, 12))
        seq = rng.integers(0, 300, groups) * (rng.random(groups) > 0.3)
        cu = np.concatenate([[0], np.cumsum((seq + align - 1) // align * align)])
        total = int(cu[-1]) + int(rng.integers(0, 200))
        ids = rng.permutation(groups).astype(np.int32)
        st, ct = torch.from_numpy(seq.astype(np.int32)), torch.from_numpy(cu.astype(np.int32))
        assert np.array_equal(dg.build_grouped_layout(st, ct, total, alignment=align).numpy(), _loop_layout(seq, cu, total))
        got = dg.build_grouped_layout(st, ct, total, alignment=align, group_ids=torch.from_numpy(ids), validate=False)
        assert np.array_equal(got.numpy(), _loop_layout(seq, cu, total, ids))


def test_build_grouped_layout_refusals():
    seq = torch.tensor([5, 3], dtype=torch.int32)
    with pytest.raises(ValueError):
        dg.build_grouped_layout(seq, torch.tensor([0, 64, 128], dtype=torch.int32), 200)            # 64 is not 128-aligned
    dg.build_grouped_layout(seq, torch.tensor([0, 64, 128], dtype=torch.int32), 200, alignment=64)
    with pytest.raises(ValueError):
        dg.build_grouped_layout(seq, torch.tensor([0, 128, 256], dtype=torch.int32), 200)           # exceeds the rows
    with pytest.raises(ValueError):
        dg.build_grouped_layout(seq, torch.tensor([0, 128], dtype=torch.int32), 200)
    with pytest.raises(ValueError):
        dg.build_grouped_layout(seq, torch.tensor([0, 128, 256], dtype=torch.int32), 300, group_ids=torch.zeros(3, dtype=torch.int32))
    assert dg.deepgemm_m_alignment() == 128


def test_dense_group_view_and_scale_shim():
    arena = torch.arange(4 * 6 * 8, dtype=torch.float32)
    members = [arena[i * 48:(i + 1) * 48].view(6, 8) for i in range(4)]
    v = dg.dense_group_view(members)
    assert v.shape == (4, 6, 8) and v.data_ptr() == arena.data_ptr() and torch.equal(v, arena.view(4, 6, 8))
    with pytest.raises(ValueError):
        dg.dense_group_view([])
    with pytest.raises(ValueError):
        dg.dense_group_view([members[0], members[2]])                                                # a gap
    with pytest.raises(ValueError):
        dg.dense_group_view([members[0], members[1].clone()])                                        # another allocation
    with pytest.raises(ValueError):
        dg.dense_group_view([members[0], members[1].view(8, 6)])
    with pytest.raises(ValueError):
        dg.dense_group_view([arena.view(4, 48).t()])                                                  # not contiguous
    with pytest.raises(ValueError):
        dg.dense_group_view([arena[96:144].view(6, 8), arena[144:192].view(6, 8), arena[144:192].view(6, 8)])
    s = torch.arange(3 * 10, dtype=torch.float32).view(3, 10)
    t = dg._scale_rows_first(s, 7)
    assert t.shape == (7, 3) and t.is_contiguous() and torch.equal(t, s[:, :7].t())
    with pytest.raises(ValueError):
        dg._scale_rows_first(s, 11)


def test_masked_chain_host_contract():
    assert mk.expected_m_per_expert(local_rows=128, world_size=1, topk=1, num_experts_global=8) == 17
    assert mk.expected_m_per_expert(local_rows=32, world_size=8, topk=8, num_experts_global=256) == 9
    with pytest.raises(ValueError):
        mk.expected_m_per_expert(local_rows=32, world_size=8, topk=0, num_experts_global=256)
    good = torch.zeros(4, 7, 8).transpose(1, 2)
    assert mk.is_mn_major_tma_aligned(good) and good.shape == (4, 8, 7)
    assert not mk.is_mn_major_tma_aligned(good.contiguous())
    assert not mk.is_mn_major_tma_aligned(torch.zeros(4, 7, 6).transpose(1, 2))                       # 6 rows: not padded to 4
    assert not mk.is_mn_major_tma_aligned(good.double())
    with pytest.raises(RuntimeError, match="MN-major"):
        mk.require_mn_major_tma_aligned(good.contiguous(), "x_scales")
