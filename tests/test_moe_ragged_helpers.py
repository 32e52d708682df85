"""Host-side helpers of the ragged workspace module (no GPU): values worked out by hand from the definitions."""
import pytest
import torch


def _mod():
    from batchgen_amd.moe import moe_ragged
    return moe_ragged


def test_tile_hint_and_capacity():
    m = _mod()
    assert m.gemm_tilem_avg(256, 8, 256) == 8
    assert m.gemm_tilem_avg(1, 8, 256) == 1                       # 8 // 256 = 0, floored at 1
    assert m.gemm_tilem_avg_effective(4096, 8, 256) == 128
    with pytest.raises(ValueError):
        m.gemm_tilem_avg(4, 8, 0)
    assert m.ragged_row_capacity(256, 8, 32) == 4096              # 2048 + 32 * 63 = 4064 -> next multiple of 128
    assert m.ragged_row_capacity(100, 8, 32, 128) == 4864         # 800 + 32 * 127 = 4864 = 38 * 128
    assert m.ragged_row_capacity(0, 8, 1, 64) == 128              # 63 -> 128
    q, s = m.make_quant_buffers(10, 256, torch.device("cpu"))
    assert q.dtype == torch.uint8 and tuple(q.shape) == (10, 256)
    assert s.dtype == torch.float32 and tuple(s.shape) == (2, 10) and not s.any()
    with pytest.raises(ValueError):
        m.make_quant_buffers(10, 200, torch.device("cpu"))


def test_recv_count_histogram():
    m = _mod()
    assert m.recv_count_histogram_width(256, 64) == 7             # steps, rows, tiles 0..4
    assert m.recv_count_histogram_width(100, 64) == 5
    with pytest.raises(ValueError):
        m.recv_count_histogram_width(0, 64)
    hist = torch.zeros(7, dtype=torch.int64)
    assert m.format_recv_count_histogram(hist, 64) == "recv-count histogram: no accumulation yet"
    counts = torch.tensor([0, 1, 64, 65, 256, 300], dtype=torch.int32)   # tiles 0, 1, 1, 2, 4, 5 -> clamped to 4
    m.accumulate_recv_count_histogram(hist, counts, 64)
    assert hist.tolist() == [1, 686, 1, 2, 1, 0, 2]
    m.accumulate_recv_count_histogram(hist, counts, 64)
    assert hist.tolist() == [2, 1372, 2, 4, 2, 0, 4]
    line = m.format_recv_count_histogram(hist, 64)
    assert "layer-steps=2 expert-slots=12 rows=1372" in line and "over_one_tile=6(50.000%)" in line
    assert "0t=2(16.67%) 1t=4(33.33%) 2t=2(16.67%) 4t=4(33.33%)" in line
    with pytest.raises(RuntimeError):
        m.accumulate_recv_count_histogram(torch.zeros(7, dtype=torch.int32), counts, 64)
    with pytest.raises(RuntimeError):
        m.accumulate_recv_count_histogram(hist, counts.view(2, 3), 64)


def test_norm_quant_fuse_policy(monkeypatch):
    from batchgen_amd.attention import norm_quant_fuse_policy as p
    assert p.glm5_norm_quant_fuse_enabled() is True
    assert all(p.glm5_norm_quant_fuse_site_enabled(s) for s in p.GLM5_NORM_QUANT_FUSE_SITES)
    with pytest.raises(ValueError):
        p.glm5_norm_quant_fuse_site_enabled("shared")
    monkeypatch.setattr(p, "GLM5_NORM_QUANT_FUSE_DISABLED_SITES", ("q_a",))
    assert not p.glm5_norm_quant_fuse_site_enabled("q_a") and p.glm5_norm_quant_fuse_site_enabled("shared_expert")
    monkeypatch.setattr(p, "GLM5_NORM_QUANT_FUSE_DISABLED_SITES", ("q_b",))
    with pytest.raises(ValueError):
        p.glm5_norm_quant_fuse_site_enabled("q_a")
    monkeypatch.setattr(p, "GLM5_NORM_QUANT_FUSE_DISABLED_SITES", "q_a")
    with pytest.raises(TypeError):
        p.glm5_norm_quant_fuse_site_enabled("q_a")
    monkeypatch.setattr(p, "GLM5_NORM_QUANT_FUSE_DISABLED_SITES", ())
    monkeypatch.setattr(p, "GLM5_NORM_QUANT_FUSE", False)
    assert not p.glm5_norm_quant_fuse_site_enabled("shared_expert")
    monkeypatch.setattr(p, "GLM5_NORM_QUANT_FUSE", 1)
    with pytest.raises(TypeError):
        p.glm5_norm_quant_fuse_enabled()
