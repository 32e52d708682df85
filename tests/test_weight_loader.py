"""Checkpoint tensors -> stacked expert weights: naming, shapes, padding, fused gate/up views, release order."""
import numpy as np
import pytest
import torch

from batchgen_amd.moe import weight_loader as wl_


def _fp8_stacks(g, el, inter, hidden):
    def one(n, k):
        q = torch.randint(0, 255, (el, n, k), generator=g, dtype=torch.uint8)
        q[q == 0x7F] = 0
        q[q == 0xFF] = 0x80                      # no NaN bytes
        s = torch.rand(el, n // 128, k // 128, generator=g) * 0.01 + 1e-3
        return q, s
    w = {}
    w["gate_q"], w["gate_s"] = one(inter, hidden)
    w["up_q"], w["up_s"] = one(inter, hidden)
    w["down_q"], w["down_s"] = one(hidden, inter)
    return w


def _checkpoint(tmp_path, tensors):
    from safetensors.torch import save_file
    half = len(tensors) // 2
    names = sorted(tensors)
    paths = [str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors")]
    save_file({k: tensors[k] for k in names[:half]}, paths[0])
    save_file({k: tensors[k] for k in names[half:]}, paths[1])
    return paths


@pytest.mark.parametrize("pad4,fuse", [(False, False), (True, False), (False, True), (True, True)])
def test_fp8_layer_round_trip_through_safetensors(tmp_path, pad4, fuse):
    g = torch.Generator().manual_seed(1)
    e_total, start, el, hidden, inter = 12, 4, 5, 384, 256          # 3 and 2 scale blocks: pad4 changes both
    w = _fp8_stacks(g, el, inter, hidden)
    sh = _fp8_stacks(g, 1, inter, hidden)
    bias = torch.randn(e_total, generator=g)
    rw = torch.randn(e_total, hidden, generator=g).to(torch.bfloat16)
    ck = wl_.export_fp8_moe_layer("model.layers.3.mlp.", w, sh, bias, rw, expert_start=start)
    assert "model.layers.3.mlp.experts.4.gate_proj.weight_scale_inv" in ck
    assert ck["model.layers.3.mlp.experts.8.down_proj.weight"].dtype == torch.float8_e4m3fn
    src = wl_.SafetensorsSource(_checkpoint(tmp_path, ck))
    assert len(src) == len(ck)
    released = []
    experts = wl_.stack_fp8_experts(src, "model.layers.3.mlp.", range(start, start + el), hidden, inter, "cpu",
                                    scale_pad4=pad4, fuse_gate_up=fuse, release=released.append)
    for k in ("gate_q", "gate_s", "up_q", "up_s", "down_q", "down_s"):
        assert torch.equal(experts[k], w[k]), k
        assert tuple(experts[k].shape) == tuple(w[k].shape)
    assert experts["gate_s"].stride(1) == (4 if pad4 else 3) and experts["down_s"].stride(1) == (4 if pad4 else 2)
    if pad4:   # the padding is zeros
        store = experts["gate_up_s"] if fuse else experts["gate_s"]
        assert float(torch.as_strided(store, (el, store.size(1), 4), store.stride())[..., 3].abs().max()) == 0.0
    if fuse:
        block = experts["gate_up_q"]
        assert tuple(block.shape) == (el, 2 * inter, hidden)
        assert experts["gate_q"].data_ptr() == block.data_ptr()
        assert experts["up_q"].data_ptr() == block.data_ptr() + inter * hidden
        assert torch.equal(block[:, inter:], w["up_q"])
    assert len(released) == 6 * el and released[0].endswith("experts.4.gate_proj.weight")
    # the whole layer in one call
    ex2, sh2, bias2, rw2 = wl_.load_fp8_moe_layer_weights(src, "model.layers.3.mlp.", e_total, start, el, hidden,
                                                          inter, "cpu", shared_inter=inter, scale_pad4=pad4)
    assert torch.equal(sh2["down_q"], sh["down_q"]) and torch.equal(sh2["up_s"], sh["up_s"])
    assert torch.equal(bias2, bias) and torch.equal(rw2, rw)


def test_fp8_loader_errors():
    g = torch.Generator().manual_seed(2)
    w = _fp8_stacks(g, 2, 128, 256)
    ck = wl_.export_fp8_moe_layer("m.", w, None, torch.zeros(4), torch.zeros(4, 256, dtype=torch.bfloat16))
    with pytest.raises(wl_.WeightLayoutError, match="no tensor"):
        wl_.stack_fp8_experts(ck, "m.", [0, 1, 2], 256, 128, "cpu")
    with pytest.raises(wl_.WeightLayoutError, match="expected"):
        wl_.stack_fp8_experts(ck, "m.", [0, 1], 128, 256, "cpu")
    bad = dict(ck)
    bad["m.experts.1.up_proj.weight_scale_inv"] = bad["m.experts.1.up_proj.weight_scale_inv"].double()
    with pytest.raises(wl_.WeightLayoutError, match="fp32"):
        wl_.stack_fp8_experts(bad, "m.", [0, 1], 256, 128, "cpu")
    bad = dict(ck)
    bad["m.experts.0.gate_proj.weight"] = bad["m.experts.0.gate_proj.weight"].view(torch.uint8).to(torch.int32)
    with pytest.raises(wl_.WeightLayoutError, match="float8_e4m3fn"):
        wl_.stack_fp8_experts(bad, "m.", [0, 1], 256, 128, "cpu")
    with pytest.raises(wl_.WeightLayoutError, match="multiples"):
        wl_.stack_fp8_experts(ck, "m.", [0], 250, 128, "cpu")
    with pytest.raises(wl_.WeightLayoutError, match="router"):
        wl_.load_fp8_moe_layer_weights(ck, "m.", 5, 0, 2, 256, 128, "cpu")


def test_mxfp4_stacking_maps_w1_w2_w3():
    g = torch.Generator().manual_seed(3)
    hidden, inter, ids = 64, 96, [7, 9]
    ck, want = {}, {}
    for name, proj, (n, k) in (("gate", "w1", (inter, hidden)), ("down", "w2", (hidden, inter)),
                               ("up", "w3", (inter, hidden))):
        want[name + "_p"] = torch.randint(0, 256, (2, n, k // 2), generator=g, dtype=torch.uint8)
        want[name + "_s"] = torch.randint(100, 140, (2, n, k // 32), generator=g, dtype=torch.uint8)
        for i, e in enumerate(ids):
            ck[f"blk.experts.{e}.{proj}.weight_packed"] = want[name + "_p"][i].clone()
            ck[f"blk.experts.{e}.{proj}.weight_scale"] = want[name + "_s"][i].clone()
    got = wl_.stack_mxfp4_experts(ck, "blk.", ids, hidden, inter, "cpu")
    for k in want:
        assert torch.equal(got[k], want[k]), k
    ck["blk.experts.7.w2.weight_scale"] = ck["blk.experts.7.w2.weight_scale"][:, :-1].contiguous()
    with pytest.raises(wl_.WeightLayoutError, match="uint8"):
        wl_.stack_mxfp4_experts(ck, "blk.", ids, hidden, inter, "cpu")
