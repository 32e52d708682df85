"""The FP8 layer end to end on the CPU emulator: the package's own host code (``Fp8MoELayer``: buffers, descriptor
tables, the C layer driver behind it) with CPU tensors standing for device memory, every kernel of the chain
(router with its DPP reductions, one-launch index + quantise + scatter, both grouped GEMMs, combine) run by
tests/emu.  Checked against the oracle exactly as the GPU test of the layer does it."""
import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from oracle import gemm as og
from oracle import layer as ol
from tests import emu


@pytest.fixture
def on_emulator(monkeypatch):
    return emu.run_package_on_emulator(monkeypatch)


def _rcfg(cfg):
    return dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf)


CASES = {
    "masked_folded_shared": wl.scaled(wl.CONFIGS[1], n_tokens=48, hidden=256, inter=128, shared_inter=128, max_tokens=48),
    "masked_unfolded_shared": wl.scaled(wl.CONFIGS[1], n_tokens=40, hidden=256, inter=256, shared_inter=128, max_tokens=40),
    "ragged": wl.scaled(wl.CONFIGS[2], n_tokens=300, hidden=256, inter=128, shared_inter=128),
}


def check_layer(layer, out, cfg, inp, w, sh):
    ref = ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(), _rcfg(cfg), wl.weights_to_numpy(w),
                           cfg.expert_start, cfg.e_local, layout=cfg.layout, max_tokens=cfg.max_tokens,
                           row_align=cfg.row_align, shared=wl.weights_to_numpy(sh))
    el = cfg.e_local
    assert np.array_equal(layer.topk_ids.numpy(), ref["ids"])
    np.testing.assert_allclose(layer.topk_weights.numpy(), ref["weights"], rtol=2e-7, atol=0)
    assert np.array_equal(layer.expert_counts[:el].numpy(), ref["counts"])
    assert np.array_equal(layer.cu_seqlens[:el].numpy(), ref["cu"][:el])
    assert np.array_equal(layer.topk_pos.numpy(), ref["pos"])
    live = np.zeros(layer.cap_rows, dtype=bool)
    for e in range(el):
        live[ref["cu"][e]:ref["cu"][e] + ref["counts"][e]] = True
    nrows = ref["xq"].shape[0]
    xq, xs = layer.xq[:layer.cap_rows].numpy(), layer.xs[:layer.cap_rows].numpy()
    assert np.array_equal(xq[:nrows][live[:nrows]], ref["xq"][live[:nrows]])
    assert np.array_equal(xs[:nrows][live[:nrows]].view(np.uint32), ref["xs"][live[:nrows]].view(np.uint32))
    assert og.rel_frobenius(out.float().numpy(), ref["out"]) < 1e-2
    hq = layer.hq[:nrows].numpy()[live[:nrows]]
    assert (hq == ref["hq"][live[:nrows]]).mean() > 0.97 if hq.size else True
    return ref


@pytest.mark.parametrize("name", list(CASES))
def test_fp8_layer_on_the_emulator_matches_the_oracle(on_emulator, name):
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = CASES[name]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    layer = Fp8MoELayer(cfg, w, sh, inp["bias"])
    out = layer(inp["x"], inp["logits"]).clone()
    check_layer(layer, out, cfg, inp, w, sh)
    assert torch.equal(out, layer(inp["x"], inp["logits"]))            # reusable, deterministic


def test_bench_measurement_code_on_the_emulator(on_emulator, monkeypatch):
    """bench.py's measurement of both halves of the metric (timed passes, the cache-flushed decode passes, the
    per-kernel timing pass, roofline and traffic objects, the JSON line) run through with configurations 1 and 2
    scaled down and the emulator standing for the GPU: the times mean nothing, the code path and the accounting do."""
    import json
    from types import SimpleNamespace
    import bench
    small = {
        1: wl.scaled(wl.CONFIGS[1], n_tokens=32, hidden=256, inter=128, shared_inter=128, max_tokens=32),
        2: wl.scaled(wl.CONFIGS[2], n_tokens=300, hidden=256, inter=128, shared_inter=128),
    }
    monkeypatch.setattr(bench, "DEVICE", "cpu")
    monkeypatch.setattr(bench, "FLUSH_BYTES", 1 << 20)
    monkeypatch.setitem(wl.CONFIGS, 1, small[1])
    monkeypatch.setitem(wl.CONFIGS, 2, small[2])
    a = SimpleNamespace(steps=2, warmup=1, graph=False, copy_calibration=False, dense_backend=None, tiled_variant=0,
                        tall_min_rows=0, mxfp4_variant=0, fold_gather=False, template=True, no_cpu_baseline=False)
    for config in (1, 2):
        out = bench.measure_layer(a, config, with_cpu=False)
        line = json.loads(json.dumps(out))                       # everything in it serialises
        decode = config == 1
        assert line["unit"] == ("GB/s" if decode else "TFLOP/s") and line["value"] > 0 and line["ms_per_step"] > 0
        assert line["config"]["workload"] == small[config].name and line["n_gpus"] == 1
        roof = line["roofline"]
        assert roof["bound"] == ("hbm" if decode else "mfma") and roof["achieved"] > 0 and 0 < roof["frac"]
        assert ("cache_flushed" in line and "back_to_back" in line) == decode
        if decode:
            assert line["value"] == pytest.approx(line["cache_flushed"]["layer_hbm_GBps"])
            assert line["timing"].startswith("median")
        tl = line["template_layer"]                              # its own gate weights: other routes than the one-call layer's
        assert tl["ms_per_step"] > 0 and 0 < tl["routed_rows"] <= small[config].n_tokens * small[config].top_k
        assert sum(line["expert_counts"][:small[config].e_local]) == line["routed_rows"]
