"""The C-ABI library and the host-side mirror of the reference interface, without a GPU: the library loads,
exports every symbol include/bgmoe.h declares, its structs have the layout the Python binding assumes, the op
modules export the reference extension's names, and the wrappers keep the reference's frozen parameter lists
(tests/contracts/test_pin_moe.py of the reference) and argument policy."""
import ctypes
import inspect
import os
import re
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bgmoe.h")


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(bgmoe_[a-z0-9_]+)\s*\(", src)))


def test_library_loads_and_exports_every_declared_symbol():
    from batchgen_amd import _lib
    import batchgen_amd.moe.fp8_layer  # noqa: F401
    handle = _lib.lib()
    names = _declared_functions()
    assert len(names) >= 25
    for n in names:
        assert hasattr(handle, n), f"libbgmoe.so does not export {n}"
    assert set(_lib.exported_symbols()) <= set(names) | {"bgmoe_last_error"}
    assert handle.bgmoe_version() >= 1


def test_struct_layout_matches_the_header(tmp_path):
    from batchgen_amd import _lib
    from batchgen_amd.moe.fp8_layer import LayerStruct
    from batchgen_amd.moe.mxfp4_layer import Mxfp4LayerStruct
    prog = tmp_path / "sz.c"
    prog.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "bgmoe.h"\n'
                    'int main(){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(bgmoe_fp8_weight),'
                    'sizeof(bgmoe_fp8_act),'
                    'sizeof(bgmoe_moe_fp8_layer), offsetof(bgmoe_moe_fp8_layer, cap_rows),'
                    'offsetof(bgmoe_moe_fp8_layer, gate), offsetof(bgmoe_moe_fp8_layer, out),'
                    'sizeof(bgmoe_mxfp4_weight), sizeof(bgmoe_moe_mxfp4_layer), offsetof(bgmoe_moe_mxfp4_layer, gate),'
                    'offsetof(bgmoe_moe_mxfp4_layer, activation), offsetof(bgmoe_moe_mxfp4_layer, row_pair));'
                    'return 0;}\n')
    exe = tmp_path / "sz"
    subprocess.run(["gcc", f"-I{os.path.join(ROOT, 'include')}", str(prog), "-o", str(exe)], check=True)
    got = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    want = [ctypes.sizeof(_lib.Fp8Weight), ctypes.sizeof(_lib.Fp8Act), ctypes.sizeof(LayerStruct),
            LayerStruct.cap_rows.offset, LayerStruct.gate.offset, LayerStruct.out.offset,
            ctypes.sizeof(_lib.Mxfp4Weight), ctypes.sizeof(Mxfp4LayerStruct), Mxfp4LayerStruct.gate.offset,
            Mxfp4LayerStruct.activation.offset, Mxfp4LayerStruct.row_pair.offset]
    assert got == want


def test_errors_are_reported_without_a_gpu():
    """Argument errors are detected before anything is launched, so they can be exercised on the CPU."""
    from batchgen_amd import _lib
    h = _lib.lib()
    assert h.bgmoe_fused_gate(None, None, 4, 16, 3, 2, 4, 1.0, 0, None, None, None) != 0
    assert b"divisible" in h.bgmoe_last_error()
    assert h.bgmoe_gate_sigmoid_topk(None, 16, None, 4, 16, 3, 1.0, None, 0, None, None, None, 0, None, 0, 0, None) != 0
    assert b"Unsupported k=3" in h.bgmoe_last_error()
    assert h.bgmoe_act_quant_ragged(None, None, None, 4, 10, 128, None, None, 48, None) != 0
    assert b"power of two" in h.bgmoe_last_error()
    assert h.bgmoe_dispatch_scatter_ragged(None, None, 8, 2, 64, ctypes.c_void_p(16), 64, 0, 4, ctypes.c_void_p(16),
                                           None, ctypes.c_void_p(16), ctypes.c_void_p(16), 64, None, 0, None) != 0
    assert b"act_buffer rows" in h.bgmoe_last_error()
    assert h.bgmoe_dispatch_workspace_bytes(2048, 32) == 0 and h.bgmoe_dispatch_workspace_bytes(131072, 32) == 64 * 32 * 4
    assert h.bgmoe_fp8_weight_repack(None, None, 1, 100, 128, None) != 0
    p16 = ctypes.c_void_p(16)
    assert h.bgmoe_dispatch_index_3d(p16, 4, 2, 0, 4, 8, p16, None, p16, None, None, 0, None) != 0
    assert b"null output" in h.bgmoe_last_error()
    assert h.bgmoe_dispatch_index_3d(p16, 4, 2, 0, 4, 0, p16, None, p16, p16, None, 0, None) != 0
    assert b"max_tokens_padded" in h.bgmoe_last_error()
    assert h.bgmoe_mxfp4_fused_s1_gather(p16, 1 << 20, p16, 8, None, None, p16, p16, 4, 64, 128, 4096, p16, None, 0, 0,
                                         None) != 0
    assert b"exceeds 4 GiB" in h.bgmoe_last_error()


def test_tuning_switches_check_their_arguments():
    """The process-wide switches are host-side state: bad values are refused with a message, good ones accepted
    (and the defaults restored here)."""
    from batchgen_amd import _lib
    h = _lib.lib()
    for bad in (-1, 3, 7):
        assert h.bgmoe_set_tiled_variant(bad) != 0 and b"variant" in h.bgmoe_last_error()
    for good in (1, 2, 0):
        assert h.bgmoe_set_tiled_variant(good) == 0
    w8 = ctypes.c_int * 8
    for bad in ([1] + [64] * 7, [0] + [8] * 7, [65] + [8] * 7, [64] * 7 + [1]):
        assert h.bgmoe_set_streamk_xcd_weights(w8(*bad)) != 0, bad
    assert b"32 times the smallest" in h.bgmoe_last_error()
    assert h.bgmoe_set_streamk_xcd_weights(None) != 0
    for good in ([8] * 8, [2, 3] * 4, [23, 21] * 4):
        assert h.bgmoe_set_streamk_xcd_weights(w8(*good)) == 0, good
    assert h.bgmoe_debug_streamk_status(None) != 0
    for bad in (-1, 1, 31):
        assert h.bgmoe_set_skinny_tall_min_rows(bad) != 0 and b"at least 32" in h.bgmoe_last_error()
    for good in (32, 64, 200, 0):
        assert h.bgmoe_set_skinny_tall_min_rows(good) == 0
    for bad in (-1, 0, 1, 5, 7):
        assert h.bgmoe_set_skinny_gemm_stages(bad) != 0 and b"2, 3, 4 or 6" in h.bgmoe_last_error()
    for good in (3, 4, 6, 2):
        assert h.bgmoe_set_skinny_gemm_stages(good) == 0
    for bad in (0, 2, 5):
        assert h.bgmoe_set_skinny_s1_stages(bad) != 0 and b"3 or 4" in h.bgmoe_last_error()
    for good in (4, 3):
        assert h.bgmoe_set_skinny_s1_stages(good) == 0
    for bad in (-1, 4):
        assert h.bgmoe_set_mxfp4_variant(bad) != 0 and b"variant" in h.bgmoe_last_error()
    for good in (1, 2, 3, 0):
        assert h.bgmoe_set_mxfp4_variant(good) == 0


def test_loader_and_op_names():
    from batchgen_amd.kernels import load_extension
    want = {
        "batchgen_kernels.common._C_mgn_ops": ["moe_fused_gate", "fused_moe_token_dispatch", "compact_expert_data",
                                               "expert_bincount"],
        "batchgen_kernels.moe._C_routing": ["gate_sigmoid_topk", "gate_sigmoid_topk_warp", "dispatch_count_gather",
                                            "reduce_weighted_scatter"],
        "batchgen_kernels.moe._C_dispatch_scatter_3d": ["dispatch_scatter_3d", "dispatch_scatter_ragged",
                                                        "reduce_weighted_scatter", "reduce_weighted_scatter_fp32",
                                                        "reduce_weighted_scatter_bf16_ordered"],
        "batchgen_kernels.moe._C_fp8_blockwise_ops": ["act_quant_3d", "act_quant_ragged", "silu_mul_3d",
                                                      "fused_silu_quant_3d"],
        "batchgen_kernels.moe._C_fp8_blockwise_gemm": ["fp8_blockwise_grouped_gemm", "fp8_blockwise_fused_s1",
                                                       "fp8_blockwise_grouped_gemm_ptrs",
                                                       "fp8_blockwise_fused_s1_ptrs",
                                                       "fp8_blockwise_prepare_s1_s3_tma"],
    }
    for mod, names in want.items():
        m = load_extension(mod)
        for n in names:
            assert callable(getattr(m, n)), f"{mod}.{n}"
    with pytest.raises(ImportError):
        load_extension("batchgen_kernels.moe._C_not_built")


# frozen parameter lists of the reference's Python wrappers (tests/contracts/test_pin_moe.py:63-140, 321-368)
PINS = {
    ("batchgen_amd.moe.dispatch_scatter_3d", "dispatch_scatter_3d"):
        ["x", "topk_indices", "act_buffer", "expert_start", "num_local_experts", "max_tokens_padded",
         "expert_counts", "expert_counters", "topk_pos"],
    ("batchgen_amd.moe.dispatch_scatter_3d", "dispatch_scatter_ragged"):
        ["x", "topk_indices", "act_buffer", "expert_start", "num_local_experts", "expert_counts",
         "expert_counters", "topk_pos", "cu_seqlens", "row_align"],
    ("batchgen_amd.moe.dispatch_scatter_3d", "reduce_weighted_scatter"):
        ["expert_output", "topk_pos", "topk_weights", "N", "H", "K", "output"],
    ("batchgen_amd.moe.dispatch_scatter_3d", "reduce_weighted_scatter_fp32"):
        ["expert_output", "topk_pos", "topk_weights", "N", "H", "K", "output"],
    ("batchgen_amd.moe.routing.cuda_routing", "dispatch_count_gather_cuda"):
        ["x", "topk_indices", "expert_start", "num_local_experts", "expert_counts", "expert_offsets",
         "expert_counters", "dispatched_x", "topk_pos", "num_valid_tokens"],
    ("batchgen_amd.moe.routing.cuda_routing", "gate_sigmoid_topk_cuda"):
        ["router_logits", "e_score_correction", "k", "routed_scaling_factor", "topk_indices", "topk_weights",
         "num_valid_tokens", "latent_out", "latent_offset", "rank_token_counts", "rows_per_rank"],
    ("batchgen_amd.moe.routing.cuda_routing", "gate_sigmoid_topk_warp_cuda"):
        ["router_logits", "e_score_correction", "k", "routed_scaling_factor", "topk_indices", "topk_weights",
         "num_valid_tokens", "rank_token_counts", "rows_per_rank"],
    ("batchgen_amd.moe.grouped_fp8_blockwise_moe", "grouped_fp8_blockwise_gemm"):
        ["x_fp8", "weight_3d", "seqlens", "cu_seqlens", "x_scale", "w_scale_3d", "num_seq_per_group_avg", "output",
         "tma_desc", "tma_plan"],
    ("batchgen_amd.moe.grouped_fp8_blockwise_moe", "grouped_fp8_blockwise_fused_s1"):
        ["x_fp8", "gate_weight_3d", "up_weight_3d", "seqlens", "cu_seqlens", "x_scale", "gate_w_scale_3d",
         "up_w_scale_3d", "num_seq_per_group_avg", "output", "tma_desc", "tma_plan"],
}


@pytest.mark.parametrize("key", list(PINS))
def test_wrapper_signatures_are_the_reference_ones(key):
    import importlib
    mod, name = key
    fn = getattr(importlib.import_module(mod), name)
    assert list(inspect.signature(fn).parameters) == PINS[key]


def test_gate_padding_argument_policy():
    """cuda_routing.py:102-121 of the reference: ValueError before any launch."""
    import torch
    from batchgen_amd.moe.routing import gate_sigmoid_topk_cuda, gate_sigmoid_topk_warp_cuda
    lg, b = torch.zeros(4, 16), torch.zeros(16)
    one = torch.zeros(1, dtype=torch.int32)
    rc = torch.zeros(2, dtype=torch.int64)
    with pytest.raises(ValueError):
        gate_sigmoid_topk_cuda(lg, b, 4, 1.0, num_valid_tokens=one, rank_token_counts=rc, rows_per_rank=2)
    with pytest.raises(ValueError):
        gate_sigmoid_topk_cuda(lg, b, 4, 1.0, rank_token_counts=rc)
    with pytest.raises(ValueError):
        gate_sigmoid_topk_cuda(lg, b, 4, 1.0, rank_token_counts=rc, rows_per_rank=0)
    with pytest.raises(ValueError):
        gate_sigmoid_topk_cuda(lg, b, 4, 1.0, rows_per_rank=2)
    with pytest.raises(TypeError):
        gate_sigmoid_topk_warp_cuda(lg.double(), b, 4, 1.0)
    with pytest.raises(ValueError):
        gate_sigmoid_topk_warp_cuda(torch.zeros(4, 300), torch.zeros(300), 4, 1.0)
    with pytest.raises(TypeError):
        gate_sigmoid_topk_warp_cuda(lg, b, 4, 1.0, topk_indices=torch.zeros(4, 4, dtype=torch.int16))


def test_tile_m_buckets_and_plan_checks():
    import torch
    from batchgen_amd.moe import grouped_fp8_blockwise_moe as g
    assert [g.grouped_fp8_tile_m(v) for v in (1, 16, 17, 32, 33, 48, 64, 500)] == [16, 16, 32, 32, 64, 64, 64, 64]
    a, b = torch.zeros(4, 128), torch.zeros(4, 256)
    plan = g.GroupedFp8TmaPlan(None, None, None, None, 16, 1, 2, a.data_ptr(), b.data_ptr(), 0, 0, 4, 128, 256, 0, 0)
    sl, cu = torch.zeros(1, dtype=torch.int32), torch.zeros(2, dtype=torch.int32)
    with pytest.raises(ValueError):
        g._check_plan(plan, "s1", a, None, sl, cu, 16)                 # no output buffer
    with pytest.raises(ValueError):
        g._check_plan(plan, "s1", a, b, sl, cu, 16)                    # other seqlens tensors
    with pytest.raises(ValueError):
        g._check_plan(plan, "s1", a, b, sl, cu, 64)                    # other TileM


def test_ragged_capacity_formula():
    from batchgen_amd.moe.dispatch_scatter_3d import ragged_row_capacity
    assert ragged_row_capacity(256, 8, 32, 64) == (2048 + 63 * 32) // 64 * 64
    assert ragged_row_capacity(1, 2, 32, 64) == (2 + 63 * 2) // 64 * 64
    assert ragged_row_capacity(16384, 8, 32, 128) == (131072 + 127 * 32) // 128 * 128


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_config4_routing_has_the_skew_the_baseline_names():
    """Config 4 is the skewed workload: Zipf-distributed expert popularity with roughly 30% of the experts
    receiving no token and a hot expert with thousands of rows (the empty-group and long-group paths)."""
    import numpy as np
    from batchgen_amd import workloads as wl
    from oracle import layer as ol
    cfg = wl.CONFIGS[4]
    inp = wl.make_inputs(cfg, "cpu")
    ids, _ = ol.route(inp["logits"].numpy(), inp["bias"].numpy(),
                      dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf))
    counts = np.bincount(ids.ravel(), minlength=cfg.n_experts)
    empty = float((counts == 0).mean())
    assert 0.2 <= empty <= 0.4, empty
    assert counts.max() > 2000
    assert counts.sum() == cfg.n_tokens * cfg.top_k


def test_bf16_linear_workspace_bound_covers_every_row_count():
    """The layer sizes its GEMM workspace once: the bound must cover what the library asks for at every row count
    up to the maximum (the launch shape, and with it the need, is not monotonic in the rows)."""
    from batchgen_amd._lib import lib
    from batchgen_amd.moe.latent import bf16_linear_workspace_bytes
    for n_max, h, e in [(512, 7168, 4096), (512, 2048, 7168), (96, 1024, 1024), (64, 7168, 4096), (300, 3584, 7168)]:
        bound = bf16_linear_workspace_bytes(n_max, h, e)
        for n in range(1, n_max + 1):
            assert lib().bgmoe_router_gemm_workspace_bytes(n, h, e) <= bound, (n_max, h, e, n)


def test_moe_base_template_names_and_config_mapping():
    """The template class carries the reference's names (batchgen/moe/moe_base.py:75-264) and maps a model
    configuration object to this package's workload description; a world of more than one rank is refused."""
    from types import SimpleNamespace
    from batchgen_amd.moe import moe_base as mb
    for name in ("gate", "expert_compute_persistent", "expert_compute_mixed", "shared_expert_forward", "forward",
                 "_forward_decode", "_forward_prefill", "init_buffer_manager", "init_num_tokens",
                 "set_num_tokens_per_rank"):
        assert callable(getattr(mb.MoEBase, name)), name
    cfg = SimpleNamespace(hidden_size=7168, moe_intermediate_size=2048, n_routed_experts=256, num_experts_per_tok=8,
                          n_group=8, topk_group=4, routed_scaling_factor=2.5, norm_topk_prob=True, n_shared_experts=1)
    base = mb.MoEBase(cfg)
    assert (base.rank, base.world_size, base.experts_per_rank, base.routed_expert_end_idx) == (0, 1, 256, 256)
    assert base.num_persistent_local_experts == 256 and base.enable_ep_offloading is False
    with pytest.raises(NotImplementedError):
        base.gate(None)
    m = mb._moe_config(cfg, 256, 32, 64, True)
    assert (m.hidden, m.inter, m.n_experts, m.e_local, m.expert_start, m.top_k, m.n_group, m.topk_group) == \
        (7168, 2048, 256, 32, 64, 8, 8, 4)
    assert (m.layout, m.max_tokens, m.shared_inter, m.rsf) == ("masked", 256, 2048, 2.5)
    big = mb._moe_config(cfg, 16384, 256, 0, False)
    assert (big.layout, big.row_align, big.shared_inter) == ("ragged", 128, 0)


def test_bench_accounting_and_traffic_records(tmp_path, monkeypatch):
    """The figures bench.py divides by the measured times: algorithmic bytes and flops of config 1 worked out by
    hand for a given routing draw (19 active experts, 297 routed rows), and the rule for `roofline.traffic`: a
    record under profiles/ counts only while every kernel source it names still has the recorded SHA-256."""
    import hashlib
    import json
    import bench
    from batchgen_amd import workloads as wl
    cfg = wl.CONFIGS[1]
    weights = 3 * 7168 * 2048 + 3 * 56 * 16 * 4                    # gate, up, down bytes + their 128x128 block scales
    by_hand = 19 * weights + weights + 256 * 7168 * 2 * 2 + 297 * (7168 + 2048) * 3
    assert wl.algorithmic_bytes_fp8(cfg, 19, 297) == by_hand == 896570368
    assert wl.flops_routed(cfg, 297) == 297 * 6 * 7168 * 2048
    src = tmp_path / "kernel.hip"
    src.write_text("v1")
    (tmp_path / "profiles").mkdir()
    rec = dict(key="layer:1", fetch_bytes=1000, write_bytes=24, commit="abc1234",
               sources={"kernel.hip": hashlib.sha256(b"v1").hexdigest()})
    (tmp_path / "profiles" / "p.md").write_text(f"text\n<!-- traffic-record: {json.dumps(rec)} -->\n")
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    got, where = bench.traffic_record("layer:1")
    assert got == 1024 and "abc1234" in where
    assert bench.traffic_record("layer:2") == (None, "no record under profiles/")
    src.write_text("v2")
    got, where = bench.traffic_record("layer:1")
    assert got is None and "kernel.hip changed" in where and "abc1234" in where


def test_moe_base_decode_template_on_a_toy_layer():
    """The template's own steps (pad to the announced capacity, gate, expert compute on the padded rows, live rows
    + shared expert, shapes, the shared buffer manager, the overflow error) with a layer whose pieces are plain
    tensor arithmetic, on the CPU."""
    from types import SimpleNamespace
    from batchgen_amd.moe import moe_base as mb
    seen = {}

    class Toy(mb.MoEBase):
        def gate(self, x):
            seen["gate_rows"] = x.shape[0]
            seen["pad_is_zero"] = bool((x[5:] == 0).all())
            return torch.zeros(x.shape[0], 2, dtype=torch.int32), torch.ones(x.shape[0], 2)

        def expert_compute_persistent(self, global_x, topk_idx, topk_weight):
            return global_x * topk_weight.sum(dim=1, keepdim=True).to(global_x.dtype)     # 2 x

        def shared_expert_forward(self, identity):
            return identity * 3

    cfg = SimpleNamespace(hidden_size=16, num_experts_per_tok=2, n_routed_experts=4, phase="decode")
    layer = Toy(cfg)
    x = torch.randn(5, 16).to(torch.bfloat16)
    with pytest.raises(RuntimeError):
        layer(x)                                                       # capacity not announced
    layer.init_num_tokens(8)
    out = layer(x)
    assert seen == {"gate_rows": 8, "pad_is_zero": True}
    assert torch.equal(out, x * 2 + x * 3) and out.dtype == torch.bfloat16
    assert layer(x.view(1, 5, 16)).shape == (1, 5, 16)
    with pytest.raises(RuntimeError, match="buffer overflow"):
        layer(torch.zeros(9, 16, dtype=torch.bfloat16))
    Toy.init_buffer_manager(8, 1, 16, torch.device("cpu"))
    try:
        assert mb.MoEBase._buffer_mgr is None, "the manager belongs to the class it was set on"
        Toy._buffer_mgr.all_tokens.fill_(7.0)                          # stale rows of an earlier call
        assert torch.equal(layer(x), out) and seen["pad_is_zero"]
        layer.set_num_tokens_per_rank(12)
        assert Toy._buffer_mgr.num_tokens_per_rank == 12 and Toy._buffer_mgr.all_tokens.shape == (12, 16)
        assert torch.equal(layer(x), out) and seen["gate_rows"] == 12
    finally:
        Toy._buffer_mgr = None
    mgr = mb.MoEBufferManager(4, 3, 16, torch.device("cpu"))           # both buffers are views of one allocation
    assert mgr.all_tokens.shape == (12, 16) and mgr.padded_hidden_states.shape == (4, 16)
    assert mgr.padded_hidden_states.data_ptr() == mgr.all_tokens.data_ptr() + 12 * 16 * 2
    before = mgr.all_tokens.data_ptr()
    mgr.resize_if_needed(3)
    assert mgr.all_tokens.data_ptr() == before and mgr.num_tokens_per_rank == 4      # never shrinks
    mgr.resize_if_needed(6)
    assert mgr.all_tokens.shape == (18, 16) and mgr.padded_hidden_states.shape == (6, 16)
    layer.enable_ep_offloading = True
    with pytest.raises(NotImplementedError):
        layer(x)                                                       # the toy has no mixed path
    cfg.phase = "prefill"
    with pytest.raises(NotImplementedError):
        layer(x)


def test_build_gate_rejects_flat_memory_instructions(tmp_path):
    """The streaming kernels' device assembly is scanned on every build: a flat load, store or atomic fails it (and
    removes the object), directives and comments that merely contain the word do not."""
    from batchgen_amd import build as b

    class Done:
        returncode = 0

        def communicate(self):
            return "", ""

    def run(text):
        obj = tmp_path / "k.o"
        obj.write_bytes(b"x")
        (tmp_path / "k.s").write_text(text)
        b._check_no_flat("k.hip", str(obj), Done())
        return obj

    ok = run("\t.amdhsa_user_sgpr_flat_scratch_init 0\n\tglobal_store_dwordx2 v[0:1], v[2:3], off ; not flat_store\n")
    assert ok.exists() and not (tmp_path / "k.s").exists()
    with pytest.raises(RuntimeError, match="flat_store_dwordx2"):
        run("\tglobal_load_dwordx4 v[0:3], v[4:5], off\n\tflat_store_dwordx2 v[0:1], v[2:3]\n")
    assert not (tmp_path / "k.o").exists()


def test_isa_audit_reads_rings_and_flat_instructions():
    """The assembly reader behind `python -m batchgen_amd.isa_audit`: an innermost loop with barriers and matrix
    instructions is a ring whose waits are listed in order; an enclosing loop is not reported again; flat memory
    instructions are named."""
    from batchgen_amd.isa_audit import audit
    step = "\ts_waitcnt vmcnt(4)\n\ts_barrier\n\tglobal_load_dwordx4 v[0:3], v[4:5], off\n" + \
           "\ts_waitcnt vmcnt(10)\n" + "\tv_mfma_f32_16x16x128_f8f6f4 a[0:3], v[0:7], v[8:15], a[0:3]\n" * 4
    asm = ("_Z6kernelv: ; @_Z6kernelv\n.LBB0_1:\n\tflat_store_dwordx2 v[0:1], v[2:3]\n.LBB0_2:\n" + step * 2 +
           "\ts_cbranch_scc1 .LBB0_2\n\ts_waitcnt vmcnt(0)\n\ts_cbranch_vccnz .LBB0_1\n\ts_endpgm\n")
    (rec,) = audit(asm)
    assert rec["kernel"] == "_Z6kernelv" and rec["flat"] == ["flat_store_dwordx2"]
    (ring,) = rec["rings"]
    assert ring["barriers"] == 2 and ring["mfma"] == 8 and ring["waits"] == [4, 10, 4, 10]
