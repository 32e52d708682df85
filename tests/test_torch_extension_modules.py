"""The PyTorch C++ extension modules (batchgen_amd/ext/bgmoe_torch.cc) import under the reference's module names
and export its op names with its keyword names (batchgen_kernels/src/moe/routing/routing_extension.cc:11-137,
mgn/mgn_extension.cc:17-62, dispatch_scatter_3d.cu:671-683, fp8_blockwise/fp8_blockwise_gemm.cu:1253-1299,
fp8_blockwise_ops.cu:800-814, attention/csrc/add_rmsnorm_fp8_quant.cu:553-566).  No compute without a GPU."""
import importlib
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXT_ROOT = os.path.join(ROOT, "batchgen_amd", "ext", "build")

OPS = {
    "batchgen_kernels.moe._C_routing": {
        "dispatch_count_gather": ["x", "topk_indices", "expert_start", "num_local_experts", "expert_counts", "expert_offsets",
                                  "expert_counters", "dispatched_x", "topk_pos", "rank_token_counts", "rows_per_rank"],
        "gate_sigmoid_topk": ["router_logits", "e_score_correction", "k", "routed_scaling_factor", "topk_indices",
                              "topk_weights", "num_valid_tokens", "latent_out", "latent_offset", "rank_token_counts",
                              "rows_per_rank"],
        "gate_sigmoid_topk_warp": ["router_logits", "e_score_correction", "k", "routed_scaling_factor", "topk_indices",
                                   "topk_weights", "num_valid_tokens", "rank_token_counts", "rows_per_rank"],
        "glm5_router_gemm": ["hidden_states", "router_weight", "rank_token_counts", "output", "bucket_size", "world_size"],
        "reduce_weighted_scatter": ["expert_output", "topk_pos", "topk_weights", "N", "H", "K", "output", "num_valid_tokens"],
    },
    "batchgen_kernels.common._C_mgn_ops": {
        "moe_fused_gate": ["scores", "e_score_correction_bias", "n_group", "topk_group", "n_routed_experts", "top_k",
                           "routed_scaling_factor"],
        "expert_bincount": ["eids", "routed_expert_start_idx", "experts_per_rank", "device"],
        "fused_moe_token_dispatch": ["global_x", "topk_idx", "token_idx", "topk_pos", "routed_expert_start_idx",
                                     "routed_expert_end_idx"],
        "compact_expert_data": ["expert_counts"],
    },
    "batchgen_kernels.moe._C_dispatch_scatter_3d": {
        "dispatch_scatter_3d": None, "dispatch_scatter_ragged": None, "reduce_weighted_scatter": None,
        "reduce_weighted_scatter_fp32": None, "reduce_weighted_scatter_bf16_ordered": None,
    },
    "batchgen_kernels.moe._C_fp8_blockwise_gemm": {
        "fp8_blockwise_grouped_gemm": ["x", "weight", "seqlens", "cu_seqlens", "x_scale", "w_scale", "num_seq_per_group_avg",
                                       "output", "tma_desc", "tiles", "cu_tiles", "update_tma"],
        "fp8_blockwise_grouped_gemm_ptrs": ["x", "weight_prototype", "weight_ptrs", "seqlens", "cu_seqlens", "x_scale",
                                            "w_scale_prototype", "w_scale_ptrs", "num_seq_per_group_avg", "output", "tma_desc",
                                            "tiles", "cu_tiles"],
        "fp8_blockwise_fused_s1": ["x", "gate_weight", "up_weight", "seqlens", "cu_seqlens", "x_scale", "gate_w_scale",
                                   "up_w_scale", "num_seq_per_group_avg", "output", "tma_desc", "tiles", "cu_tiles", "update_tma"],
        "fp8_blockwise_prepare_s1_s3_tma": ["s1_x", "s1_output", "s3_x", "s3_output", "seqlens", "cu_seqlens",
                                            "num_seq_per_group_avg", "s1_tma_desc", "s3_tma_desc", "tiles", "cu_tiles"],
        "fp8_blockwise_fused_s1_ptrs": ["x", "gate_weight_prototype", "gate_weight_ptrs", "up_weight_prototype", "up_weight_ptrs",
                                        "seqlens", "cu_seqlens", "x_scale", "gate_w_scale_prototype", "gate_w_scale_ptrs",
                                        "up_w_scale_prototype", "up_w_scale_ptrs", "num_seq_per_group_avg", "output", "tma_desc",
                                        "tiles", "cu_tiles"],
    },
    "batchgen_kernels.moe._C_fp8_blockwise_ops": {
        "act_quant_3d": None, "act_quant_ragged": None, "silu_mul_3d": None, "fused_silu_quant_3d": None,
        "deepep_ll_scale_repack": None,
    },
    "batchgen_kernels.attention._C_add_rmsnorm_fp8_quant": {
        "add_rmsnorm_fp8_quant_forward": ["residual", "hidden", "weight", "eps", "norm_num_valid_tokens",
                                          "quant_num_valid_tokens", "row_valid_mask", "scale_tma_aligned"],
    },
}


def load(name):
    if not os.path.isdir(os.path.join(EXT_ROOT, "batchgen_kernels")):
        pytest.skip("extension modules not built (python -m batchgen_amd.build --ext)")
    if EXT_ROOT not in sys.path:
        sys.path.insert(0, EXT_ROOT)
    return importlib.import_module(name)


@pytest.mark.parametrize("name", sorted(OPS))
def test_modules_export_the_reference_ops(name):
    mod = load(name)
    for op, kwargs in OPS[name].items():
        fn = getattr(mod, op)
        assert callable(fn)
        if kwargs:
            doc = fn.__doc__.split("\n")[0]
            for kw in kwargs:
                assert f"{kw}:" in doc, f"{name}.{op}: keyword {kw} missing from {doc}"


def test_argument_errors_are_runtime_errors():
    rt = load("batchgen_kernels.moe._C_routing")
    with pytest.raises(RuntimeError):          # a CPU tensor where the op wants device memory
        rt.gate_sigmoid_topk(torch.zeros(2, 4), torch.zeros(4), 2, 1.0, torch.zeros(0), torch.zeros(0))
    ops = load("batchgen_kernels.moe._C_fp8_blockwise_ops")
    with pytest.raises(RuntimeError):
        ops.act_quant_3d(torch.zeros(2, 4), torch.zeros(2, dtype=torch.int32))
