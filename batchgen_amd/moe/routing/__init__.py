from .cuda_routing import (  # noqa: F401
    dispatch_count_gather_cuda,
    gate_sigmoid_topk_cuda,
    gate_sigmoid_topk_warp_cuda,
    glm5_router_gemm_cuda,
    reduce_weighted_scatter_cuda,
    router_gemm_gate_sigmoid_topk,
)
