"""The router GEMM / bf16 linear kernel with 128-token x 64-output block tiles (plan 5 of
``bgmoe_set_router_gemm_plan``) on the GPU: bit for bit the results of the launch shape chosen from the sizes, as
every other plan, for the linear layers of the MXFP4 layer's shared expert (512 rows), outputs that are not
multiples of 64 or 4, a last token tile with a few rows, and the fp32 logits with a padding mask.

The kernel has not run on a GPU yet, so this file carries a name pytest does not collect (run it by naming the
file); once it is green it becomes tests/test_gpu_y_router_gemm_narrow.py."""
import pytest
import torch

from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,h,e", [(512, 7168, 4096), (512, 2048, 7168), (300, 1024, 100), (1000, 512, 257), (129, 64, 64),
                                   (16384, 1024, 256)])
def test_narrow_block_tiles_give_the_same_bits(dev, n, h, e):
    from batchgen_amd._lib import check, lib
    from batchgen_amd.moe.latent import bf16_linear
    from batchgen_amd.moe.routing.cuda_routing import glm5_router_gemm_cuda
    say("router gemm 128x64 tiles", n, h, e)
    g = torch.Generator().manual_seed(n + h + e)
    x = rand_bf16(g, n, h).to(dev)
    w = rand_bf16(g, e, h, scale=0.05).to(dev)
    base16, base32 = bf16_linear(x, w).clone(), glm5_router_gemm_cuda(x, w).clone()
    try:
        check(lib().bgmoe_set_router_gemm_plan(-1, 5))
        got16, got32 = bf16_linear(x, w).clone(), glm5_router_gemm_cuda(x, w).clone()
    finally:
        check(lib().bgmoe_set_router_gemm_plan(-1, -1))
    assert torch.equal(got32, base32), "fp32 logits differ from the default launch shape"
    assert torch.equal(got16, base16), "bf16 outputs differ from the default launch shape"
    ref = x.float().cpu() @ w.float().cpu().t()
    assert float((got32.cpu() - ref).norm() / ref.norm()) < 1e-5
