"""The bf16 dense parts of the MXFP4 layer (shared expert, latent projections) on this library's own kernels:
``bgmoe_bf16_linear`` against fp32, ``bgmoe_silu_and_mul`` bit for bit against the oracle, and the layer with its
dense parts on the library's GEMM (the default) and on the vendor's."""
import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from oracle import quant as oq
from tests.util import rand_bf16, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("latent", [False, True])
def test_dense_backends_agree_and_hip_allocates_nothing(dev, latent):
    """The bf16 shared expert and the latent projections on this library's bf16 GEMM against the same layer on
    ``F.linear``: bf16 outputs of two fp32 summation orders; and the library path allocates nothing in forward."""
    from batchgen_amd import workloads as wl
    from batchgen_amd.moe.mxfp4_layer import Mxfp4MoELayer
    base = wl.K3_LATENT if latent else wl.CONFIGS[3]
    kw = dict(n_tokens=96, hidden=1024, inter=256, shared_inter=512, n_experts=224, e_local=28, expert_start=56,
              max_tokens=96)
    if latent:
        kw["latent"] = 512
    cfg = wl.scaled(base, **kw)
    say("dense backends", cfg.name, "latent", latent)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_mxfp4_weights(cfg, dev)
    lat = wl.make_latent_weights(cfg, dev) if cfg.latent else None
    hip = Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat, dense_backend="hip")
    ven = Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat, dense_backend="vendor")
    a = hip(inp["x"], inp["logits"]).float().cpu()
    b = ven(inp["x"], inp["logits"]).float().cpu()
    err = float((a - b).norm() / b.norm())
    say("   hip vs vendor dense parts, rel. Frobenius:", err)
    assert err < 4e-3
    x17, l17 = inp["x"][:17].contiguous(), inp["logits"][:17].contiguous()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    y = hip(inp["x"], inp["logits"])
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before, "forward allocated device memory"
    assert torch.equal(y.float().cpu(), a)
    a17 = hip(x17, l17).float().cpu()
    assert float((a17 - a[:17]).norm() / a[:17].norm()) < 4e-3      # another launch shape of the routed kernels
    # the default is this library's own GEMM: nothing of the layer runs on the vendor library unless asked for
    default = Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat)
    assert default.dense_backend == "hip"
    assert torch.equal(default(inp["x"], inp["logits"]).float().cpu(), a)
    with pytest.raises(ValueError):
        Mxfp4MoELayer(cfg, w, sh, inp["bias"], latent=lat, dense_backend="auto")


@pytest.mark.parametrize("n,h,e", [(1, 512, 8), (17, 1024, 512), (96, 7168, 260), (300, 2048, 1024), (512, 1024, 4096)])
def test_bf16_linear_against_fp32(dev, n, h, e):
    """``x @ W^T`` with bf16 operands, fp32 sums, one rounding to bf16: against torch in fp32 on the CPU (the sum's
    order differs, so the comparison allows one bf16 step)."""
    from batchgen_amd.moe.latent import bf16_linear
    say("bf16_linear", n, h, e)
    g = torch.Generator().manual_seed(n + h + e)
    x = rand_bf16(g, n, h).to(dev)
    w = rand_bf16(g, e, h, scale=0.05).to(dev)
    ref = (x.float().cpu() @ w.float().cpu().t())
    y = bf16_linear(x, w)
    out = torch.full((n, e), 3.0, dtype=torch.bfloat16, device=dev)
    ws = torch.empty(max(int(lib_().bgmoe_router_gemm_workspace_bytes(n, h, e)), 16), dtype=torch.uint8, device=dev)
    y2 = bf16_linear(x, w, out, ws)
    assert y2 is out and torch.equal(y, y2)
    d = (y.float().cpu() - ref).abs()
    assert float(d.max()) <= 2.0 ** -8 * float(ref.abs().max()) + 1e-6
    assert float((y.float().cpu() - ref).norm() / ref.norm()) < 3e-3
    with pytest.raises(RuntimeError):
        bf16_linear(x, w, out[:, :-1])
    with pytest.raises(RuntimeError):
        bf16_linear(x.float(), w)


def lib_():
    from batchgen_amd._lib import lib
    return lib()


@pytest.mark.parametrize("rows,d", [(1, 8), (33, 520), (96, 2048)])
def test_silu_and_mul_bits(dev, rows, d):
    """``bf16(bf16(silu(gate)) * up)``, PyTorch's ``F.silu(gate) * up`` on bf16 tensors (silu in fp32 as exp, add,
    division; rounded to bf16; then the product rounded to bf16): bit for bit against the oracle
    (``oracle.quant.silu_mul_bf16``, whose exp is the correctly rounded one), and against torch on the CPU up to
    the handful of elements where its library exp differs from the correctly rounded one by an ulp."""
    import torch.nn.functional as F
    from batchgen_amd.moe.latent import silu_and_mul
    say("silu_and_mul", rows, d)
    x = rand_bf16(torch.Generator().manual_seed(rows + d), rows, 2 * d, scale=4.0)
    x[0, 0], x[0, d - 1] = 90.0, -90.0                      # the saturated ends of the exponential
    y = silu_and_mul(x.to(dev)).cpu()
    want = oq.silu_mul_bf16(x[:, :d], x[:, d:])
    assert np.array_equal(y.float().numpy(), want)
    out = torch.full((rows, d + 8), 3.0, dtype=torch.bfloat16, device=dev)
    y2 = silu_and_mul(x.to(dev), out=out[:, :d])            # a strided output
    assert torch.equal(y2.cpu(), y) and bool((out[:, d:] == 3.0).all())
    ref = F.silu(x[:, :d].float()).to(torch.bfloat16) * x[:, d:]
    bad = int((y.view(torch.int16) != ref.view(torch.int16)).sum())
    assert bad <= max(2, rows * d // 2000), bad


@pytest.mark.parametrize("which", ["config3_small", "latent_small", "config3_full_size", "latent_full_size"])
def test_mxfp4_layers_on_the_default_backend(dev, which):
    """The oracle checks of the MXFP4 layers (tests/test_gpu_mxfp4.py, test_gpu_situ_latent.py, test_gpu_full_size.py)
    with the layer's default dense backend, this library's own bf16 GEMM, at 96 and at 512 tokens; the full-size
    run of configuration 3 includes the token-order check (a row's sums do not depend on its position)."""
    say("default dense backend", which)
    if which == "config3_small":
        from tests.test_gpu_mxfp4 import check_mxfp4_layer_against_oracle
        check_mxfp4_layer_against_oracle(dev, "hip")
    elif which == "latent_small":
        from tests.test_gpu_situ_latent import check_latent_layer_against_oracle
        check_latent_layer_against_oracle(dev, "hip")
    elif which == "config3_full_size":
        from tests.test_gpu_full_size import check_full_size_mxfp4_layer
        check_full_size_mxfp4_layer(dev, "hip")
    else:
        from tests.test_gpu_situ_latent import check_latent_layer_full_size_sample
        check_latent_layer_full_size_sample(dev, "hip")
