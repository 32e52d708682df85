"""The FP8 MoE layer at the FULL sizes of the benchmark configurations.

The CPU oracle cannot finish a whole 16K-token layer in seconds, so full-size runs are checked through
properties that do not depend on the size:

* determinism: two passes over the same inputs give the same bits;
* token-order equivariance: a token's result is a function of that token only (routing, quantisation, the
  expert rows and the k-ascending combine never mix tokens), so permuting the tokens permutes the output rows
  bit for bit -- although every row then sits in a different place of the permuted buffers, in a different
  chunk / tile / lane of the GEMM kernels;
* a sample of tokens (first, last, and the ones routed to the fullest local expert) is run through the oracle
  on its own -- legitimate for the same reason -- and compared to the bar of the small-size tests: router ids
  bit-exact, output within 1e-2 relative Frobenius error.
"""
import numpy as np
import pytest
import torch

from batchgen_amd import workloads as wl
from oracle import gemm as og
from oracle import layer as ol
from tests.util import say

pytestmark = pytest.mark.gpu


def _rcfg(cfg):
    return dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf)


@pytest.mark.parametrize("idx", [1, 2, 4])
def test_full_size_layer_properties(dev, idx):
    from batchgen_amd.moe.fp8_layer import Fp8MoELayer
    cfg = wl.CONFIGS[idx]
    say("full size", cfg.name)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_fp8_weights(cfg, dev)
    layer = Fp8MoELayer(cfg, w, sh, inp["bias"])
    x, logits = inp["x"], inp["logits"]
    n = cfg.n_tokens

    out = layer(x, logits).clone()
    ids = layer.topk_ids.clone()
    counts = layer.expert_counts[:cfg.e_local].cpu().numpy()
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()

    out2 = layer(x, logits)
    assert torch.equal(out, out2), "two passes over the same input differ"

    gen = torch.Generator().manual_seed(1234 + idx)
    perm = torch.randperm(n, generator=gen).to(dev)
    outp = layer(x[perm].contiguous(), logits[perm].contiguous())
    assert torch.equal(layer.topk_ids, ids[perm]), "router result depends on the token's position"
    assert torch.equal(outp, out[perm]), "a token's output depends on where it sits in the batch"
    assert np.array_equal(layer.expert_counts[:cfg.e_local].cpu().numpy(), counts)

    # sample: first and last token + two tokens of the fullest local expert
    fullest = int(np.argmax(counts)) + cfg.expert_start
    hit = torch.nonzero((ids == fullest).any(dim=1)).flatten().cpu().numpy()
    sample = sorted(set([0, n - 1] + hit[:2].tolist()))
    say("   sample tokens", sample, "fullest local expert", fullest, "rows", int(counts.max()))
    sub = torch.tensor(sample, device=dev)
    ref = ol.moe_layer_fp8(x[sub].cpu(), logits[sub].cpu().numpy(), inp["bias"].cpu().numpy(), _rcfg(cfg),
                           wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local, layout=cfg.layout,
                           max_tokens=cfg.max_tokens, row_align=cfg.row_align, shared=wl.weights_to_numpy(sh))
    assert np.array_equal(ids[sub].cpu().numpy(), ref["ids"])
    err = og.rel_frobenius(out[sub].float().cpu().numpy(), ref["out"])
    say("   rel frobenius of the sample vs fp32 oracle:", err)
    assert err < 1e-2


def check_full_size_mxfp4_layer(dev, backend):
    """Config 3 (MXFP4 weights, bf16 activations) at full size: determinism, a sample of tokens against the
    oracle and, with the bf16 shared expert on this library's own GEMM ("hip": a row's sums are a fixed chain
    over K whatever the row's position), token-order equivariance bit for bit.  The vendor GEMM library does
    not promise position-independent rows, so "vendor" is not held to that."""
    from batchgen_amd.moe.mxfp4_layer import Mxfp4MoELayer
    cfg = wl.CONFIGS[3]
    say("full size", cfg.name, backend)
    inp = wl.make_inputs(cfg, dev)
    w, sh = wl.make_mxfp4_weights(cfg, dev)
    layer = Mxfp4MoELayer(cfg, w, sh, inp["bias"], dense_backend=backend)
    x, logits = inp["x"], inp["logits"]
    n = cfg.n_tokens
    out = layer(x, logits).clone()
    ids = layer.topk_ids.clone()
    counts = layer.expert_counts[:cfg.e_local].cpu().numpy()
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out, layer(x, logits))
    if backend == "hip":
        perm = torch.randperm(n, generator=torch.Generator().manual_seed(1237)).to(dev)
        outp = layer(x[perm].contiguous(), logits[perm].contiguous())
        assert torch.equal(layer.topk_ids, ids[perm]), "router result depends on the token's position"
        assert torch.equal(outp, out[perm]), "a token's output depends on where it sits in the batch"
        assert np.array_equal(layer.expert_counts[:cfg.e_local].cpu().numpy(), counts)
    fullest = int(np.argmax(counts)) + cfg.expert_start
    hit = torch.nonzero((ids == fullest).any(dim=1)).flatten().cpu().numpy()
    sample = sorted(set([0, n - 1] + hit[:2].tolist()))
    say("   sample tokens", sample, "fullest local expert", fullest, "rows", int(counts.max()))
    sub = torch.tensor(sample, device=dev)
    ref = ol.moe_layer_mxfp4(x[sub].cpu(), logits[sub].cpu().numpy(), inp["bias"].cpu().numpy(),
                             dict(top_k=cfg.top_k, n_group=1, topk_group=1, rsf=cfg.rsf),
                             {k: v.cpu().numpy() for k, v in w.items()}, cfg.expert_start, cfg.e_local,
                             layout="masked", max_tokens=cfg.max_tokens,
                             shared_bf16={k: v.float().cpu().numpy() for k, v in sh.items()})
    assert np.array_equal(ids[sub].cpu().numpy(), ref["ids"])
    err = og.rel_frobenius(out[sub].float().cpu().numpy(), ref["out"])
    say("   rel frobenius of the sample vs oracle:", err)
    assert err < 1e-2


def test_full_size_mxfp4_layer_properties(dev):
    """The bf16 shared expert on the vendor GEMM; with the layer's default (this library's own GEMM), token-order
    check included: tests/test_gpu_x_dense_backend.py::test_mxfp4_layers_on_the_default_backend."""
    check_full_size_mxfp4_layer(dev, "vendor")
