"""Writes tests/golden/c0_layer.npz: inputs' checksums and the oracle's outputs for config 0 of
the benchmark set (64 tokens, hidden 1024, intermediate 512, 16 experts, top-4, 4 groups / 2, 1 shared
expert).  The vectors come from this build's own CPU oracle (the reference's kernels cannot run here);
they freeze the oracle so that a later change to it shows up as a diff, and they give the GPU tests a
second, file-based target.

    python tests/golden/make_c0_golden.py
"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from batchgen_amd import workloads as wl  # noqa: E402
from oracle import layer as ol  # noqa: E402


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def compute():
    cfg = wl.CONFIGS[0]
    inp = wl.make_inputs(cfg, "cpu")
    w, sh = wl.make_fp8_weights(cfg, "cpu")
    ref = ol.moe_layer_fp8(inp["x"], inp["logits"].numpy(), inp["bias"].numpy(),
                           dict(top_k=cfg.top_k, n_group=cfg.n_group, topk_group=cfg.topk_group, rsf=cfg.rsf),
                           wl.weights_to_numpy(w), cfg.expert_start, cfg.e_local, layout=cfg.layout,
                           max_tokens=cfg.max_tokens, shared=wl.weights_to_numpy(sh))
    wn = wl.weights_to_numpy(w)
    return dict(
        x_sha=np.array(sha(inp["x"].float().numpy())), logits_sha=np.array(sha(inp["logits"].numpy())),
        gate_q_sha=np.array(sha(wn["gate_q"])), down_s_sha=np.array(sha(wn["down_s"])),
        ids=ref["ids"], weights=ref["weights"], counts=ref["counts"], pos=ref["pos"],
        xq_tok_sha=np.array(sha(ref["xq_tok"])), xs_tok=ref["xs_tok"],
        out=ref["out"].astype(np.float32))


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c0_layer.npz")
    np.savez_compressed(path, **compute())
    print("wrote", path, os.path.getsize(path), "bytes")
