"""The reference's GPU parity ladder for its MXFP4 kernels (tests/moe/gpu_parity_mxfp4_marlin.py), restated for
this build at the Kimi-K3 shapes (w1/w3: K 3584 -> N 3072, w2: K 3072 -> N 3584):

  M sweep        single-expert down projection and fused gate + up + SiTU at M in {1, 16, 63, 64, 65, 512}
                 under the reference's numerical gate (its `gate()`, :142-159): |err| <= 1e-5 + 1.6e-2 |ref| on
                 all but < 1e-4 of the elements, max relative error < 1.6e-2 where |ref| > 0.1 rms, all finite;
                 weights = random bytes, half of the experts "half heavy" (80 % +-0.5 codes), scales 112..122
  grouped        28 experts with skewed counts including 0, 1, 8, 9, 64, 65 and 70 rows and non-zero starts,
                 fused stage 1 and down projection, NaN canaries in every row no expert owns, an all-empty launch
                 that writes nothing
  mutations      gate/up swap, scale groups rolled by one, SwiGLU instead of SiTU: each must FAIL the gate while
                 the control passes
  graph          stage 1 + down projection captured in one HIP graph, replayed twice with eager work between
                 the replays: both replays bit-identical to the eager launches

The oracle is dequantise-then-matmul in fp32 with both branches rounded to bf16 before SiTU, as in the
reference's `t3_s1_situ_parity` (:304-325)."""
import numpy as np
import pytest
import torch

from oracle import mxfp4 as mx
from oracle import quant as oq
from oracle import situ as os_
from tests.util import say

pytestmark = pytest.mark.gpu

K3_K, K3_N = 3584, 3072


def _mg():
    from batchgen_amd.kernels import load_extension
    return load_extension("batchgen_kernels.moe._C_marlin_grouped_gemm")


def gate(out, ref, name):
    out = np.asarray(out, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    finite = bool(np.isfinite(out).all())
    err = np.abs(out - ref)
    fail_frac = float(np.mean(err > 1e-5 + 1.6e-2 * np.abs(ref)))
    rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
    mask = np.abs(ref) > 0.1 * rms
    max_rel = float((err[mask] / np.abs(ref[mask])).max()) if mask.any() else 0.0
    ok = finite and fail_frac < 1e-4 and max_rel < 1.6e-2
    say(f"    {name}: {'gate-PASS' if ok else 'gate-FAIL'} fail_frac={fail_frac:.2e} max_rel={max_rel:.2e} finite={finite}")
    return ok


def rand_expert(k, n, seed, half_heavy=False):
    g = torch.Generator().manual_seed(seed)
    if half_heavy:
        nib = torch.where(torch.rand(n, k, generator=g) < 0.8,
                          torch.where(torch.rand(n, k, generator=g) < 0.5, torch.tensor(0x1), torch.tensor(0x9)),
                          torch.randint(0, 16, (n, k), generator=g))
        packed = (nib[:, 0::2] | (nib[:, 1::2] << 4)).to(torch.uint8)
    else:
        packed = torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.int16).to(torch.uint8)
    scale = torch.randint(112, 123, (n, k // 32), generator=g, dtype=torch.int16).to(torch.uint8)
    return packed.numpy(), scale.numpy()


class Expert:
    """One expert's three projections: checkpoint bytes, fp32 dequantised copies, resident device tensors."""

    def __init__(self, seed, dev, half_heavy=False):
        self.raw = {"w1": rand_expert(K3_K, K3_N, seed, half_heavy), "w3": rand_expert(K3_K, K3_N, seed + 1, half_heavy),
                    "w2": rand_expert(K3_N, K3_K, seed + 2, half_heavy)}
        self.deq = {k: torch.from_numpy(mx.dequant(*v)) for k, v in self.raw.items()}
        self.dev = {}
        for k, (p, s) in self.raw.items():
            pd, sd = _mg().mxfp4_weight_repack(torch.from_numpy(p).to(dev)[None], torch.from_numpy(s).to(dev)[None])
            self.dev[k] = (pd, sd)

    def s1_ref(self, x):
        xf = x.float()
        return os_.situ_fused((xf @ self.deq["w1"].T).numpy(), (xf @ self.deq["w3"].T).numpy())

    def s3_ref(self, h):
        return oq.bf16_round((h.float() @ self.deq["w2"].T).numpy())


@pytest.fixture(scope="module")
def experts(dev):
    say("building 4 K3-shaped experts")
    return [Expert(100 + 10 * i, dev, half_heavy=bool(i & 1)) for i in range(4)]


def _one(dev, m):
    return (torch.tensor([m], dtype=torch.int32, device=dev), torch.tensor([0, m], dtype=torch.int32, device=dev))


@pytest.mark.parametrize("m", [1, 16, 63, 64, 65, 512])
def test_m_sweep_down_projection_and_fused_situ(dev, experts, m):
    e = experts[m % 4]
    g = torch.Generator().manual_seed(1000 + m)
    x = torch.randn(m, K3_K, generator=g).to(torch.bfloat16)
    h_in = torch.randn(m, K3_N, generator=g).to(torch.bfloat16)
    cnt, cu = _one(dev, m)
    (gp, gs), (up, us), (dp, ds) = e.dev["w1"], e.dev["w3"], e.dev["w2"]
    h = _mg().mxfp4_fused_s1(x.to(dev), gp, gs, up, us, cnt, cu, weight_layout="tile_major", activation="situ")
    assert gate(h.float().cpu().numpy(), e.s1_ref(x), f"S1+SiTU M={m}")
    y = _mg().mxfp4_grouped_gemm(h_in.to(dev), dp, ds, cnt, cu, weight_layout="tile_major")
    assert gate(y.float().cpu().numpy(), e.s3_ref(h_in), f"down M={m}")


def _grouped_problem(dev, experts):
    counts = np.array([0, 1, 8, 9, 64, 65, 70, 3, 0, 16, 17, 31, 32, 33, 2, 0, 5, 40, 1, 12, 0, 7, 24, 48, 0, 6, 11, 4],
                      dtype=np.int32)
    starts = np.concatenate([[0], np.cumsum((counts + 15) // 16 * 16 + 16)]).astype(np.int32)   # gaps between experts
    return counts, starts, int(starts[-1])


def _tables(dev, experts, key, e):
    w = torch.tensor([experts[i % 4].dev[key][0].data_ptr() for i in range(e)], dtype=torch.int64, device=dev)
    s = torch.tensor([experts[i % 4].dev[key][1].data_ptr() for i in range(e)], dtype=torch.int64, device=dev)
    return w, s


def test_grouped_skewed_counts_with_canaries(dev, experts):
    counts, starts, rows = _grouped_problem(dev, experts)
    e = len(counts)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(rows, K3_K, generator=g).to(torch.bfloat16)
    xd = x.to(dev)
    cnt_d, st_d = torch.from_numpy(counts).to(dev), torch.from_numpy(starts[:e].copy()).to(dev)
    owned = np.zeros(rows, dtype=bool)
    for i, c in enumerate(counts):
        owned[starts[i]:starts[i] + c] = True

    def ptrs(buf):
        return torch.tensor([buf[int(starts[i])].data_ptr() for i in range(e)], dtype=torch.int64, device=dev)

    gw, gsc = _tables(dev, experts, "w1", e)
    uw, usc = _tables(dev, experts, "w3", e)
    dw, dsc = _tables(dev, experts, "w2", e)
    h = torch.full((rows, K3_N), float("nan"), dtype=torch.bfloat16, device=dev)
    _mg().grouped_marlin_gemm_m16_s1_mxfp4_situ(xd, gw, uw, ptrs(h), gsc, usc, st_d, cnt_d, e, K3_N, K3_K, None,
                                                K3_N // 256, 5)
    hn = h.float().cpu().numpy()
    assert np.isnan(hn[~owned]).all(), "a row no expert owns was written"
    ref = np.zeros((rows, K3_N), dtype=np.float32)
    for i, c in enumerate(counts):
        if c:
            ref[starts[i]:starts[i] + c] = experts[i % 4].s1_ref(x[starts[i]:starts[i] + c])
    assert gate(hn[owned], ref[owned], "grouped S1+SiTU, 28 experts")
    y = torch.full((rows, K3_K), float("nan"), dtype=torch.bfloat16, device=dev)
    hb = torch.nan_to_num(h, nan=0.0)
    _mg().marlin_grouped_m16_mxfp4(hb, dw, ptrs(y), dsc, st_d, cnt_d, e, K3_K, K3_N, None, 1, K3_K // 256, 5)
    yn = y.float().cpu().numpy()
    assert np.isnan(yn[~owned]).all()
    yref = np.zeros((rows, K3_K), dtype=np.float32)
    hcpu = hb.cpu()
    for i, c in enumerate(counts):
        if c:
            yref[starts[i]:starts[i] + c] = experts[i % 4].s3_ref(hcpu[starts[i]:starts[i] + c])
    assert gate(yn[owned], yref[owned], "grouped down, 28 experts")
    # an all-empty launch writes nothing
    zero = torch.zeros_like(cnt_d)
    h2 = torch.full_like(h, float("nan"))
    _mg().grouped_marlin_gemm_m16_s1_mxfp4_situ(xd, gw, uw, ptrs(h2), gsc, usc, st_d, zero, e, K3_N, K3_K, None,
                                                K3_N // 256, 5)
    assert torch.isnan(h2.float()).all()


def test_mutations_fail_the_gate(dev, experts):
    e = experts[0]
    m = 64
    g = torch.Generator().manual_seed(505)
    x = torch.randn(m, K3_K, generator=g).to(torch.bfloat16)
    cnt, cu = _one(dev, m)
    (gp, gs), (up, us) = e.dev["w1"], e.dev["w3"]
    ref = e.s1_ref(x)
    run = lambda a, b, c, d, act="situ": _mg().mxfp4_fused_s1(x.to(dev), a, b, c, d, cnt, cu, weight_layout="tile_major",
                                                              activation=act).float().cpu().numpy()
    assert gate(run(gp, gs, up, us), ref, "control")
    caught = 0
    caught += not gate(run(up, us, gp, gs), ref, "m2 gate/up swap")
    # scale groups rolled by one along K, on the checkpoint layout, then made resident again
    p, s = e.raw["w1"]
    pr, sr = _mg().mxfp4_weight_repack(torch.from_numpy(p).to(dev)[None],
                                       torch.from_numpy(np.roll(s, 1, axis=1).copy()).to(dev)[None])
    caught += not gate(run(pr, sr, up, us), ref, "m3 scale groups off by one")
    caught += not gate(run(gp, gs, up, us, act="swiglu"), ref, "m4 SwiGLU instead of SiTU")
    assert caught == 3


def test_stage1_and_down_in_one_graph_replayed_twice(dev, experts):
    counts, starts, rows = _grouped_problem(dev, experts)
    e = len(counts)
    g = torch.Generator().manual_seed(8)
    xd = torch.randn(rows, K3_K, generator=g).to(torch.bfloat16).to(dev)
    cnt_d, st_d = torch.from_numpy(counts).to(dev), torch.from_numpy(starts[:e].copy()).to(dev)
    gw, gsc = _tables(dev, experts, "w1", e)
    uw, usc = _tables(dev, experts, "w3", e)
    dw, dsc = _tables(dev, experts, "w2", e)
    h = torch.zeros((rows, K3_N), dtype=torch.bfloat16, device=dev)
    y = torch.zeros((rows, K3_K), dtype=torch.bfloat16, device=dev)
    ptrs = lambda buf: torch.tensor([buf[int(starts[i])].data_ptr() for i in range(e)], dtype=torch.int64, device=dev)
    hp, yp = ptrs(h), ptrs(y)

    def chain():
        _mg().grouped_marlin_gemm_m16_s1_mxfp4_situ(xd, gw, uw, hp, gsc, usc, st_d, cnt_d, e, K3_N, K3_K, None,
                                                    K3_N // 256, 5)
        _mg().marlin_grouped_m16_mxfp4(h, dw, yp, dsc, st_d, cnt_d, e, K3_K, K3_N, None, 1, K3_K // 256, 5)

    chain()
    torch.cuda.synchronize()
    h_eager, y_eager = h.clone(), y.clone()
    side = torch.cuda.Stream(device=dev)
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain()                                   # warm-up on the capture stream
        with torch.cuda.graph(graph, stream=side):
            chain()
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(2):
        h.zero_()
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(h, h_eager) and torch.equal(y, y_eager), f"replay {replay} differs from the eager launches"
        (xd.float().sum() + 1).item()             # eager work and a synchronisation between the replays
