"""The balanced GEMM's safety net on the GPU: its sticky status word stays zero over launches of every kind of cut,
and the XCD weightings that could leave a share without work are rejected by the setter (the arithmetic behind
both is walked on the CPU in tests/test_hostcheck.py)."""
import ctypes as C

import pytest
import torch

from tests.test_gpu_streamk import _problem, gm
from tests.util import say

pytestmark = pytest.mark.gpu


def _status():
    from batchgen_amd._lib import check, lib
    out = C.c_int32(-1)
    check(lib().bgmoe_debug_streamk_status(C.byref(out)))
    return out.value


def test_status_word_stays_zero_and_bad_weights_are_rejected(dev):
    from batchgen_amd._lib import lib
    m_ = gm()
    _status()                                                           # clear whatever earlier tests left
    default = (C.c_int * 8)(23, 21, 23, 21, 23, 21, 23, 21)
    for w in ([1] + [64] * 7, [0] + [8] * 7, [65] + [8] * 7):
        assert lib().bgmoe_set_streamk_xcd_weights((C.c_int * 8)(*w)) != 0, w
    try:
        for w in ([23, 21] * 4, [8] * 8, [2, 3, 2, 3, 2, 3, 2, 3]):
            assert lib().bgmoe_set_streamk_xcd_weights((C.c_int * 8)(*w)) == 0, w
            for counts in ([16] * 8, [1, 0, 17, 64, 0, 3, 33, 65, 130, 256], [5] * 31):
                say("streamk status", w, counts)
                groups, cap, n, k = len(counts), 256, 512, 2048
                wq, ws, uq, us, xq, xs, cu, m = _problem(dev, groups, n, k, cap, seed=11)
                cnt = torch.tensor(counts, dtype=torch.int32, device=dev)
                wsb = m_.streamk_workspace(dev)
                y0 = torch.zeros((m, n), dtype=torch.bfloat16, device=dev)
                y1 = torch.zeros((m, n), dtype=torch.bfloat16, device=dev)
                wq_t = m_.fp8_weight_repack(wq)
                m_.fp8_blockwise_grouped_gemm(xq, wq_t, cnt, cu, xs, ws, 16, y0, weight_layout="tile_major")
                m_.fp8_blockwise_grouped_gemm(xq, wq_t, cnt, cu, xs, ws, 16, y1, weight_layout="tile_major",
                                              max_group_rows=256, workspace=wsb)
                assert _status() == 0
                a, b = y0.float(), y1.float()
                assert float((a - b).norm() / a.norm().clamp_min(1e-30)) < 2e-3
    finally:
        assert lib().bgmoe_set_streamk_xcd_weights(default) == 0
