"""CPU oracle for the MoE expert-layer hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this
directory.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may call it, and only as the checker.

Every function restates, in NumPy / PyTorch-CPU, the arithmetic of one
reference function (file:line under the reference tree is cited in each
docstring).  All fp32 steps are written as separate, individually rounded
IEEE operations (no fused multiply-add), which is what the checked HIP
kernels also do.

How each function is pinned (what a test checks it against, other than its
own formula):

* ``fp8.e4m3fn_encode``          torch's ``.to(float8_e4m3fn)`` on every bf16
                                 bit pattern in [-448, 448] and random fp32;
                                 decode against the 256-entry closed form.
* ``quant.act_quant``            zero block -> bytes 0 / scale 1e-12*(1/448);
                                 form A == form C whenever amax >= 2^-16;
                                 dequantised value within half an fp8 ulp;
                                 sentinel write-set model for the ragged form.
* ``router.fused_gate``          independent torch.topk transcription of the
                                 PyTorch gate (no ties), brute force on tiny
                                 inputs, tie rule cases of the reference tests
                                 (all-equal row -> ids 0..K-1, ...), sum(w)=rsf.
* ``router.gate_sigmoid_topk``   same, plus padding rows (-1 / 0.0).
* ``permute.*``                  sequential per-pair loop (the reference test's
                                 ``ref_dispatch``) and the layout invariants;
                                 ``dispatch_masked_arrivals`` (the slot counter's
                                 final value, dispatch_scatter_3d.cu:66) against a
                                 running counter over the pairs, kept and dropped.
* ``combine.*``                  per-token Python loop, all-(-1) -> zeros.
* ``mxfp4.dequant``              the frozen 16-byte vector of the reference and
                                 its unit cases.
* ``mxfp4.quantize``             parity unpinned in the reference (it holds no
                                 MXFP4 quantiser); pinned to the OCP MX v1.0
                                 closed form: round trip of representable
                                 values is exact, scale = 2^(floor(log2 amax)-2).
* ``gemm.*`` / ``layer.*``       closed-form constant case, dense per-token
                                 brute force, composition of the above.
"""
