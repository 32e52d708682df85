"""Router GEMM on the CPU: logits[n,e] = hidden[n,h] (bf16) x weight[e,h]^T (bf16) in fp32.
Oracle code: test infrastructure only.

Three statements of the same product:

* ``router_gemm_exact``     -- the mathematical value: float64 dot products of the bf16 operands (every
  product of two bf16 numbers is exact in float64), rounded once to float32.  This is what the tests
  hold the HIP kernel to, within a bound proportional to sum_k |x_k w_k|.
* ``router_gemm_ref_order`` -- the reference kernel's own summation order
  (batchgen_kernels/src/moe/routing/glm5_router_gemm.cu:35-105): 256 threads, thread t runs the fp32 FMA
  chain over k = t, t+256, ...; 32-lane shuffle-down trees (offsets 16..1) per warp; the 8 warp sums
  go through the same tree in lanes 0..7 of warp 0 (other lanes hold 0).  fmaf(x, w, acc) with bf16 x, w
  equals float32(acc + x*w) because x*w is exact in float32.
* ``router_gemm_segmented`` -- the summation STRUCTURE of this build's kernel: K in segments of 512, the
  logit is (((0 + p_0) + p_1) + ...) in float32 with every p_s rounded to float32.  The inside of a
  segment is an MFMA chain whose internal rounding is not published, so p_s is taken from float64 here:
  this function is a second, tighter yardstick (it differs from the device result only by the rounding
  inside a 512-element segment), not a bit-exact model.

Padding rows (``rank_token_counts``: row i is padding when i % bucket >= counts[i // bucket], or when
i // bucket >= world_size) are zero in all three (glm5_router_gemm.cu:62-80).
"""
from __future__ import annotations

import numpy as np

F32 = np.float32
SEGMENT = 512


def bf16_to_f32(bits_or_tensor) -> np.ndarray:
    """uint16/int16 bf16 bit patterns (numpy) or a torch bf16 tensor -> float32 array."""
    if hasattr(bits_or_tensor, "dtype") and str(bits_or_tensor.dtype) == "torch.bfloat16":
        import torch
        bits_or_tensor = bits_or_tensor.contiguous().view(torch.int16).cpu().numpy()
    b = np.asarray(bits_or_tensor).view(np.uint16).astype(np.uint32) << 16
    return b.view(np.float32)


def padding_rows(n: int, rank_token_counts, bucket_size: int, world_size: int) -> np.ndarray:
    """Boolean [n]: True where the row is padding."""
    if rank_token_counts is None:
        return np.zeros(n, dtype=bool)
    counts = np.asarray(rank_token_counts, dtype=np.int64)
    rows = np.arange(n)
    rank = rows // bucket_size
    local = rows - rank * bucket_size
    inside = rank < world_size
    valid = np.zeros(n, dtype=bool)
    valid[inside] = local[inside] < counts[rank[inside]]
    return ~valid


def _mask(out, rank_token_counts, bucket_size, world_size):
    if rank_token_counts is not None:
        out[padding_rows(out.shape[0], rank_token_counts, bucket_size, world_size)] = 0.0
    return out


def router_gemm_exact(hidden, weight, rank_token_counts=None, bucket_size=0, world_size=1) -> np.ndarray:
    x = bf16_to_f32(hidden).astype(np.float64)
    w = bf16_to_f32(weight).astype(np.float64)
    if rank_token_counts is not None:       # padding rows may hold NaN: keep them out of the product
        x = x.copy()
        x[padding_rows(x.shape[0], rank_token_counts, bucket_size, world_size)] = 0.0
    return _mask((x @ w.T).astype(F32), rank_token_counts, bucket_size, world_size)


def abs_product_sum(hidden, weight) -> np.ndarray:
    """sum_k |x_k w_k| per output: the scale of the fp32 summation error."""
    x = np.abs(bf16_to_f32(hidden).astype(np.float64))
    w = np.abs(bf16_to_f32(weight).astype(np.float64))
    return np.nan_to_num(x, nan=0.0) @ w.T


def router_gemm_ref_order(hidden, weight, rank_token_counts=None, bucket_size=0, world_size=1,
                          threads: int = 256, warp: int = 32) -> np.ndarray:
    x = bf16_to_f32(hidden)
    w = bf16_to_f32(weight)
    n, h = x.shape
    e = w.shape[0]
    if rank_token_counts is not None:
        x = x.copy()
        x[padding_rows(n, rank_token_counts, bucket_size, world_size)] = 0.0
    acc = np.zeros((n, e, threads), dtype=F32)
    for k0 in range(0, h, threads):                       # glm5_router_gemm.cu:85-87
        width = min(threads, h - k0)
        prod = x[:, None, k0:k0 + width] * w[None, :, k0:k0 + width]      # exact in float32
        acc[:, :, :width] = acc[:, :, :width] + prod                      # one rounding = fmaf
    v = acc.reshape(n, e, threads // warp, warp)
    off = warp // 2
    while off >= 1:                                       # warp_reduce_sum, :27-33
        v = v[..., :off] + v[..., off:2 * off]
        off //= 2
    sums = np.zeros((n, e, warp), dtype=F32)              # :96-101
    sums[:, :, :threads // warp] = v[..., 0]
    off = warp // 2
    while off >= 1:
        sums = sums[..., :off] + sums[..., off:2 * off]
        off //= 2
    return _mask(np.ascontiguousarray(sums[..., 0]), rank_token_counts, bucket_size, world_size)


def router_gemm_segmented(hidden, weight, rank_token_counts=None, bucket_size=0, world_size=1) -> np.ndarray:
    x = bf16_to_f32(hidden).astype(np.float64)
    w = bf16_to_f32(weight).astype(np.float64)
    n, h = x.shape
    if rank_token_counts is not None:
        x = x.copy()
        x[padding_rows(n, rank_token_counts, bucket_size, world_size)] = 0.0
    total = np.zeros((n, w.shape[0]), dtype=F32)
    for k0 in range(0, h, SEGMENT):
        part = (x[:, k0:k0 + SEGMENT] @ w[:, k0:k0 + SEGMENT].T).astype(F32)
        total = total + part
    return _mask(total, rank_token_counts, bucket_size, world_size)
