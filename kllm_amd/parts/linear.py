"""Matrix products of the parts: choice of kernel and of a split of K.

``linear`` computes x . w^T for x [n, k] and w [m, k].  With a float32 result
it returns partial sums [nsplit, n, m] that the consuming kernel adds (norm,
rotary + append, SiLU gate); with the compute dtype as result it returns
[n, m].  Which kernel runs depends only on the dtype and on n:

  float32   n <= 8: gemv      else: tiled FMA (true 32-bit)
  bfloat16  n <= 8: gemv      n <= 64: MFMA skinny      else: MFMA tiles,
            or the vendor library (torch.matmul) when the engine option
            ``gemm`` is "library" -- the reference uses its vendor library for
            every product (backend/model.cu:494-503)

Sizes that the MFMA kernels do not take (K not a multiple of 8) go to the plain
kernel.
"""

from __future__ import annotations

import torch

from .. import kernels as K

TARGET_WAVES = 2048


def _split_for(n, m, k, rows_per_wave, min_slice):
    """How many slices of K: enough waves to fill the chip, but partial sums
    must stay small beside the weights they come from."""
    tiles = -(-m // rows_per_wave)
    by_fill = max(1, TARGET_WAVES // max(tiles, 1))
    by_traffic = max(1, k // (16 * n))
    by_slice = max(1, k // min_slice)
    return int(max(1, min(by_fill, by_traffic, by_slice, 16)))


def choose(dtype, n, m, k, options=None):
    """(algorithm, nsplit) for a product of these sizes."""
    options = options or {}
    forced = options.get("gemm_algo")
    if forced is not None:
        return forced, 1
    if n <= 8:
        return K.GEMM_GEMV, _split_for(n, m, k, 1, 1024)
    if dtype == torch.float32:
        return K.GEMM_TILED_F32, 1
    if k % 8 != 0:
        return K.GEMM_PLAIN, 1
    if n <= 64:
        return K.GEMM_SKINNY_BF16, _split_for(n, m, k, 16, 128)
    if options.get("gemm") == "library":
        return "library", 1
    return K.GEMM_MFMA_BF16, 1


def linear(ctx, x, w, tag, out_dtype=torch.float32, split=True):
    """x [n, k] . w [m, k]^T.  float32 result: [nsplit, n, m]; else [n, m]."""
    n, k = x.shape
    m = w.shape[0]
    rt = ctx.runtime
    algo, nsplit = choose(x.dtype, n, m, k, rt.options)
    if not split or out_dtype != torch.float32:
        nsplit = 1
    if algo == "library":
        y = ctx.buf(tag, (n, m), x.dtype)
        torch.matmul(x, w.t(), out=y)
        if out_dtype == torch.float32:
            y32 = ctx.buf(tag + ".f32", (1, n, m), torch.float32)
            y32[0].copy_(y)
            return y32
        return y
    if out_dtype == torch.float32:
        y = ctx.buf(tag, (nsplit, n, m), torch.float32)
        K.gemm(x, w, y, algo, nsplit)
        return y
    if algo in (K.GEMM_GEMV, K.GEMM_SKINNY_BF16) or (algo == K.GEMM_TILED_F32):
        # These write float32 only; round once afterwards.
        y32 = ctx.buf(tag + ".f32", (1, n, m), torch.float32)
        K.gemm(x, w, y32, algo, 1)
        y = ctx.buf(tag, (n, m), out_dtype)
        y.copy_(y32[0])
        return y
    y = ctx.buf(tag, (n, m), out_dtype)
    K.gemm(x, w, y, algo, 1)
    return y
