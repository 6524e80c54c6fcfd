"""Matrix products of the parts: choice of kernel and of a split of K.

``linear`` computes x . w^T for x [n, k] and w [m, k].  With a float32 result
it returns partial sums [nsplit, n, m] that the consuming kernel adds (norm,
rotary + append, SiLU gate); with the compute dtype as result it returns
[n, m].  Which kernel runs depends only on the dtype and on n:

  n <= 8    float32: gemv with X in LDS and the whole of K in one wave (no
            partial sums), if the sizes fit; bfloat16 up to 4 rows: the streaming
            gemv, K cut into slices for long rows (measured faster than the
            former for a plain product; the fused epilogues are another matter)
  float32   else: MFMA tiles with 32-bit operands (true 32-bit; K in slices for
            few rows, where one wave's chain of products bounds the time), or
            tiled FMA where K is no multiple of 4
  bfloat16  n <= 64: MFMA skinny (n <= 16 and one float32 result wanted: the
            decode-batch kernel with all of K in a workgroup; from 17 rows on: MFMA
            tiles of 64 rows)
            else: MFMA tiles (K in slices where the tiles alone do not fill the chip),
            or the vendor library (torch.matmul) when the engine option
            ``gemm`` is "library" -- the reference uses its vendor library for
            every product (backend/model.cu:494-503)

Sizes that the MFMA kernels do not take (K not a multiple of 8) go to the plain
kernel.
"""

from __future__ import annotations

import functools

import torch

from .. import kernels as K

def _gemv_split(dtype, n, m, k):
    """Slices of K for the streaming gemv: a wave covers two rows and up to
    2048 (bfloat16) or 1024 (float32) of K with all loads in flight; K is cut
    unless the rows alone already give the chip enough waves."""
    per = 2048 if dtype == torch.bfloat16 else 1024
    if m // 2 >= 4096:
        return 1
    return int(max(1, min(16, -(-k // per))))


def _skinny_split(n, m, k):
    """Slices of K for the skinny MFMA kernel: at most 512 of K per workgroup
    (its LDS stage); more slices while the chip has no workgroup per CU and a
    slice keeps 128 of K.  Idle CUs cost more than the partial sums that a
    further slice writes (measured up to 64 rows)."""
    nsplit = -(-k // 512)
    wgs = -(-m // 64)
    while wgs * nsplit < K.device_cus() and k // (nsplit * 2) >= 128:
        nsplit *= 2
    while (-(-(-(-k // nsplit)) // 32) * 32) * (nsplit - 1) >= k:   # no empty slice
        nsplit -= 1
    return int(nsplit)


def _mfma_split(n, m, k):
    """Slices of K for the tiled MFMA kernel.  A product with fewer 128 x 128
    tiles than the chip has room for workgroups (a portion of a prompt, a
    projection to a narrow output) is bound by how many workgroups stream the
    weights: up to 8 slices of at least 512 of K bring it to about 512
    workgroups (measured, 72 rows: 2048 -> 2560 in 9 us instead of 26 us,
    5632 -> 2048 in 13 us instead of 62 us; 2048 rows, 5632 -> 2048: 57 us
    instead of 68 us with two slices, the second sum's traffic included)."""
    tiles = -(-n // 128) * -(-m // 128)
    nsplit = 1
    # slices of at least 512 of K (512 rows, 2,048 -> 2,048 with the norm behind it: 22.1 us in
    # 4 slices, 23.5 in 8); a deep K bears twice the workgroups if the tiles alone leave CUs idle (1,024 rows, 14,336 -> 4,096:
    # 136 us in 4 slices, 160 in 2; 512 rows: 83 us in 8, 94 in 4)
    reach = (4 if k >= 8192 and tiles <= K.device_cus() else 2) * K.device_cus()
    while nsplit * 2 <= min(8, reach // tiles, k // 512):
        nsplit *= 2
    if nsplit == 1 and n > 64:
        # More 128 x 128 tiles than workgroups fit, but few 256 x 256 ones: slices of at least
        # 2,048 of K that make those one full round of the chip (2,048 rows, 4,096 wide, with the
        # norm behind: K = 4,096 114 us in 2 slices against 126 us; 11,008: 208 against 246;
        # 14,336: 263 against 305)
        big, cus = -(-n // 256) * -(-m // 256), K.device_cus()
        for slices in (2, 3, 4):
            if k // slices >= 2048 and 4 * slices * big >= 3 * cus and slices * big <= cus:
                nsplit = slices
                break
    while nsplit > 1 and (-(-(-(-k // nsplit)) // 64) * 64) * (nsplit - 1) >= k:   # no empty slice
        nsplit -= 1
    return nsplit


def _mfma_f32_split(n, m, k):
    """Slices of K for the float32 MFMA kernel.  With 32-bit operands a wave's
    own chain of products bounds the time (64 cycles for 32 x 32 x 2), not the
    loads, so a product should give every SIMD a wave or two: up to 16 slices
    of at least 128 of K."""
    if n <= 64:
        waves = -(-m // 128) * 2                      # tiles of 64 rows, two waves
    else:
        waves = -(-n // 128) * -(-m // 128) * 4
    nsplit = max(1, min(16, k // 128, -(-4 * K.device_cus() // waves)))
    while nsplit > 1 and (-(-(-(-k // nsplit)) // 32) * 32) * (nsplit - 1) >= k:   # no empty slice
        nsplit -= 1
    return int(nsplit)


def _tiles_beat_skinny(n, m, k):
    """Decode batches of more than 16 rows (two or more of the skinny kernel's 16-row
    tiles): the tiled kernel (tiles of 64 rows, both operands through LDS in whole cache lines) takes nearly
    the same time from 24 to 64 rows, the time of its weights; the skinny one, whose
    workgroups each stage all rows of X for 512 of K and leave up to 28 partial sums, grows
    with the rows.  Measured, tiled against skinny in us (tiles of 64 columns below 40 M
    weights, of 128 above), at 64 rows: 2,048 x 5,632: 9.8 / 13.5; 2,560 x 2,048: 7.0 / 8.6;
    2,048 x 2,048: 6.1 / 6.9; 11,264 x 2,048: 14.3 / 19.7; 4,096 x 4,096: 10.3 / 15.1; 4,096 x
    14,336: 28.7 / 41.1; 28,672 x 4,096: 58.0 / 72.7.  At 24 rows: 8.6 / 9.5; 6.4 / 6.4; 5.6 /
    5.4; 12.3 / 13.5; 9.3 / 10.8; 27.8 / 30.5.  At 16 rows the largest gain 4,096 x 14,336: 26.9
    / 28.2, but none in a whole step (8B sizes: 2,745 against 2,731 tok/s).  At 20 rows:
    8.6 / 9.4; 6.2 / 6.4; 5.6 / 5.4; 12.3 / 13.4; 9.4 / 10.6; 26.1 / 30.0."""
    return n > 16


def _decode_tile_split(n, m, k):
    """Slices of K for a decode batch on the tiled kernel.  Against the largest weights: as
    for prompts.  Below (tiles of 64 columns): slices of at least 256 of K until every CU
    has a workgroup, then further ones of at least 512, up to 16 (measured at 64 rows, in us
    by slices: 2,048 x 5,632: 14.9 with 4, 9.8 with 8; 11,264 x 2,048: 17.3 with 2, 14.3 with 4,
    17.7 with 8; 4,096 x 4,096: 12.2 with 4, 10.3 with 8, 11.2 with 16)."""
    cols = K.gemm_decode_tile_cols(n, m, k)     # the library's choice: 64 below 40 M weights
    if cols != 64:
        return _mfma_split(n, m, k)
    tiles, cus = -(-m // cols), K.device_cus()
    nsplit = 1
    while nsplit < 16 and ((tiles * nsplit < cus and k // (2 * nsplit) >= 256) or k // (2 * nsplit) >= 512):
        nsplit *= 2
    while nsplit > 1 and (-(-(-(-k // nsplit)) // 64) * 64) * (nsplit - 1) >= k:   # no empty slice
        nsplit -= 1
    return nsplit


def choose(dtype, n, m, k, options=None):
    """(algorithm, nsplit) for a product of these sizes."""
    options = options or {}
    forced = options.get("gemm_algo")
    if forced is not None:
        return forced, 1
    if dtype == torch.float32 and K.gemv_fits(n, m, k, dtype) and not options.get("no_fused_gemv"):
        return K.GEMM_GEMV_LDS, 1
    if n <= 4 or (n <= 8 and dtype == torch.float32):
        return K.GEMM_GEMV, _gemv_split(dtype, n, m, k)
    if dtype == torch.float32:
        if k % 4 == 0 and not options.get("no_mfma_f32"):
            return K.GEMM_MFMA_F32, _mfma_f32_split(n, m, k)
        return K.GEMM_TILED_F32, 1
    if k % 8 != 0:
        return (K.GEMM_GEMV, 1) if n <= 8 else (K.GEMM_PLAIN, 1)
    if n <= 64:
        if _tiles_beat_skinny(n, m, k) and options.get("gemm") != "library":
            return K.GEMM_MFMA_BF16, _decode_tile_split(n, m, k)
        return K.GEMM_SKINNY_BF16, _skinny_split(n, m, k)
    if options.get("gemm") == "library":
        return "library", 1
    return K.GEMM_MFMA_BF16, _mfma_split(n, m, k)


@functools.lru_cache(maxsize=4096)
def _resid_tiles(n, m, k):
    """(tiles per workgroup, partial sums of squares per row) of a decode batch's residual
    product: as few tiles to a workgroup as keep the sums of squares within what the
    consumer reads (one tile where the rows go through LDS in passes over K); (1, 0) if the
    kernel does not take the sizes."""
    passes = K.fused_linear_passes(n, k)
    if passes == 0 or (passes > 1 and (passes > K.FUSED_LINEAR_BEST_PASSES or n > K.FUSED_LINEAR_PASSES_BEST_ROWS)):
        return 1, 0
    tpw = 1
    while K.fused_resid_parts(n, m, k, tpw) == 0 and tpw < 64 and passes == 1:
        tpw *= 2
    return tpw, K.fused_resid_parts(n, m, k, tpw)


def tiled_copy(runtime, w, kind, rope=None):
    """A second copy of a weight matrix in the order the decode-batch kernel's lanes read it
    (``K.fused_linear_tile``), or None where that kernel does not run: other dtypes, sizes it
    does not take, or ``EngineOptions.extra["no_tiled_weights"]`` (the copies double the
    memory of the weights they are made of; decode batches of 2 to 16 tokens stream them 20 to
    30 % faster than the row-major matrix)."""
    if (w is None or w.dtype != torch.bfloat16 or not w.is_cuda or w.shape[1] % 8
            or runtime.options.get("no_tiled_weights") or runtime.options.get("no_fused_linear")):
        return None
    return K.fused_linear_tile(w, kind, rope)


def linear_into(ctx, x, w, sink, tag, w_tiled=None):
    """x . w^T added to the residual stream of ``sink`` in the product's own
    epilogue, for up to four tokens: returns the ``Normed`` that stands for the
    norm behind the addition, or None if the kernel with that epilogue does
    not take these sizes (the caller then returns the product and the norm
    adds it).  Measured at width 2048: 4 % of a decode step at one token; for
    decode batches on the matrix cores the same was built and lost 4 % at
    eight tokens (every workgroup of the consuming product then stages 72 KB
    of float32 rows where it staged 32 KB of bfloat16), so it stops at four; in
    float32, where rows are staged in 32 bits either way, the kernels for eight
    rows with these epilogues are the slower ones (2.53 against 2.27 ms a step
    at five to eight tokens)."""
    from .base import Normed
    n, k = x.shape
    m = w.shape[0]
    rt = ctx.runtime
    if rt.options.get("no_fused_norm") or rt.options.get("gemm_algo") is not None:
        return None
    if rt.options.get("no_fused_gemv"):
        return None
    norm = sink.norm
    if tuple(sink.x.shape) != (n, m) or norm.weight is None or norm.weight.numel() != m:
        return None
    parts = K.resid_parts(n, m, k, x.dtype)
    if parts:
        ss = ctx.buf(tag + ".ss", (n, -(-parts // 4) * 4), torch.float32)
        K.linear_resid(x, w, sink.x, ss)
        return Normed(sink.x, ss, parts, norm)
    if x.dtype != torch.bfloat16 or n > K.FUSED_NORM_BEST_ROWS or rt.options.get("no_fused_linear"):
        return None
    # a decode batch on the matrix cores: all of K in a workgroup, the addition in the epilogue, and
    # beside the stream its rows times the norm's weight in 16 bits for a consumer that scales its sums
    tpw, parts = _resid_tiles(n, m, k)
    if parts == 0:
        return None
    ss = ctx.buf(tag + ".ss", (n, -(-parts // 4) * 4), torch.float32)
    xw = ctx.buf(tag + ".xw", (n, m), torch.bfloat16)
    K.fused_linear(w_tiled if w_tiled is not None else w, xw, K.LINEAR_RESID, x=x, tiles_per_wg=tpw, resid=sink.x,
                   norm_weight=norm.weight, ss_out=ss)
    return Normed(sink.x, ss, parts, norm, xw=xw)


def linear(ctx, x, w, tag, out_dtype=torch.float32, split=True, w_tiled=None):
    """x [n, k] . w [m, k]^T.  With a float32 result and ``split``: partial
    sums [nsplit, n, m] for a consumer that adds them; otherwise one [n, m]
    tensor of ``out_dtype``.  ``w_tiled``: the tiled copy of w (``tiled_copy`` with
    LINEAR_PARTS), taken where the decode-batch kernel runs."""
    n, k = x.shape
    m = w.shape[0]
    rt = ctx.runtime
    algo, nsplit = choose(x.dtype, n, m, k, rt.options)
    whole = not split or out_dtype != torch.float32
    if (algo == K.GEMM_SKINNY_BF16 and whole and out_dtype == torch.float32 and n <= 16
            and K.fused_linear_fits(n, k) and not rt.options.get("no_fused_linear")):
        # one float32 result from a decode batch (the logits): all of K in one workgroup, so
        # that no partial sums have to be added afterwards
        y = ctx.buf(tag, (1, n, m), torch.float32)
        K.fused_linear(w_tiled if w_tiled is not None else w, y, K.LINEAR_PARTS, x=x, tiles_per_wg=4 if m >= 16384 else 1)
        return y[0]
    if algo == "library":
        K.bypass_recorded()             # the library is called through torch: behind what was recorded
        if out_dtype == torch.float32:
            # float32 sums straight from the library's accumulators: a result that the caller
            # wants in 32-bit (a residual delta, logits) is never rounded to bfloat16 on the way
            y32 = ctx.buf(tag + ".f32", (1, n, m), torch.float32)
            torch.mm(x, w.t(), out_dtype=torch.float32, out=y32[0])
            return y32[0] if whole else y32
        y = ctx.buf(tag, (n, m), x.dtype)
        torch.matmul(x, w.t(), out=y)
        return y
    if (algo == K.GEMM_MFMA_BF16 or algo == K.GEMM_PLAIN
            or (algo == K.GEMM_MFMA_F32 and (nsplit == 1 or not whole))):   # write either dtype themselves
        if whole:
            y = ctx.buf(tag, (n, m), out_dtype)
            K.gemm(x, w, y, algo, 1)
            return y
        y = ctx.buf(tag, (nsplit, n, m), torch.float32)
        K.gemm(x, w, y, algo, nsplit)
        return y
    parts = ctx.buf(tag, (nsplit, n, m), torch.float32)       # float32 partial sums only
    K.gemm(x, w, parts, algo, nsplit)
    if not whole:
        return parts
    if nsplit == 1 and out_dtype == torch.float32:
        return parts[0]
    y = ctx.buf(tag + ".sum", (n, m), out_dtype)
    K.sum_splits(parts, y)
    return y
