"""Each kernel alone against its plain reference, at other sizes than the
engine's tiny models use: widths and vocabularies that are no power of two,
head sizes in steps of 16, odd numbers of heads and groups."""

import math

import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu

DEV = "cuda"


def K():
    from kllm_amd import kernels
    return kernels


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def tol(dtype):
    return 1e-5 if dtype == torch.float32 else 2e-2


# ------------------------------------------------------------------ embedding, norm

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    table = rnd(131, 72, dtype=dtype)
    ids = torch.tensor([0, 130, 5, 5, 77], dtype=torch.int32, device=DEV)
    out = torch.empty(5, 72, device=DEV)
    K().embed(out, table, ids)
    assert torch.equal(out.cpu(), P.embedding(ids.cpu().tolist(), table.cpu().float()))


SPLITS = [1, 3, 4, 7, 8, 11, 12, 15, 16]


@pytest.mark.parametrize("n,d", [(7, 72), (7, 100), (5, 1000), (7, 2048), (3, 3000), (7, 4100), (2, 9000), (300, 2048)])
@pytest.mark.parametrize("out_dtype,delta_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.float32),
                                                   (torch.bfloat16, torch.bfloat16)])
def test_add_rmsnorm(n, d, out_dtype, delta_dtype):
    """Every number of partial sums that a split product hands over (the consumer's 8-wide,
    4-wide and one-by-one branches), at row lengths a thread keeps 2, 4 or 8 elements of (and
    longer ones), with 256 and with 1024 threads a row."""
    eps = 1e-5
    x, w = rnd(n, d, seed=1, scale=3.0), (1 + 0.2 * rnd(d, seed=2))
    out = torch.empty(n, d, dtype=out_dtype, device=DEV)
    # norm only
    x0 = x.clone()
    K().add_rmsnorm(x0, weight=w, out=out, eps=eps)
    assert torch.equal(x0, x)
    ref0 = P.rmsnorm(x.cpu().double(), w.cpu().double(), eps)
    assert (out.cpu().double() - ref0).abs().max() < tol(out_dtype) * 3
    rows = torch.tensor([n - 1, 0, n // 2], dtype=torch.int32, device=DEV)
    for nsplit in SPLITS:
        delta = rnd(nsplit, n, d, seed=3 + nsplit, dtype=delta_dtype)
        want_x = x.cpu().double() + delta.cpu().double().sum(0)
        want = P.rmsnorm(want_x, w.cpu().double(), eps)
        # add (partial sums) + norm, x updated
        x1 = x.clone()
        out.fill_(float("nan"))
        K().add_rmsnorm(x1, delta=delta, weight=w, out=out, eps=eps)
        assert (x1.cpu().double() - want_x).abs().max() < 2e-5, nsplit
        assert (out.cpu().double() - want).abs().max() < tol(out_dtype) * 3, nsplit
        # add only (all partial sums, and a single one given as a matrix)
        x2 = x.clone()
        K().add_rmsnorm(x2, delta=delta, write_x=True)
        assert torch.equal(x2, x1), nsplit
        x2 = x.clone()
        K().add_rmsnorm(x2, delta=delta[0], write_x=True)
        assert torch.allclose(x2, x + delta[0].float())
        # gathered rows: x untouched
        x3 = x.clone()
        out3 = torch.empty(3, d, dtype=out_dtype, device=DEV)
        K().add_rmsnorm(x3, delta=delta, weight=w, out=out3, rows=rows, eps=eps)
        assert torch.equal(x3, x)
        assert (out3.cpu().double() - want[rows.cpu().long()]).abs().max() < tol(out_dtype) * 3, nsplit


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_sum_splits(out_dtype):
    for nsplit, shape in [(1, (3, 130)), (4, (8, 257)), (7, (5, 100)), (8, (64, 515)), (11, (64, 2048)), (16, (2, 33))]:
        parts = rnd(nsplit, *shape, seed=nsplit)
        out = torch.full(shape, float("nan"), dtype=out_dtype, device=DEV)
        K().sum_splits(parts, out)
        want = parts.cpu().double().sum(0)
        assert (out.cpu().double() - want).abs().max() < tol(out_dtype) * 3, nsplit


def test_rmsnorm_zero_row_and_eps_inside_the_root():
    x = torch.zeros(2, 64, device=DEV)
    x[1] = 2.0
    out = torch.empty(2, 64, device=DEV)
    K().add_rmsnorm(x, weight=torch.ones(64, device=DEV), out=out, eps=5.0)
    assert torch.equal(out[0].cpu(), torch.zeros(64))
    assert torch.allclose(out[1].cpu(), torch.full((64,), 2.0 / 3.0), atol=1e-6)


# ------------------------------------------------------------------ rotary, append

@pytest.mark.parametrize("hd,theta", [(16, 10000.0), (48, 1000.0), (128, 500000.0)])
def test_rope_tables_large_positions(hd, theta):
    pos = torch.tensor([0, 1, 17, 4095, 100000], dtype=torch.int32, device=DEV)
    cos = torch.empty(5, hd // 2, device=DEV)
    sin = torch.empty(5, hd // 2, device=DEV)
    K().rope_tables(cos, sin, pos, hd, theta)
    ang = P.rope_angles(pos.cpu().tolist(), hd, theta)
    assert (cos.cpu().double() - torch.cos(ang)).abs().max() < 1e-6
    assert (sin.cpu().double() - torch.sin(ang)).abs().max() < 1e-6


def read_cache(cache, table, length, KV, hd, ps):
    """Keys and values [length, KV*hd] of one request out of the paged layout."""
    c = cache.cpu().float()
    k = torch.zeros(length, KV, hd)
    v = torch.zeros(length, KV, hd)
    for p in range(length):
        page, slot = table[p // ps], p % ps
        for h in range(KV):
            k[p, h] = c[page, 0, h].reshape(ps, hd)[slot]
            v[p, h] = c[page, 1, h].reshape(hd, ps)[:, slot]
    return k.reshape(length, KV * hd), v.reshape(length, KV * hd)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KV,hd,ps", [(4, 2, 16, 16), (3, 1, 32, 16), (5, 5, 48, 32), (6, 3, 80, 16)])
@pytest.mark.parametrize("nsplit", [1, 2, 4, 7, 8, 11, 16])
def test_rope_append(dtype, H, KV, hd, ps, nsplit):
    theta = 10000.0
    # two spans: positions 30..36 of request 0 and 0..4 of request 1, scattered pages
    spans = [(30, 7), (0, 5)]
    n = sum(l for _, l in spans)
    pos = torch.tensor([p0 + i for p0, l in spans for i in range(l)], dtype=torch.int32, device=DEV)
    sot = torch.tensor([s for s, (_, l) in enumerate(spans) for _ in range(l)], dtype=torch.int32, device=DEV)
    tables = [[9, 4, 11], [2, -1, -1]]
    bt = torch.tensor(tables, dtype=torch.int32, device=DEV)
    qd, kvd = H * hd, KV * hd
    qkv = rnd(nsplit, n, qd + 2 * kvd, seed=5)
    cos = torch.empty(n, hd // 2, device=DEV)
    sin = torch.empty(n, hd // 2, device=DEV)
    K().rope_tables(cos, sin, pos, hd, theta)
    cache = torch.full((12, 2, KV, ps * hd), float("nan"), dtype=dtype, device=DEV)
    q_out = torch.empty(n, qd, dtype=dtype, device=DEV)
    K().rope_append(qkv, q_out, cos, sin, cache, pos, sot, bt, ps, H, KV, hd)
    full = qkv.cpu().double().sum(0)
    want_q = P.rope(full[:, :qd], pos.cpu().tolist(), H, hd, theta)
    want_k = P.rope(full[:, qd:qd + kvd], pos.cpu().tolist(), KV, hd, theta)
    want_v = full[:, qd + kvd:]
    assert (q_out.cpu().double() - want_q).abs().max() < tol(dtype) * 4
    off = 0
    for s, (p0, l) in enumerate(spans):
        k, v = read_cache(cache, tables[s], p0 + l, KV, hd, ps)
        assert (k[p0:].double() - want_k[off:off + l]).abs().max() < tol(dtype) * 4
        assert (v[p0:].double() - want_v[off:off + l]).abs().max() < tol(dtype) * 4
        assert torch.isnan(k[:p0]).all()          # nothing else was written
        off += l
    # without tables: no rotation; without cache: q only
    q2 = torch.empty(n, qd, dtype=dtype, device=DEV)
    K().rope_append(qkv[0, :, :qd].contiguous(), q2, None, None, None, None, None, None, ps, H, KV, hd)
    assert (q2.cpu().double() - qkv[0, :, :qd].cpu().double()).abs().max() < tol(dtype) * 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KV,hd,ps,nsplit", [(8, 8, 128, 16, 1), (32, 4, 64, 16, 3), (5, 5, 48, 32, 2), (2, 2, 256, 8, 1)])
def test_rope_append_many_tokens(dtype, H, KV, hd, ps, nsplit):
    """Hundreds of tokens in three spans that begin inside a page and cross many: the kernel
    takes runs of 16 neighbouring tokens, which here begin and end anywhere in spans and pages,
    and the values of a run are written by lanes side by side; the last run is not full."""
    theta = 10000.0
    spans = [(21, 150), (0, 37), (100, 118)]
    n = sum(l for _, l in spans)
    pos = torch.tensor([p0 + i for p0, l in spans for i in range(l)], dtype=torch.int32, device=DEV)
    sot = torch.tensor([s for s, (_, l) in enumerate(spans) for _ in range(l)], dtype=torch.int32, device=DEV)
    width = max(-(-(p0 + l) // ps) for p0, l in spans)
    order = torch.randperm(3 * width, generator=torch.Generator().manual_seed(3)).tolist()
    tables = [order[s * width:(s + 1) * width] for s in range(3)]
    bt = torch.tensor(tables, dtype=torch.int32, device=DEV)
    qd, kvd = H * hd, KV * hd
    qkv = rnd(nsplit, n, qd + 2 * kvd, seed=6)
    cos = torch.empty(n, hd // 2, device=DEV)
    sin = torch.empty(n, hd // 2, device=DEV)
    K().rope_tables(cos, sin, pos, hd, theta)
    cache = torch.full((3 * width, 2, KV, ps * hd), float("nan"), dtype=dtype, device=DEV)
    q_out = torch.empty(n, qd, dtype=dtype, device=DEV)
    K().rope_append(qkv, q_out, cos, sin, cache, pos, sot, bt, ps, H, KV, hd)
    full = qkv.cpu().double().sum(0)
    want_q = P.rope(full[:, :qd], pos.cpu().tolist(), H, hd, theta)
    want_k = P.rope(full[:, qd:qd + kvd], pos.cpu().tolist(), KV, hd, theta)
    want_v = full[:, qd + kvd:]
    assert (q_out.cpu().double() - want_q).abs().max() < tol(dtype) * 4
    off, written = 0, 0
    for s, (p0, l) in enumerate(spans):
        k, v = read_cache(cache, tables[s], p0 + l, KV, hd, ps)
        assert (k[p0:].double() - want_k[off:off + l]).abs().max() < tol(dtype) * 4
        assert (v[p0:].double() - want_v[off:off + l]).abs().max() < tol(dtype) * 4
        assert torch.isnan(k[:p0]).all() and torch.isnan(v[:p0]).all()
        off += l
        written += l
    assert int((~torch.isnan(cache)).sum()) == 2 * written * kvd          # nothing else was written


# ------------------------------------------------------------------ silu gate

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd,rot,interleaved", [(16, 16, True), (32, 8, False), (48, 24, True), (64, 0, False), (80, 80, True)])
def test_rope_append_with_another_pairing_and_extent(dtype, hd, rot, interleaved):
    """The rotation's pairing and extent are arguments: neighbouring pairs, a part of the
    head, no rotation at all; what is not rotated passes through."""
    k_ = K()
    H, KV, ps, n = 3, 2, 16, 7
    pos = torch.tensor([5, 6, 7, 0, 40, 41, 15], dtype=torch.int32, device=DEV)
    sot = torch.tensor([0, 0, 0, 1, 2, 2, 3], dtype=torch.int32, device=DEV)
    tables = [[3, -1, -1], [5, -1, -1], [1, 0, 4], [2, -1, -1]]
    bt = torch.tensor(tables, dtype=torch.int32, device=DEV)
    qd, kvd = H * hd, KV * hd
    qkv = rnd(2, n, qd + 2 * kvd, seed=4)
    g = torch.Generator().manual_seed(3)
    ang = torch.rand(n, rot // 2, generator=g, dtype=torch.float64) * 6.0
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    cache = torch.full((6, 2, KV, ps * hd), float("nan"), dtype=dtype, device=DEV)
    q_out = torch.full((n, qd), float("nan"), dtype=dtype, device=DEV)
    k_.rope_append(qkv, q_out, cos if rot else None, sin if rot else None, cache, pos, sot, bt, ps, H, KV, hd, rot, interleaved)
    full = qkv.cpu().double().sum(0)

    def rotate(x, heads):
        x = x.reshape(n, heads, hd).clone()
        ia = torch.arange(0, rot, 2) if interleaved else torch.arange(rot // 2)
        ib = ia + 1 if interleaved else ia + rot // 2
        a, b = x[..., ia].clone(), x[..., ib].clone()
        x[..., ia] = a * torch.cos(ang)[:, None, :] - b * torch.sin(ang)[:, None, :]
        x[..., ib] = b * torch.cos(ang)[:, None, :] + a * torch.sin(ang)[:, None, :]
        return x.reshape(n, heads * hd)

    want_q, want_k, want_v = rotate(full[:, :qd], H), rotate(full[:, qd:qd + kvd], KV), full[:, qd + kvd:]
    t = 1e-5 if dtype == torch.float32 else 0.01 * full.abs().max()
    assert (q_out.cpu().double() - want_q).abs().max() < t
    for i in range(n):
        page, slot = tables[int(sot[i])][int(pos[i]) // ps], int(pos[i]) % ps
        for h in range(KV):
            got_k = cache[page, 0, h].view(ps, hd)[slot].cpu().double()
            got_v = cache[page, 1, h].view(hd, ps)[:, slot].cpu().double()
            assert (got_k - want_k[i, h * hd:(h + 1) * hd]).abs().max() < t
            assert (got_v - want_v[i, h * hd:(h + 1) * hd]).abs().max() < t
    with pytest.raises(k_.KernelError, match="rotary dimension"):
        k_.rope_append(qkv, q_out, None, None, cache, pos, sot, bt, ps, H, KV, hd, hd + 2, False)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nsplit", [1, 2, 4, 7, 8, 11, 16])
def test_silu_mul(out_dtype, nsplit):
    n, f = 5, 176
    gu = rnd(nsplit, n, 2 * f, seed=4, scale=3.0 / nsplit ** 0.5)
    gu[:, 0, 0] = -60.0 / nsplit                  # far negative gate: 0, not NaN
    out = torch.empty(n, f, dtype=out_dtype, device=DEV)
    K().silu_mul(gu, out)
    s = gu.cpu().double().sum(0)
    want = P.silu(s[:, :f]) * s[:, f:]
    assert torch.isfinite(out).all()
    bound = 1e-4 if out_dtype == torch.float32 else 0.01 * want.abs().max()    # eight bits of the largest value
    assert (out.cpu().double() - want).abs().max() < bound


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_every_kernel_with_a_gate_takes_the_activation(dtype):
    """The gate's activation is an argument: the tanh approximation of GELU through the
    separate gate kernel, the two fused small-batch kernels and the tiled product's
    epilogue, against the plain formula; and an activation nobody built is refused."""
    k_ = K()
    act = k_.ACT_GELU_TANH
    f, k = 176, 264
    w = rnd(2 * f, k, seed=2, dtype=dtype, scale=0.12)
    wd = w.cpu().double()
    tol = (lambda want: 1e-4) if dtype == torch.float32 else (lambda want: 0.01 * want.abs().max() + 1e-3)
    for n in (3, 8, 20, 150):
        x = rnd(n, k, seed=n, dtype=dtype, scale=0.7)
        xd = x.cpu().double()
        g, u = P.linear(xd, wd[:f]), P.linear(xd, wd[f:])
        want = P.gelu_tanh(g) * u
        assert (want - P.silu(g) * u).abs().max() > 0.05          # the two gates differ visibly
        outs = {}
        gu = torch.cat([g, u], dim=1).float().to(DEV).contiguous()
        outs["gate kernel"] = torch.empty(n, f, dtype=dtype, device=DEV)
        k_.silu_mul(gu.view(1, n, 2 * f), outs["gate kernel"], act)
        if n <= 8:
            outs["gemv"] = torch.empty(n, f, dtype=dtype, device=DEV)
            k_.gemv_swiglu(x, w, outs["gemv"], act)
        if dtype == torch.bfloat16 and n <= 32:
            outs["fused_linear"] = torch.empty(n, f, dtype=dtype, device=DEV)
            k_.fused_linear(w, outs["fused_linear"], k_.LINEAR_SWIGLU, x, act=act)
        outs["tiles"] = torch.empty(n, f, dtype=dtype, device=DEV)
        k_.gemm_swiglu(x, w, outs["tiles"], act)
        for name, h in outs.items():
            assert (h.cpu().double() - want).abs().max() < tol(want), (name, n)
    with pytest.raises(k_.KernelError, match="unknown activation"):
        k_.gemm_swiglu(x, w, outs["tiles"], 7)
    with pytest.raises(k_.KernelError, match="unknown activation"):
        k_.silu_mul(gu.view(1, n, 2 * f), outs["gate kernel"], -1)


# ------------------------------------------------------------------ matrix products

GEMM_SIZES = [(1, 64, 64), (2, 131, 88), (5, 100, 72), (8, 515, 2048), (3, 130, 5632), (8, 64, 20480),
              (7, 258, 4100), (17, 96, 176),
              (33, 320, 96), (64, 200, 264), (65, 130, 40), (130, 515, 1032), (300, 257, 520)]


@pytest.mark.parametrize("n,m,k", GEMM_SIZES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gemm_kernels_against_plain(n, m, k, dtype):
    k_ = K()
    x, w = rnd(n, k, seed=1, dtype=dtype), rnd(m, k, seed=2, dtype=dtype)
    want = P.linear(x.cpu().double(), w.cpu().double())
    bound = 1e-5 * k ** 0.5 * 8
    algos = [(k_.GEMM_PLAIN, 1)]
    if dtype == torch.float32:
        algos.append((k_.GEMM_TILED_F32, 1))
        if k % 4 == 0:
            algos.append((k_.GEMM_MFMA_F32, 1))
            if k >= 64:
                algos += [(k_.GEMM_MFMA_F32, 2)] + ([(k_.GEMM_MFMA_F32, 3)] if k >= 100 else [])
            if k >= 2048 and (-(-(-(-k // 16)) // 32) * 32) * 15 < k:     # 16 slices, none empty
                algos.append((k_.GEMM_MFMA_F32, 16))
    elif k % 8 == 0:
        algos.append((k_.GEMM_MFMA_BF16, 1))
        if k >= 128:
            algos += [(k_.GEMM_MFMA_BF16, 2)] + ([(k_.GEMM_MFMA_BF16, 3)] if k >= 200 else [])
        if n <= 64:
            base = -(-k // 512)
            algos += [(k_.GEMM_SKINNY_BF16, base)] + ([(k_.GEMM_SKINNY_BF16, base * 2)] if k >= 256 else [])
    if n <= 8:
        algos += [(k_.GEMM_GEMV, 1)] + ([(k_.GEMM_GEMV, 2)] if k >= 2048 else [])
        if m % 2 == 0 and k % (4 if dtype == torch.float32 else 8) == 0:
            algos.append((k_.GEMM_GEMV_LDS, 1))
    for algo, ns in algos:
        y = torch.full((ns, n, m), float("nan"), device=DEV)
        k_.gemm(x, w, y, algo, ns)
        err = (y.cpu().double().sum(0) - want).abs().max()
        assert err < bound, (algo, ns, float(err))
    if dtype == torch.bfloat16 and k % 8 == 0:      # rounded output
        y = torch.empty(n, m, dtype=dtype, device=DEV)
        k_.gemm(x, w, y, k_.GEMM_MFMA_BF16)
        assert (y.cpu().double() - want).abs().max() < 0.01 * want.abs().max()


def _gpu_reference(x, w):
    """x . w^T in double on the GPU with the library's product: the yardstick for
    sizes at which the CPU would take minutes.  (The library is the reference
    here, never the product path.)"""
    return x.double() @ w.double().t()


@pytest.mark.parametrize("n,m,k,nsplit", [
    (2048, 2560, 2048, 1),      # more tiles than CUs: two stages, 128-row tiles
    (2048, 2048, 5632, 2),      # two slices of K
    (2048, 2048, 5632, 1),
    (2048, 11264, 2048, 1),     # 256-row tiles, eight waves
    (1000, 5000, 2056, 1),      # ragged in every direction, 256-row tiles
    (1000, 5000, 2056, 3),
    (700, 2100, 264, 1),        # two stages, ragged
    (4096, 4096, 4096, 1),
    (2048, 4096, 4096, 2),      # what the engine takes here: 256 x 256 tiles, one round of the chip in two slices of K
    (2048, 32000, 2048, 1),     # the logits of a whole prompt: 256 x 256 tiles (two rounds of them per CU)
    (1000, 16284, 264, 1),      # 256 x 256 tiles (one full round of them), ragged in every direction
    (1000, 8100, 520, 2),       # ... in two slices of K
    (1000, 11000, 264, 1),      # 256 x 192 tiles (2,048 x 11,264 x 2,048 above takes them too), ragged
    (1000, 5600, 520, 2),       # ... in two slices of K
    (64, 11264, 2048, 4),       # a decode batch on tiles of 64 rows and 64 columns, more tiles than CUs: two stages
    (40, 2048, 5632, 8),        # ... as many tiles as CUs: three stages
    (33, 1000, 264, 1),         # ... ragged
    (40, 4096, 14336, 8),       # against the largest weights tiles of 128 columns, few: three stages
    (33, 160000, 264, 1),       # ... many, ragged: two stages
])
@pytest.mark.parametrize("dtype,out_dtype", [(torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                             (torch.float32, torch.float32)])
def test_gemm_mfma_at_prompt_sizes(n, m, k, nsplit, dtype, out_dtype):
    """The tile variants that only products of prompt size reach (256-row tiles with eight
    waves; two stages when there are more tiles than CUs), whole and in slices of K, with
    bfloat16 and with 32-bit operands."""
    if out_dtype == torch.bfloat16 and nsplit > 1:
        pytest.skip("K is split only for float32 partial sums")
    k_ = K()
    x, w = rnd(n, k, seed=1, dtype=dtype), rnd(m, k, seed=2, dtype=dtype)
    want = _gpu_reference(x, w)
    y = torch.full((nsplit, n, m), float("nan"), dtype=out_dtype, device=DEV)
    algo = k_.GEMM_MFMA_BF16 if dtype == torch.bfloat16 else k_.GEMM_MFMA_F32
    k_.gemm(x, w, y if nsplit > 1 or out_dtype == torch.float32 else y[0], algo, nsplit)
    err = (y.double().sum(0) - want).abs().max()
    if out_dtype == torch.float32:
        assert err < 1e-5 * k ** 0.5 * 8, float(err)
    else:
        assert err < 0.01 * want.abs().max(), float(err)
    # one row and one column against the plain kernel's way of summing, on the CPU in double
    r, c = n - 1, m - 1
    assert abs(float(y.double().sum(0)[r, c]) - float(P.linear(x[r:r + 1].cpu().double(), w[c:c + 1].cpu().double()))) < \
        (1e-3 if out_dtype == torch.float32 else 0.01 * float(want.abs().max()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,f,k", [(2048, 5632, 2048), (1000, 2500, 2056), (2048, 14336, 4096), (300, 5632, 2048),
                                   (1000, 8100, 264),     # (2048, 14336, 4096) and this one: 256 x 256 tiles, whole and ragged
                                   (64, 14336, 4096), (40, 20000, 264),    # decode batches: tiles of 64 rows, three and two stages
                                   (1000, 5500, 264)])    # 256 x 192 tiles whose column tiles gate and up share (the first case too), ragged
def test_gemm_swiglu_at_prompt_sizes(n, f, k, dtype):
    x, w = rnd(n, k, seed=1, dtype=dtype, scale=0.5), rnd(2 * f, k, seed=2, dtype=dtype, scale=0.05)
    h = torch.full((n, f), float("nan"), dtype=dtype, device=DEV)
    K().gemm_swiglu(x, w, h)
    g, u = _gpu_reference(x, w[:f]), _gpu_reference(x, w[f:])
    want = P.silu(g) * u
    assert (h.double() - want).abs().max() < (0.01 * want.abs().max() + 1e-3 if dtype == torch.bfloat16
                                              else 1e-5 * want.abs().max() + 1e-5)


@pytest.mark.parametrize("n", [5, 8, 16, 33, 64])
@pytest.mark.parametrize("m,k", [(2048, 2048), (2048, 5632), (4096, 14336), (2560, 2048)])
def test_split_product_into_its_consumers(n, m, k):
    """A decode batch's product with the kernel and with K in as many slices as the engine
    chooses at these sizes (skinny: 8 at K = 2048, 11 at 5632, 28 at 14,336; from 17 rows on
    the tiles of 64 rows, 8 slices), consumed by the norm and
    by the sum kernel."""
    from kllm_amd.parts.linear import choose
    k_ = K()
    algo, nsplit = choose(torch.bfloat16, n, m, k)
    tiled = n > 16
    assert algo == (k_.GEMM_MFMA_BF16 if tiled else k_.GEMM_SKINNY_BF16) and nsplit >= 4
    x, w = rnd(n, k, seed=1, dtype=torch.bfloat16, scale=0.5), rnd(m, k, seed=2, dtype=torch.bfloat16, scale=0.05)
    parts = torch.full((nsplit, n, m), float("nan"), device=DEV)
    k_.gemm(x, w, parts, algo, nsplit)
    want = _gpu_reference(x, w).cpu()
    assert (parts.cpu().double().sum(0) - want).abs().max() < 1e-5 * k ** 0.5 * 8
    res, nw = rnd(n, m, seed=3), 1 + 0.2 * rnd(m, seed=4)
    out = torch.empty(n, m, dtype=torch.bfloat16, device=DEV)
    x1 = res.clone()
    k_.add_rmsnorm(x1, delta=parts, weight=nw, out=out, eps=1e-5)
    want_x = res.cpu().double() + want
    assert (x1.cpu().double() - want_x).abs().max() < 1e-4
    assert (out.cpu().double() - P.rmsnorm(want_x, nw.cpu().double(), 1e-5)).abs().max() < 6e-2
    y = torch.empty(n, m, device=DEV)
    k_.sum_splits(parts, y)
    assert (y.cpu().double() - want).abs().max() < 1e-5 * k ** 0.5 * 8


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,f,k", [(1, 176, 64), (3, 120, 88), (8, 5632, 2048), (5, 33, 4104)])
def test_gemv_swiglu(dtype, n, f, k):
    x, w = rnd(n, k, seed=1, dtype=dtype, scale=0.5), rnd(2 * f, k, seed=2, dtype=dtype, scale=0.1)
    h = torch.full((n, f), float("nan"), dtype=dtype, device=DEV)
    K().gemv_swiglu(x, w, h)
    xd, wd = x.cpu().double(), w.cpu().double()
    want = P.silu(P.linear(xd, wd[:f])) * P.linear(xd, wd[f:])
    assert (h.cpu().double() - want).abs().max() < (1e-4 if dtype == torch.float32 else 0.01 * want.abs().max() + 1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n,f,k", [(65, 176, 64), (130, 120, 88), (300, 515, 264), (128, 5632, 2048)])
def test_gemm_swiglu(n, f, k, dtype):
    x, w = rnd(n, k, seed=1, dtype=dtype, scale=0.5), rnd(2 * f, k, seed=2, dtype=dtype, scale=0.1)
    h = torch.full((n, f), float("nan"), dtype=dtype, device=DEV)
    K().gemm_swiglu(x, w, h)
    xd, wd = x.cpu().double(), w.cpu().double()
    want = P.silu(P.linear(xd, wd[:f])) * P.linear(xd, wd[f:])
    assert (h.cpu().double() - want).abs().max() < (1e-5 * want.abs().max() + 1e-5 if dtype == torch.float32
                                                    else 0.01 * want.abs().max() + 1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KV,hd,ps,d", [(4, 2, 16, 16, 64), (3, 1, 32, 16, 96), (5, 5, 48, 32, 88), (32, 4, 64, 16, 2048)])
def test_gemv_rope_append(dtype, H, KV, hd, ps, d):
    """Projections, rotation and append in one launch, against the plain functions."""
    theta = 10000.0
    spans = [(37, 3), (0, 2), (ps - 1, 1)]                # six tokens of three requests
    n = sum(l for _, l in spans)
    pos = torch.tensor([p0 + i for p0, l in spans for i in range(l)], dtype=torch.int32, device=DEV)
    sot = torch.tensor([s for s, (_, l) in enumerate(spans) for _ in range(l)], dtype=torch.int32, device=DEV)
    tables = [[9, 4, 11], [2, -1, -1], [7, -1, -1]]
    bt = torch.tensor(tables, dtype=torch.int32, device=DEV)
    qd, kvd = H * hd, KV * hd
    x = rnd(n, d, seed=3, dtype=dtype, scale=0.5)
    w = rnd(qd + 2 * kvd, d, seed=4, dtype=dtype, scale=0.1)
    cos = torch.empty(n, hd // 2, device=DEV)
    sin = torch.empty(n, hd // 2, device=DEV)
    K().rope_tables(cos, sin, pos, hd, theta)
    cache = torch.full((12, 2, KV, ps * hd), float("nan"), dtype=dtype, device=DEV)
    q_out = torch.full((n, qd), float("nan"), dtype=dtype, device=DEV)
    K().gemv_rope_append(x, w, q_out, cos, sin, cache, pos, sot, bt, ps, H, KV, hd)
    full = P.linear(x.cpu().double(), w.cpu().double())
    want_q = P.rope(full[:, :qd], pos.cpu().tolist(), H, hd, theta)
    want_k = P.rope(full[:, qd:qd + kvd], pos.cpu().tolist(), KV, hd, theta)
    want_v = full[:, qd + kvd:]
    t = 1e-4 if dtype == torch.float32 else 3e-2
    assert (q_out.cpu().double() - want_q).abs().max() < t
    off = 0
    for s, (p0, l) in enumerate(spans):
        k, v = read_cache(cache, tables[s], p0 + l, KV, hd, ps)
        assert (k[p0:].double() - want_k[off:off + l]).abs().max() < t
        assert (v[p0:].double() - want_v[off:off + l]).abs().max() < t
        assert torch.isnan(k[:p0]).all() and torch.isnan(v[:p0]).all()
        off += l
    # query only (a run that reads another run's cache), without rotation
    q2 = torch.full((n, qd), float("nan"), dtype=dtype, device=DEV)
    K().gemv_rope_append(x, w[:qd].contiguous(), q2, None, None, None, None, None, None, ps, H, KV, hd)
    assert (q2.cpu().double() - full[:, :qd]).abs().max() < t


# ------------------------------------------------------------------ decode-batch products

def _bf(*shape, seed, scale):
    return rnd(*shape, seed=seed, dtype=torch.bfloat16, scale=scale)


@pytest.mark.parametrize("n,m,k,nsplit,tpw", [(1, 48, 64, 1, 1), (8, 2048, 2048, 1, 1), (5, 100, 264, 1, 3),
                                              (16, 72, 520, 2, 1), (19, 33, 4104, 3, 2), (32, 257, 1000, 1, 4),
                                              (8, 176, 5632, 1, 1), (16, 48, 5632, 1, 1), (32, 257, 5000, 1, 1),
                                              (8, 64, 14336, 1, 1), (27, 40, 9992, 2, 1)])
def test_fused_linear_parts(n, m, k, nsplit, tpw):
    """bfloat16 rows in, float32 sums (or partial sums over slices of K) out; the last sizes are
    rows that do not fit into LDS at once and go in passes over K (two and three, the last one
    shorter than the others)."""
    k_ = K()
    x, w = _bf(n, k, seed=1, scale=0.5), _bf(m, k, seed=2, scale=0.1)
    want = P.linear(x.cpu().double(), w.cpu().double())
    bound = 1e-3 * math.sqrt(k) * 0.05 + 1e-4
    y = torch.full((nsplit, n, m), float("nan"), device=DEV)
    k_.fused_linear(w, y, k_.LINEAR_PARTS, x, nsplit=nsplit, tiles_per_wg=tpw)
    assert (y.cpu().double().sum(0) - want).abs().max() < bound
    if nsplit == 1:
        # a view with a row stride (columns of a wider buffer)
        wide = torch.zeros(n, k + 16, dtype=torch.bfloat16, device=DEV)
        wide[:, 8:8 + k] = x
        y2 = torch.full((1, n, m), float("nan"), device=DEV)
        k_.fused_linear(w, y2, k_.LINEAR_PARTS, wide[:, 8:8 + k], tiles_per_wg=tpw)
        assert torch.equal(y2, y)


@pytest.mark.parametrize("n,f,k,tpw", [(1, 176, 64, 1), (3, 120, 88, 2), (8, 5632, 2048, 1), (20, 33, 520, 1),
                                       (16, 100, 264, 3)])
def test_fused_linear_swiglu(n, f, k, tpw):
    k_ = K()
    w = _bf(2 * f, k, seed=2, scale=0.1)
    h = torch.full((n, f), float("nan"), dtype=torch.bfloat16, device=DEV)
    x = _bf(n, k, seed=1, scale=0.5)
    k_.fused_linear(w, h, k_.LINEAR_SWIGLU, x, tiles_per_wg=tpw)
    xd, wd = x.cpu().double(), w.cpu().double()
    want = P.silu(P.linear(xd, wd[:f])) * P.linear(xd, wd[f:])
    assert (h.cpu().double() - want).abs().max() < 0.01 * want.abs().max() + 1e-3


@pytest.mark.parametrize("H,KV,hd,ps,d", [(4, 2, 16, 16, 64), (3, 1, 32, 16, 96), (5, 5, 48, 32, 88),
                                          (32, 4, 64, 16, 2048), (3, 3, 80, 16, 104)])
@pytest.mark.parametrize("tpw", [1, 2])
def test_fused_linear_rope_append(H, KV, hd, ps, d, tpw):
    """Projections, rotation and append in one launch, against the plain functions; a
    workgroup takes one tile of 16 rows of W, or two in turn."""
    k_ = K()
    theta = 10000.0
    spans = [(37, 3), (0, 2), (ps - 1, 1), (5, 11)]       # seventeen tokens of four requests
    n = sum(l for _, l in spans)
    pos = torch.tensor([p0 + i for p0, l in spans for i in range(l)], dtype=torch.int32, device=DEV)
    sot = torch.tensor([s for s, (_, l) in enumerate(spans) for _ in range(l)], dtype=torch.int32, device=DEV)
    tables = [[9, 4, 11], [2, -1, -1], [7, -1, -1], [3, -1, -1]]
    bt = torch.tensor(tables, dtype=torch.int32, device=DEV)
    qd, kvd = H * hd, KV * hd
    x = _bf(n, d, seed=3, scale=0.5)
    w = _bf(qd + 2 * kvd, d, seed=4, scale=0.1)
    cos = torch.empty(n, hd // 2, device=DEV)
    sin = torch.empty(n, hd // 2, device=DEV)
    k_.rope_tables(cos, sin, pos, hd, theta)
    cache = torch.full((12, 2, KV, ps * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    q_out = torch.full((n, qd), float("nan"), dtype=torch.bfloat16, device=DEV)
    k_.fused_linear(w, q_out, k_.LINEAR_ROPE, x, tiles_per_wg=tpw,
                    rope=k_.Rope(cos, sin, cache, pos, sot, bt, ps, H, KV, hd))
    full = P.linear(x.cpu().double(), w.cpu().double())
    want_q = P.rope(full[:, :qd], pos.cpu().tolist(), H, hd, theta)
    want_k = P.rope(full[:, qd:qd + kvd], pos.cpu().tolist(), KV, hd, theta)
    want_v = full[:, qd + kvd:]
    t = 0.01 * full.abs().max() + 1e-3
    assert (q_out.cpu().double() - want_q).abs().max() < t
    off = 0
    for s, (p0, l) in enumerate(spans):
        k, v = read_cache(cache, tables[s], p0 + l, KV, hd, ps)
        assert (k[p0:].double() - want_k[off:off + l]).abs().max() < t
        assert (v[p0:].double() - want_v[off:off + l]).abs().max() < t
        assert torch.isnan(k[:p0]).all() and torch.isnan(v[:p0]).all()
        off += l
    # query only (a run that reads another run's cache), without rotation
    xb = _bf(n, d, seed=8, scale=0.5)
    q2 = torch.full((n, qd), float("nan"), dtype=torch.bfloat16, device=DEV)
    k_.fused_linear(w[:qd].contiguous(), q2, k_.LINEAR_ROPE, xb,
                    rope=k_.Rope(None, None, None, None, None, None, ps, H, KV, hd))
    want2 = P.linear(xb.cpu().double(), w[:qd].cpu().double())
    assert (q2.cpu().double() - want2).abs().max() < 0.01 * want2.abs().max() + 1e-3


@pytest.mark.parametrize("n,m,k,tpw", [(1, 48, 64, 1), (3, 72, 88, 1), (8, 2048, 2048, 1), (8, 2048, 5632, 1),
                                       (13, 2048, 5632, 2), (16, 100, 264, 3), (19, 33, 3080, 1), (32, 257, 1000, 2),
                                       (5, 4096, 14336, 1), (12, 4096, 4096, 1), (16, 2048, 5632, 1),
                                       (8, 4096, 14336, 1), (24, 4088, 4096, 1)])
def test_fused_linear_resid_then_scaled_consumers(n, m, k, tpw):
    """A decode batch's product added to the residual stream in its own epilogue, with what
    the RMS norm behind the addition needs left beside it; then the two consumers that apply
    the norm's row scale to their own sums (gate and rotation), against the plain functions
    in float64: add, norm, product, epilogue."""
    k_ = K()
    eps = 1e-5
    x, w = _bf(n, k, seed=1, scale=0.5), _bf(m, k, seed=2, scale=0.1)
    resid = rnd(n, m, seed=3, scale=2.0)
    nw = 1 + 0.2 * rnd(m, seed=4)
    parts = k_.fused_resid_parts(n, m, k, tpw)
    assert parts == -(-(-(-m // 16)) // tpw)
    stride = -(-parts // 4) * 4
    ss = torch.full((n, stride), float("nan"), device=DEV)
    xw = torch.full((n, m), float("nan"), dtype=torch.bfloat16, device=DEV)
    stream = resid.clone()
    k_.fused_linear(w, xw, k_.LINEAR_RESID, x, tiles_per_wg=tpw, resid=stream, norm_weight=nw, ss_out=ss)
    want_x = resid.cpu().double() + P.linear(x.cpu().double(), w.cpu().double())
    bound = 1e-3 * math.sqrt(k) * 0.05 + 1e-4
    assert (stream.cpu().double() - want_x).abs().max() < bound
    assert (xw.cpu().double() - want_x * nw.cpu().double()).abs().max() < 0.005 * want_x.abs().max() * 1.2 + 1e-3
    got_ss = ss[:, :parts].cpu().double().sum(1)
    assert ((got_ss - (want_x ** 2).sum(1)).abs() / (want_x ** 2).sum(1)).max() < 1e-4
    # the consumers: x * w in 16 bits as input, the row scale applied to the sums
    want_n = P.rmsnorm(want_x, nw.cpu().double(), eps)
    sr = k_.ScaledRows(xw, ss, parts, eps)
    f = 40
    wg = _bf(2 * f, m, seed=5, scale=0.1)
    if k_.fused_linear_passes(n, m) >= 1:      # (24 rows of 4,088: in two passes)
        h = torch.full((n, f), float("nan"), dtype=torch.bfloat16, device=DEV)
        k_.fused_linear(wg, h, k_.LINEAR_SWIGLU, sr)
        wd = wg.cpu().double()
        want = P.silu(P.linear(want_n, wd[:f])) * P.linear(want_n, wd[f:])
        assert (h.cpu().double() - want).abs().max() < 0.01 * want.abs().max() + 2e-3
        # the same numbers as the norm kernel's rows through the unscaled product, within rounding
        xn = torch.empty(n, m, dtype=torch.bfloat16, device=DEV)
        k_.add_rmsnorm(stream, weight=nw, out=xn, eps=eps)
        h2 = torch.empty_like(h)
        k_.fused_linear(wg, h2, k_.LINEAR_SWIGLU, xn)
        assert (h.float() - h2.float()).abs().max() < 0.01 * want.abs().max() + 2e-3
        # rotation epilogue: two heads of 16, queries only
        H, hd = 2, 16
        wq = _bf(H * hd, m, seed=6, scale=0.1)
        pos = torch.arange(5, 5 + n, dtype=torch.int32, device=DEV)
        cos = torch.empty(n, hd // 2, device=DEV)
        sin = torch.empty(n, hd // 2, device=DEV)
        k_.rope_tables(cos, sin, pos, hd, 10000.0)
        q = torch.full((n, H * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
        k_.fused_linear(wq, q, k_.LINEAR_ROPE, sr, rope=k_.Rope(cos, sin, None, None, None, None, 16, H, 1, hd))
        want_q = P.rope(P.linear(want_n, wq.cpu().double()), pos.cpu().tolist(), H, hd, 10000.0)
        assert (q.cpu().double() - want_q).abs().max() < 0.01 * want_q.abs().max() + 2e-3


@pytest.mark.parametrize("n,m,k,tpw", [(1, 48, 64, 1), (8, 2048, 2048, 1), (5, 100, 264, 3), (19, 34, 3080, 2),
                                       (8, 2048, 5632, 1), (16, 520, 1000, 4)])
def test_fused_linear_with_tiled_weights_gives_the_same_bits(n, m, k, tpw):
    """The copy of the weights in the order the kernel's lanes read them changes addresses
    only: every output kind gives, bit for bit, what the row-major weights give (K no
    multiple of 32, rows no multiple of 16, several tiles to a workgroup, K in slices)."""
    k_ = K()
    x, w = _bf(n, k, seed=1, scale=0.5), _bf(m, k, seed=2, scale=0.1)
    tiled = k_.fused_linear_tile(w, k_.LINEAR_PARTS)
    for nsplit in (1, 2):
        if not k_.fused_linear_fits(n, k, nsplit):
            continue
        a = torch.full((nsplit, n, m), float("nan"), device=DEV)
        b = torch.full((nsplit, n, m), float("nan"), device=DEV)
        k_.fused_linear(w, a, k_.LINEAR_PARTS, x, nsplit=nsplit, tiles_per_wg=tpw)
        k_.fused_linear(tiled, b, k_.LINEAR_PARTS, x, nsplit=nsplit, tiles_per_wg=tpw)
        assert torch.isfinite(a).all() and torch.equal(a, b), nsplit
    if not k_.fused_linear_fits(n, k):
        return
    # residual epilogue: the same tiled copy
    nw = 1 + 0.2 * rnd(m, seed=4)
    parts = k_.fused_resid_parts(n, m, k, tpw)
    outs = []
    for wt in (w, tiled):
        stream = rnd(n, m, seed=3, scale=2.0)
        ss = torch.full((n, -(-parts // 4) * 4), float("nan"), device=DEV)
        xw = torch.full((n, m), float("nan"), dtype=torch.bfloat16, device=DEV)
        k_.fused_linear(wt, xw, k_.LINEAR_RESID, x, tiles_per_wg=tpw, resid=stream, norm_weight=nw, ss_out=ss)
        outs.append((stream, xw, ss[:, :parts].clone()))
    for a, b in zip(*outs):
        assert torch.isfinite(a.float()).all() and torch.equal(a, b)
    if m % 2 == 0:
        # gate: rows (p, f + p) meet in a tile
        f = m // 2
        h1 = torch.full((n, f), float("nan"), dtype=torch.bfloat16, device=DEV)
        h2 = torch.full_like(h1, float("nan"))
        k_.fused_linear(w, h1, k_.LINEAR_SWIGLU, x, tiles_per_wg=tpw)
        k_.fused_linear(k_.fused_linear_tile(w, k_.LINEAR_SWIGLU), h2, k_.LINEAR_SWIGLU, x, tiles_per_wg=tpw)
        assert torch.isfinite(h1.float()).all() and torch.equal(h1, h2)
    with pytest.raises(k_.KernelError, match="made for output kind"):
        k_.fused_linear(tiled, torch.empty(n, m // 2, dtype=torch.bfloat16, device=DEV), k_.LINEAR_SWIGLU, x)


@pytest.mark.parametrize("H,KV,hd,ps,d", [(4, 2, 16, 16, 64), (3, 1, 32, 16, 96), (32, 4, 64, 16, 2048), (3, 3, 80, 16, 104)])
def test_fused_linear_rope_append_with_tiled_weights(H, KV, hd, ps, d):
    """Projections, rotation and append from the tiled copy of [q; k; v] (rows j and j + hd/2
    of a head meet in a tile): the same bits in q_out and in the pages as from the row-major
    weights; a copy made for other heads is refused."""
    k_ = K()
    spans = [(37, 3), (0, 2), (ps - 1, 1), (5, 5)]
    n = sum(l for _, l in spans)
    pos = torch.tensor([p0 + i for p0, l in spans for i in range(l)], dtype=torch.int32, device=DEV)
    sot = torch.tensor([s for s, (_, l) in enumerate(spans) for _ in range(l)], dtype=torch.int32, device=DEV)
    bt = torch.tensor([[9, 4, 11], [2, -1, -1], [7, -1, -1], [3, -1, -1]], dtype=torch.int32, device=DEV)
    qd, kvd = H * hd, KV * hd
    x, w = _bf(n, d, seed=3, scale=0.5), _bf(qd + 2 * kvd, d, seed=4, scale=0.1)
    cos = torch.empty(n, hd // 2, device=DEV)
    sin = torch.empty(n, hd // 2, device=DEV)
    k_.rope_tables(cos, sin, pos, hd, 10000.0)
    got = []
    for tile in (False, True):
        cache = torch.zeros((12, 2, KV, ps * hd), dtype=torch.bfloat16, device=DEV)
        q_out = torch.full((n, qd), float("nan"), dtype=torch.bfloat16, device=DEV)
        rope = k_.Rope(cos, sin, cache, pos, sot, bt, ps, H, KV, hd)
        k_.fused_linear(k_.fused_linear_tile(w, k_.LINEAR_ROPE, rope) if tile else w, q_out, k_.LINEAR_ROPE, x, rope=rope)
        got.append((q_out, cache))
    assert torch.isfinite(got[0][0].float()).all() and float(got[0][1].float().abs().sum()) > 0
    assert torch.equal(got[0][0], got[1][0]) and torch.equal(got[0][1], got[1][1])
    other = k_.Rope(cos, sin, None, None, None, None, ps, H, KV, hd)
    with pytest.raises(k_.KernelError, match="other heads"):
        k_.fused_linear(k_.fused_linear_tile(w[:qd].contiguous(), k_.LINEAR_ROPE, other), got[0][0], k_.LINEAR_ROPE, x,
                        rope=k_.Rope(cos, sin, got[0][1], pos, sot, bt, ps, H, KV, hd))


def test_fused_linear_resid_refusals():
    k_ = K()
    n, m, k = 4, 64, 64
    x, w = _bf(n, k, seed=1, scale=0.5), _bf(m, k, seed=2, scale=0.1)
    xw = torch.empty(n, m, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(k_.KernelError):       # no stream
        k_.fused_linear(w, xw, k_.LINEAR_RESID, x)
    with pytest.raises(k_.KernelError):       # sums of squares of the wrong width
        k_.fused_linear(w, xw, k_.LINEAR_RESID, x, resid=torch.zeros(n, m, device=DEV),
                        norm_weight=torch.ones(m, device=DEV), ss_out=torch.zeros(n, 8, device=DEV))
    with pytest.raises(k_.KernelError):       # partial sums do not take a row scale
        k_.fused_linear(w, torch.empty(1, n, m, device=DEV), k_.LINEAR_PARTS,
                        k_.ScaledRows(x, torch.zeros(n, 4, device=DEV), 4, 1e-5))
    assert k_.fused_resid_parts(8, 16 * 300, 64) == 0 and k_.fused_resid_parts(8, 16 * 300, 64, 2) == 150


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [1, 2, 3, 4])
@pytest.mark.parametrize("d,kin,f", [(64, 48, 88), (2048, 2048, 5632), (2048, 5632, 256), (104, 264, 72), (4096, 512, 64)])
def test_a_product_adds_itself_to_the_stream_and_its_consumer_normalises(dtype, n, d, kin, f):
    """The residual product (x += a . w^T in the epilogue, partial sums of squares left
    behind) and the consumers that normalise the stream while they stage their input,
    against the plain add, RMS norm and products, and against the norm kernel's own bits."""
    k_ = K()
    parts = k_.resid_parts(n, d, kin, dtype, best=False)     # what the kernels take, chosen by the engine or not
    if parts == 0:
        pytest.skip("no kernel with a residual epilogue takes these sizes")
    eps = 1e-5
    a, w = rnd(n, kin, seed=1, dtype=dtype, scale=0.5), rnd(d, kin, seed=2, dtype=dtype, scale=0.05)
    x0 = rnd(n, d, seed=3)
    nw = (1 + 0.2 * rnd(d, seed=4)).contiguous()
    x = x0.clone()
    ss = torch.full((n, -(-parts // 4) * 4), float("nan"), device=DEV)
    assert k_.linear_resid(a, w, x, ss) == parts
    want_x = x0.cpu().double() + P.linear(a.cpu().double(), w.cpu().double())
    tol_x = 1e-5 * kin ** 0.5 if dtype == torch.float32 else 1e-4 * kin ** 0.5
    assert (x.cpu().double() - want_x).abs().max() < tol_x
    got_ss = ss.cpu().double()[:, :parts].sum(1)
    assert ((got_ss - (x.cpu().double() ** 2).sum(1)).abs() / got_ss).max() < 1e-5
    normed = k_.NormedInput(x, nw, ss, parts, eps)
    xn_kernel = torch.empty(n, d, dtype=dtype, device=DEV)            # the norm kernel on the same stream
    k_.add_rmsnorm(x.clone(), weight=nw, out=xn_kernel, eps=eps)
    xn = P.rmsnorm(want_x, nw.cpu().double(), eps)
    rel = 1e-4 if dtype == torch.float32 else 2e-2
    # gate + up with the activation
    wgu = rnd(2 * f, d, seed=5, dtype=dtype, scale=0.1)
    want_h = P.silu(P.linear(xn, wgu.cpu().double()[:f])) * P.linear(xn, wgu.cpu().double()[f:])
    h, h2 = (torch.full((n, f), float("nan"), dtype=dtype, device=DEV) for _ in range(2))
    if k_.gemv_fits(n, 2 * f, d, dtype, best=False):
        k_.gemv_swiglu(normed, wgu, h)
        k_.gemv_swiglu(xn_kernel, wgu, h2)
    if not torch.isnan(h).all():
        assert (h.cpu().double() - want_h).abs().max() < rel * want_h.abs().max() + 1e-4
        # normalising while staging gives what the norm kernel gives, up to the last bit of the row's scale
        assert (h.float() - h2.float()).abs().max() <= (1e-5 if dtype == torch.float32 else 0.008) * want_h.abs().max()
    # q, k, v with rotation and append
    H, KV, hd, ps = 2, 1, 16, 16
    wq = rnd((H + 2 * KV) * hd, d, seed=6, dtype=dtype, scale=0.1)
    pos = torch.arange(3, 3 + n, dtype=torch.int32, device=DEV)
    sot = torch.zeros(n, dtype=torch.int32, device=DEV)
    bt = torch.tensor([[1, 0, 2]], dtype=torch.int32, device=DEV)
    cos, sin = torch.empty(n, hd // 2, device=DEV), torch.empty(n, hd // 2, device=DEV)
    k_.rope_tables(cos, sin, pos, hd, 10000.0)
    cache = torch.full((3, 2, KV, ps * hd), float("nan"), dtype=dtype, device=DEV)
    q = torch.full((n, H * hd), float("nan"), dtype=dtype, device=DEV)
    k_.gemv_rope_append(normed, wq, q, cos, sin, cache, pos, sot, bt, ps, H, KV, hd)
    full = P.linear(xn, wq.cpu().double())
    want_q = P.rope(full[:, :H * hd], pos.cpu().tolist(), H, hd, 10000.0)
    assert (q.cpu().double() - want_q).abs().max() < rel * full.abs().max() + 1e-4
    kk, vv = read_cache(cache, [1, 0, 2], 3 + n, KV, hd, ps)
    want_k = P.rope(full[:, H * hd:(H + KV) * hd], pos.cpu().tolist(), KV, hd, 10000.0)
    assert (kk[3:].double() - want_k).abs().max() < rel * full.abs().max() + 1e-4
    assert (vv[3:].double() - full[:, (H + KV) * hd:]).abs().max() < rel * full.abs().max() + 1e-4
    with pytest.raises(k_.KernelError, match="up to 4 rows"):
        five = k_.NormedInput(torch.zeros(5, d, device=DEV), nw, torch.zeros(5, ss.shape[1], device=DEV), parts, eps)
        k_.gemv_swiglu(five, rnd(2 * f, d, seed=5, dtype=torch.float32, scale=0.1), torch.empty(5, f, device=DEV))


def test_fused_linear_refuses_what_it_does_not_take():
    k_ = K()
    w = _bf(32, 64, seed=1, scale=0.1)
    y = torch.empty(1, 33, 32, device=DEV)
    with pytest.raises(k_.KernelError, match="outside"):
        k_.fused_linear(w, y, k_.LINEAR_PARTS, _bf(33, 64, seed=2, scale=1.0))
    with pytest.raises(k_.KernelError, match="multiple of 8"):
        k_.fused_linear(_bf(32, 60, seed=1, scale=0.1), torch.empty(1, 4, 32, device=DEV), k_.LINEAR_PARTS,
                        _bf(4, 60, seed=2, scale=1.0))
    # 32 rows of 8,192 do not fit into LDS at once: they go in passes, with one tile to a workgroup only
    with pytest.raises(k_.KernelError, match="in passes a workgroup takes one tile"):
        k_.fused_linear(_bf(32, 8192, seed=1, scale=0.1), torch.empty(1, 32, 32, device=DEV), k_.LINEAR_PARTS,
                        _bf(32, 8192, seed=2, scale=1.0), tiles_per_wg=2)
    with pytest.raises(k_.KernelError, match="LDS"):        # ... and not in more than eight passes
        k_.fused_linear(_bf(16, 32768, seed=1, scale=0.1), torch.empty(1, 32, 16, device=DEV), k_.LINEAR_PARTS,
                        _bf(32, 32768, seed=2, scale=1.0))
    assert not k_.fused_linear_fits(32, 8192) and k_.fused_linear_fits(32, 8192, 4) and k_.fused_linear_fits(8, 5632)
    assert k_.fused_linear_passes(32, 8192) == 4 and k_.fused_linear_passes(8, 5632) == 1
    assert k_.fused_linear_passes(32, 32768) == 0 and k_.fused_linear_passes(16, 5632) == 2
    with pytest.raises(k_.KernelError, match="split"):
        k_.fused_linear(_bf(32, 64, seed=1, scale=0.1), torch.empty(4, 16, dtype=torch.bfloat16, device=DEV),
                        k_.LINEAR_SWIGLU, _bf(4, 64, seed=2, scale=1.0), nsplit=2)


def test_fused_gemv_refuses_what_it_does_not_take():
    k_ = K()
    x = rnd(9, 64, dtype=torch.bfloat16)
    with pytest.raises(k_.KernelError, match="outside"):
        k_.gemv_swiglu(x, rnd(32, 64, dtype=torch.bfloat16), torch.empty(9, 16, dtype=torch.bfloat16, device=DEV))
    x = rnd(2, 60, dtype=torch.bfloat16)
    with pytest.raises(k_.KernelError, match="multiple of 8"):
        k_.gemv_swiglu(x, rnd(32, 60, dtype=torch.bfloat16), torch.empty(2, 16, dtype=torch.bfloat16, device=DEV))
    assert not k_.gemv_fits(2, 131, 64, torch.bfloat16) and not k_.gemv_fits(9, 64, 64, torch.float32)
    assert k_.gemv_fits(8, 64, 100, torch.float32) and not k_.gemv_fits(1, 64, 100, torch.bfloat16)
    # in bfloat16 the matrix-core kernels are the faster choice at every row count; these take up to eight
    assert not k_.gemv_fits(1, 64, 64, torch.bfloat16) and k_.gemv_fits(1, 64, 64, torch.bfloat16, best=False)
    assert k_.gemv_fits(8, 64, 64, torch.bfloat16, best=False) and not k_.gemv_fits(9, 64, 64, torch.bfloat16, best=False)


def test_gemm_refuses_what_it_does_not_take():
    k_ = K()
    x, w = rnd(70, 72, dtype=torch.bfloat16), rnd(16, 72, dtype=torch.bfloat16)
    y = torch.empty(1, 70, 16, device=DEV)
    with pytest.raises(k_.KernelError, match="exceeds 64"):
        k_.gemm(x, w, y, k_.GEMM_SKINNY_BF16)
    x2, w2 = rnd(4, 12, dtype=torch.bfloat16), rnd(16, 12, dtype=torch.bfloat16)
    with pytest.raises(k_.KernelError, match="multiple of 8"):
        k_.gemm(x2, w2, torch.empty(1, 4, 16, device=DEV), k_.GEMM_MFMA_BF16)
    with pytest.raises(k_.KernelError, match="GPU only"):
        k_.gemm(x2.cpu(), w2, torch.empty(1, 4, 16, device=DEV), k_.GEMM_PLAIN)


def test_linear_chooses_a_kernel_for_every_size():
    from kllm_amd.parts.linear import choose
    k_ = K()
    assert choose(torch.float32, 1, 64, 64)[0] == k_.GEMM_GEMV_LDS
    assert choose(torch.float32, 1, 65, 64)[0] == k_.GEMM_GEMV          # odd number of rows of W
    assert choose(torch.bfloat16, 4, 2560, 2048) == (k_.GEMM_GEMV, 1)
    assert choose(torch.bfloat16, 1, 2048, 5632) == (k_.GEMM_GEMV, 3)
    assert choose(torch.float32, 8, 2560, 2048) == (k_.GEMM_GEMV_LDS, 1)
    assert choose(torch.bfloat16, 8, 2560, 2048) == (k_.GEMM_SKINNY_BF16, 8)
    assert choose(torch.float32, 100, 64, 64) == (k_.GEMM_MFMA_F32, 1)
    assert choose(torch.float32, 100, 64, 66)[0] == k_.GEMM_TILED_F32        # K not a multiple of 4
    assert choose(torch.float32, 64, 2048, 5632) == (k_.GEMM_MFMA_F32, 16)   # few rows: many slices of K
    for n, m, k in [(9, 100, 72), (64, 2048, 5632), (300, 257, 520), (70, 64, 4104), (2048, 2048, 5632)]:
        ns = choose(torch.float32, n, m, k)[1]
        assert 1 <= ns <= 16 and (-(-(-(-k // ns)) // 32) * 32) * (ns - 1) < k, (n, m, k, ns)
    assert choose(torch.bfloat16, 16, 64, 64)[0] == k_.GEMM_SKINNY_BF16
    assert choose(torch.bfloat16, 40, 64, 60)[0] == k_.GEMM_PLAIN          # K not a multiple of 8
    assert choose(torch.bfloat16, 16, 2048, 5632) == (k_.GEMM_SKINNY_BF16, 11)
    assert choose(torch.bfloat16, 40, 64, 64) == (k_.GEMM_MFMA_BF16, 1)          # from 17 rows: tiles of 64 rows
    assert choose(torch.bfloat16, 64, 2048, 5632) == (k_.GEMM_MFMA_BF16, 8)
    assert choose(torch.bfloat16, 64, 11264, 2048) == (k_.GEMM_MFMA_BF16, 4)
    assert choose(torch.bfloat16, 17, 11264, 2048) == (k_.GEMM_MFMA_BF16, 4)
    assert choose(torch.bfloat16, 17, 4096, 14336) == (k_.GEMM_MFMA_BF16, 8)
    assert choose(torch.bfloat16, 64, 11264, 2048, {"gemm": "library"})[0] == k_.GEMM_SKINNY_BF16
    assert choose(torch.bfloat16, 3, 32001, 2048) == (k_.GEMM_GEMV, 1)
    for n, m, k in [(5, 100, 72), (16, 2048, 5632), (13, 96, 176), (9, 320, 520), (12, 64, 4104)]:
        ns = choose(torch.bfloat16, n, m, k)[1]
        kslice = -(-(-(-k // ns)) // 32) * 32
        assert kslice <= 512 and kslice * (ns - 1) < k, (n, m, k, ns)
    assert choose(torch.bfloat16, 400, 64, 64) == (k_.GEMM_MFMA_BF16, 1)
    assert choose(torch.bfloat16, 2048, 2048, 5632) == (k_.GEMM_MFMA_BF16, 2)     # few tiles: slices of K
    assert choose(torch.bfloat16, 72, 2048, 5632) == (k_.GEMM_MFMA_BF16, 8)
    assert choose(torch.bfloat16, 512, 2560, 2048) == (k_.GEMM_MFMA_BF16, 4)
    assert choose(torch.bfloat16, 2048, 11264, 2048) == (k_.GEMM_MFMA_BF16, 1)
    for n, m, k in [(65, 130, 40), (130, 515, 1032), (300, 257, 520), (70, 64, 4104), (100, 2048, 264)]:
        ns = choose(torch.bfloat16, n, m, k)[1]
        assert ns >= 1 and (-(-(-(-k // ns)) // 64) * 64) * (ns - 1) < k, (n, m, k, ns)
    assert choose(torch.bfloat16, 400, 64, 64, {"gemm": "library"})[0] == "library"
    a, ns = choose(torch.bfloat16, 1, 2049, 5632)
    assert a == k_.GEMM_GEMV and 1 <= ns <= 16


# ------------------------------------------------------------------ attention

def build_paged(k, v, tables, lens, KV, hd, ps, num_pages, dtype, poison=True):
    """Put [len, KV*hd] keys/values of several requests into a paged cache."""
    cache = torch.full((num_pages, 2, KV, ps * hd), float("nan") if poison else 0.0)
    for s, L in enumerate(lens):
        for p in range(L):
            page, slot = tables[s][p // ps], p % ps
            for h in range(KV):
                cache[page, 0, h].view(ps, hd)[slot] = k[s][p, h * hd:(h + 1) * hd]
                cache[page, 1, h].view(hd, ps)[:, slot] = v[s][p, h * hd:(h + 1) * hd]
    return cache.to(dtype).to(DEV)


def attention_case(H, KV, hd, ps, dtype, window, spans, seed=0):
    """spans: list of (cached_len, new_len).  Returns (engine output, reference)."""
    lens = [a + b for a, b in spans]
    maxp = max(-(-L // ps) for L in lens)
    num_pages = sum(-(-L // ps) for L in lens) + 3
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, used = [], 0
    for L in lens:
        cnt = -(-L // ps)
        tables.append(perm[used:used + cnt] + [-1] * (maxp - cnt))
        used += cnt
    ks = [torch.randn(L, KV * hd, generator=g).to(dtype).float() for L in lens]
    vs = [torch.randn(L, KV * hd, generator=g).to(dtype).float() for L in lens]
    qs = [torch.randn(b, H * hd, generator=g).to(dtype).float() * 2 for _, b in spans]
    cache = build_paged(ks, vs, tables, lens, KV, hd, ps, num_pages, dtype)
    q = torch.cat(qs).to(dtype).to(DEV)
    pos = torch.tensor([a + i for a, b in spans for i in range(b)], dtype=torch.int32, device=DEV)
    sot = torch.tensor([s for s, (_, b) in enumerate(spans) for _ in range(b)], dtype=torch.int32, device=DEV)
    bt = torch.tensor(tables, dtype=torch.int32, device=DEV)
    want = torch.cat([
        P.attention(qs[s].double(), ks[s].double(), vs[s].double(), range(a, a + b), H, KV, hd, window)
        for s, (a, b) in enumerate(spans)])
    starts = [0]
    for _, b in spans:
        starts.append(starts[-1] + b)
    return dict(q=q, cache=cache, pos=pos, sot=sot, bt=bt, want=want, ps=ps, H=H, KV=KV, hd=hd,
                window=window, scale=1.0 / math.sqrt(hd), tables=tables, lens=lens, spans=spans,
                span_start=torch.tensor(starts, dtype=torch.int32, device=DEV),
                span_pos=torch.tensor([a for a, _ in spans], dtype=torch.int32, device=DEV))


def run_prefill(c, min_len=1, keys=(0, 0), part=None):
    """The prompt kernel over the spans of at least min_len tokens; returns
    (output, mask of the rows it computed).  ``keys``: what the caller says
    about the keys that the blocks read (all together, the longest block).  ``part``:
    room for the partial results of slices of the keys."""
    tiles, rows = [], torch.zeros(c["q"].shape[0], dtype=torch.bool)
    start = 0
    for s, (_, b) in enumerate(c["spans"]):
        if b >= min_len:
            tiles += [(t, s) for t in range(start, start + b, K().PREFILL_QUERY_BLOCK)]
            rows[start:start + b] = True
        start += b
    qt = torch.tensor(tiles, dtype=torch.int32, device=DEV)
    out = torch.full_like(c["q"], float("nan"))
    K().attn_prefill(c["q"], out, c["cache"], qt, len(tiles), c["span_start"], c["span_pos"], c["bt"],
                     c["ps"], c["H"], c["KV"], c["hd"], c["window"], c["scale"], *keys, part=part)
    return out, rows


def run_attention(kernel, q, cache, pos, sot, bt, ps, H, KV, hd, window, scale, nslices=None):
    out = torch.full_like(q, float("nan"))
    if kernel == "generic":
        K().attn_generic(q, out, cache, pos, sot, bt, ps, H, KV, hd, window, scale)
    else:
        n = q.shape[0]
        ns = 1 if kernel == "decode_whole" else nslices or K().attn_decode_slices(n, KV, H, hd, q.dtype)
        part = torch.full((n * H * ns * (hd + 2),), float("nan"), device=DEV)
        K().attn_decode(q, out, part, cache, pos, sot, bt, ps, H, KV, hd, window, scale, ns)
    return out


def kernels_for(dtype):
    # "decode_whole": one slice, so that one workgroup takes all keys of a token and writes
    # the output without a merge (what large batches run)
    return ["generic", "decode", "decode_whole"]


def attn_tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


ATTN_SHAPES = [(4, 2, 16, 16), (3, 1, 32, 16), (5, 5, 48, 16), (8, 2, 64, 16), (6, 3, 80, 32),
               (2, 1, 128, 16), (2, 2, 256, 16), (32, 4, 64, 64)]


@pytest.mark.parametrize("H,KV,hd,ps", ATTN_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_generic(H, KV, hd, ps, dtype, window):
    # a whole prompt, a portion behind 300 cached keys, a decode token at a
    # page's first slot, one at its last, and a sequence's very first token
    c = attention_case(H, KV, hd, ps, dtype, window, [(0, 45), (300, 9), (ps * 3, 1), (ps * 2 - 1, 1), (0, 1)])
    for kernel in kernels_for(dtype):
        out = run_attention(kernel, c["q"], c["cache"], c["pos"], c["sot"], c["bt"], ps, H, KV, hd, window, c["scale"])
        err = (out.cpu().double() - c["want"]).abs().max()
        assert torch.isfinite(out).all(), kernel
        assert err < (2e-5 if dtype == torch.float32 else 2e-2), (kernel, float(err))


@pytest.mark.parametrize("H,KV,hd,ps", [(4, 2, 32, 16), (3, 1, 64, 16), (8, 2, 64, 32), (5, 5, 96, 16),
                                        (2, 1, 128, 16), (2, 2, 192, 16), (2, 1, 256, 16), (32, 4, 64, 16),
                                        (4, 2, 64, 48), (2, 1, 128, 48), (2, 2, 192, 80), (12, 4, 128, 16),
                                        (16, 2, 128, 32), (6, 6, 256, 16)])
@pytest.mark.parametrize("window", [0, 37, 200])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_attention_prefill(H, KV, hd, ps, window, dtype):
    """Whole prompts of ragged lengths, portions behind cached keys that start
    and end inside pages and query tiles, and a one-token span, in one launch.  With heads of
    128 and more and so few blocks, the blocks' keys go in four or two slices over workgroups
    (a slice may hold no key of a query) and a second kernel merges them."""
    c = attention_case(H, KV, hd, ps, dtype, window,
                       [(0, 45), (300, 9), (0, 100), (37, 70), (5, 1), (16, 32), (31, 33)], seed=5)
    out, rows = run_prefill(c)
    assert rows.all() and torch.isfinite(out).all()
    err = (out.cpu().double() - c["want"]).abs().max()
    assert err < attn_tol(dtype), float(err)
    if dtype == torch.bfloat16:
        want_slices = {(2, 128): 4, (2, 192): 4, (2, 256): 4, (12, 128): 2, (16, 128): 2, (6, 256): 4}.get((H, hd), 1)
        assert K().attn_prefill_slices(7, H, hd) == want_slices       # (the seven spans are seven blocks)
    # told that the longest block reads many keys, the launch takes the slices (where there are any)
    slices = K().attn_prefill_slices(7, H, hd, dtype)
    part = torch.full((c["q"].shape[0] * H * slices * (hd + 2),), float("nan"), device=DEV)
    out3, _ = run_prefill(c, keys=(20000, 4000), part=part)
    assert torch.isfinite(out3).all() and (out3.cpu().double() - c["want"]).abs().max() < attn_tol(dtype)
    assert bool(torch.isfinite(part).any()) == (slices > 1)      # the slices' results went through it
    _, _ = run_prefill(c, part=part.fill_(float("nan")))
    assert not torch.isfinite(part).any()                         # ... and not when nothing is said about the keys
    # only the listed spans are touched (fewer query blocks: possibly another of the kernels)
    for keys in ((0, 0), (20000, 4000)):
        out2, rows2 = run_prefill(c, min_len=33, keys=keys)
        assert torch.isnan(out2.cpu()[~rows2]).all() and torch.isfinite(out2.cpu()[rows2]).all()
        assert (out2.cpu().double() - c["want"])[rows2].abs().max() < attn_tol(dtype)


def test_attention_prefill_refuses_tables_beyond_its_page_arithmetic():
    """The prompt kernel finds a key's page with a multiplication that is exact for
    requests of up to 2^24 tokens and pages of up to 2,048: a wider block table or a
    larger page is refused, not computed wrongly."""
    k_ = K()
    c = attention_case(4, 2, 64, 16, torch.bfloat16, 0, [(0, 40)], seed=1)
    qt = torch.tensor([(0, 0)], dtype=torch.int32, device=DEV)
    out = torch.empty_like(c["q"])
    wide = torch.zeros((1, (1 << 24) // 16 + 1), dtype=torch.int32, device=DEV)
    wide[:, :c["bt"].shape[1]] = c["bt"]
    with pytest.raises(k_.KernelError, match="per request"):
        k_.attn_prefill(c["q"], out, c["cache"], qt, 1, c["span_start"], c["span_pos"], wide, c["ps"], c["H"],
                        c["KV"], c["hd"], 0, c["scale"])
    k_.attn_prefill(c["q"], out, c["cache"], qt, 1, c["span_start"], c["span_pos"], wide[:, :(1 << 24) // 16],
                    c["ps"], c["H"], c["KV"], c["hd"], 0, c["scale"])
    assert (out.cpu().double() - c["want"]).abs().max() < attn_tol(torch.bfloat16)


@pytest.mark.parametrize("H,KV,hd,ps", [(24, 4, 32, 16), (24, 3, 64, 16), (22, 2, 96, 32), (22, 11, 128, 16),
                                        (24, 6, 64, 48)])
@pytest.mark.parametrize("window", [0, 150])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("twice", [False, True])
def test_attention_prefill_many_blocks(H, KV, hd, ps, window, dtype, twice):
    """More query blocks than CUs: the kernel that passes the keys through LDS, with two
    groups of waves that take the tiles in turn (up to two blocks per CU) and with one (more:
    the list of spans twice), with blocks of 128 queries that end inside a tile, long chains of
    tiles, portions behind cached keys, and a window that ends inside a block."""
    spans = [(0, 300), (500, 260), (100, 129), (37, 70), (5, 1), (16, 32), (31, 33)] * (2 if twice else 1)
    c = attention_case(H, KV, hd, ps, dtype, window, spans, seed=6)
    blocks = sum(-(-b // K().PREFILL_QUERY_BLOCK) for _, b in spans)
    assert (blocks * H > 512) == twice and blocks * H > 256
    out, rows = run_prefill(c)
    assert rows.all() and torch.isfinite(out).all()
    err = (out.cpu().double() - c["want"]).abs().max()
    assert err < attn_tol(dtype), float(err)
    # told that every block reads many keys (a portion far into its context), the launch
    # takes one group of waves also for few blocks per CU; told that one block reads nearly
    # all of them, two groups
    for keys in ((10 ** 9, 1000), (1000, 1000)):
        out2, _ = run_prefill(c, keys=keys)
        assert (out2.cpu().double() - c["want"]).abs().max() < attn_tol(dtype), keys


@pytest.mark.parametrize("H,KV,hd,ps", [(5, 5, 48, 16), (6, 3, 80, 32), (3, 1, 40, 12), (2, 1, 8, 4), (2, 2, 136, 20),
                                        (70, 2, 16, 16)])
@pytest.mark.parametrize("window", [0, 37])
def test_attention_float32_takes_head_sizes_in_steps_of_8(H, KV, hd, ps, window):
    """Head sizes that are no multiple of 32, pages that are no multiple of 16 and more than
    32 heads to a KV head, on the prompt and on the decode path of the float32 kernel."""
    spans = [(0, 45), (300, 9), (0, 100), (37, 70), (5, 1), (16, 32), (31, 33), (ps * 3, 1), (ps * 2 - 1, 1), (0, 1)]
    c = attention_case(H, KV, hd, ps, torch.float32, window, spans, seed=8)
    out, rows = run_prefill(c)
    assert rows.all() and torch.isfinite(out).all()
    assert (out.cpu().double() - c["want"]).abs().max() < 2e-5
    for nslices in (None, 1, 5):
        out = run_attention("decode", c["q"], c["cache"], c["pos"], c["sot"], c["bt"], ps, H, KV, hd, window,
                            c["scale"], nslices)
        assert torch.isfinite(out).all()
        assert (out.cpu().double() - c["want"]).abs().max() < 2e-5, nslices


@pytest.mark.parametrize("H,KV,ps,news", [(80, 2, 16, (260, 200, 129)), (66, 2, 16, (260, 200, 129)),
                                          (6, 2, 48, (140, 1, 70))])
def test_attention_prefill_far_into_long_contexts(H, KV, ps, news):
    """Portions of prompts behind 70,000 cached keys: the page of a key is found by a
    multiplication instead of a division, and addresses inside a page are 32-bit; both are
    shown here at large key numbers, for the prompt kernels (many query blocks, some, few),
    against the decode kernel, which divides."""
    k_ = K()
    hd, dtype = 64, torch.bfloat16
    spans = list(zip((70000, 65003, 100), news))
    lens = [a + b for a, b in spans]
    counts = [-(-L // ps) for L in lens]
    maxp, num_pages = max(counts), sum(counts) + 2
    g = torch.Generator(device=DEV).manual_seed(11)
    cache = torch.full((num_pages, 2, KV, ps * hd), float("nan"), dtype=dtype, device=DEV)
    tables, used = [], 1
    for L, cnt in zip(lens, counts):
        ids = list(range(used + cnt - 1, used - 1, -1))          # a request's pages in falling order
        used += cnt
        tables.append(ids + [-1] * (maxp - cnt))
        kv = torch.randn(2, cnt * ps, KV, hd, generator=g, device=DEV).to(dtype)
        idx = torch.tensor(ids, device=DEV)
        cache[idx, 0] = kv[0].view(cnt, ps, KV, hd).permute(0, 2, 1, 3).reshape(cnt, KV, ps * hd)
        cache[idx, 1] = kv[1].view(cnt, ps, KV, hd).permute(0, 2, 3, 1).reshape(cnt, KV, hd * ps)
    n = sum(news)
    q = (torch.randn(n, H * hd, generator=g, device=DEV) * 2).to(dtype)
    pos = torch.tensor([a + i for a, b in spans for i in range(b)], dtype=torch.int32, device=DEV)
    sot = torch.tensor([s_ for s_, (_, b) in enumerate(spans) for _ in range(b)], dtype=torch.int32, device=DEV)
    bt = torch.tensor(tables, dtype=torch.int32, device=DEV)
    starts = [0]
    for b in news:
        starts.append(starts[-1] + b)
    scale = 1.0 / math.sqrt(hd)
    want = run_attention("decode", q, cache, pos, sot, bt, ps, H, KV, hd, 0, scale)
    tiles = [(t, s_) for s_, b in enumerate(news) for t in range(starts[s_], starts[s_] + b, k_.PREFILL_QUERY_BLOCK)]
    assert (len(tiles) * H > 256) == (H > 6)
    out = torch.full_like(q, float("nan"))
    k_.attn_prefill(q, out, cache, torch.tensor(tiles, dtype=torch.int32, device=DEV), len(tiles),
                    torch.tensor(starts, dtype=torch.int32, device=DEV),
                    torch.tensor([a for a, _ in spans], dtype=torch.int32, device=DEV), bt, ps, H, KV, hd, 0, scale)
    assert torch.isfinite(out).all()
    assert (out.float() - want.float()).abs().max() < attn_tol(dtype)


def test_attention_prefill_refuses_what_it_does_not_take():
    k_ = K()
    c = attention_case(2, 1, 48, 16, torch.bfloat16, 0, [(0, 40)])
    with pytest.raises(k_.KernelError, match="head_dim 48"):
        run_prefill(c)


@pytest.mark.parametrize("H,KV,hd,ps", [(40, 2, 32, 16), (17, 1, 64, 16), (12, 4, 192, 16), (8, 8, 112, 48)])
@pytest.mark.parametrize("nslices", [4, 8, 64])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_attention_decode_many_heads_and_slices(H, KV, hd, ps, nslices, dtype):
    """More than 16 query heads per KV head (several head tiles), odd groups,
    more slices than there are keys."""
    c = attention_case(H, KV, hd, ps, dtype, 0, [(700, 1), (ps - 1, 1), (0, 1), (33, 2)], seed=3)
    out = run_attention("decode", c["q"], c["cache"], c["pos"], c["sot"], c["bt"], ps, H, KV, hd, 0, c["scale"], nslices)
    assert torch.isfinite(out).all()
    assert (out.cpu().double() - c["want"]).abs().max() < attn_tol(dtype)


def test_attention_decode_takes_more_slices_for_longer_contexts():
    """The proposed number of slices grows with the longest context the caller
    announces (one token over 20,000 keys would otherwise run on 64 waves),
    and the many partial results merge to the same output; one slice writes
    the output without a merge."""
    k_ = K()
    H, KV, hd, ps, dtype = 8, 2, 64, 16, torch.bfloat16
    few = k_.attn_decode_slices(1, KV, H, hd, dtype, 2048)
    assert few == k_.attn_decode_slices(1, KV, H, hd, dtype) == 16
    assert k_.attn_decode_slices(1, KV, H, hd, dtype, 4096) == 32 and k_.attn_decode_slices(1, KV, H, hd, dtype, 8192) == 64
    assert k_.attn_decode_slices(k_.device_cus(), 1, 8, hd, dtype) == 1     # a workgroup to a token
    c = attention_case(H, KV, hd, ps, dtype, 0, [(20000, 1), (37, 1)], seed=9)
    many = k_.attn_decode_slices(2, KV, H, hd, dtype, c["bt"].shape[1] * ps)
    assert few < many <= 64
    for ns in (1, 2, 7, few, 17, 32, 33, many, 65, 100, 256):      # (up to 64 slices: the merge that asks for all at once)
        out = run_attention("decode", c["q"], c["cache"], c["pos"], c["sot"], c["bt"], ps, H, KV, hd, 0, c["scale"], ns)
        assert (out.cpu().double() - c["want"]).abs().max() < attn_tol(dtype), ns


def standout_case(H, KV, hd, key_pos, ctx_len):
    """One decode token whose query matches exactly one key, far stronger than
    all others (score 40 against about 0): the output must be that key's
    value.  A kernel that skips the key (a page's edge, the first or last key)
    or reads beyond the context (the slot after the last key holds a still
    stronger key, score 120) shows at once."""
    g = torch.Generator().manual_seed(1000 + key_pos)
    L, G = ctx_len, H // KV
    k = torch.randn(L + 1, KV * hd, generator=g) * 0.1
    v = torch.randn(L + 1, KV * hd, generator=g)
    u = torch.randn(KV, hd, generator=g)
    u = u / u.norm(dim=1, keepdim=True)
    a = math.sqrt(40.0 * math.sqrt(hd))
    k[key_pos] = (a * u).reshape(-1)
    k[L] = (3.0 * a * u).reshape(-1)
    q = (a * u).repeat_interleave(G, dim=0).reshape(1, H * hd)
    return q, k, v, L


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("key_pos,ctx", [(0, 500), (15, 500), (16, 500), (255, 500), (256, 500),
                                         (499, 500), (311, 312), (0, 1), (16, 17)])
def test_attention_finds_one_key_among_hundreds(dtype, key_pos, ctx):
    H, KV, hd, ps = 4, 2, 32, 16
    q, k, v, L = standout_case(H, KV, hd, key_pos, ctx)
    pages = -(-(L + 1) // ps)
    table = list(range(pages - 1, -1, -1))
    cache = build_paged([k], [v], [table], [L + 1], KV, hd, ps, pages, dtype, poison=False)
    qd = q.to(dtype).to(DEV)
    pos = torch.tensor([L - 1], dtype=torch.int32, device=DEV)
    sot = torch.zeros(1, dtype=torch.int32, device=DEV)
    bt = torch.tensor([table], dtype=torch.int32, device=DEV)
    want = v[key_pos].to(dtype).float().reshape(KV, hd).repeat_interleave(H // KV, 0).reshape(-1)
    for kernel in kernels_for(dtype):
        out = run_attention(kernel, qd, cache, pos, sot, bt, ps, H, KV, hd, 0, 1.0 / math.sqrt(hd))
        assert (out.cpu().float()[0] - want).abs().max() < (1e-3 if dtype == torch.float32 else 3e-2), kernel


@pytest.mark.parametrize("window", [1, 16, 17, 33])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_window_edge(window, dtype):
    H, KV, hd, ps, L = 2, 1, 32, 16, 100
    # the key just outside the window is overwhelming; it must not be seen
    g = torch.Generator().manual_seed(window)
    k = torch.randn(L, hd, generator=g) * 0.1
    v = torch.randn(L, hd, generator=g)
    q = torch.randn(1, H * hd, generator=g)
    q[0, hd:] = q[0, :hd]
    outside, inside = L - 1 - window, L - window
    k[outside] = 50.0 * q[0, :hd]
    table = list(range(-(-L // ps)))
    cache = build_paged([k], [v], [table], [L], KV, hd, ps, len(table), dtype, poison=False)
    q, k, v = (t.to(dtype).float() for t in (q, k, v))
    qd = q.to(dtype).to(DEV)
    pos = torch.tensor([L - 1], dtype=torch.int32, device=DEV)
    sot = torch.zeros(1, dtype=torch.int32, device=DEV)
    bt = torch.tensor([table], dtype=torch.int32, device=DEV)
    want = P.attention(q.double(), k.double(), v.double(), [L - 1], H, KV, hd, window)
    for kernel in kernels_for(dtype):
        out = run_attention(kernel, qd, cache, pos, sot, bt, ps, H, KV, hd, window, 1.0 / math.sqrt(hd))
        assert (out.cpu().double() - want).abs().max() < (1e-4 if dtype == torch.float32 else 2e-2), kernel
        assert (out.cpu().float()[0, :hd] - v[outside]).abs().max() > 0.1
        # pages wholly before the window may be gone (-1 in the table)
        gone = inside // ps
        bt2 = bt.clone()
        bt2[0, :gone] = -1
        out2 = run_attention(kernel, qd, cache, pos, sot, bt2, ps, H, KV, hd, window, 1.0 / math.sqrt(hd))
        assert torch.equal(out2, out), kernel


def test_attention_refuses_sizes_it_does_not_take():
    k_ = K()
    q = torch.zeros(1, 2 * 272, device=DEV)
    cache = torch.zeros(1, 2, 1, 16 * 272, device=DEV)
    i32 = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(k_.KernelError, match="head_dim"):
        k_.attn_generic(q, torch.empty_like(q), cache, i32, i32, i32.view(1, 1), 16, 2, 1, 272, 0, 1.0)


# ------------------------------------------------------------------ sampling

def test_sample_greedy_first_maximum():
    logits = rnd(6, 1031, seed=9)
    logits[2, 77] = logits[2, 900] = 50.0
    logits[3, 1030] = 60.0
    logits[4, 0] = 60.0
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    K().sample(out, logits)
    want = [P.argmax_first(r) for r in logits.cpu()]
    assert out.tolist() == want and want[2] == 77 and want[3] == 1030 and want[4] == 0


@pytest.mark.parametrize("temperature", [0.3, 1.0, 2.0])
def test_sample_temperature_inverts_the_cdf(temperature):
    from kllm_amd.sampling import uniform
    rows, vocab = 64, 517
    logits = rnd(rows, vocab, seed=3, scale=2.0)
    us = [uniform(5, i) for i in range(rows)]
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    t = torch.full((rows,), temperature, device=DEV)
    K().sample(out, logits, t, torch.tensor(us, device=DEV))
    got = out.tolist()
    for r in range(rows):
        p = P.softmax_temperature(logits[r].cpu(), temperature)
        cdf = torch.cumsum(p, 0)
        lo = float(cdf[got[r] - 1]) if got[r] > 0 else 0.0
        hi = float(cdf[got[r]])
        assert lo - 1e-5 <= us[r] < hi + 1e-5, (r, got[r], lo, us[r], hi)
    # mixed rows: temperature 0 is greedy
    t[::2] = 0.0
    K().sample(out, logits, t, torch.tensor(us, device=DEV))
    assert out.tolist()[::2] == [P.argmax_first(r) for r in logits.cpu()[::2]]


def test_sample_frequencies_follow_softmax():
    from kllm_amd.sampling import uniform
    n = 4096
    row = torch.tensor([0.0, math.log(2.0), math.log(5.0), -40.0])
    logits = row.repeat(n, 1).to(DEV)
    us = torch.tensor([uniform(2, i) for i in range(n)], device=DEV)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    K().sample(out, logits, torch.ones(n, device=DEV), us)
    counts = torch.bincount(out.cpu().long(), minlength=4).tolist()
    want = [1 / 8, 2 / 8, 5 / 8]
    chi2 = sum((counts[k] - n * want[k]) ** 2 / (n * want[k]) for k in range(3))
    assert chi2 < 13.8 and counts[3] == 0
