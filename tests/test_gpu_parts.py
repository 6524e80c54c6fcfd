"""Each part alone, built from a PartSpec as a model would build it, against
the plain function of the same name."""

import pytest
import torch

import part_tools as T
import plain_llama as P
from kllm_amd.parts import LayerSpec, PartSpec, make_part

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def tol(dtype, k=1.0):
    return (3e-5 if dtype == torch.float32 else 3e-2) * k


def as_stored(w, dtype):
    """Host float32 copy of what the part holds (matrices in the compute dtype)."""
    return {k: (v.to(dtype).float() if v.dim() > 1 else v.float()) for k, v in w.items()}


def bind(part, w, dtype):
    dev = {}
    for s in part.weight_specs():
        t = w[s.name]
        assert tuple(t.shape) == tuple(s.shape), s
        dev[s.name] = t.to(dtype if s.role == "matrix" else torch.float32).to(T.DEV)
    part.bind(dev)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    rt = T.runtime(dtype)
    norm = make_part("norm", PartSpec("rmsnorm", "blk.ln", size=88, eps=1e-4), rt)
    assert [s.name for s in norm.weight_specs()] == ["blk.ln.weight"]
    w = {"blk.ln.weight": 1 + 0.3 * rnd(88, seed=1)}
    bind(norm, w, dtype)
    ctx = T.context(rt, [(0, 6)])
    x = rnd(6, 88, seed=2, scale=2.0).to(T.DEV)
    delta = rnd(6, 88, seed=3).to(T.DEV)
    out = norm.forward(ctx, x.clone())
    assert (out.float().cpu() - P.rmsnorm(x.cpu(), w["blk.ln.weight"], 1e-4)).abs().max() < tol(dtype, 4)
    x2 = x.clone()
    out = norm.forward(ctx, x2, delta=delta)
    assert torch.allclose(x2, x + delta)
    assert (out.float().cpu() - P.rmsnorm((x + delta).cpu(), w["blk.ln.weight"], 1e-4)).abs().max() < tol(dtype, 4)
    x3 = x.clone()
    norm.add(ctx, x3, delta)
    assert torch.allclose(x3, x + delta)


def test_rotary_part_tables():
    rt = T.runtime(torch.float32)
    rot = make_part("position", PartSpec("rotary", head_dim=48, theta=1000.0), rt)
    assert rot.weight_specs() == []
    ctx = T.context(rt, [(100, 3), (0, 2)])
    rot.prepare(ctx)
    cos, sin = rot.tables(ctx)
    ang = P.rope_angles([100, 101, 102, 0, 1], 48, 1000.0)
    assert (cos.cpu().double() - torch.cos(ang)).abs().max() < 1e-6
    assert (sin.cpu().double() - torch.sin(ang)).abs().max() < 1e-6


ATTN = [dict(hidden=64, heads=4, kv_heads=2, head_dim=16), dict(hidden=96, heads=3, kv_heads=1, head_dim=32),
        dict(hidden=88, heads=5, kv_heads=5, head_dim=48), dict(hidden=72, heads=6, kv_heads=2, head_dim=64)]


def attn_weights(p, prefix, seed):
    qd, kvd, d = p["heads"] * p["head_dim"], p["kv_heads"] * p["head_dim"], p["hidden"]
    return {f"{prefix}.q_proj.weight": rnd(qd, d, seed=seed, scale=0.2),
            f"{prefix}.k_proj.weight": rnd(kvd, d, seed=seed + 1, scale=0.2),
            f"{prefix}.v_proj.weight": rnd(kvd, d, seed=seed + 2, scale=0.2),
            f"{prefix}.o_proj.weight": rnd(d, qd, seed=seed + 3, scale=0.2)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("p", ATTN)
@pytest.mark.parametrize("window", [0, 21])
def test_attention_part_over_two_steps(dtype, p, window):
    """A prompt portion, then a second portion and a decode token of another
    request in one batch: the part against whole-sequence plain attention."""
    rt = T.runtime(dtype)
    rot = PartSpec("rotary", head_dim=p["head_dim"], theta=10000.0)
    part = make_part("mixer", PartSpec("attention", "l.self_attn", window=window, position=rot, **p), rt)
    need = part.cache_need()
    assert (need.kind, need.kv_heads, need.head_dim, need.window) == ("paged", p["kv_heads"], p["head_dim"], window)
    w = attn_weights(p, "l.self_attn", 5)
    bind(part, w, dtype)
    ws = as_stored(w, dtype)
    c = dict(H=p["heads"], KV=p["kv_heads"], hd=p["head_dim"], theta=10000.0)
    cache = T.empty_cache(9, p["kv_heads"], p["head_dim"], 16, dtype)
    xa = rnd(50, p["hidden"], seed=7).to(dtype).float()       # request a: 50 tokens
    xb = rnd(33, p["hidden"], seed=8).to(dtype).float()       # request b: 33 tokens
    tables = {"a": [7, 2, 5, 0], "b": [3, 8, 1]}
    want_a, _ = P.attention_sublayer(ws, "l.", xa, torch.arange(50), c, window)
    want_b, _ = P.attention_sublayer(ws, "l.", xb, torch.arange(33), c, window)

    def step(spans, tabs, xs):
        ctx = T.context(rt, spans, tables=tabs)
        for _, sp in rt.shared.values():
            sp.prepare(ctx)
        xn = torch.cat(xs).to(dtype).to(T.DEV)
        out = part.forward(ctx, xn, T.view(cache, ctx))
        return out.float().sum(0).cpu()
    o1 = step([(0, 30), (0, 32)], [tables["a"], tables["b"]], [xa[:30], xb[:32]])
    o2 = step([(32, 1), (30, 20)], [tables["b"], tables["a"]], [xb[32:], xa[30:]])
    got_a = torch.cat([o1[:30], o2[1:]])
    got_b = torch.cat([o1[30:], o2[:1]])
    assert (got_a - want_a).abs().max() < tol(dtype, 10)
    assert (got_b - want_b).abs().max() < tol(dtype, 10)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part_reading_another_runs_cache(dtype):
    rt = T.runtime(dtype)
    p = ATTN[0]
    rot = PartSpec("rotary", head_dim=16, theta=10000.0)
    owner = make_part("mixer", PartSpec("attention", "a.self_attn", position=rot, **p), rt)
    reader = make_part("mixer", PartSpec("attention", "b.self_attn", position=rot, own_kv=False, **p), rt)
    assert [s.name for s in reader.weight_specs()] == ["b.self_attn.q_proj.weight", "b.self_attn.o_proj.weight"]
    wa, wb = attn_weights(p, "a.self_attn", 1), attn_weights(p, "b.self_attn", 9)
    bind(owner, wa, dtype), bind(reader, wb, dtype)
    cache = T.empty_cache(3, 2, 16, 16, dtype)
    ctx = T.context(rt, [(0, 20)])
    for _, sp in rt.shared.values():
        sp.prepare(ctx)
    x = rnd(20, 64, seed=3).to(dtype)
    owner.forward(ctx, x.to(T.DEV), T.view(cache, ctx))
    got = reader.forward(ctx, x.to(T.DEV), T.view(cache, ctx, write=False)).float().sum(0).cpu()
    c = dict(H=4, KV=2, hd=16, theta=10000.0)
    wsa, wsb = as_stored(wa, dtype), as_stored(wb, dtype)
    _, kv = P.attention_sublayer({k.replace("a.", "l."): v for k, v in wsa.items()}, "l.", x.float(), torch.arange(20), c)
    kv = tuple(t.to(dtype).float() for t in kv)
    want, _ = P.attention_sublayer({k.replace("b.", "l."): v for k, v in wsb.items()}, "l.", x.float(), torch.arange(20), c, kv=kv)
    assert (got - want).abs().max() < tol(dtype, 10)
    with pytest.raises(ValueError, match="write"):
        reader.forward(ctx, x.to(T.DEV), T.view(cache, ctx, write=True))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d,f,n", [(64, 176, 5), (88, 120, 70), (96, 256, 200)])
def test_gated_feed_forward_part(dtype, d, f, n):
    rt = T.runtime(dtype)
    part = make_part("feed_forward", PartSpec("gated_mlp", "l.mlp", hidden=d, intermediate=f), rt)
    w = {"l.mlp.gate_proj.weight": rnd(f, d, seed=1, scale=0.2), "l.mlp.up_proj.weight": rnd(f, d, seed=2, scale=0.2),
         "l.mlp.down_proj.weight": rnd(d, f, seed=3, scale=0.2)}
    bind(part, w, dtype)
    ws = as_stored(w, dtype)
    x = rnd(n, d, seed=4).to(dtype)
    got = part.forward(T.context(rt, [(0, n)]), x.to(T.DEV)).float().sum(0).cpu()
    want = P.swiglu(x.float(), ws["l.mlp.gate_proj.weight"], ws["l.mlp.up_proj.weight"], ws["l.mlp.down_proj.weight"])
    assert (got - want).abs().max() < tol(dtype, 10)
    with pytest.raises(ValueError, match="activation"):
        make_part("feed_forward", PartSpec("gated_mlp", "x", hidden=8, intermediate=8, activation="gelu"), rt)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_parts(dtype):
    rt = T.runtime(dtype)
    emb = make_part("embedding", PartSpec("token_embedding", "tok", vocab=131, hidden=88), rt)
    head = make_part("head", PartSpec("linear_head", "tok", vocab=131, hidden=88), rt)      # tied: same tensor
    w = {"tok.weight": rnd(131, 88, seed=1)}
    bind(emb, w, dtype), bind(head, w, dtype)
    assert emb.table.data_ptr() != 0 and emb.weight_specs() == head.weight_specs()
    ids = [130, 0, 7, 7]
    ctx = T.context(rt, [(0, 4)], token_ids=ids)
    x = emb.forward(ctx, ctx.token_ids)
    table = w["tok.weight"].to(dtype).float()
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), table[ids])
    xn = rnd(3, 88, seed=2).to(dtype)
    logits = head.forward(ctx, xn.to(T.DEV))
    assert logits.dtype == torch.float32 and tuple(logits.shape) == (3, 131)
    assert (logits.cpu() - P.linear(xn.float(), table)).abs().max() < tol(dtype, 4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_pre_norm_block_is_a_decoder_layer(dtype):
    rt = T.runtime(dtype)
    d, f, p = 64, 176, ATTN[0]
    rot = PartSpec("rotary", head_dim=16, theta=10000.0)
    layer = LayerSpec(
        norm_mixer=PartSpec("rmsnorm", "model.layers.0.input_layernorm", size=d, eps=1e-5),
        mixer=PartSpec("attention", "model.layers.0.self_attn", position=rot, **p),
        norm_feed_forward=PartSpec("rmsnorm", "model.layers.0.post_attention_layernorm", size=d, eps=1e-5),
        feed_forward=PartSpec("gated_mlp", "model.layers.0.mlp", hidden=d, intermediate=f))
    block = make_part("block", PartSpec("pre_norm", layer=layer), rt)
    w = attn_weights(p, "model.layers.0.self_attn", 3)
    w.update({"model.layers.0.mlp.gate_proj.weight": rnd(f, d, seed=11, scale=0.2),
              "model.layers.0.mlp.up_proj.weight": rnd(f, d, seed=12, scale=0.2),
              "model.layers.0.mlp.down_proj.weight": rnd(d, f, seed=13, scale=0.2),
              "model.layers.0.input_layernorm.weight": 1 + 0.2 * rnd(d, seed=14),
              "model.layers.0.post_attention_layernorm.weight": 1 + 0.2 * rnd(d, seed=15)})
    assert sorted(s.name for s in block.weight_specs()) == sorted(w)
    bind(block, w, dtype)
    ctx = T.context(rt, [(0, 25)])
    for _, sp in rt.shared.values():
        sp.prepare(ctx)
    cache = T.empty_cache(2, 2, 16, 16, dtype)
    x0 = rnd(25, d, seed=20)
    carried = rnd(25, d, seed=21).to(T.DEV)                  # a delta not yet added
    x, pending = block.forward(ctx, x0.clone().to(T.DEV), carried, T.view(cache, ctx))
    got = (x + pending.float().sum(0)).cpu()
    c = dict(H=4, KV=2, hd=16, theta=10000.0, eps=1e-5)
    want, _ = P.decoder_layer(as_stored(w, dtype), 0, x0 + carried.cpu(), torch.arange(25), c)
    assert (got - want).abs().max() < tol(dtype, 20)


def test_unknown_part_kind_names_the_registered_ones():
    rt = T.runtime(torch.float32)
    with pytest.raises(ValueError, match="rmsnorm"):
        make_part("norm", PartSpec("layernorm", size=8, eps=1e-5), rt)


def test_weights_drawn_on_the_gpu_equal_those_drawn_on_the_cpu():
    """The seeded generator is integer mixing and one exact conversion: bit for bit the
    same on both devices, in any piece, for every role and dtype."""
    from kllm_amd.parts import WeightSpec
    from kllm_amd.weights import random_tensor
    from kllm_amd.weights.random_init import unit_variates
    for spec, dtype in [(WeightSpec("a.weight", (300, 257)), torch.float32), (WeightSpec("a.weight", (300, 257)), torch.bfloat16),
                        (WeightSpec("n.weight", (1000,), "vector"), torch.float32)]:
        cpu = random_tensor(spec, 9, dtype, 0.05, 0.1, "cpu")
        gpu = random_tensor(spec, 9, dtype, 0.05, 0.1, "cuda")
        assert torch.equal(cpu, gpu.cpu()) and gpu.dtype == dtype
    far = (1 << 33) + 12345                              # beyond 32 bits of element index
    assert torch.equal(unit_variates(9, "t", far, 1000, "cpu"), unit_variates(9, "t", far, 1000, "cuda").cpu())
    assert not torch.equal(unit_variates(9, "t", far, 1000, "cpu"), unit_variates(9, "t", far - (1 << 32), 1000, "cpu"))
