"""Pins the plain implementation by what fixes it beside the reference's text:
special cases that reduce to a library routine, invariants, and vectors the
reference's own files hold.  Each check is chosen so that a plausible mistake
(a wrong sign or pairing, a norm in the wrong place, a wrong head mapping)
fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
import tiny


def rnd(*shape, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=dtype)


# ------------------------------------------------------------------ linear, embedding

def test_linear_is_x_times_w_transposed():
    x, w = rnd(5, 7), rnd(3, 7, seed=1)
    assert torch.allclose(P.linear(x, w), F.linear(x, w))
    # a single 1 in W picks one input channel for one output channel
    w = torch.zeros(3, 7, dtype=torch.float64)
    w[2, 4] = 1.0
    assert torch.equal(P.linear(x, w)[:, 2], x[:, 4])


def test_embedding_is_a_row_lookup():
    table = rnd(11, 4)
    ids = [3, 0, 10, 3]
    assert torch.equal(P.embedding(ids, table), F.embedding(torch.tensor(ids), table))


# ------------------------------------------------------------------ rmsnorm

def test_rmsnorm_matches_library():
    x, w = rnd(6, 40), rnd(40, seed=2)
    for eps in (1e-5, 1e-6, 0.3):
        assert torch.allclose(P.rmsnorm(x, w, eps), F.rms_norm(x, (40,), w, eps), atol=1e-12)


def test_rmsnorm_invariants():
    x = rnd(4, 32)
    one = torch.ones(32, dtype=torch.float64)
    out = P.rmsnorm(x, one, 0.0)
    assert torch.allclose((out * out).mean(-1), torch.ones(4, dtype=torch.float64))   # RMS is 1
    assert torch.allclose(P.rmsnorm(3.7 * x, one, 0.0), out)                           # scale-free
    assert torch.equal(P.rmsnorm(torch.zeros(2, 8), torch.ones(8), 1e-5), torch.zeros(2, 8))
    # eps is added to the mean, not to the sum and not outside the root
    v = torch.full((1, 4), 2.0, dtype=torch.float64)
    assert torch.allclose(P.rmsnorm(v, torch.ones(4, dtype=torch.float64), 5.0),
                          v / math.sqrt(4.0 + 5.0))
    # the weight is w, not 1 + w
    assert torch.allclose(P.rmsnorm(x, torch.zeros(32, dtype=torch.float64), 1e-6),
                          torch.zeros(4, 32, dtype=torch.float64))


# ------------------------------------------------------------------ rotary

def test_rope_position_zero_is_identity_and_norms_are_kept():
    x = rnd(1, 2 * 16)
    assert torch.allclose(P.rope(x, [0], 2, 16, 10000.0), x)
    y = P.rope(rnd(3, 32), [5, 900, 4095], 2, 16, 500000.0)
    x3 = rnd(3, 32)
    pairs = lambda t: t.reshape(3, 2, 2, 8).pow(2).sum(2)   # |(j, j+half)|^2
    assert torch.allclose(pairs(y), pairs(x3))


def test_rope_is_complex_multiplication_on_half_split_pairs():
    hd, theta = 16, 10000.0
    x = rnd(4, hd)
    pos = [3, 17, 250, 4095]
    y = P.rope(x, pos, 1, hd, theta)
    j = torch.arange(hd // 2, dtype=torch.float64)
    ang = torch.tensor(pos, dtype=torch.float64)[:, None] * theta ** (-2.0 * j / hd)
    z = torch.complex(x[:, :hd // 2], x[:, hd // 2:]) * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(y, torch.cat([z.real, z.imag], -1), atol=1e-12)
    # ... and it is not the interleaved pairing (2j, 2j+1)
    zi = torch.view_as_complex(x.reshape(4, hd // 2, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)
    assert not torch.allclose(y, torch.view_as_real(zi).reshape(4, hd), atol=1e-3)


def test_rope_scores_depend_on_distance_only():
    hd = 32
    q, k = rnd(1, hd, seed=3), rnd(1, hd, seed=4)

    def score(t, u, theta):
        return float((P.rope(q, [t], 1, hd, theta) * P.rope(k, [u], 1, hd, theta)).sum())
    for theta in (10000.0, 500000.0):
        assert abs(score(10, 3, theta) - score(1010, 1003, theta)) < 1e-9
        assert abs(score(10, 3, theta) - score(3, 10, theta)) > 1e-3     # direction matters


def test_rope_first_frequency_is_one_radian_per_position():
    # pair j = 0 turns by exactly pos radians whatever theta is
    x = torch.zeros(1, 8, dtype=torch.float64)
    x[0, 0] = 1.0
    y = P.rope(x, [2], 1, 8, 12345.0)
    assert abs(float(y[0, 0]) - math.cos(2.0)) < 1e-12 and abs(float(y[0, 4]) - math.sin(2.0)) < 1e-12


# ------------------------------------------------------------------ attention

def sdpa(q, k, v, H, KV, hd, mask=None, causal=False):
    T, S = q.shape[0], k.shape[0]
    qh = q.reshape(T, H, hd).transpose(0, 1)
    kh = k.reshape(S, KV, hd).transpose(0, 1).repeat_interleave(H // KV, dim=0)
    vh = v.reshape(S, KV, hd).transpose(0, 1).repeat_interleave(H // KV, dim=0)
    o = F.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask, is_causal=causal)
    return o.transpose(0, 1).reshape(T, H * hd)


@pytest.mark.parametrize("H,KV,hd", [(4, 2, 16), (3, 1, 32), (5, 5, 48), (1, 1, 16)])
def test_attention_whole_prompt_matches_library(H, KV, hd):
    T = 13
    q, k, v = rnd(T, H * hd), rnd(T, KV * hd, seed=1), rnd(T, KV * hd, seed=2)
    got = P.attention(q, k, v, range(T), H, KV, hd)
    assert torch.allclose(got, sdpa(q, k, v, H, KV, hd, causal=True), atol=1e-10)


def test_attention_portion_after_cached_keys_matches_library_with_trapezoid_mask():
    H, KV, hd, S, T = 4, 2, 16, 20, 6
    q, k, v = rnd(T, H * hd), rnd(S, KV * hd, seed=1), rnd(S, KV * hd, seed=2)
    qpos = torch.arange(S - T, S)
    mask = torch.arange(S)[None, :] <= qpos[:, None]
    got = P.attention(q, k, v, qpos, H, KV, hd)
    assert torch.allclose(got, sdpa(q, k, v, H, KV, hd, mask=mask), atol=1e-10)


def test_attention_special_cases():
    H, KV, hd, T = 4, 2, 16, 9
    q, k, v = rnd(T, H * hd), rnd(T, KV * hd, seed=1), rnd(T, KV * hd, seed=2)
    out = P.attention(q, k, v, range(T), H, KV, hd)
    # the first token sees only itself: its output is its value, per KV group
    first = v[0].reshape(KV, hd).repeat_interleave(H // KV, dim=0).reshape(-1)
    assert torch.allclose(out[0], first)
    # q = 0: uniform weights, the mean of the values seen so far
    mean = P.attention(torch.zeros_like(q), k, v, range(T), H, KV, hd)
    want = (v.cumsum(0) / torch.arange(1, T + 1)[:, None]).reshape(T, KV, hd)
    assert torch.allclose(mean, want.repeat_interleave(H // KV, dim=1).reshape(T, -1))
    # head h reads KV head h // (H/KV), not h % KV
    v2 = v.clone()
    v2[:, hd:] += 1.0                       # change KV head 1 only
    changed = (P.attention(q, k, v2, range(T), H, KV, hd) - out).abs().reshape(T, H, hd).amax((0, 2))
    assert (changed[:2] == 0).all() and (changed[2:] > 0.5).all()
    # the scale is 1/sqrt(head_dim): one query, two keys, known weights
    qq = torch.zeros(2, hd, dtype=torch.float64)
    qq[1, 0] = 4.0
    kk = torch.zeros(2, hd, dtype=torch.float64)
    kk[1, 0] = 1.0
    vv = torch.zeros(2, hd, dtype=torch.float64)
    vv[1, 0] = 1.0
    o = P.attention(qq, kk, vv, range(2), 1, 1, hd)
    assert abs(float(o[1, 0]) - 1.0 / (1.0 + math.exp(-4.0 / math.sqrt(hd)))) < 1e-12


def test_attention_window_keeps_the_last_w_keys():
    H, KV, hd, T, W = 2, 1, 16, 12, 4
    q, k, v = rnd(T, H * hd), rnd(T, KV * hd, seed=1), rnd(T, KV * hd, seed=2)
    got = P.attention(q, k, v, range(T), H, KV, hd, window=W)
    pos = torch.arange(T)
    mask = (pos[None, :] <= pos[:, None]) & (pos[None, :] > pos[:, None] - W)
    assert torch.allclose(got, sdpa(q, k, v, H, KV, hd, mask=mask), atol=1e-10)
    # at the edge: position W-1 still sees key 0, position W does not
    v2 = v.clone()
    v2[0] += 5.0
    d = (P.attention(q, k, v2, range(T), H, KV, hd, window=W) - got).abs().amax(1)
    assert (d[:W] > 0).all() and (d[W:] == 0).all()


# ------------------------------------------------------------------ feed-forward

def test_swiglu_matches_library():
    x, wg, wu, wd = rnd(5, 12), rnd(20, 12, seed=1), rnd(20, 12, seed=2), rnd(12, 20, seed=3)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(P.swiglu(x, wg, wu, wd), want, atol=1e-12)
    assert float(P.silu(torch.tensor(0.0))) == 0.0
    assert abs(float(P.silu(torch.tensor(-80.0, dtype=torch.float64)))) < 1e-30
    # the gate, not the up branch, goes through the activation
    assert not torch.allclose(P.swiglu(x, wu, wg, wd), want, atol=1e-3)


# ------------------------------------------------------------------ whole model

def one_layer_by_library(w, cfg, ids):
    """A one-layer model written a second time with library routines only."""
    c = P._cfg(cfg)
    T = len(ids)
    x = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    p = "model.layers.0."
    xn = F.rms_norm(x, (c["d"],), w[p + "input_layernorm.weight"], c["eps"])
    q = F.linear(xn, w[p + "self_attn.q_proj.weight"])
    k = F.linear(xn, w[p + "self_attn.k_proj.weight"])
    v = F.linear(xn, w[p + "self_attn.v_proj.weight"])

    def rot(t, heads):
        hd = c["hd"]
        j = torch.arange(hd // 2, dtype=torch.float64)
        ang = torch.arange(T, dtype=torch.float64)[:, None] * c["theta"] ** (-2.0 * j / hd)
        th = t.reshape(T, heads, hd)
        z = torch.complex(th[..., :hd // 2], th[..., hd // 2:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
        return torch.cat([z.real, z.imag], -1).reshape(T, heads * hd)
    a = sdpa(rot(q, c["H"]), rot(k, c["KV"]), v, c["H"], c["KV"], c["hd"], causal=True)
    x = x + F.linear(a, w[p + "self_attn.o_proj.weight"])
    xn = F.rms_norm(x, (c["d"],), w[p + "post_attention_layernorm.weight"], c["eps"])
    x = x + F.linear(F.silu(F.linear(xn, w[p + "mlp.gate_proj.weight"])) *
                     F.linear(xn, w[p + "mlp.up_proj.weight"]), w[p + "mlp.down_proj.weight"])
    xn = F.rms_norm(x, (c["d"],), w["model.norm.weight"], c["eps"])
    return F.linear(xn, w["lm_head.weight"])


def test_one_layer_model_matches_library_composition():
    cfg = tiny.CONFIGS["C"]
    w = P.random_weights(cfg, 7, std=0.08, norm_std=0.2, dtype=torch.float64)
    ids = tiny.tokens(cfg, 15, 1)
    got = P.forward(w, cfg, ids, dtype=torch.float64)
    assert torch.allclose(got, one_layer_by_library(w, cfg, ids), atol=1e-10)


@pytest.mark.parametrize("name", ["A", "B"])
def test_model_invariants(name):
    cfg = tiny.CONFIGS[name]
    w = P.random_weights(cfg, 11, std=0.08, norm_std=0.2, dtype=torch.float64)
    ids = tiny.tokens(cfg, 24, 2)
    logits, hidden = P.forward(w, cfg, ids, dtype=torch.float64, return_hidden=True)
    L = cfg["num_hidden_layers"]
    assert len(hidden) == L + 2 and logits.shape == (24, cfg["vocab_size"])
    # only distances between positions count: shift every position
    shifted = P.forward(w, cfg, ids, dtype=torch.float64, pos0=777)
    assert torch.allclose(logits, shifted, atol=1e-9)
    # causal: logits of a prefix do not depend on what follows
    assert torch.allclose(P.forward(w, cfg, ids[:10], dtype=torch.float64), logits[:10], atol=1e-10)
    # tied head reads the embedding table; untied reads lm_head
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    assert torch.allclose(logits, hidden[-1] @ head.T)
    # residual stream: zero output projections leave a layer's input unchanged
    w0 = dict(w)
    w0["model.layers.0.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.0.self_attn.o_proj.weight"])
    w0["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.0.mlp.down_proj.weight"])
    _, h0 = P.forward(w0, cfg, ids, dtype=torch.float64, return_hidden=True)
    assert torch.equal(h0[1], h0[0])


def test_reference_tiny_model_shapes_and_prompts():
    """The reference's own tiny model (tools/make_test_model.py:47-100) and its
    prompts (tools/prompts_tiny.txt): the tensor list and shapes are the ones
    the reference requires at finalize (backend/model.cu:873-892)."""
    cfg = tiny.CONFIGS["R"]
    shapes = P.weight_shapes(cfg)
    assert len(shapes) == 3 + 9 * 2
    assert shapes["model.layers.1.self_attn.k_proj.weight"] == (32, 64)
    assert shapes["model.layers.0.mlp.down_proj.weight"] == (64, 128)
    assert shapes["lm_head.weight"] == (512, 64)
    w = P.random_weights(cfg, 0)
    for prompt in tiny.REFERENCE_PROMPTS:
        out = P.generate_greedy(w, cfg, prompt, 4)
        assert len(out) == 4 and all(0 <= t < 512 for t in out)


def test_greedy_takes_the_first_maximum():
    assert P.argmax_first(torch.tensor([1.0, 3.0, 3.0, 2.0])) == 1      # engine/engine.go:216-224
    assert P.argmax_first(torch.tensor([5.0, 5.0])) == 0


def test_sampling_reference():
    row = torch.tensor([0.0, math.log(2.0), math.log(5.0)])              # p = 1/8, 2/8, 5/8
    assert P.sample_inverse_cdf(row, 1.0, 0.0) == 0
    assert P.sample_inverse_cdf(row, 1.0, 0.124) == 0
    assert P.sample_inverse_cdf(row, 1.0, 0.126) == 1
    assert P.sample_inverse_cdf(row, 1.0, 0.374) == 1
    assert P.sample_inverse_cdf(row, 1.0, 0.376) == 2
    assert P.sample_inverse_cdf(row, 1.0, 0.999999) == 2
    assert P.sample_inverse_cdf(row, 0, 0.0) == 2
    # temperature sharpens: at T = 0.5 the weights are squared (1, 4, 25)/30
    assert P.sample_inverse_cdf(row, 0.5, 0.034) == 1


def test_storage_rounding_changes_little_and_nothing_when_it_is_the_identity():
    """``store`` marks where an engine with narrower storage keeps activations: the
    identity must give the default's logits (but for the order of the softmax's division),
    bfloat16 rounding logits that differ by rounding noise only (far less than the
    logits' own size)."""
    import tiny
    cfg = tiny.CONFIGS["A"]
    w = P.random_weights(cfg, 2, std=0.05, norm_std=0.1)
    ids = tiny.tokens(cfg, 40, 1)
    base = P.forward(w, cfg, ids)
    assert float((P.forward(w, cfg, ids, store=lambda t: t) - base).abs().max()) < 2e-6
    rounded = P.forward(w, cfg, ids, store=P.round_bfloat16)
    err = float((rounded - base).abs().max())
    assert 0 < err < 0.02 * float(base.abs().max())


def test_gelu_tanh_is_the_library_routine():
    x = torch.linspace(-8, 8, 4001, dtype=torch.float64)
    want = torch.nn.functional.gelu(x, approximate="tanh")
    assert (P.gelu_tanh(x) - want).abs().max() < 1e-12
    assert abs(float(P.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12
