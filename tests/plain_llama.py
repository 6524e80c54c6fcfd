"""Plain, slow Llama decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference (paths are relative to the
reference checkout); it shares no code with the package under test.  Every
function takes ordinary torch CPU tensors and computes in the dtype of its
inputs (float32 by default, float64 for a tighter yardstick).

Weights are a dict ``name -> tensor`` with the HuggingFace names the reference
requires (backend/model.cu:873-892).  All linear weights are ``[out, in]`` and
``y = x @ W.T`` (backend/model.cu:494-503); there are no biases.
"""

from __future__ import annotations

import math

import torch


# --------------------------------------------------------------------------- parts

def embedding(ids, table):
    """x[t, :] = E[id_t, :], no scaling for Llama (backend/model.cu:89-95, :1056-1060)."""
    ids = torch.as_tensor(ids, dtype=torch.long)
    return table[ids]


def rmsnorm(x, w, eps):
    """out = x * rsqrt(mean(x^2) + eps) * w (backend/model.cu:101-122;
    numpy form tools/gen_reference_numpy_moe.py:28-30).  eps is added to the
    mean, inside the square root; the weight multiplies after normalisation."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(ms + eps) * w


def linear(x, w):
    """Y[n, m] = X[n, k] . W[m, k]^T (backend/model.cu:494-503)."""
    return x @ w.transpose(0, 1)


def rope_angles(positions, head_dim, theta):
    """ang[t, j] = pos_t * theta^(-2j/head_dim) in float64
    (backend/model.cu:176-178; tools/gen_reference_numpy_moe.py:37-39)."""
    half = head_dim // 2
    j = torch.arange(half, dtype=torch.float64)
    freq = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * j / head_dim)
    pos = torch.as_tensor(positions, dtype=torch.float64)
    return pos[:, None] * freq[None, :]


def rope(x, positions, n_heads, head_dim, theta):
    """Half-split rotary encoding: the pair is (j, j + head_dim/2);
    a' = a*cos - b*sin, b' = b*cos + a*sin (backend/model.cu:170-184;
    tools/gen_reference_numpy_moe.py:33-45).  x is [T, n_heads*head_dim]."""
    T = x.shape[0]
    half = head_dim // 2
    ang = rope_angles(positions, head_dim, theta)
    cos = torch.cos(ang).to(x.dtype)[:, None, :]
    sin = torch.sin(ang).to(x.dtype)[:, None, :]
    xh = x.reshape(T, n_heads, head_dim)
    a, b = xh[:, :, :half], xh[:, :, half:]
    out = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
    return out.reshape(T, n_heads * head_dim)


def attention(q, k, v, q_positions, n_heads, n_kv_heads, head_dim, window=0, store=None):
    """Causal softmax attention of one sequence over its own keys.

    q is [T, H*hd] at absolute positions ``q_positions``; k and v are
    [S, KV*hd] and hold the keys of positions 0..S-1.  Query head h reads KV
    head h // (H/KV) (backend/model.cu:358).  A query at position p sees keys
    [0, p] (backend/model.cu:361), or the last ``window`` of them when
    window > 0 (backend/model.cu:224-225, :362).  score = (q.k) * 1/sqrt(hd)
    (backend/model.cu:1063-1064); softmax with the maximum subtracted
    (backend/model.cu:365-407; tools/gen_reference_numpy_moe.py:105-118).
    ``store`` (see ``forward``) rounds the exponentials before they meet the
    values; their sum is then taken over the rounded numbers."""
    T, S = q.shape[0], k.shape[0]
    group = n_heads // n_kv_heads
    qpos = torch.as_tensor(q_positions, dtype=torch.long)
    kpos = torch.arange(S, dtype=torch.long)
    mask = kpos[None, :] <= qpos[:, None]
    if window and window > 0:
        mask = mask & (kpos[None, :] > qpos[:, None] - window)
    scale = 1.0 / math.sqrt(head_dim)
    out = torch.zeros(T, n_heads * head_dim, dtype=q.dtype)
    for h in range(n_heads):
        kvh = h // group
        qh = q[:, h * head_dim:(h + 1) * head_dim]
        kh = k[:, kvh * head_dim:(kvh + 1) * head_dim]
        vh = v[:, kvh * head_dim:(kvh + 1) * head_dim]
        sc = (qh @ kh.transpose(0, 1)) * scale
        sc = torch.where(mask, sc, torch.full_like(sc, float("-inf")))
        sc = sc - sc.max(dim=1, keepdim=True).values
        p = torch.exp(sc)
        if store is not None:
            p = store(p)
            out[:, h * head_dim:(h + 1) * head_dim] = (p @ vh) / p.sum(dim=1, keepdim=True)
            continue
        p = p / p.sum(dim=1, keepdim=True)
        out[:, h * head_dim:(h + 1) * head_dim] = p @ vh
    return out


def silu(x):
    """x / (1 + exp(-x)) (backend/model.cu:477-483; tools/gen_reference_numpy_moe.py:48-49)."""
    return x / (1.0 + torch.exp(-x))


def gelu_tanh(x):
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) (backend/model.cu:131-139): the
    gate of the reference's other gated feed-forward; here for the kernels' activation
    argument, no model in this package uses it."""
    return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)))


def swiglu(xn, w_gate, w_up, w_down, store=None):
    """down(silu(gate(x)) * up(x)) (backend/model.cu:1112-1115)."""
    h = silu(linear(xn, w_gate)) * linear(xn, w_up)
    return linear(h if store is None else store(h), w_down)


# --------------------------------------------------------------------------- model

def _cfg(cfg):
    """The handful of numbers the forward pass needs, with the reference's
    defaults (models/config.go:107-119)."""
    H = cfg["num_attention_heads"]
    d = cfg["hidden_size"]
    return dict(
        L=cfg["num_hidden_layers"], d=d, H=H,
        KV=cfg.get("num_key_value_heads") or H,
        hd=cfg.get("head_dim") or d // H,
        eps=cfg.get("rms_norm_eps", 1e-6),
        theta=cfg.get("rope_theta", 10000.0),
        tied=bool(cfg.get("tie_word_embeddings", False)),
    )


def attention_sublayer(w, prefix, xn, positions, c, window=0, kv=None, store=None):
    """q, k, v projections, rotary on q and k before they are kept, attention,
    output projection (backend/model.cu:1090-1104).  With ``kv`` given (the
    rotated keys and the values another layer made) only q is projected.
    Returns (output, (k, v))."""
    keep = store if store is not None else (lambda t: t)
    q = linear(xn, w[prefix + "self_attn.q_proj.weight"])
    q = keep(rope(q, positions, c["H"], c["hd"], c["theta"]))
    if kv is None:
        k = linear(xn, w[prefix + "self_attn.k_proj.weight"])
        v = keep(linear(xn, w[prefix + "self_attn.v_proj.weight"]))
        k = keep(rope(k, positions, c["KV"], c["hd"], c["theta"]))
    else:
        k, v = kv
    a = keep(attention(q, k, v, torch.arange(len(positions)), c["H"], c["KV"], c["hd"], window, store))
    return linear(a, w[prefix + "self_attn.o_proj.weight"]), (k, v)


def decoder_layer(w, layer, x, positions, c, window=0, kv=None, store=None):
    """a = h + Attn(Norm_in(h)); h' = a + FFN(Norm_post(a))
    (backend/model.cu:1083-1117; the reference defers the second add into the
    next norm, which does not change the sum)."""
    p = f"model.layers.{layer}."
    keep = store if store is not None else (lambda t: t)
    xn = keep(rmsnorm(x, w[p + "input_layernorm.weight"], c["eps"]))
    a, kv_out = attention_sublayer(w, p, xn, positions, c, window, kv, store)
    x = x + a
    xn = keep(rmsnorm(x, w[p + "post_attention_layernorm.weight"], c["eps"]))
    x = x + swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                   w[p + "mlp.down_proj.weight"], store)
    return x, kv_out


def round_bfloat16(t):
    """A value as an engine with bfloat16 storage keeps it: rounded to nearest even."""
    return t.to(torch.bfloat16).to(t.dtype)


def forward(w, cfg, ids, dtype=torch.float32, return_hidden=False, schedule=None, pos0=0,
            windows=None, kv_from=None, store=None):
    """Logits [T, vocab] at every position of one whole sequence whose first
    token stands at position ``pos0`` (0 for a real sequence; another value
    only shifts every rotary angle, which must not change anything).
    ``hidden`` follows the reference's capture order: [0] the embedding, [j]
    the input of layer j, last the final norm's output (backend/model.cu:1061,
    :1085, :1123-1124; engine/e2e/e2e_test.go:117-131).  ``schedule`` is the
    order in which layers run (default 0..L-1); ``windows`` maps a layer to
    its attention window; ``kv_from`` maps a run of the schedule to the earlier
    run whose keys and values it reads.  ``store`` (for instance
    ``round_bfloat16``) is applied wherever an engine with narrower storage
    keeps an activation: the normalised rows that feed a product, rotated
    queries, kept keys and values, attention's exponentials and output, the
    gated activation.  The residual stream, every sum and the logits stay in
    ``dtype``; weights are rounded by the caller."""
    c = _cfg(cfg)
    w = {k: v.to(dtype) for k, v in w.items()}
    T = len(ids)
    positions = torch.arange(pos0, pos0 + T)
    x = embedding(ids, w["model.embed_tokens.weight"])
    hidden = [x.clone()]
    order = list(range(c["L"])) if schedule is None else list(schedule)
    kept = {}
    for run, layer in enumerate(order):
        kv = kept[kv_from[run]] if kv_from and run in kv_from else None
        win = (windows or {}).get(layer, 0)
        x, kept[run] = decoder_layer(w, layer, x, positions, c, win, kv, store)
        hidden.append(x.clone())
    xn = rmsnorm(x, w["model.norm.weight"], c["eps"])
    if store is not None:
        xn = store(xn)
    hidden.append(xn.clone())
    head = w["model.embed_tokens.weight"] if c["tied"] else w["lm_head.weight"]
    logits = linear(xn, head)
    if return_hidden:
        return logits, hidden
    return logits


def argmax_first(row):
    """Greedy choice; the first maximum wins (engine/engine.go:216-224)."""
    best, best_val = 0, float(row[0])
    for i in range(1, row.shape[0]):
        v = float(row[i])
        if v > best_val:
            best, best_val = i, v
    return best


def generate_greedy(w, cfg, prompt, max_new_tokens, dtype=torch.float32, eos=None):
    """Greedy generation by recomputing the whole sequence for each new token
    (the loop of engine/engine.go:192-213, without its cache)."""
    ids = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        logits = forward(w, cfg, ids, dtype=dtype)
        nxt = argmax_first(logits[-1])
        out.append(nxt)
        ids.append(nxt)
        if eos is not None and nxt in eos:
            break
    return out


# --------------------------------------------------------------------------- sampling

def softmax_temperature(logits_row, temperature):
    """p = softmax(logits / T) in float64 with the maximum subtracted."""
    z = logits_row.to(torch.float64) / float(temperature)
    z = z - z.max()
    e = torch.exp(z)
    return e / e.sum()


def sample_inverse_cdf(logits_row, temperature, u):
    """Smallest index whose cumulative probability exceeds u; greedy when
    temperature is 0."""
    if temperature == 0:
        return argmax_first(logits_row)
    p = softmax_temperature(logits_row, temperature)
    cdf = torch.cumsum(p, dim=0)
    idx = int(torch.searchsorted(cdf, torch.tensor(u * float(cdf[-1]), dtype=torch.float64), right=True))
    return min(idx, logits_row.shape[0] - 1)


# --------------------------------------------------------------------------- weights

def weight_shapes(cfg):
    """Name -> shape of every tensor the model needs (backend/model.cu:873-892),
    in the creation order of tools/make_test_model.py:82-96."""
    c = _cfg(cfg)
    d, f, V = c["d"], cfg["intermediate_size"], cfg["vocab_size"]
    qd, kvd = c["H"] * c["hd"], c["KV"] * c["hd"]
    shapes = {"model.embed_tokens.weight": (V, d)}
    for i in range(c["L"]):
        p = f"model.layers.{i}."
        shapes[p + "self_attn.q_proj.weight"] = (qd, d)
        shapes[p + "self_attn.k_proj.weight"] = (kvd, d)
        shapes[p + "self_attn.v_proj.weight"] = (kvd, d)
        shapes[p + "self_attn.o_proj.weight"] = (d, qd)
        shapes[p + "mlp.gate_proj.weight"] = (f, d)
        shapes[p + "mlp.up_proj.weight"] = (f, d)
        shapes[p + "mlp.down_proj.weight"] = (d, f)
        shapes[p + "input_layernorm.weight"] = (d,)
        shapes[p + "post_attention_layernorm.weight"] = (d,)
    shapes["model.norm.weight"] = (d,)
    if not c["tied"]:
        shapes["lm_head.weight"] = (V, d)
    return shapes


def random_weights(cfg, seed, std=0.02, norm_std=0.02, dtype=torch.float32):
    """Seeded weights in the manner of tools/make_test_model.py:59-80: linear
    and embedding ~ N(0, std), norm weights 1 + N(0, norm_std)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in weight_shapes(cfg).items():
        r = torch.randn(shape, generator=g, dtype=torch.float32)
        if len(shape) == 1:
            out[name] = (1.0 + norm_std * r).to(dtype)
        else:
            out[name] = (std * r).to(dtype)
    return out
