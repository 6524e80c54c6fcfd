"""That the engine takes parts and architectures it has never seen, without a
change to its files: a toy mixer with state of its own, a toy feed-forward
with routing, another position encoding, a running order that names a layer
twice and lets a layer read another layer's cache, and layers with a window
beside layers without (two cache groups).  The toy parts are written with
ordinary torch operations here in the test; they are no model of anyone's."""

import math

import pytest
import torch

import plain_llama as P
import tiny
import traces
from kllm_amd.config import LlamaConfig, register_architecture, unregister_architecture
from kllm_amd.parts import (CacheNeed, LayerSpec, ModelSpec, Part, PartSpec, Run, WeightSpec,
                            register_part, unregister_part)

pytestmark = pytest.mark.gpu


# ----------------------------------------------------------------------------- toy parts

class ToyDecayMixer(Part):
    """s_t = decay * s_{t-1} + W_in x_t ;  out_t = W_out s_t.  The state s is
    one vector per request, kept in a slot between steps."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden, self.width, self.decay = self.param("hidden"), self.param("width"), self.param("decay")

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("in.weight"), (self.width, self.hidden)),
                WeightSpec(self.tensor_name("out.weight"), (self.hidden, self.width))]

    def bind(self, weights):
        self.w_in = weights[self.tensor_name("in.weight")].float()
        self.w_out = weights[self.tensor_name("out.weight")].float()

    def cache_need(self):
        return CacheNeed("state", state_shape=(self.width,))

    def forward(self, ctx, xn, cache):
        u = xn.float() @ self.w_in.t()
        out = torch.empty(ctx.n, self.hidden, dtype=torch.float32, device=xn.device)
        slots = cache.slots.tolist()
        for s in range(ctx.n_spans):
            a, b = ctx.h_span_start[s], ctx.h_span_start[s + 1]
            state = cache.state[slots[s]]
            if ctx.h_span_pos[s] == 0:
                state.zero_()                       # a new request starts from nothing
            for t in range(a, b):
                state.mul_(self.decay).add_(u[t])
                out[t] = self.w_out @ state
        return out


class ToyRoutedFeedForward(Part):
    """Two tiny experts; each token goes to the one its router prefers."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden, self.width = self.param("hidden"), self.param("width")

    def weight_specs(self):
        specs = [WeightSpec(self.tensor_name("router.weight"), (2, self.hidden))]
        for e in range(2):
            specs += [WeightSpec(self.tensor_name(f"experts.{e}.up.weight"), (self.width, self.hidden)),
                      WeightSpec(self.tensor_name(f"experts.{e}.down.weight"), (self.hidden, self.width))]
        return specs

    def bind(self, weights):
        self.router = weights[self.tensor_name("router.weight")].float()
        self.up = [weights[self.tensor_name(f"experts.{e}.up.weight")].float() for e in range(2)]
        self.down = [weights[self.tensor_name(f"experts.{e}.down.weight")].float() for e in range(2)]

    def forward(self, ctx, xn):
        x = xn.float()
        choice = (x @ self.router.t()).argmax(-1)
        out = torch.zeros_like(x)
        for e in range(2):
            m = choice == e
            out[m] = torch.relu(x[m] @ self.up[e].t()) @ self.down[e].t()
        return out


class ToyAdditivePositions(Part):
    """Adds sin(position * rate) to every channel of the embedded tokens."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.rate = self.param("rate")

    def prepare(self, ctx):
        pass

    def on_embedding(self, ctx, x):
        x.add_(torch.sin(ctx.positions[:ctx.n].float() * self.rate)[:, None])


def toy_reference(w, cfg, ids, dtype_round):
    """The toy architecture written plainly, whole sequence, on the CPU.
    Returns (logits, margins): margins[t] is the gap between the router's two
    scores at position t; where it is tiny, rounding may send the token to the
    other expert, and everything after it in the sequence differs."""
    d, eps = cfg["hidden_size"], cfg["rms_norm_eps"]
    r = (lambda t: t.to(torch.bfloat16).float()) if dtype_round else (lambda t: t)
    T = len(ids)
    pos = torch.arange(T)
    x = P.embedding(ids, w["model.embed_tokens.weight"]) + torch.sin(pos.float() * 0.37)[:, None]
    c = P._cfg(cfg)
    # layer 0: attention (no rotary here: positions come from the embedding) + routed feed-forward
    xn = r(P.rmsnorm(x, w["model.layers.0.input_layernorm.weight"], eps))
    q = P.linear(xn, w["model.layers.0.self_attn.q_proj.weight"])
    k = P.linear(xn, w["model.layers.0.self_attn.k_proj.weight"])
    v = P.linear(xn, w["model.layers.0.self_attn.v_proj.weight"])
    a = P.attention(r(q), r(k), r(v), pos, c["H"], c["KV"], c["hd"])
    x = x + P.linear(r(a), w["model.layers.0.self_attn.o_proj.weight"])
    xn = r(P.rmsnorm(x, w["model.layers.0.post_attention_layernorm.weight"], eps))
    scores = xn @ w["model.layers.0.moe.router.weight"].t()
    choice = scores.argmax(-1)
    margins = (scores[:, 0] - scores[:, 1]).abs()
    ff = torch.zeros_like(x)
    for e in range(2):
        m = choice == e
        ff[m] = torch.relu(xn[m] @ w[f"model.layers.0.moe.experts.{e}.up.weight"].t()) @ \
            w[f"model.layers.0.moe.experts.{e}.down.weight"].t()
    x = x + ff
    # layer 1: decay mixer + gated feed-forward
    xn = r(P.rmsnorm(x, w["model.layers.1.input_layernorm.weight"], eps))
    u = xn @ w["model.layers.1.mix.in.weight"].t()
    s = torch.zeros(u.shape[1])
    mix = torch.zeros_like(x)
    for t in range(T):
        s = 0.9 * s + u[t]
        mix[t] = w["model.layers.1.mix.out.weight"] @ s
    x = x + mix
    xn = r(P.rmsnorm(x, w["model.layers.1.post_attention_layernorm.weight"], eps))
    x = x + P.swiglu(xn, w["model.layers.1.mlp.gate_proj.weight"], w["model.layers.1.mlp.up_proj.weight"],
                     w["model.layers.1.mlp.down_proj.weight"]) if not dtype_round else x + P.linear(
        r(P.silu(P.linear(xn, w["model.layers.1.mlp.gate_proj.weight"])) * P.linear(xn, w["model.layers.1.mlp.up_proj.weight"])),
        w["model.layers.1.mlp.down_proj.weight"])
    xn = r(P.rmsnorm(x, w["model.norm.weight"], eps))
    return P.linear(xn, w["lm_head.weight"]), margins


def build_toy(cfg: LlamaConfig) -> ModelSpec:
    d = cfg.hidden_size
    positions = PartSpec("toy_additive", rate=0.37)
    norm = lambda name: PartSpec("rmsnorm", name, size=d, eps=cfg.rms_norm_eps)
    layers = [
        LayerSpec(norm_mixer=norm("model.layers.0.input_layernorm"),
                  mixer=PartSpec("attention", "model.layers.0.self_attn", hidden=d, heads=cfg.num_attention_heads,
                                 kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim, position=positions),
                  norm_feed_forward=norm("model.layers.0.post_attention_layernorm"),
                  feed_forward=PartSpec("toy_routed", "model.layers.0.moe", hidden=d, width=24)),
        LayerSpec(norm_mixer=norm("model.layers.1.input_layernorm"),
                  mixer=PartSpec("toy_decay", "model.layers.1.mix", hidden=d, width=40, decay=0.9),
                  norm_feed_forward=norm("model.layers.1.post_attention_layernorm"),
                  feed_forward=PartSpec("gated_mlp", "model.layers.1.mlp", hidden=d,
                                        intermediate=cfg.intermediate_size)),
    ]
    return ModelSpec(
        embedding=PartSpec("token_embedding", "model.embed_tokens", vocab=cfg.vocab_size, hidden=d),
        layers=layers, schedule=[Run(0), Run(1)], final_norm=norm("model.norm"),
        head=PartSpec("linear_head", "lm_head", vocab=cfg.vocab_size, hidden=d),
        vocab_size=cfg.vocab_size, hidden_size=d)


@pytest.fixture
def toy_registered():
    register_part("mixer", "toy_decay", ToyDecayMixer)
    register_part("feed_forward", "toy_routed", ToyRoutedFeedForward)
    register_part("position", "toy_additive", ToyAdditivePositions)
    register_architecture("ToyForCausalLM", LlamaConfig, build_toy)
    yield dict(tiny.CONFIGS["A"], architectures=["ToyForCausalLM"])
    unregister_architecture("ToyForCausalLM")
    for cat, kind in (("mixer", "toy_decay"), ("feed_forward", "toy_routed"), ("position", "toy_additive")):
        unregister_part(cat, kind)


def engine_weights_seed(eng, seed):
    """name -> float32 CPU tensor of what the engine's parts were given."""
    from kllm_amd.weights import random_weights
    return {k: v.float().cpu() for k, v in random_weights(eng.model.weight_specs(), seed, eng.dtype, "cpu", 0.08, 0.2).items()}


def engine_weights(eng):
    return engine_weights_seed(eng, 5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(toy_registered, dtype):
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    cfg = toy_registered
    eng = Engine.from_random(cfg, 5, EngineOptions(dtype=dtype, max_tokens=256, max_requests=3), std=0.08, norm_std=0.2)
    plan = eng.model.cache_plan
    assert [g.need.kind for g in plan.groups] == ["paged", "state"] and plan.runs == [(0, 0, True), (1, 0, True)]
    assert tuple(eng.state[1].shape) == (1, 3, 40)
    # the toy parts use torch operations: the engine calls them with its recorded launches run, and
    # does not run such a model's steps again from recorded commands
    assert eng.records_launches and not eng._repeat_steps
    w = engine_weights(eng)
    reqs = {"a": tiny.tokens(cfg, 45, 1), "b": tiny.tokens(cfg, 30, 2), "c": tiny.tokens(cfg, 22, 3),
            "d": tiny.tokens(cfg, 37, 4)}
    want = {rid: toy_reference(w, cfg, toks, dtype == "bfloat16") for rid, toks in reqs.items()}
    steps, peak = traces.mixed(reqs, seed=3, max_live=3, tail=6, max_portion=9)
    outs = []
    for s in steps:
        out = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        outs.append(out.cpu().numpy())
        for rid in s["end"]:
            eng.release(rid)                      # the slot goes back and is taken again by "d"
    rows = traces.collect(steps, outs)
    compared = 0
    for rid, toks in reqs.items():
        logits, margins = want[rid]
        close = (margins < (1e-4 if dtype == "float32" else 8e-3)).nonzero()
        upto = int(close[0]) if len(close) else len(toks)     # a near-tie of the router ends the comparison
        for p in range(upto):
            err = float((torch.from_numpy(rows[(rid, p)]) - logits[p]).abs().max())
            assert err < (2e-4 if dtype == "float32" else 8e-2), (rid, p, err)
        compared += upto
    assert compared >= 60, compared
    assert eng.cache.slots.free_slots == 3 and not eng.cache.requests


# ----------------------------------------------------------------------------- running order

def build_repeat_and_share(cfg: LlamaConfig) -> ModelSpec:
    """Three layers; layer 1 runs twice (a cache for each run); layer 2 has no
    k/v projections and reads the cache of layer 1's first run."""
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    spec.layers[2].mixer.params["own_kv"] = False
    spec.schedule = [Run(0), Run(1), Run(1), Run(2, cache_of=1)]
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_twice_and_a_layer_reading_anothers_cache(dtype, tmp_path):
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_architecture("ToyScheduleForCausalLM", LlamaConfig, build_repeat_and_share)
    try:
        cfg = dict(tiny.CONFIGS["B"], architectures=["ToyScheduleForCausalLM"])
        w = P.random_weights(cfg, 4, std=0.05, norm_std=0.1)
        del w["model.layers.2.self_attn.k_proj.weight"], w["model.layers.2.self_attn.v_proj.weight"]
        d = tiny.write_model(str(tmp_path), cfg, 0, weights=w)
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=192))
        plan = eng.model.cache_plan
        assert plan.groups[0].entries == 3 and plan.runs == [(0, 0, True), (0, 1, True), (0, 2, True), (0, 1, False)]
        ids = tiny.tokens(cfg, 60, 1)
        ws = tiny.read_weights(d, as_stored_in=dtype)
        want = P.forward(ws, cfg, ids, schedule=[0, 1, 1, 2], kv_from={3: 1})
        got = torch.cat([eng.step([StepEntry("r", ids[a:b], list(range(b - a)))]).cpu()
                         for a, b in [(0, 23), (23, 25), (25, 59), (59, 60)]])
        assert float((got - want).abs().max()) < tiny.TOL[dtype]
        assert float((want - P.forward(ws | {"model.layers.2.self_attn.k_proj.weight": ws["model.layers.1.self_attn.k_proj.weight"],
                                             "model.layers.2.self_attn.v_proj.weight": ws["model.layers.1.self_attn.v_proj.weight"]},
                                       cfg, ids, schedule=[0, 1, 1, 2])).abs().max()) > 1e-3
    finally:
        unregister_architecture("ToyScheduleForCausalLM")


def test_a_bad_running_order_is_refused():
    from kllm_amd.engine.model import Model
    from kllm_amd.models.llama import build_llama
    from kllm_amd.config import config_from_dict
    from kllm_amd.parts import Runtime
    cfg = config_from_dict(tiny.CONFIGS["B"])
    rt = lambda: Runtime(device=torch.device("cpu"), dtype=torch.float32)
    spec = build_llama(cfg)
    spec.schedule = [Run(0), Run(5)]
    with pytest.raises(ValueError, match="names layer 5"):
        Model(spec, rt())
    spec.schedule = [Run(0, cache_of=0)]
    with pytest.raises(ValueError, match="earlier entry"):
        Model(spec, rt())


# ----------------------------------------------------------------------------- windows

WINDOW = 20


def build_windowed(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    for i in (0, 2):
        spec.layers[i].mixer.params["window"] = WINDOW
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_with_a_window_have_pages_of_their_own(dtype, model_dirs, tmp_path):
    import json
    import os
    import shutil
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_architecture("ToyWindowForCausalLM", LlamaConfig, build_windowed)
    try:
        cfg = dict(tiny.CONFIGS["B"], architectures=["ToyWindowForCausalLM"])
        d = str(tmp_path / "m")
        shutil.copytree(model_dirs("B"), d)
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(cfg, f)
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, num_pages=14, max_model_len=1 << 20,
                                               poison_freed_pages=True))
        plan = eng.model.cache_plan
        assert [(g.need.window, g.entries) for g in plan.groups] == [(WINDOW, 2), (0, 1)]
        ids = tiny.tokens(cfg, 200, 1)
        want = P.forward(tiny.read_weights(d, as_stored_in=dtype), cfg, ids, windows={0: WINDOW, 2: WINDOW})
        cuts = [0, 37, 39, 70, 71, 72, 130, 133] + list(range(134, 201))
        got = []
        for a, b in zip(cuts, cuts[1:]):
            got.append(eng.step([StepEntry("r", ids[a:b], list(range(b - a)))]).cpu())
            win, full = eng.cache.pools
            assert win.used_pages <= -(-(WINDOW + (b - a)) // 16) + 1     # the window's pages only
            assert full.used_pages == -(-b // 16)
        got = torch.cat(got)
        assert torch.isfinite(got).all()
        assert float((got - want).abs().max()) < tiny.TOL[dtype]
        assert eng.cache.pools[0].total_allocs == 13 and eng.cache.pools[0].used_pages <= 3
        eng.release("r")
        eng.cache.check_invariants()
    finally:
        unregister_architecture("ToyWindowForCausalLM")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_of_the_windowed_model_as_graphs(dtype):
    """Two cache groups, one of them windowed (its tables lose pages at the back while the
    other's grow): single-token steps of two requests queued as recorded HIP graphs give, bit
    for bit, what the eager step gives, across a change of the growing table's width."""
    import numpy as np
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_architecture("ToyWindowForCausalLM", LlamaConfig, build_windowed)
    try:
        cfg = dict(tiny.CONFIGS["B"], architectures=["ToyWindowForCausalLM"])
        reqs = {"a": tiny.tokens(cfg, 150, 1), "b": tiny.tokens(cfg, 97, 2)}
        prompt = {"a": 110, "b": 60}
        outs = {}
        for mode in ("eager", "graph"):
            eng = Engine.from_random(cfg, 3, EngineOptions(dtype=dtype, num_pages=24, max_model_len=1 << 20,
                                                           poison_freed_pages=True, graph_after_steps=1),
                                     std=0.05, norm_std=0.1)
            eng.step([StepEntry(r, reqs[r][:prompt[r]], []) for r in reqs])
            got = []
            for k in range(37):
                entries = [StepEntry(r, [reqs[r][prompt[r] + k]], [0]) for r in reqs]
                if mode == "eager":
                    got.append(eng.step(entries).cpu().numpy().copy())
                else:
                    assert eng.can_sample_ahead(entries)
                    h = eng.step_sample_ahead(entries, [0.0, 0.0], [0.0, 0.0])
                    h.tokens()
                    got.append(h.logits.cpu().numpy().copy())
            if mode == "graph":
                assert len(eng._graphs.recordings) >= 2          # request a's table grew from 7 to 10 pages
                assert eng.cache.pools[0].used_pages <= 2 * 3     # the window's pages only
            eng.cache.check_invariants()
            outs[mode] = got
        for k, (a, b) in enumerate(zip(outs["eager"], outs["graph"])):
            assert np.isfinite(a).all() and np.array_equal(a, b), k
    finally:
        unregister_architecture("ToyWindowForCausalLM")


def test_pools_are_sized_per_group_and_from_a_byte_budget():
    """A windowed group gets no more pages than its requests can hold; a byte budget
    shrinks every pool; page sizes no kernel takes and portions larger than the engine
    was sized for are refused when they are asked for, not at the first launch."""
    from kllm_amd.cache.manager import window_pages
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    from kllm_amd.engine.engine import StepError
    register_architecture("ToyWindowForCausalLM", LlamaConfig, build_windowed)
    try:
        cfg = dict(tiny.CONFIGS["B"], architectures=["ToyWindowForCausalLM"])
        base = dict(dtype="float32", num_pages=1000, max_requests=4, max_model_len=400, max_step_tokens=32)
        eng = Engine.from_random(cfg, 1, EngineOptions(**base))
        per_request = window_pages(400, 32, 16, WINDOW)
        assert per_request == 5
        assert [p.num_pages for p in eng.cache.pools] == [4 * per_request, 1000]
        assert eng.kv[0].shape[1] == 20 and eng.kv[1].shape[1] == 1000
        report = eng.capacity_report()
        assert "window 20: 20 pages" in report and "asked for 1000 pages" in report and "1000 pages of 16" in report
        with pytest.raises(StepError, match="sized for 32"):
            eng.step([StepEntry("r", tiny.tokens(cfg, 33, 1), [32])])
        assert eng.cache.pools[0].free_pages == 20 and "r" not in eng.cache
        # a 200-token request in portions of 32 runs in the small windowed pool
        ids = tiny.tokens(cfg, 200, 2)
        for a in range(0, 200, 32):
            eng.step([StepEntry("r", ids[a:a + 32], [])])
        assert eng.cache.pools[0].high_water <= per_request
        # a byte budget: one page of the windowed group (2 layers) and of the other (1 layer)
        page_bytes = [2 * 2 * 1 * 16 * 32 * 4, 1 * 2 * 1 * 16 * 32 * 4]
        full = 20 * page_bytes[0] + 1000 * page_bytes[1]
        eng2 = Engine.from_random(cfg, 1, EngineOptions(**base, memory_bytes=full // 4))
        pages = [p.num_pages for p in eng2.cache.pools]
        assert pages == [5, 250] and eng2.cache_bytes() <= full // 4
        assert "budget" in eng2.capacity_report()
        with pytest.raises(ValueError, match="no room for a cache page"):
            Engine.from_random(cfg, 1, EngineOptions(**base, memory_bytes=1000))
        with pytest.raises(ValueError, match="pages of 512 tokens"):
            Engine.from_random(cfg, 1, EngineOptions(dtype="float32", page_size=512))
    finally:
        unregister_architecture("ToyWindowForCausalLM")


# ----------------------------------------------------------------------------- a mixer with its own tiling

class ToyTiledMixer(Part):
    """out_t = W x_t, computed tile by tile over tiles of at most TILE rows that never
    cross a span: the tiling is this part's own, asked for through ``step_lists`` and
    found on the device in ``ctx.lists``.  Rows that no tile covers stay NaN."""
    step_lists_key = "toy.tiled"
    TILE = 5
    seen = []                                    # (starts, lens, tiles as the device held them)

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = self.param("hidden")

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("weight"), (self.hidden, self.hidden))]

    def bind(self, weights):
        self.w = weights[self.tensor_name("weight")].float()

    def step_lists(self, starts, lens):
        tiles = []
        for a, n in zip(starts, lens):
            for t in range(a, a + n, self.TILE):
                tiles += [t, min(self.TILE, a + n - t)]
        return {"tiles": tiles}

    def forward(self, ctx, xn, cache):
        tiles = ctx.lists["toy.tiled.tiles"]
        assert tiles.dtype == torch.int32 and tiles.is_cuda
        host = tiles.tolist()
        ToyTiledMixer.seen.append((list(ctx.h_span_start), list(ctx.h_span_len), host))
        out = torch.full((ctx.n, self.hidden), float("nan"), dtype=torch.float32, device=xn.device)
        for row, count in zip(host[0::2], host[1::2]):
            out[row:row + count] = xn[row:row + count].float() @ self.w.t()
        return out


def build_tiled(cfg: LlamaConfig) -> ModelSpec:
    """Layer 0: the tiled toy mixer and a feed-forward gated by the tanh approximation of
    GELU; layer 1: attention (whose own span lists travel beside the toy's) and the
    SiLU-gated feed-forward."""
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    spec.layers[0].mixer = PartSpec("toy_tiled", "model.layers.0.mix", hidden=cfg.hidden_size)
    spec.layers[0].feed_forward.params["activation"] = "gelu_tanh"
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_with_its_own_tiling_and_a_gelu_gated_feed_forward(dtype):
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_part("mixer", "toy_tiled", ToyTiledMixer)
    register_architecture("ToyTiledForCausalLM", LlamaConfig, build_tiled)
    try:
        cfg = dict(tiny.CONFIGS["A"], architectures=["ToyTiledForCausalLM"])
        eng = Engine.from_random(cfg, 5, EngineOptions(dtype=dtype, max_tokens=256, max_requests=4),
                                 std=0.08, norm_std=0.2)
        assert sorted(eng.model.step_lists([0, 3, 4], [3, 1])) == ["attention.spans.blocks", "attention.spans.short",
                                                                   "toy.tiled.tiles"]
        w = engine_weights(eng)
        r = (lambda t: t.to(torch.bfloat16).float()) if dtype == "bfloat16" else (lambda t: t)
        c = P._cfg(cfg)

        def reference(ids):
            x = P.embedding(ids, w["model.embed_tokens.weight"])
            xn = r(P.rmsnorm(x, w["model.layers.0.input_layernorm.weight"], c["eps"]))
            x = x + P.linear(xn, w["model.layers.0.mix.weight"])
            xn = r(P.rmsnorm(x, w["model.layers.0.post_attention_layernorm.weight"], c["eps"]))
            h = P.gelu_tanh(P.linear(xn, w["model.layers.0.mlp.gate_proj.weight"])) * \
                P.linear(xn, w["model.layers.0.mlp.up_proj.weight"])
            x = x + P.linear(r(h), w["model.layers.0.mlp.down_proj.weight"])
            x, _ = P.decoder_layer(w, 1, x, torch.arange(len(ids)), c, store=r if dtype == "bfloat16" else None)
            return P.linear(r(P.rmsnorm(x, w["model.norm.weight"], c["eps"])), w["lm_head.weight"])

        reqs = {"a": tiny.tokens(cfg, 45, 1), "b": tiny.tokens(cfg, 30, 2), "c": tiny.tokens(cfg, 22, 3)}
        steps, _ = traces.mixed(reqs, seed=3, max_live=3, tail=6, max_portion=13)
        ToyTiledMixer.seen.clear()
        outs = []
        for s in steps:
            outs.append(eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]).cpu().numpy())
            for rid in s["end"]:
                eng.release(rid)
        rows = traces.collect(steps, outs)
        for rid, toks in reqs.items():
            want = reference(toks)
            for p in range(len(toks)):
                err = float((torch.from_numpy(rows[(rid, p)]) - want[p]).abs().max())
                assert err < (2e-4 if dtype == "float32" else 8e-2), (rid, p, err)
        # every step carried this part's tiling of exactly its spans
        assert len(ToyTiledMixer.seen) == len(steps)
        part = eng.model.blocks[0].mixer
        for starts, lens, tiles in ToyTiledMixer.seen:
            assert tiles == part.step_lists(starts, lens)["tiles"]
            assert sum(tiles[1::2]) == sum(lens) and max(tiles[1::2]) <= ToyTiledMixer.TILE
        assert any(len(l) > 1 and max(l) > ToyTiledMixer.TILE for _, l, _ in ToyTiledMixer.seen)
        # the gate matters: SiLU instead of GELU moves the logits far beyond the tolerance
        ids = reqs["a"]
        x = P.embedding(ids, w["model.embed_tokens.weight"])
        xn = P.rmsnorm(x + P.linear(P.rmsnorm(x, w["model.layers.0.input_layernorm.weight"], c["eps"]),
                                    w["model.layers.0.mix.weight"]), w["model.layers.0.post_attention_layernorm.weight"], c["eps"])
        g = P.linear(xn, w["model.layers.0.mlp.gate_proj.weight"])
        assert float((P.gelu_tanh(g) - P.silu(g)).abs().max()) > 0.05
    finally:
        unregister_architecture("ToyTiledForCausalLM")
        unregister_part("mixer", "toy_tiled")


# ----------------------------------------------------------------------------- another rotation

class ToyPartialInterleavedRotary(Part):
    """Rotates only the first ``rotary_dim`` elements of a head, in neighbouring pairs
    (2j, 2j + 1), with angles position * base^(-j / pairs): neither the pairing nor the
    extent of the built-in rotary part.  The tables are made with torch in the test."""
    interleaved = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.rotary_dim, self.base = int(self.param("rotary_dim")), float(self.param("base"))

    @staticmethod
    def angles(positions, rotary_dim, base):
        pairs = rotary_dim // 2
        freq = base ** (-torch.arange(pairs, dtype=torch.float64) / pairs)
        return positions.double()[:, None] * freq[None, :]

    def prepare(self, ctx):
        ang = self.angles(ctx.positions[:ctx.n].cpu(), self.rotary_dim, self.base)
        ctx.scratch[("toy_rot", id(self))] = (torch.cos(ang).float().to(ctx.positions.device).contiguous(),
                                              torch.sin(ang).float().to(ctx.positions.device).contiguous())

    def tables(self, ctx):
        return ctx.scratch[("toy_rot", id(self))]


ROT_DIM, ROT_BASE = 8, 50.0


def build_other_rotation(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    pos = PartSpec("toy_partial_interleaved", rotary_dim=ROT_DIM, base=ROT_BASE)
    for layer in spec.layers:
        layer.mixer.params["position"] = pos
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_rotation_with_another_pairing_and_extent(dtype):
    """A position part that rotates half of each head in neighbouring pairs is registered
    and used without a change to the package: the attention part reads the pairing from the
    position part and the rotate-and-append kernel takes it as arguments."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_part("position", "toy_partial_interleaved", ToyPartialInterleavedRotary)
    register_architecture("ToyRotationForCausalLM", LlamaConfig, build_other_rotation)
    try:
        cfg = dict(tiny.CONFIGS["A"], architectures=["ToyRotationForCausalLM"])
        eng = Engine.from_random(cfg, 7, EngineOptions(dtype=dtype, max_tokens=256, max_requests=4), std=0.08, norm_std=0.2)
        w = engine_weights_seed(eng, 7)
        c = P._cfg(cfg)
        r = (lambda t: t.to(torch.bfloat16).float()) if dtype == "bfloat16" else (lambda t: t)

        def rotate(x, positions, heads):
            ang = ToyPartialInterleavedRotary.angles(positions, ROT_DIM, ROT_BASE).float()
            cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            x = x.view(len(positions), heads, c["hd"]).clone()
            a, b = x[..., 0:ROT_DIM:2].clone(), x[..., 1:ROT_DIM:2].clone()
            x[..., 0:ROT_DIM:2] = a * cos - b * sin
            x[..., 1:ROT_DIM:2] = b * cos + a * sin
            return x.reshape(len(positions), heads * c["hd"])

        def reference(ids):
            T = len(ids)
            pos = torch.arange(T)
            x = P.embedding(ids, w["model.embed_tokens.weight"])
            for l in range(c["L"]):
                p = f"model.layers.{l}."
                xn = r(P.rmsnorm(x, w[p + "input_layernorm.weight"], c["eps"]))
                q = r(rotate(P.linear(xn, w[p + "self_attn.q_proj.weight"]), pos, c["H"]))
                k = r(rotate(P.linear(xn, w[p + "self_attn.k_proj.weight"]), pos, c["KV"]))
                v = r(P.linear(xn, w[p + "self_attn.v_proj.weight"]))
                a = r(P.attention(q, k, v, pos, c["H"], c["KV"], c["hd"], store=r if dtype == "bfloat16" else None))
                x = x + P.linear(a, w[p + "self_attn.o_proj.weight"])
                xn = r(P.rmsnorm(x, w[p + "post_attention_layernorm.weight"], c["eps"]))
                x = x + P.swiglu(xn, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                                 w[p + "mlp.down_proj.weight"], r if dtype == "bfloat16" else None)
            return P.linear(r(P.rmsnorm(x, w["model.norm.weight"], c["eps"])), w["lm_head.weight"])

        reqs = {"a": tiny.tokens(cfg, 45, 1), "b": tiny.tokens(cfg, 30, 2), "c": tiny.tokens(cfg, 22, 3)}
        steps, _ = traces.mixed(reqs, seed=5, max_live=3, tail=6, max_portion=13)
        outs = []
        for s in steps:
            outs.append(eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]).cpu().numpy())
            for rid in s["end"]:
                eng.release(rid)
        rows = traces.collect(steps, outs)
        for rid, toks in reqs.items():
            want = reference(toks)
            for p in range(len(toks)):
                err = float((torch.from_numpy(rows[(rid, p)]) - want[p]).abs().max())
                assert err < (2e-4 if dtype == "float32" else 8e-2), (rid, p, err)
        # the rotation matters, and so do its pairing and extent: the built-in rotation over the
        # same weights gives other logits
        plain = P.forward(w, cfg, reqs["a"])
        assert float((plain - reference(reqs["a"])).abs().max()) > 0.05
    finally:
        unregister_architecture("ToyRotationForCausalLM")
        unregister_part("position", "toy_partial_interleaved")


# ----------------------------------------------------------------------------- another norm, another arrangement

class ToyCenteredNorm(Part):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * w + b, written with torch operations.  It
    takes what every norm takes: a ``delta`` (one tensor or a stack of partial sums over
    slices of K) that is added into the float32 stream first, or ``rows`` to read."""
    graph_safe = False

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.size, self.eps = int(self.param("size")), float(self.param("eps"))

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("weight"), (self.size,), "vector"),
                WeightSpec(self.tensor_name("bias"), (self.size,), "vector")]

    def bind(self, weights):
        self.weight, self.bias = weights[self.tensor_name("weight")], weights[self.tensor_name("bias")]

    def add(self, ctx, x, delta):
        x += delta.sum(0) if delta.dim() == 3 else delta
        return x

    def normalise(self, x):
        mu = x.mean(-1, keepdim=True)
        var = ((x - mu) ** 2).mean(-1, keepdim=True)
        return (x - mu) / torch.sqrt(var + self.eps) * self.weight + self.bias

    def forward(self, ctx, x, delta=None, rows=None, tag="xn", normed_ok=False):
        if delta is not None and rows is None:
            self.add(ctx, x, delta)
        src = x if rows is None else x[rows.long()]
        return self.normalise(src).to(self.runtime.dtype)


class ToyPostNormBlock(Part):
    """h = Norm1(h + Mixer(h)); h' = Norm2(h + FeedForward(h)): the norms stand behind the
    additions and their result is the stream.  Built from the same kinds of parts as the
    arrangement the package has; leaves nothing pending."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        from kllm_amd.parts import make_part
        layer = self.param("layer")
        self.norm_mixer = make_part("norm", layer.norm_mixer, runtime)
        self.mixer = make_part("mixer", layer.mixer, runtime)
        self.norm_ff = make_part("norm", layer.norm_feed_forward, runtime)
        self.feed_forward = make_part("feed_forward", layer.feed_forward, runtime)

    graph_safe = False

    def children(self):
        return [self.norm_mixer, self.mixer, self.norm_ff, self.feed_forward]

    def weight_specs(self):
        return [s for p in self.children() for s in p.weight_specs()]

    def bind(self, weights):
        for p in self.children():
            p.bind(weights)

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, ctx, x, pending, cache, next_norm=None):
        assert pending is None                         # no layer before this kind leaves anything pending
        dtype = self.runtime.dtype
        a = self.mixer.forward(ctx, x.to(dtype), cache)
        x.copy_(self.norm_mixer.forward(ctx, x, delta=a).float())
        f = self.feed_forward.forward(ctx, x.to(dtype))
        x.copy_(self.norm_ff.forward(ctx, x, delta=f).float())
        return x, None


def build_post_norm(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    for i, layer in enumerate(spec.layers):
        layer.block = "toy_post_norm"
        layer.norm_mixer = PartSpec("toy_centered", f"model.layers.{i}.norm_a", size=cfg.hidden_size, eps=1e-3)
        layer.norm_feed_forward = PartSpec("toy_centered", f"model.layers.{i}.norm_b", size=cfg.hidden_size, eps=1e-3)
    spec.final_norm = PartSpec("toy_centered", "model.final", size=cfg.hidden_size, eps=1e-3)
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_norm_with_a_bias_and_an_arrangement_with_the_norms_behind_the_additions(dtype):
    """Another norm (centred, with a bias) and another arrangement of a layer (post-norm) are
    registered from here and run with the package's attention and feed-forward: mixed
    steps with page reuse against a plain computation of the same formulas."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_part("norm", "toy_centered", ToyCenteredNorm)
    register_part("block", "toy_post_norm", ToyPostNormBlock)
    register_architecture("ToyPostNormForCausalLM", LlamaConfig, build_post_norm)
    try:
        cfg = dict(tiny.CONFIGS["B"], architectures=["ToyPostNormForCausalLM"])
        eng = Engine.from_random(cfg, 5, EngineOptions(dtype=dtype, max_tokens=192, max_requests=4),
                                 std=0.08, norm_std=0.2)
        w = engine_weights(eng)
        assert "model.layers.0.norm_a.bias" in w and "model.final.weight" in w
        r = (lambda t: t.to(torch.bfloat16).float()) if dtype == "bfloat16" else (lambda t: t)
        c = P._cfg(cfg)

        def centred(x, name):
            mu = x.mean(-1, keepdim=True)
            var = ((x - mu) ** 2).mean(-1, keepdim=True)
            return (x - mu) / torch.sqrt(var + 1e-3) * w[name + ".weight"] + w[name + ".bias"]

        def reference(ids):
            x = P.embedding(ids, w["model.embed_tokens.weight"])
            pos = torch.arange(len(ids))
            for i in range(c["L"]):
                p = f"model.layers.{i}."
                a, _ = P.attention_sublayer(w, p, r(x), pos, c, store=r if dtype == "bfloat16" else None)
                x = r(centred(x + a, p + "norm_a"))
                f = P.swiglu(r(x), w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                             w[p + "mlp.down_proj.weight"], r if dtype == "bfloat16" else None)
                x = r(centred(x + f, p + "norm_b"))
            head = w["model.embed_tokens.weight"] if c["tied"] else w["lm_head.weight"]
            return P.linear(r(centred(x, "model.final")), head)

        reqs = {"a": tiny.tokens(cfg, 45, 1), "b": tiny.tokens(cfg, 30, 2), "c": tiny.tokens(cfg, 22, 3),
                "d": tiny.tokens(cfg, 37, 4)}
        steps, _ = traces.mixed(reqs, seed=5, max_live=3, tail=6, max_portion=11)
        outs = []
        for s in steps:
            outs.append(eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]).cpu().numpy())
            for rid in s["end"]:
                eng.release(rid)
        rows = traces.collect(steps, outs)
        for rid, toks in reqs.items():
            want = reference(toks)
            for p in range(len(toks)):
                err = float((torch.from_numpy(rows[(rid, p)]) - want[p]).abs().max())
                assert err < (2e-4 if dtype == "float32" else 8e-2), (rid, p, err)
        assert not eng.cache.requests
    finally:
        unregister_architecture("ToyPostNormForCausalLM")
        unregister_part("block", "toy_post_norm")
        unregister_part("norm", "toy_centered")


# ----------------------------------------------------------------------------- other cache shapes

class ToyLatentMixer(Part):
    """Caches one compressed vector per token, c_t = W_c x_t of ``width`` elements: a paged
    cache with keys of ``width`` and no values (``value_dim=0``), so a page is a flat run that
    this part lays out as [page_size, width].  out_t = W_o sum_j softmax_j(q_t . c_j) c_j over
    j <= t with q_t = W_q x_t.  It also keeps the number of tokens it has seen of a request
    in an int32 state slot and scales its output by 1 / (tokens seen so far)."""

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden, self.width = self.param("hidden"), self.param("width")

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("c.weight"), (self.width, self.hidden)),
                WeightSpec(self.tensor_name("q.weight"), (self.width, self.hidden)),
                WeightSpec(self.tensor_name("o.weight"), (self.hidden, self.width))]

    def bind(self, weights):
        self.w_c, self.w_q, self.w_o = (weights[self.tensor_name(n + ".weight")].float() for n in "cqo")

    def cache_need(self):
        return CacheNeed("paged", kv_heads=1, head_dim=self.width, value_dim=0, dtype="float32")

    def forward(self, ctx, xn, cache):
        ps = cache.page_size
        assert cache.pages.dim() == 2 and cache.pages.shape[1] == ps * self.width and cache.pages.dtype == torch.float32
        pages = cache.pages.view(-1, ps, self.width)
        x = xn.float()
        c, q = x @ self.w_c.t(), x @ self.w_q.t()
        out = torch.empty(ctx.n, self.hidden, dtype=torch.float32, device=xn.device)
        tables = cache.block_table.tolist()
        for s in range(ctx.n_spans):
            a, p0 = ctx.h_span_start[s], ctx.h_span_pos[s]
            for i in range(ctx.h_span_len[s]):
                p = p0 + i
                pages[tables[s][p // ps], p % ps] = c[a + i]
                keys = torch.stack([pages[tables[s][j // ps], j % ps] for j in range(p + 1)])
                out[a + i] = self.w_o @ (torch.softmax(keys @ q[a + i], 0) @ keys)
        return out


class ToyCountMixer(Part):
    """out_t = x_t / (tokens of the request seen so far, this one included); the count lives
    in an int32 state slot."""

    def cache_need(self):
        return CacheNeed("state", state_shape=(1,), dtype="int32")

    def forward(self, ctx, xn, cache):
        assert cache.state.dtype == torch.int32
        out = torch.empty(ctx.n, xn.shape[1], dtype=torch.float32, device=xn.device)
        slots = cache.slots.tolist()
        for s in range(ctx.n_spans):
            a, b = ctx.h_span_start[s], ctx.h_span_start[s + 1]
            if ctx.h_span_pos[s] == 0:
                cache.state[slots[s]].zero_()
            for t in range(a, b):
                cache.state[slots[s]] += 1
                assert int(cache.state[slots[s]]) == ctx.h_span_pos[s] + (t - a) + 1
                out[t] = xn[t].float() / cache.state[slots[s]].float()
        return out


def build_latent(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    spec.layers[0].mixer = PartSpec("toy_latent", "model.layers.0.mix", hidden=cfg.hidden_size, width=24)
    spec.layers[1].mixer = PartSpec("toy_count", "model.layers.1.mix")
    return spec


def latent_reference(w, cfg, ids, dtype_round):
    """The same model written plainly over a whole sequence on the CPU."""
    eps = cfg["rms_norm_eps"]
    r = (lambda t: t.to(torch.bfloat16).float()) if dtype_round else (lambda t: t)
    T = len(ids)
    x = P.embedding(ids, w["model.embed_tokens.weight"])
    for i in range(cfg["num_hidden_layers"]):
        pre = f"model.layers.{i}"
        xn = r(P.rmsnorm(x, w[pre + ".input_layernorm.weight"], eps))
        if i == 0:
            c, q = xn @ w[pre + ".mix.c.weight"].t(), xn @ w[pre + ".mix.q.weight"].t()
            mix = torch.stack([w[pre + ".mix.o.weight"] @ (torch.softmax(c[:t + 1] @ q[t], 0) @ c[:t + 1])
                               for t in range(T)])
        elif i == 1:
            mix = xn / torch.arange(1, T + 1).float()[:, None]
        else:
            pos = torch.arange(T)
            cc = P._cfg(cfg)
            qq = P.rope(P.linear(xn, w[pre + ".self_attn.q_proj.weight"]), pos.tolist(), cc["H"], cc["hd"], cc["theta"])
            kk = P.rope(P.linear(xn, w[pre + ".self_attn.k_proj.weight"]), pos.tolist(), cc["KV"], cc["hd"], cc["theta"])
            vv = P.linear(xn, w[pre + ".self_attn.v_proj.weight"])
            mix = P.linear(r(P.attention(r(qq), r(kk), r(vv), pos, cc["H"], cc["KV"], cc["hd"])),
                           w[pre + ".self_attn.o_proj.weight"])
        x = x + mix
        xn = r(P.rmsnorm(x, w[pre + ".post_attention_layernorm.weight"], eps))
        h = r(P.silu(P.linear(xn, w[pre + ".mlp.gate_proj.weight"])) * P.linear(xn, w[pre + ".mlp.up_proj.weight"]))
        x = x + P.linear(h, w[pre + ".mlp.down_proj.weight"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return P.linear(r(P.rmsnorm(x, w["model.norm.weight"], eps)), head)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_cache_of_one_vector_per_token_and_an_integer_state(dtype):
    """A mixer whose cache entry is one vector per token (keys of another width than the model's
    heads, no values, float32 whatever the engine computes in) and a mixer with an int32
    state are registered from here, get pools of their own beside attention's, and are
    stepped in portions and mixed batches with pages used again."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_part("mixer", "toy_latent", ToyLatentMixer)
    register_part("mixer", "toy_count", ToyCountMixer)
    register_architecture("ToyLatentForCausalLM", LlamaConfig, build_latent)
    try:
        cfg = dict(tiny.CONFIGS["B"], architectures=["ToyLatentForCausalLM"])
        eng = Engine.from_random(cfg, 7, EngineOptions(dtype=dtype, num_pages=9, max_requests=3,
                                                       poison_freed_pages=True), std=0.08, norm_std=0.2)
        plan = eng.model.cache_plan
        kinds = [(g.need.kind, g.need.head_dim, g.need.value_width, g.need.dtype) for g in plan.groups]
        assert kinds == [("paged", 24, 0, "float32"), ("state", 0, 0, "int32"), ("paged", 32, 32, None)]
        assert tuple(eng.kv[0].shape) == (1, 9, 16 * 24) and eng.kv[0].dtype == torch.float32
        assert tuple(eng.kv[2].shape) == (1, 9, 2, 1, 16 * 32) and eng.state[1].dtype == torch.int32
        assert "values of 0" in eng.capacity_report()
        w = engine_weights_seed(eng, 7)
        reqs = {"a": tiny.tokens(cfg, 45, 1), "b": tiny.tokens(cfg, 30, 2), "c": tiny.tokens(cfg, 22, 3),
                "d": tiny.tokens(cfg, 37, 4)}
        steps, peak = traces.mixed(reqs, seed=5, max_live=3, tail=5, max_portion=11)
        outs = []
        for s in steps:
            out = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
            outs.append(out.cpu().numpy())
            for rid in s["end"]:
                eng.release(rid)
        rows = traces.collect(steps, outs)
        assert eng.cache.pools[0].total_allocs > 9                 # pages were used again
        worst = 0.0
        for rid, toks in reqs.items():
            want = latent_reference(w, cfg, toks, dtype == "bfloat16")
            for p in range(len(toks)):
                worst = max(worst, float((torch.from_numpy(rows[(rid, p)]) - want[p]).abs().max()))
        assert worst < (2e-4 if dtype == "float32" else 8e-2), worst
        eng.cache.check_invariants()
    finally:
        unregister_architecture("ToyLatentForCausalLM")
        unregister_part("mixer", "toy_latent")
        unregister_part("mixer", "toy_count")
