"""That a step walks through only the first two of the layers that are alike and writes the
others' commands from the first's (kllm_amd/engine/repeat.py): the logits are, bit for bit,
those of an engine that walks through every layer, and both fit the plain implementation;
for the dense model with more layers than the other tests' configurations have, for layers
of two kinds in turn (a window, none: two cache groups), for a running order that names a
layer five times and lets the last layer read its cache, and for parts that do not lend
themselves to it (a mixer of torch operations; a feed-forward whose scratch buffers alternate
from layer to layer), where the engine must fall back to walking."""

import pytest
import torch

import plain_llama as P
import tiny
import traces
from kllm_amd.config import LlamaConfig, register_architecture, unregister_architecture
from kllm_amd.parts import ModelSpec, Part, PartSpec, Run, register_part, unregister_part

pytestmark = pytest.mark.gpu

DEEP = {
    "L": dict(tiny.CONFIGS["B"], num_hidden_layers=7),
    "M": dict(tiny.CONFIGS["A"], num_hidden_layers=10, intermediate_size=208, vocab_size=300),
}


def engines(cfg, dtype, model_dir=None, **opts):
    """The same model twice: layers repeated, and every layer walked through."""
    from kllm_amd.engine import Engine, EngineOptions
    out = []
    for extra in ({}, {"no_repeated_layers": True}):
        o = EngineOptions(dtype=dtype, extra=extra, **opts)
        out.append(Engine.from_dir(model_dir, o) if model_dir else Engine.from_random(cfg, 3, o, std=0.05, norm_std=0.1))
    assert out[0].model._repeater is not None and out[1].model._repeater is None
    return out


def replay_both(engs, steps):
    """The trace through both engines; every step's logits must be the same bits."""
    from kllm_amd.engine import StepEntry
    outs = []
    for s in steps:
        got = [e.step([StepEntry(x["id"], x["tokens"], x["want"]) for x in s["entries"]]) for e in engs]
        assert torch.equal(got[0], got[1]), s["step"]
        outs.append(got[0].cpu().numpy())
        for rid in s["end"]:
            for e in engs:
                e.release(rid)
    return outs


def check_rows(steps, outs, want, tol):
    rows = traces.collect(steps, outs)
    for (rid, p), row in rows.items():
        err = float((torch.from_numpy(row) - want[rid][p]).abs().max())
        assert err < tol, (rid, p, err)
    return len(rows)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["L", "M"])
def test_layers_that_are_alike_are_walked_through_twice(name, dtype, tmp_path):
    cfg = DEEP[name]
    d = tiny.write_model(str(tmp_path), cfg, 11)
    engs = engines(cfg, dtype, d, max_tokens=512)
    ws = tiny.read_weights(d, as_stored_in=dtype)
    reqs = {"a": tiny.tokens(cfg, 90, 1), "b": tiny.tokens(cfg, 61, 2), "c": tiny.tokens(cfg, 47, 3),
            "d": tiny.tokens(cfg, 70, 4), "e": tiny.tokens(cfg, 33, 5)}
    want = {rid: P.forward(ws, cfg, toks) for rid, toks in reqs.items()}
    layers, walked = cfg["num_hidden_layers"], 0
    for family in (traces.whole(reqs), traces.bulk_then_tail(reqs, tail=20), traces.portions(reqs, seed=1),
                   traces.mixed(reqs, seed=2, max_live=4, tail=10, max_portion=17)[0]):
        outs = replay_both(engs, family)
        assert check_rows(family, outs, want, tiny.TOL[dtype]) == sum(len(t) for t in reqs.values())
        walked += len(family)
    eng = engs[0]
    # (a step that repeats an earlier one's commands walks through nothing, one whose scratch
    # buffers grow walks through everything)
    through_parts = walked - eng.steps_repeated
    assert eng.steps_repeated > 20 and through_parts > 25, (eng.steps_repeated, through_parts)
    assert eng.model.runs_repeated >= (layers - 4) * (through_parts - 12), (eng.model.runs_repeated, through_parts)
    assert engs[1].model.runs_repeated == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_repeated_layers_in_steps_that_run_again_from_their_commands(dtype):
    """Decode steps of one shape at advancing positions run from the first one's commands with
    the new step's values in them; the values sit in the repeated layers' commands too."""
    from kllm_amd.engine import StepEntry
    cfg = DEEP["L"]
    engs = engines(cfg, dtype, max_tokens=1024, max_model_len=256)
    prompts = {rid: tiny.tokens(cfg, n, seed) for seed, (rid, n) in enumerate([("a", 70), ("b", 5), ("c", 130)])}
    for rid, toks in prompts.items():
        for e in engs:
            e.step([StepEntry(rid, toks, [])])
    before = engs[0].steps_repeated
    for step in range(40):        # (the attention's kernel choice depends on the longest context: a value of the step)
        entries = [StepEntry(rid, [(7 * step + k) % cfg["vocab_size"]], [0]) for k, rid in enumerate(prompts)]
        got = [e.step(entries) for e in engs]
        assert torch.equal(got[0], got[1]), step
    assert engs[0].steps_repeated - before >= 30 and engs[0].model.runs_repeated >= 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_repeated_layers_in_a_recorded_graph(dtype):
    """A batch of decode tokens recorded as a HIP graph: the recording walks through two
    layers of a kind as any step does; its replays sample what the walked engine samples."""
    from kllm_amd.engine import StepEntry, TokenRef
    cfg = DEEP["M"]
    engs = engines(cfg, dtype, max_tokens=1024, max_model_len=256, graph_after_steps=1)
    prompts = {rid: tiny.tokens(cfg, n, seed) for seed, (rid, n) in enumerate([("a", 40), ("b", 9), ("c", 75)])}
    for rid, toks in prompts.items():
        for e in engs:
            e.step([StepEntry(rid, toks, [])])
    before = engs[0].model.runs_repeated
    last, ids = [None, None], [[3, 4, 5], [3, 4, 5]]
    for step in range(24):
        for k, e in enumerate(engs):
            entries = [StepEntry(rid, [ids[k][j] if last[k] is None else TokenRef(last[k], j)], [0])
                       for j, rid in enumerate(prompts)]
            last[k] = e.step_sample_ahead(entries, [0.0, 0.7, 1.3], [0.0, 0.31 + 0.01 * step, 0.77])
        got = [h.tokens() for h in last]
        assert got[0] == got[1], step
        assert torch.equal(last[0].logits, last[1].logits), step
    assert engs[0]._graphs.captures >= 1 and sum(r.replays for r in engs[0]._graphs.recordings.values()) >= 20
    assert engs[0].model.runs_repeated > before            # (both runs of a recording: 2 x 6 of 10 layers)


def build_windows_in_turn(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    for i in range(0, cfg.num_hidden_layers, 2):
        spec.layers[i].mixer.params["window"] = 24
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_two_kinds_in_turn(dtype, tmp_path):
    register_architecture("ToyTurnsForCausalLM", LlamaConfig, build_windows_in_turn)
    try:
        cfg = dict(DEEP["M"], architectures=["ToyTurnsForCausalLM"])
        d = tiny.write_model(str(tmp_path), cfg, 12)
        engs = engines(cfg, dtype, d, max_tokens=512, max_model_len=1 << 16)
        assert [(g.need.window, g.entries) for g in engs[0].model.cache_plan.groups] == [(24, 5), (0, 5)]
        ws = tiny.read_weights(d, as_stored_in=dtype)
        reqs = {"a": tiny.tokens(cfg, 100, 1), "b": tiny.tokens(cfg, 75, 2), "c": tiny.tokens(cfg, 58, 3)}
        want = {rid: P.forward(ws, cfg, toks, windows={i: 24 for i in range(0, 10, 2)}) for rid, toks in reqs.items()}
        steps = traces.mixed(reqs, seed=5, max_live=3, tail=30, max_portion=21)[0]
        outs = replay_both(engs, steps)
        assert check_rows(steps, outs, want, tiny.TOL[dtype]) == 233
        # per step that is walked through: of each kind the first, the second, and of the
        # windowed kind the model's first layer, of the other its last
        assert engs[0].model.runs_repeated >= 4 * (len(steps) - engs[0].steps_repeated - 10)
        assert engs[0].model.runs_repeated > 40
    finally:
        unregister_architecture("ToyTurnsForCausalLM")


def build_one_layer_five_times(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    spec.layers[2].mixer.params["own_kv"] = False
    spec.schedule = [Run(0)] + [Run(1)] * 5 + [Run(2, cache_of=3)]
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_that_follows_itself(dtype, tmp_path):
    """The runs of one layer are alike but for their caches; the last of them is followed by
    another layer and is walked through."""
    register_architecture("ToyFiveForCausalLM", LlamaConfig, build_one_layer_five_times)
    try:
        cfg = dict(tiny.CONFIGS["B"], architectures=["ToyFiveForCausalLM"])
        w = P.random_weights(cfg, 4, std=0.05, norm_std=0.1)
        del w["model.layers.2.self_attn.k_proj.weight"], w["model.layers.2.self_attn.v_proj.weight"]
        d = tiny.write_model(str(tmp_path), cfg, 0, weights=w)
        engs = engines(cfg, dtype, d, max_tokens=256)
        assert engs[0].model.cache_plan.groups[0].entries == 6
        ws = tiny.read_weights(d, as_stored_in=dtype)
        reqs = {"a": tiny.tokens(cfg, 64, 1), "b": tiny.tokens(cfg, 40, 2)}
        want = {rid: P.forward(ws, cfg, toks, schedule=[0, 1, 1, 1, 1, 1, 2], kv_from={6: 3}) for rid, toks in reqs.items()}
        steps = traces.mixed(reqs, seed=1, max_live=2, tail=12, max_portion=15)[0]
        outs = replay_both(engs, steps)
        assert check_rows(steps, outs, want, tiny.TOL[dtype]) == 104
        through_parts = len(steps) - engs[0].steps_repeated
        assert engs[0].model.runs_repeated >= 2 * max(1, through_parts - 6), (engs[0].model.runs_repeated, through_parts)
    finally:
        unregister_architecture("ToyFiveForCausalLM")


# ----------------------------------------------------------------------------- parts that do not lend themselves to it

class _TurnedContext:
    """A step's context whose scratch buffers are one of two sets."""

    def __init__(self, ctx, turn):
        self._ctx, self._turn = ctx, turn

    def __getattr__(self, name):
        return getattr(self._ctx, name)

    def buf(self, tag, shape, dtype):
        return self._ctx.buf(f"turn{self._turn}.{tag}", shape, dtype)


class ToyTurningFeedForward(Part):
    """The dense feed-forward, but with two sets of scratch buffers that it uses in turn: the
    commands of two layers then differ in words that no tensor of the layers explains."""
    graph_safe = True
    records_launches = True
    calls = 0

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        from kllm_amd.parts.base import make_part
        self.inner = make_part("feed_forward", PartSpec("gated_mlp", spec.prefix, **spec.params), runtime)

    def children(self):
        return [self.inner]

    def weight_specs(self):
        return self.inner.weight_specs()

    def bind(self, weights):
        self.inner.bind(weights)

    def read_bytes(self, tokens):
        return self.inner.read_bytes(tokens)

    def forward(self, ctx, xn):
        ToyTurningFeedForward.calls += 1
        return self.inner.forward(_TurnedContext(ctx, ToyTurningFeedForward.calls % 2), xn)


def build_turning(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    for layer in spec.layers:
        layer.feed_forward = PartSpec("toy_turning", layer.feed_forward.prefix, **layer.feed_forward.params)
    return spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_scratch_buffers_that_alternate_between_layers_end_the_repeating(dtype, tmp_path):
    register_part("feed_forward", "toy_turning", ToyTurningFeedForward)
    register_architecture("ToyTurningForCausalLM", LlamaConfig, build_turning)
    try:
        cfg = dict(DEEP["L"], architectures=["ToyTurningForCausalLM"])
        d = tiny.write_model(str(tmp_path), cfg, 13)
        engs = engines(cfg, dtype, d, max_tokens=256)
        ws = tiny.read_weights(d, as_stored_in=dtype)
        reqs = {"a": tiny.tokens(cfg, 50, 1), "b": tiny.tokens(cfg, 37, 2)}
        want = {rid: P.forward(ws, cfg, toks) for rid, toks in reqs.items()}
        steps = traces.mixed(reqs, seed=4, max_live=2, tail=8, max_portion=13)[0]
        outs = replay_both(engs, steps)
        assert check_rows(steps, outs, want, tiny.TOL[dtype]) == 87
        assert engs[0].model.runs_repeated == 0
        why = engs[0].model._repeater.last.why
        assert why and all("buffers" in w or "no tensor" in w for w in why), why
    finally:
        unregister_architecture("ToyTurningForCausalLM")
        unregister_part("feed_forward", "toy_turning")


class ToyTorchMixer(Part):
    """A mixer without memory made of torch operations (the engine calls it with what was
    recorded already run)."""
    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.w = None

    def weight_specs(self):
        from kllm_amd.parts import WeightSpec
        d = int(self.param("hidden"))
        return [WeightSpec(self.tensor_name("mix.weight"), (d, d))]

    def bind(self, weights):
        self.w = weights[self.tensor_name("mix.weight")]

    def forward(self, ctx, xn, cache):
        return torch.tanh(xn.float() @ self.w.float().t()).to(xn.dtype)


def build_torch_mixers(cfg: LlamaConfig) -> ModelSpec:
    from kllm_amd.models.llama import build_llama
    spec = build_llama(cfg)
    for i, layer in enumerate(spec.layers):
        layer.mixer = PartSpec("toy_torch", f"model.layers.{i}", hidden=cfg.hidden_size)
    return spec


def test_parts_of_torch_operations_are_walked_through():
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    register_part("mixer", "toy_torch", ToyTorchMixer)
    register_architecture("ToyTorchForCausalLM", LlamaConfig, build_torch_mixers)
    try:
        cfg = dict(DEEP["L"], architectures=["ToyTorchForCausalLM"])
        eng = Engine.from_random(cfg, 3, EngineOptions(dtype="float32", max_tokens=128), std=0.2, norm_std=0.1)
        assert eng.model._repeater is None and not eng.model.repeatable      # nothing to repeat where parts launch for themselves
        ids = tiny.tokens(cfg, 12, 1)
        whole = eng.step([StepEntry("a", ids, list(range(12)))]).cpu()
        cut = torch.cat([eng.step([StepEntry("b", ids[a:b], list(range(b - a)))]).cpu() for a, b in [(0, 5), (5, 7), (7, 12)]])
        assert float((whole - cut).abs().max()) < 1e-5 and float(whole.std()) > 1e-3
    finally:
        unregister_architecture("ToyTorchForCausalLM")
        unregister_part("mixer", "toy_torch")
