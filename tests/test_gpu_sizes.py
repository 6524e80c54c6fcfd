"""The engine against the plain implementation at the layer sizes that the
measurements run (TinyLlama 1.1B, Llama-3 8B, Llama-2 7B: their widths, head
sizes, groups and feed-forward widths, with few layers), in 32-bit and in
bfloat16: whole prompts (one of 2,048 tokens), bulk + the last 32 tokens one by
one, portions of changing size, mixed batches with pages used again, a decode
step of 64 requests, and decode steps replayed as HIP graphs and compared by
their logits over two widths of the block table.  These sizes reach kernels
that no tiny configuration reaches: the prompt products' 256-row and two-stage
tiles, products of decode batches with K in 8 or 11 slices, attention at head
sizes 64 and 128 over long tables.  The reference checks itself at full size
the same way (engine/e2e/e2e_test.go:107-170)."""

import numpy as np
import pytest
import torch

import plain_llama as P
import tiny
import traces

pytestmark = pytest.mark.gpu


def _cfg(**kw):
    base = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu",
            "tie_word_embeddings": False, "rms_norm_eps": 1e-5}
    base.update(kw)
    return base


# Layer sizes of the three models that the measurements name, with few layers (and the 8B
# model's vocabulary cut to 32,000: the product with the output matrix is the same kernel).
SIZES = {
    "tinyllama": _cfg(num_hidden_layers=2, hidden_size=2048, num_attention_heads=32, num_key_value_heads=4,
                      head_dim=64, intermediate_size=5632, vocab_size=32000, rope_theta=10000.0,
                      max_position_embeddings=2048),
    "llama3-8b": _cfg(num_hidden_layers=1, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                      head_dim=128, intermediate_size=14336, vocab_size=32000, rope_theta=500000.0,
                      max_position_embeddings=8192),
    "llama2-7b": _cfg(num_hidden_layers=1, hidden_size=4096, num_attention_heads=32, num_key_value_heads=32,
                      head_dim=128, intermediate_size=11008, vocab_size=32000, rope_theta=10000.0,
                      max_position_embeddings=4096),
}
LENGTHS = {"tinyllama": [300, 150, 77, 33, 120, 64], "llama3-8b": [200, 130, 70, 33, 90, 45],
           "llama2-7b": [200, 130, 70, 33, 90, 45]}
SEED = 11
DTYPES = ["float32", "bfloat16"]

_weights, _expected = {}, {}


def weights(name):
    """name -> float32 CPU tensor, from the package's seeded generator (drawn on the GPU,
    whose values equal the CPU's: test_weights_drawn_on_the_gpu_equal_those_drawn_on_the_cpu);
    the engine is given exactly these (rounded to bfloat16 for a bfloat16 engine, as the
    loader would)."""
    if name not in _weights:
        from kllm_amd.config import config_from_dict, resolve_architecture
        from kllm_amd.engine.model import collect_weight_specs
        from kllm_amd.weights import random_weights
        raw = SIZES[name]
        spec = resolve_architecture(raw).build(config_from_dict(raw, where=name))
        _weights[name] = {k: v.cpu() for k, v in
                          random_weights(collect_weight_specs(spec), SEED, torch.float32, "cuda").items()}
    return _weights[name]


def plain_weights(name, dtype):
    w = weights(name)
    if dtype == "bfloat16":
        return {k: (v.to(torch.bfloat16).float() if v.dim() > 1 else v) for k, v in w.items()}
    return w


def engine(name, dtype, **opts):
    from kllm_amd.config import config_from_dict
    from kllm_amd.engine import Engine, EngineOptions
    from kllm_amd.weights.loader import target_dtype
    raw = SIZES[name]
    options = EngineOptions(dtype=dtype, max_model_len=1 << 30, poison_freed_pages=True, graph_after_steps=1, **opts)
    compute = options.torch_dtype()
    w = weights(name)

    def weights_from(specs, spec):
        return {s.name: w[s.name].to("cuda").to(target_dtype(s.role, compute)).contiguous() for s in specs}
    return Engine(config_from_dict(raw, where=name), raw, weights_from, options)


def requests(name, lengths=None, seed=1):
    cfg = SIZES[name]
    return {f"r{i}": tiny.tokens(cfg, n, seed * 100 + i) for i, n in enumerate(lengths or LENGTHS[name])}


def expected(name, dtype, reqs, stored=False):
    """The plain implementation's logits; with ``stored`` it rounds to bfloat16 wherever a
    bfloat16 engine keeps an activation (the weights are rounded in both cases)."""
    out = {}
    for rid, toks in reqs.items():
        key = (name, dtype, stored, tuple(toks))
        if key not in _expected:
            _expected[key] = P.forward(plain_weights(name, dtype), SIZES[name], toks,
                                       store=P.round_bfloat16 if stored else None).numpy()
        out[rid] = _expected[key]
    return out


def run(eng, steps):
    from kllm_amd.engine import StepEntry
    outs = []
    for s in steps:
        out = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        outs.append(None if out is None else out.cpu().numpy())
        for rid in s["end"]:
            eng.release(rid)
    assert not eng.cache.requests
    eng.cache.check_invariants()
    return traces.collect(steps, outs)


def compare(rows, want, dtype, reqs, tol=None):
    tol = tol if tol is not None else tiny.TOL_SIZES[dtype]
    worst = 0.0
    for rid, toks in reqs.items():
        for p in range(len(toks)):
            got = rows[(rid, p)]
            assert np.isfinite(got).all(), (rid, p)
            worst = max(worst, float(np.abs(got - want[rid][p]).max()))
            assert worst < tol, f"{rid} position {p}: off by {worst}"
    return worst


def compare_both(name, dtype, rows, reqs):
    """Against the plain implementation; in bfloat16 also against the plain implementation
    rounding where the engine stores (a somewhat tighter yardstick: rounding noise
    that both share cancels, what a different order of sums flips does not)."""
    worst = compare(rows, expected(name, dtype, reqs), dtype, reqs)
    text = f"off by at most {worst:.3e}"
    if dtype == "bfloat16":
        near = compare(rows, expected(name, dtype, reqs, stored=True), dtype, reqs, tiny.TOL_SIZES_STORED)
        text += f" ({near:.3e} from the plain implementation with bfloat16 storage)"
    return text


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(SIZES))
def test_four_families_at_real_layer_sizes(name, dtype):
    reqs = requests(name)
    mixed, peak = traces.mixed(reqs, seed=3, max_live=3)
    families = {"whole": traces.whole(reqs), "bulk": traces.bulk_then_tail(reqs, 32),
                "portions": traces.portions(reqs, seed=2), "mixed": mixed}
    assert peak < sum(-(-len(t) // 64) * 64 for t in reqs.values())
    for fam, steps in families.items():
        eng = engine(name, dtype, max_tokens=traces.peak_tokens(steps))
        rows = run(eng, steps)
        print(f"{name} {dtype} {fam}: logits", compare_both(name, dtype, rows, reqs))
        if fam == "mixed":
            pool = eng.cache.pools[0]
            assert pool.total_allocs > pool.num_pages
        del eng


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_whole_prompt_of_2048_tokens(dtype):
    """One step of 2,048 tokens with the logits of every position (the products' largest
    tiles, sixteen query blocks a head), then the same prompt with its last 32 tokens
    decoded one by one over 126 to 128 pages."""
    name = "tinyllama"
    reqs = requests(name, [2048], seed=4)
    for steps in (traces.whole(reqs), traces.bulk_then_tail(reqs, 32)):
        eng = engine(name, dtype, max_tokens=2048)
        print(f"{name} {dtype} 2048 tokens in {len(steps)} steps: logits", compare_both(name, dtype, run(eng, steps), reqs))
        del eng


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,B", [("tinyllama", 64), ("tinyllama", 33), ("tinyllama", 24), ("tinyllama", 16),
                                    ("tinyllama", 12), ("tinyllama", 8), ("tinyllama", 4), ("tinyllama", 2),
                                    ("llama3-8b", 64), ("llama3-8b", 40), ("llama3-8b", 17), ("llama3-8b", 16),
                                    ("llama3-8b", 12), ("llama3-8b", 8), ("llama3-8b", 3)])
def test_decode_steps_of_many_requests_eager_and_as_graphs(name, B, dtype):
    """64 requests decode together (and fewer, which take other kernels for the products and for
    attention and other hand-overs between them: up to 2, 4, 16, 32 and 64 rows, with the norm
    folded into its neighbours or in a launch of its own, the down projection's rows in one
    pass through LDS or in two to four, the gate in the tiled product's
    epilogue or apart, a few more attention groups than the chip holds whole-context workgroups):
    first through the plain step function, then queued ahead
    as HIP graphs.  Both give logits; the graphs' must equal the eager ones (the same kernels
    on the same numbers; only the width of the block table differs), for every request at
    every step, over two widths of the table, and a sample of requests is compared with the
    plain implementation."""
    from kllm_amd.engine import StepEntry
    cfg = SIZES[name]
    new = 24
    lens = [100 + (7 * i) % 26 for i in range(B)]          # 100..125 tokens: tables of 7 and 8 pages,
    reqs = requests(name, [n + new for n in lens], seed=6)  # then 9 and 10 while decoding
    eng = engine(name, dtype, max_tokens=B * 192, max_requests=B)
    rids = list(reqs)
    eager, graphs = {}, {}
    for mode, store in (("eager", eager), ("graph", graphs)):
        for a in range(0, B, 16):                           # prompts, sixteen requests a step
            eng.step([StepEntry(r, reqs[r][:lens[i]], []) for i, r in enumerate(rids) if a <= i < a + 16])
        captures = eng._graphs.captures
        for k in range(new):
            entries = [StepEntry(r, [reqs[r][lens[i] + k]], [0]) for i, r in enumerate(rids)]
            if mode == "eager":
                out = eng.step(entries)
            else:
                h = eng.step_sample_ahead(entries, [0.0] * B, [0.0] * B)
                ids = h.tokens()
                out = h.logits
                assert ids == out.argmax(-1).tolist() or \
                    all(float(out[i, ids[i]]) == float(out[i].max()) for i in range(B))
            store[k] = out.cpu().numpy().copy()
        if mode == "graph":
            assert eng._graphs.captures - captures >= 2 or len(eng._graphs.recordings) >= 2
            assert sum(r.replays for r in eng._graphs.recordings.values()) >= new - 4
        for r in rids:
            eng.release(r)
    for k in range(new):
        assert np.array_equal(eager[k], graphs[k]), f"step {k}: a replayed graph and the eager step differ"
    sample = sorted({0, B // 5, min(B // 2 + 1, B - 1), B - 1})
    for stored in ([False, True] if dtype == "bfloat16" else [False]):
        want = expected(name, dtype, {rids[i]: reqs[rids[i]] for i in sample}, stored)
        worst = 0.0
        for i in sample:
            for k in range(new):
                worst = max(worst, float(np.abs(eager[k][i] - want[rids[i]][lens[i] + k]).max()))
        print(f"{name} {dtype} decode of {B}: logits off by at most {worst:.3e}" + (" (bfloat16 storage)" if stored else ""))
        assert worst < (tiny.TOL_SIZES_STORED if stored else tiny.TOL_SIZES[dtype]), worst


def test_prompt_portions_of_512_tokens_beside_decode_tokens():
    """What a scheduler with a budget of 512 tokens sends at these sizes: a 512-token portion
    of one prompt beside single decode tokens of other requests, in bfloat16."""
    name, dtype = "tinyllama", "bfloat16"
    reqs = requests(name, [1100, 60, 45], seed=8)
    a, b, c = (reqs[r] for r in ("r0", "r1", "r2"))
    steps = [{"entries": [{"id": "r1", "tokens": b[:40], "want": list(range(40))},
                          {"id": "r2", "tokens": c[:30], "want": list(range(30))}], "end": []}]
    fed = {"r0": 0, "r1": 40, "r2": 30}
    while fed["r0"] < len(a):
        n = min(512, len(a) - fed["r0"])
        entries = [{"id": "r0", "tokens": a[fed["r0"]:fed["r0"] + n], "want": list(range(n))}]
        fed["r0"] += n
        for rid, toks in (("r1", b), ("r2", c)):
            if fed[rid] < len(toks):
                entries.insert(0, {"id": rid, "tokens": toks[fed[rid]:fed[rid] + 1], "want": [0]})
                fed[rid] += 1
        steps.append({"entries": entries, "end": []})
    while fed["r1"] < len(b) or fed["r2"] < len(c):
        entries = []
        for rid, toks in (("r1", b), ("r2", c)):
            if fed[rid] < len(toks):
                entries.append({"id": rid, "tokens": toks[fed[rid]:fed[rid] + 1], "want": [0]})
                fed[rid] += 1
        steps.append({"entries": entries, "end": []})
    steps[-1]["end"] = ["r0", "r1", "r2"]
    for i, s in enumerate(steps):
        s["step"] = i
    eng = engine(name, dtype, max_tokens=traces.peak_tokens(steps))
    print(f"{name} {dtype} 512-token portions beside decode tokens: logits", compare_both(name, dtype, run(eng, steps), reqs))


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_scheduler_with_portions_of_512_tokens_beside_decode_tokens(dtype):
    """The scheduler itself at these sizes (the reference's end-to-end check of its scheduler:
    engine/scheduler.go:160-189, engine/e2e/e2e_test.go:256-312): five requests, two of them
    with prompts of more than 512 tokens, submitted together under a budget of 512 prompt
    tokens a step, so that portions of 512 run beside the decode tokens of the requests that
    are already generating and steps end on whole tiles of rows.  Every generated token must
    be the plain implementation's greedy choice given the tokens before it, or lie within
    the tolerance of it (bfloat16 may part ways at a near-tie; what follows is then judged
    from the engine's own tokens)."""
    from kllm_amd.engine.scheduler import Scheduler
    name, new = "tinyllama", 12
    cfg = SIZES[name]
    prompts = [tiny.tokens(cfg, n, 400 + i) for i, n in enumerate([1100, 60, 700, 45, 300])]
    eng = engine(name, dtype, max_tokens=sum(len(p) + new + 16 for p in prompts), max_requests=8)
    sched = Scheduler(eng, max_batch=5, max_step_tokens=512 + 5, chunk_size=512)
    ids = [sched.submit(p, new) for p in prompts]
    results = sched.run_until_done()
    assert sched.stats["steps"] >= 6 and sched.stats["preemptions"] == 0
    assert not eng.cache.requests
    eng.cache.check_invariants()
    w = plain_weights(name, dtype)
    tol = tiny.TOL_SIZES[dtype]
    ties = 0
    for i, p in zip(ids, prompts):
        assert results[i].error is None and len(results[i].tokens) == new
        logits = P.forward(w, cfg, list(p) + results[i].tokens[:-1])[len(p) - 1:]
        for k, tok in enumerate(results[i].tokens):
            best = int(logits[k].argmax())
            if tok != best:
                ties += 1
                assert float(logits[k][best] - logits[k][tok]) < 2 * tol, (i, k, tok, best)
    assert ties <= (0 if dtype == "float32" else 6), ties
