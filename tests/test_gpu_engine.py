"""The engine against the plain implementation, in 32-bit and in bfloat16:
each request alone and whole; most of it in one step and the last 32 tokens
one by one; in portions of changing size, down to two tokens; and mixed, up to
four live requests with so few pages that they are used again.  Then long
decoding, the first tokens of a sequence, and generation through the entry
points."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as P
import tiny
import traces

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]


def make_requests(cfg, lengths, seed):
    return {f"r{i}": tiny.tokens(cfg, n, seed * 100 + i) for i, n in enumerate(lengths)}


def expected(model_dir, cfg, requests, dtype):
    w = tiny.read_weights(model_dir, as_stored_in=dtype)
    return {rid: P.forward(w, cfg, toks).numpy() for rid, toks in requests.items()}


def replay(model_dir, dtype, steps, max_tokens, **opts):
    from kllm_amd.engine import EngineOptions
    from kllm_amd.replay import Replayer
    options = EngineOptions(dtype=dtype, max_tokens=max_tokens, max_model_len=1 << 30,
                            poison_freed_pages=True, **opts)
    rep = Replayer(model_dir, dtype, max_tokens or 0, options=options)
    outs = [rep.step(s["entries"], s["end"]) for s in steps]
    assert not rep.engine.cache.requests, "every request of the trace was ended"
    rep.engine.cache.check_invariants()
    assert all(p.free_pages == p.num_pages for p in rep.engine.cache.pools)
    return traces.collect(steps, outs), rep


def compare(rows, want, dtype, requests):
    worst = 0.0
    for rid, toks in requests.items():
        for p in range(len(toks)):
            got = rows[(rid, p)]
            assert np.isfinite(got).all(), (rid, p)
            worst = max(worst, float(np.abs(got - want[rid][p]).max()))
            assert worst < tiny.TOL[dtype], f"{rid} position {p}: off by {worst}"
    assert len(rows) == sum(len(t) for t in requests.values())
    return worst


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,lengths", [("A", [5, 17, 33, 100]), ("B", [1, 9, 40, 70, 150]),
                                          ("C", [3, 64, 65]), ("D", [2, 90])])
def test_alone_and_whole(model_dirs, name, lengths, dtype):
    cfg, d = tiny.CONFIGS[name], model_dirs(name)
    reqs = make_requests(cfg, lengths, 1)
    steps = traces.whole(reqs)
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, expected(d, cfg, reqs, dtype), dtype, reqs)


def test_a_long_prompt_with_more_query_blocks_than_cus(model_dirs):
    """2,300 tokens of a model with 16 heads in one step (the prompt kernel that passes
    keys through LDS), then its last 32 tokens one by one over the long context."""
    cfg, d = tiny.CONFIGS["E"], model_dirs("E")
    reqs = make_requests(cfg, [2300], 5)
    want = expected(d, cfg, reqs, "bfloat16")
    for steps in (traces.whole(reqs), traces.bulk_then_tail(reqs, 32)):
        rows, _ = replay(d, "bfloat16", steps, traces.peak_tokens(steps))
        compare(rows, want, "bfloat16", reqs)


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_far_into_a_long_context_with_few_large_heads(model_dirs, dtype):
    """1,900 tokens of a model with three heads of 128 in portions of 300 and less: from 1,280
    keys on, the keys of a portion's blocks go in slices over several workgroups whose results
    a second kernel merges (bfloat16); every position's logits against the plain model's, and
    the same prompt beside a second request in portions that end inside blocks."""
    from kllm_amd import kernels as K
    cfg, d = tiny.CONFIGS["F"], model_dirs("F")
    assert K.attn_prefill_slices(3, cfg["num_attention_heads"], cfg["head_dim"]) == 4
    reqs = make_requests(cfg, [1900, 1500], 6)
    want = expected(d, cfg, reqs, dtype)
    steps = traces.portions(reqs, seed=2, sizes=(300, 257, 31, 300, 128, 2, 300, 129))
    rows, rep = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, want, dtype, reqs)
    assert (("attn.block_part", torch.float32) in rep.engine.runtime.workspace._bufs) == (dtype == "bfloat16")
    steps, peak = traces.mixed(reqs, seed=3, max_live=2, tail=8, max_portion=290)
    rows, _ = replay(d, dtype, steps, peak)
    compare(rows, want, dtype, reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,lengths", [("A", [33, 100]), ("B", [40, 129]), ("C", [50]), ("D", [45])])
def test_bulk_then_last_32_one_by_one(model_dirs, name, lengths, dtype):
    cfg, d = tiny.CONFIGS[name], model_dirs(name)
    reqs = make_requests(cfg, lengths, 2)
    steps = traces.bulk_then_tail(reqs, 32)
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, expected(d, cfg, reqs, dtype), dtype, reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,lengths", [("A", [100, 37]), ("B", [150, 70]), ("C", [81]), ("D", [77])])
def test_portions_of_changing_size(model_dirs, name, lengths, dtype):
    cfg, d = tiny.CONFIGS[name], model_dirs(name)
    reqs = make_requests(cfg, lengths, 3)
    steps = traces.portions(reqs, seed=4)
    assert min(len(s["entries"][0]["tokens"]) for s in steps if not s["end"]) == 2
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps))
    compare(rows, expected(d, cfg, reqs, dtype), dtype, reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_mixed_with_pages_used_again(model_dirs, name, dtype):
    cfg, d = tiny.CONFIGS[name], model_dirs(name)
    reqs = make_requests(cfg, [70, 33, 120, 18, 64, 97, 41, 129, 5, 80], 4)
    steps, peak = traces.mixed(reqs, seed=7)
    assert peak == traces.peak_tokens(steps)
    assert peak < sum(len(t) for t in reqs.values())          # the pool is smaller than the trace
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"]) and \
        any(len(e["tokens"]) > 1 and len(s["entries"]) > 1 for s in steps for e in s["entries"])
    rows, rep = replay(d, dtype, steps, peak)
    pool = rep.engine.cache.pools[0]
    assert pool.total_allocs > pool.num_pages                 # pages were handed out again
    compare(rows, expected(d, cfg, reqs, dtype), dtype, reqs)


@pytest.mark.parametrize("dtype", DTYPES)
def test_all_families_agree_with_each_other(model_dirs, dtype):
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    reqs = make_requests(cfg, [90, 47], 5)
    families = [traces.whole(reqs), traces.bulk_then_tail(reqs), traces.portions(reqs, 1),
                traces.mixed(reqs, seed=2)[0]]
    results = [replay(d, dtype, s, traces.peak_tokens(s))[0] for s in families]
    tol = 2e-5 if dtype == "float32" else tiny.TOL[dtype]
    for other in results[1:]:
        for key, row in results[0].items():
            assert float(np.abs(other[key] - row).max()) < tol, key


@pytest.mark.parametrize("options", [
    {"extra": {"no_fused_gemv": True}},                              # few tokens through the split-K kernels
    {"extra": {"no_fused_gemv": True, "no_fused_linear": True}},     # and without the decode-batch kernel
    {"extra": {"no_fused_norm": True}},                              # every norm as a launch of its own
    {"attention": "generic"},                                        # the attention kernel that takes every size
    {"gemm": "library"},                                             # prompt-sized products from the vendor library
    {"graphs": False},
])
def test_every_choice_of_kernels_gives_the_same_logits(model_dirs, options):
    """The engine picks kernels by the number of tokens; each alternative path, forced here,
    must agree with the plain implementation just as well (bfloat16, where the choices are)."""
    cfg, d = tiny.CONFIGS["B"], model_dirs("B")
    reqs = make_requests(cfg, [150, 33, 70], 9)
    want = expected(d, cfg, reqs, "bfloat16")
    for steps in (traces.portions(reqs, 3), traces.mixed(reqs, seed=4)[0]):
        rows, _ = replay(d, "bfloat16", steps, traces.peak_tokens(steps), **options)
        compare(rows, want, "bfloat16", reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [4, 10, 12, 24, 48, 256])
def test_page_sizes_that_are_no_multiple_of_16_and_large_ones(model_dirs, page_size, dtype):
    """Pages of every size the engine accepts: those that only the kernel for every size
    takes (10; in bfloat16 also 4, 12, 24), those the float32 matrix-core kernel takes (a
    multiple of 4), and pages of 256 tokens.  Mixed steps, so that pages are used again."""
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    reqs = make_requests(cfg, [70, 33, 120, 18, 64, 97], 6)
    want = expected(d, cfg, reqs, dtype)
    steps, peak = traces.mixed(reqs, seed=9)
    held, most = {}, 0                  # exactly the pages the live requests hold at the worst step
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // page_size) for n in held.values()))
        for rid in st["end"]:
            del held[rid]
    rows, rep = replay(d, dtype, steps, None, page_size=page_size, num_pages=most)
    pool = rep.engine.cache.pools[0]
    assert pool.high_water == most and (pool.total_allocs > most or page_size == 256)   # pages were used again
    compare(rows, want, dtype, reqs)
    steps = traces.bulk_then_tail(reqs, 32)
    rows, _ = replay(d, dtype, steps, traces.peak_tokens(steps) + page_size, page_size=page_size)
    compare(rows, want, dtype, reqs)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_queued_ahead_takes_its_ids_from_the_device(model_dirs, dtype):
    """Decode steps queued one ahead, fed by TokenRef, give the ids that steps fed from the
    host give; a reference to an older step is refused and changes nothing."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry, TokenRef, StepError
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    prompts = [tiny.tokens(cfg, n, 70 + i) for i, n in enumerate([9, 33, 4])]
    runs = []
    for ahead in (False, True):
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=512))
        firsts = eng.step_sample([StepEntry(i, p, [len(p) - 1]) for i, p in enumerate(prompts)],
                                 [0.0] * 3, [0.0] * 3)
        out, ids, before, handles = [list(firsts)], list(firsts), None, []
        for _ in range(20):
            if not ahead:
                ids = eng.step_sample([StepEntry(i, [t], [0]) for i, t in enumerate(ids)], [0.0] * 3, [0.0] * 3)
                out.append(list(ids))
                continue
            feed = ids if before is None else [TokenRef(before, i) for i in range(3)]
            h = eng.step_sample_ahead([StepEntry(i, [t], [0]) for i, t in enumerate(feed)], [0.0] * 3, [0.0] * 3)
            if before is not None:
                out.append(before.tokens())
            before = h
            handles.append(h)
        if ahead:
            out.append(before.tokens())
            # a handle's logits are the recording's buffer: the last step's hold, an older step's
            # were overwritten by a step of the same shape and are refused, not handed out
            assert before.logits.argmax(-1).tolist() == out[-1]
            with pytest.raises(RuntimeError, match="overwritten"):
                handles[-2].logits
            lengths = [eng.cache.get(i).length for i in range(3)]
            with pytest.raises(ValueError, match="sampled last"):
                eng.step_sample_ahead([StepEntry(i, [TokenRef(handles[0], i)], [0]) for i in range(3)],
                                      [0.0] * 3, [0.0] * 3)
            assert [eng.cache.get(i).length for i in range(3)] == lengths
            with pytest.raises(StepError, match="TokenRef"):
                eng.step([StepEntry(0, [TokenRef(before, 0), 5], [1])])
        runs.append(out)
    assert runs[0] == runs[1]
    want = [P.generate_greedy(tiny.read_weights(d, as_stored_in=dtype), cfg, p, 21) for p in prompts]
    if dtype == "float32":
        assert [[step[i] for step in runs[1]] for i in range(3)] == want


def test_a_batch_shape_is_recorded_only_when_it_comes_back(model_dirs):
    """A decode batch is recorded as a graph the n-th time its shape is queued (here the third;
    two runs of the step and the instantiation are what a recording costs); before that it runs as any
    step does, from its recorded commands, and gives the same ids.  A scheduler whose batch
    shrinks as requests end therefore records nothing for shapes that pass once."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry, TokenRef
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    prompts = [tiny.tokens(cfg, n, 70 + i) for i, n in enumerate([9, 33, 4])]
    runs = []
    for after in (1, 3):
        eng = Engine.from_dir(d, EngineOptions(dtype="bfloat16", max_tokens=512, graph_after_steps=after))
        h = eng.step_sample_ahead([StepEntry(i, p, [len(p) - 1]) for i, p in enumerate(prompts)], [0.0] * 3, [0.0] * 3)
        out, recorded = [], []
        for _ in range(6):
            h2 = eng.step_sample_ahead([StepEntry(i, [TokenRef(h, i)], [0]) for i in range(3)], [0.0] * 3, [0.0] * 3)
            out.append(h.tokens())
            recorded.append(eng._graphs.captures)
            h = h2
        out.append(h.tokens())
        assert recorded == ([1] * 6 if after == 1 else [0, 0, 1, 1, 1, 1])
        runs.append(out)
    assert runs[0] == runs[1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_with_prompt_portions_are_queued_ahead_too(model_dirs, dtype):
    """Any step can be queued before the ids of the step before it have reached the host:
    a portion of a prompt beside decode tokens that name those ids (TokenRef), a prompt's last
    portion whose first token is sampled on the device.  The ids are the ones that the same
    steps give when every step waits for the one before and is fed from the host."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry, TokenRef, StepError
    cfg, d = tiny.CONFIGS["B"], model_dirs("B")
    a, b, c = (tiny.tokens(cfg, n, 90 + n) for n in (21, 40, 7))
    temps = {"a": 0.0, "b": 0.7, "c": 0.0}

    def u(k):
        return [0.11 * ((k * 7 + i) % 9) for i in range(3)]
    runs = []
    for ahead in (False, True):
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=512))
        take = eng.step_sample_ahead if ahead else (lambda e, t, w: eng.step_sample(e, t, w))
        seen = []
        # step 0: a whole, the first portion of b
        h0 = take([StepEntry("a", a, [len(a) - 1]), StepEntry("b", b[:16], [])], [temps["a"]], u(0)[:1])
        ref = (lambda h, i: TokenRef(h, i)) if ahead else (lambda h, i: h[i])
        # step 1: a decodes the id of step 0, b's second portion, c whole
        h1 = take([StepEntry("a", [ref(h0, 0)], [0]), StepEntry("b", b[16:32], []), StepEntry("c", c, [len(c) - 1])],
                  [temps["a"], temps["c"]], u(1)[:2])
        seen.append(h0.tokens() if ahead else h0)
        # step 2: a and c decode, b's last portion gives its first token
        h2 = take([StepEntry("a", [ref(h1, 0)], [0]), StepEntry("c", [ref(h1, 1)], [0]),
                   StepEntry("b", b[32:], [len(b) - 33])], [temps["a"], temps["c"], temps["b"]], u(2))
        seen.append(h1.tokens() if ahead else h1)
        before = h2
        for k in range(3, 9):                  # all three decode: replayed graphs from here on
            h = take([StepEntry("a", [ref(before, 0)], [0]), StepEntry("c", [ref(before, 1)], [0]),
                      StepEntry("b", [ref(before, 2)], [0])], [temps["a"], temps["c"], temps["b"]], u(k))
            seen.append(before.tokens() if ahead else before)
            before = h
        seen.append(before.tokens() if ahead else before)
        if ahead:
            with pytest.raises(StepError, match="stands alone"):
                eng.step_sample_ahead([StepEntry("a", [TokenRef(before, 0), 3], [1])], [0.0], [0.0])
            with pytest.raises(StepError, match="sampled last"):
                eng.step_sample_ahead([StepEntry("a", [TokenRef(h1, 0)], [0]), StepEntry("b", [5, 6], [1])],
                                      [0.0, 0.0], [0.0, 0.0])
        runs.append(seen)
    assert runs[0] == runs[1]
    if dtype == "float32":                      # the greedy request against the plain implementation
        w = tiny.read_weights(d, as_stored_in=dtype)
        assert [s[0] for s in runs[1]] == P.generate_greedy(w, cfg, a, len(runs[1]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_scheduler_queues_steps_with_portions_ahead(model_dirs, dtype):
    """Prompts in portions beside decoding requests, more requests than places: with every
    step queued behind the one in flight the scheduler gives the tokens it gives when it waits
    for each step, and it does queue steps with portions in them ahead."""
    from kllm_amd.engine import Engine, EngineOptions
    from kllm_amd.engine.scheduler import Scheduler
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    prompts = [tiny.tokens(cfg, n, 30 + n) for n in (50, 9, 33, 70, 4, 21)]
    got = []
    for ahead in (False, True):
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=1024, graph_after_steps=2))
        queued = []
        inner = eng.step_sample_ahead
        eng.step_sample_ahead = lambda e, t, w: (queued.append(any(len(x.tokens) > 1 for x in e)), inner(e, t, w))[1]
        sched = Scheduler(eng, max_batch=4, max_step_tokens=24, chunk_size=16, queue_ahead=ahead)
        ids = [sched.submit(list(p), 18, temperature=0.6 if i % 2 else 0.0, seed=i) for i, p in enumerate(prompts)]
        results = sched.run_until_done()
        assert all(results[i].error is None and len(results[i].tokens) == 18 for i in ids)
        assert not eng.cache.requests and all(p.free_pages == p.num_pages for p in eng.cache.pools)
        assert (sum(queued) > 5) == ahead       # steps with portions went ahead, or none did
        got.append([results[i].tokens for i in ids])
    assert got[0] == got[1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_run_again_from_their_recorded_commands(model_dirs, dtype):
    """A step's launches go to the library as one buffer of commands, and a step whose shape
    was seen before runs again from the commands recorded then, with its own positions' values
    in place.  Both give, bit for bit, what launching one by one gives: portions of equal size
    of a long prompt (whose key counts grow), beside decode tokens of other requests."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    cfg, d = tiny.CONFIGS["E"], model_dirs("E")
    long_prompt, others = tiny.tokens(cfg, 900, 1), [tiny.tokens(cfg, 40 + 3 * i, 2 + i) for i in range(3)]
    outs = {}

    def run(eng):
        got = [eng.step([StepEntry(("o", i), o[:-12], [len(o) - 13]) for i, o in enumerate(others)]).clone()]
        fed = 0
        for k in range(12):                    # 3 decode tokens + a portion of 64 tokens, twelve times
            entries = [StepEntry(("o", i), [o[len(o) - 12 + k]], [0]) for i, o in enumerate(others)]
            entries.append(StepEntry("long", long_prompt[fed:fed + 64], [0, 63]))
            fed += 64
            got.append(eng.step(entries).clone())
        got.append(eng.step([StepEntry("long", long_prompt[fed:], [len(long_prompt) - fed - 1])]).clone())
        for rid in ["long"] + [("o", i) for i in range(len(others))]:
            eng.release(rid)
        eng.cache.check_invariants()
        return [g.cpu() for g in got]
    for mode, extra in (("one by one", {"launch_one_by_one": True}), ("recorded", {"no_repeated_steps": True}),
                        ("repeated", {})):
        eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=2048, max_model_len=2048, extra=extra))
        outs[mode] = run(eng)
        if mode == "repeated":
            # the first pass grows the scratch buffers now and then (commands recorded before that
            # are dropped), the second records what was dropped, the third repeats every step
            first = eng.steps_repeated
            run(eng)
            second = eng.steps_repeated
            outs["repeated, third pass"] = run(eng)
            assert eng._repeat_steps and first >= 3 and second - first >= 6, (first, second)
            assert eng.steps_repeated - second == 14
        else:
            assert eng.steps_repeated == 0
    for mode in ("recorded", "repeated", "repeated, third pass"):
        for a, b in zip(outs["one by one"], outs[mode]):
            assert torch.equal(a, b), mode
    want = expected(d, cfg, {"long": long_prompt}, dtype)["long"]
    got = outs["repeated"][-1][0].numpy()
    assert float(np.abs(got - want[len(long_prompt) - 1]).max()) < tiny.TOL[dtype]


def test_a_recorded_launch_that_the_library_refuses_is_named():
    """Inside a recording scope the wrappers only write commands; the library's refusal of one
    comes out when the commands run, with the launch's name, and the launches before it have
    run."""
    from kllm_amd import kernels as K
    x = torch.ones(4, 64, device="cuda")
    w = torch.ones(64, device="cuda")
    out = torch.zeros(4, 64, device="cuda")
    bad_x, bad_w, bad_y = (torch.ones(4, 12, dtype=torch.bfloat16, device="cuda"),
                           torch.ones(8, 12, dtype=torch.bfloat16, device="cuda"), torch.zeros(1, 4, 8, device="cuda"))
    with pytest.raises(K.KernelError, match="gemm.*command 1 of 2"):
        with K.stream_scope(record=True):
            K.add_rmsnorm(x, weight=w, out=out, eps=0.0)
            K.gemm(bad_x, bad_w, bad_y, K.GEMM_MFMA_BF16, 1)          # K = 12 is no multiple of 8
            assert float(out.abs().sum()) == 0.0                      # nothing has run yet
    torch.cuda.synchronize()
    assert torch.allclose(out, torch.ones_like(out), atol=1e-6)       # the norm before it did run
    with K.stream_scope(record=True):                                 # work given to the stream by other ways
        K.add_rmsnorm(x, weight=w, out=out, eps=3.0)                  # comes after a flush
        K.flush_recorded()
        assert torch.allclose(out, torch.full_like(out, 0.5), atol=1e-6)
        with K.direct_launches():
            assert not K.recording()
            K.add_rmsnorm(x, weight=w, out=out, eps=0.0)
            assert torch.allclose(out, torch.ones_like(out), atol=1e-6)
        assert K.recording()


def test_no_collection_of_garbage_falls_into_a_recording(model_dirs):
    """An engine that is dropped is garbage in a reference cycle, its recorded steps with
    it.  HIP refuses to destroy a graph on a thread that records one, and the error would
    leave a destructor and end the process, so a collection must not start while a later
    engine records: with the collector set to run at every allocation, none does."""
    import gc
    from kllm_amd.engine import Engine, EngineOptions
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    prompt = tiny.tokens(cfg, 9, 3)
    started = []

    def watch(phase, info):
        if phase == "start":
            started.append(torch.cuda.is_current_stream_capturing())

    before = gc.get_threshold()
    outs = []
    gc.callbacks.append(watch)
    try:
        for _ in range(2):
            eng = Engine.from_dir(d, EngineOptions(dtype="float32", max_tokens=128, graph_after_steps=1))
            gc.set_threshold(1, 1, 1)
            outs.append(eng.generate(prompt, 6))
            gc.set_threshold(*before)
            assert eng._graphs.captures > 0
            del eng
    finally:
        gc.set_threshold(*before)
        gc.callbacks.remove(watch)
    assert len(started) > 10 and not any(started)
    assert outs[0] == outs[1] == P.generate_greedy(tiny.read_weights(d), cfg, prompt, 6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(model_dirs, dtype):
    """One token per step for 400 steps, past several pages and past the
    model's max_position_embeddings (positions are computed, not looked up)."""
    cfg, d = tiny.CONFIGS["B"], model_dirs("B")
    reqs = make_requests(cfg, [400], 6)
    steps = traces.bulk_then_tail(reqs, tail=399)
    rows, _ = replay(d, dtype, steps, 448)
    compare(rows, expected(d, cfg, reqs, dtype), dtype, reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_of_a_sequence(model_dirs, name, dtype):
    """Position 0 sees only itself; 1 and 2 see little: the first rows of a
    sequence fed one token at a time, beside another request in the batch."""
    cfg, d = tiny.CONFIGS[name], model_dirs(name)
    reqs = make_requests(cfg, [4, 3], 8)
    a, b = reqs["r0"], reqs["r1"]
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": a[:1], "want": [0]}], "end": []},
             {"step": 1, "entries": [{"id": "r0", "tokens": a[1:2], "want": [0]},
                                     {"id": "r1", "tokens": b[:1], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "r1", "tokens": b[1:3], "want": [0, 1]},
                                     {"id": "r0", "tokens": a[2:4], "want": [0, 1]}], "end": ["r0", "r1"]}]
    rows, _ = replay(d, dtype, steps, 128)
    compare(rows, expected(d, cfg, reqs, dtype), dtype, reqs)


def test_hidden_states_layer_by_layer(model_dirs):
    """The residual stream after the embedding, after every layer and after the
    final norm, as the reference's debug taps capture it
    (backend/model.cu:1061, :1085, :1123-1124), within its own bound of 1e-4
    (engine/e2e/e2e_test.go:21-24)."""
    from kllm_amd.engine import Engine, EngineOptions, StepEntry
    for name in ("A", "B"):
        cfg, d = tiny.CONFIGS[name], model_dirs(name)
        eng = Engine.from_dir(d, EngineOptions(dtype="float32", max_tokens=256))
        ids = tiny.tokens(cfg, 40, 9)
        taps = []
        eng.step([StepEntry("x", ids, [39])], taps=taps)
        _, hidden = P.forward(tiny.read_weights(d), cfg, ids, return_hidden=True)
        assert len(taps) == len(hidden) == cfg["num_hidden_layers"] + 2
        for t, h in zip(taps, hidden):
            assert float((t.cpu() - h).abs().max()) < 1e-4


def test_step_refuses_bad_input_and_leaves_the_cache_alone(model_dirs):
    from kllm_amd.cache import OutOfPages
    from kllm_amd.engine import Engine, EngineOptions, StepEntry, StepError
    eng = Engine.from_dir(model_dirs("A"), EngineOptions(dtype="float32", max_tokens=64, max_model_len=100))
    with pytest.raises(StepError, match="token id"):
        eng.step([StepEntry("a", [1, 256], [0])])
    with pytest.raises(StepError, match="wanted place"):
        eng.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(StepError, match="twice"):
        eng.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(StepError, match="at least one token"):
        eng.step([StepEntry("a", [], [])])
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1] * 40, []), StepEntry("b", [1] * 40, [])])
    assert not eng.cache.requests and eng.cache.pools[0].free_pages == 4
    eng.step([StepEntry("a", [1] * 60, [])])
    with pytest.raises(StepError, match="longest"):
        eng.step([StepEntry("c", [1] * 101, [])])
    assert eng.step([StepEntry("a", [5], [])]) is None        # nothing wanted, nothing returned
    assert eng.length("a") == 61
    eng.release("a")
    eng.cache.check_invariants()


def run_trace_program(model_dir, dtype, steps, max_tokens, out_dir, as_module=False):
    program = [sys.executable, "-m", "kllm_amd.replay"] if as_module else \
        [sys.executable, os.path.join(ROOT, "bin", "trace_run")]
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", "")) if as_module else None
    proc = subprocess.Popen(
        program + ["--model", model_dir, "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, cwd="/", env=env)
    outs = []
    for s in steps:
        proc.stdin.write(json.dumps(s) + "\n")
        proc.stdin.flush()
        line = proc.stdout.readline().strip()
        assert line == f"done {s['step']}", line       # the next step only after this line
    proc.stdin.close()
    assert proc.wait(timeout=120) == 0
    for s in steps:
        path = os.path.join(out_dir, f"{s['step']}.f32")
        wanted = sum(len(e["want"]) for e in s["entries"])
        if wanted == 0:
            assert not os.path.exists(path)
            outs.append(None)
        else:
            outs.append(np.fromfile(path, dtype="<f4").reshape(wanted, -1))
    return outs


@pytest.mark.parametrize("dtype,name", [("float32", "B"), ("bfloat16", "A")])
def test_the_trace_run_program(model_dirs, tmp_path, dtype, name):
    cfg, d = tiny.CONFIGS[name], model_dirs(name, store="bfloat16" if dtype == "bfloat16" else "float32")
    reqs = make_requests(cfg, [50, 21, 77, 30, 64, 12], 10)
    steps, peak = traces.mixed(reqs, seed=11)
    steps[3]["entries"][0]["want"] = []                       # a step may want nothing of a request
    # the program under both of its names: bin/trace_run and python -m kllm_amd.replay
    outs = run_trace_program(d, dtype, steps, peak, str(tmp_path / "out"), as_module=dtype == "float32")
    assert outs[0].shape[1] == cfg["vocab_size"]
    rows = traces.collect(steps, outs)
    want = expected(d, cfg, reqs, dtype)
    for (rid, p), got in rows.items():
        assert float(np.abs(got - want[rid][p]).max()) < tiny.TOL[dtype]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "R"])
def test_greedy_generation_through_the_entry_point(model_dirs, name, dtype):
    """Greedy tokens through Engine.generate (scheduler, sampling kernel) equal
    the plain implementation's, for prompts generated together."""
    from kllm_amd.engine import Engine, EngineOptions
    cfg, d = tiny.CONFIGS[name], model_dirs(name)
    eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=512))
    lengths = {"A": [5, 17, 33], "B": [1, 9, 40, 70]}.get(name)
    prompts = tiny.REFERENCE_PROMPTS if name == "R" else [tiny.tokens(cfg, n, 20 + n) for n in lengths]
    new = {"A": 16, "B": 24, "R": 16}[name]
    got = eng.generate(prompts, new, max_batch=4, max_step_tokens=48)
    w = tiny.read_weights(d, as_stored_in=dtype)
    for p, g in zip(prompts, got):
        want = P.generate_greedy(w, cfg, p, new, eos={cfg["eos_token_id"]} if "eos_token_id" in cfg else None)
        if dtype == "float32":
            assert g == want
        else:                                            # bfloat16 may part ways at a near-tie
            agree = next((i for i, (x, y) in enumerate(zip(g, want)) if x != y), len(want))
            if agree < len(want):
                logits = P.forward(w, cfg, p + want[:agree])[-1]
                top2 = torch.topk(logits, 2).values
                assert float(top2[0] - top2[1]) < tiny.TOL[dtype], (agree, g, want)
    assert not eng.cache.requests


def test_generate_takes_all_its_prompts_together(model_dirs):
    """Twelve prompts and no batch size given: they decode together (more than the
    scheduler's own default of eight), and each gets the plain implementation's tokens."""
    from kllm_amd.engine import Engine, EngineOptions
    from kllm_amd.engine import scheduler as S
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    eng = Engine.from_dir(d, EngineOptions(dtype="float32", max_tokens=1024))
    prompts = [tiny.tokens(cfg, 3 + 2 * i, 70 + i) for i in range(12)]
    seen = []
    run = S.Scheduler.run_until_done
    def watched(self, *a, **k):
        out = run(self, *a, **k)
        seen.append(self.stats["max_batch_seen"])
        return out
    S.Scheduler.run_until_done = watched
    try:
        got = eng.generate(prompts, 12)
    finally:
        S.Scheduler.run_until_done = run
    assert seen == [12]
    w = tiny.read_weights(d, as_stored_in="float32")
    for p, g in zip(prompts, got):
        assert g == P.generate_greedy(w, cfg, p, 12, eos={cfg["eos_token_id"]} if "eos_token_id" in cfg else None)
    assert not eng.cache.requests


@pytest.mark.parametrize("dtype", DTYPES)
def test_generation_when_pages_run_out(model_dirs, dtype):
    """A pool too small for the requests together: the scheduler gives the youngest one's
    pages back and starts it again later, decode steps are queued ahead in between, and
    every request still gets the plain implementation's tokens."""
    from kllm_amd.engine import Engine, EngineOptions
    from kllm_amd.engine.scheduler import Scheduler
    cfg, d = tiny.CONFIGS["A"], model_dirs("A")
    prompts = [tiny.tokens(cfg, n, 50 + n) for n in (40, 33, 50, 20)]
    new = 30
    eng = Engine.from_dir(d, EngineOptions(dtype=dtype, max_tokens=176, poison_freed_pages=True, graph_after_steps=2))
    sched = Scheduler(eng, max_batch=4, max_step_tokens=64)
    ids = [sched.submit(list(p), new, seed=i) for i, p in enumerate(prompts)]
    results = sched.run_until_done()
    assert sched.stats["preemptions"] > 0
    assert not eng.cache.requests and all(p.free_pages == p.num_pages for p in eng.cache.pools)
    w = tiny.read_weights(d, as_stored_in=dtype)
    for i, p in zip(ids, prompts):
        assert results[i].error is None
        g, want = results[i].tokens, P.generate_greedy(w, cfg, p, new)
        if dtype == "float32":
            assert g == want
        else:                                            # bfloat16 may part ways at a near-tie
            agree = next((k for k, (x, y) in enumerate(zip(g, want)) if x != y), len(want))
            if agree < len(want):
                top2 = torch.topk(P.forward(w, cfg, p + want[:agree])[-1], 2).values
                assert float(top2[0] - top2[1]) < tiny.TOL[dtype], (agree, g, want)


def test_temperature_generation_matches_the_plain_sampler(model_dirs):
    """Config B, temperature 0.8, seeded: the same tokens as the plain
    implementation drawing with the same uniforms, alone and in a batch."""
    from kllm_amd.engine import Engine, EngineOptions
    from kllm_amd.sampling import uniform
    cfg, d = tiny.CONFIGS["B"], model_dirs("B")
    eng = Engine.from_dir(d, EngineOptions(dtype="float32", max_tokens=512))
    prompts = [tiny.tokens(cfg, n, 30 + n) for n in (1, 9, 40, 70)]
    got = eng.generate(prompts, 24, temperature=0.8, seed=100, max_batch=3, max_step_tokens=32)
    alone = [eng.generate(p, 24, temperature=0.8, seed=100 + i) for i, p in enumerate(prompts)]
    assert got == alone
    w = tiny.read_weights(d)
    for i, p in enumerate(prompts):
        ids = list(p)
        for k, tok in enumerate(got[i]):
            row = P.forward(w, cfg, ids)[-1]
            u = uniform(100 + i, k)
            want = P.sample_inverse_cdf(row, 0.8, u)
            if want != tok:                              # only at a boundary of the CDF
                cdf = torch.cumsum(P.softmax_temperature(row, 0.8), 0)
                assert abs(float(cdf[min(want, tok)]) - u) < 1e-4
            ids.append(tok)


def test_temperature_generation_in_bfloat16_alone_and_in_a_batch(model_dirs):
    """In bfloat16 a request's logits in a batch equal those of the request alone up to
    rounding only (the kernels follow the step's size), so the drawn tokens may part ways,
    but only where the uniform number lies within that rounding of a boundary of the
    cumulative distribution; up to there they are the same tokens."""
    from kllm_amd.engine import Engine, EngineOptions
    from kllm_amd.sampling import uniform
    cfg, d = tiny.CONFIGS["B"], model_dirs("B", store="bfloat16")
    eng = Engine.from_dir(d, EngineOptions(dtype="bfloat16", max_tokens=512))
    prompts = [tiny.tokens(cfg, n, 30 + n) for n in (1, 9, 40, 70)]
    got = eng.generate(prompts, 24, temperature=0.8, seed=100, max_batch=3, max_step_tokens=32)
    alone = [eng.generate(p, 24, temperature=0.8, seed=100 + i) for i, p in enumerate(prompts)]
    w = tiny.read_weights(d, as_stored_in="bfloat16")
    same = 0
    for i, p in enumerate(prompts):
        agree = next((k for k, (x, y) in enumerate(zip(got[i], alone[i])) if x != y), len(alone[i]))
        same += agree
        if agree < len(alone[i]):
            row = P.forward(w, cfg, list(p) + got[i][:agree])[-1]
            cdf = torch.cumsum(P.softmax_temperature(row, 0.8), 0)
            a, b = sorted((got[i][agree], alone[i][agree]))
            assert b == a + 1 or float(cdf[b - 1] - cdf[a]) < 2e-2, (i, agree, a, b)    # neighbours on the CDF
            assert abs(float(cdf[a]) - uniform(100 + i, agree)) < 2e-2, (i, agree)
    assert same >= 60, same


def test_command_line_generate(model_dirs):
    """The command line in the reference's manner (cmd/generate/main.go:15-50)."""
    cfg, d = tiny.CONFIGS["R"], model_dirs("R")
    out = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "generate"), "--model", d, "--ids", "1 17 42 100 7",
         "--steps", "16", "--max-seq", "256", "--dtype", "float32"],
        capture_output=True, text=True, timeout=120, cwd="/")
    assert out.returncode == 0, out.stderr
    lines = out.stdout.strip().splitlines()
    assert lines[0] == "prompt:    [1 17 42 100 7]"
    want = P.generate_greedy(tiny.read_weights(d), cfg, [1, 17, 42, 100, 7], 16, eos={2})
    assert lines[1] == "generated: [" + " ".join(map(str, want)) + "]"


def test_command_line_options_of_the_engine_sizes(model_dirs):
    """--page-size, --num-pages, --max-step-tokens, --max-new-tokens and --sample-seed: a
    prompt longer than the step's budget is cut into portions, the tokens stay the same,
    and what the cache was sized to is printed at start."""
    cfg, d = tiny.CONFIGS["R"], model_dirs("R")
    prompt = tiny.tokens(cfg, 45, 8)
    base = [sys.executable, os.path.join(ROOT, "bin", "generate"), "--model", d, "--ids", " ".join(map(str, prompt)),
            "--dtype", "float32", "--max-seq", "256"]
    out = subprocess.run(base + ["--max-new-tokens", "12", "--page-size", "8", "--num-pages", "9", "--max-step-tokens", "7",
                                 "--sample-seed", "3"], capture_output=True, text=True, timeout=120, cwd="/")
    assert out.returncode == 0, out.stderr
    want = P.generate_greedy(tiny.read_weights(d), cfg, prompt, 12, eos={2})
    assert out.stdout.strip().splitlines()[1] == "generated: [" + " ".join(map(str, want)) + "]"
    assert "9 pages of 8 tokens" in out.stderr
    small = subprocess.run(base + ["--steps", "12", "--page-size", "8", "--num-pages", "3"],
                           capture_output=True, text=True, timeout=120, cwd="/")
    assert small.returncode == 1 and "could not run even alone" in small.stderr


def test_command_line_bench_one_kernel_and_a_sweep_of_batches(model_dirs):
    d = model_dirs("A")
    bench = [sys.executable, os.path.join(ROOT, "bin", "bench"), "--json", "--dtype", "bfloat16"]
    out = subprocess.run(bench + ["--kernel", "gemm", "--shape", "200,256,512", "--steps", "5"],
                         capture_output=True, text=True, timeout=120, cwd="/")
    assert out.returncode == 0, out.stderr
    res = json.loads(out.stdout.strip().splitlines()[-1])
    assert res["kernel"] == "gemm" and res["us"] > 0 and 0 < res["frac_of_peak"] < 1 and res["frac_of_measured"] > 0
    out = subprocess.run(bench + ["--model", d, "--prompt", "16", "--steps", "8", "--reps", "1", "--max-seq", "64",
                                  "--batch", "1,3"], capture_output=True, text=True, timeout=120, cwd="/")
    assert out.returncode == 0, out.stderr
    rows = [json.loads(l) for l in out.stdout.strip().splitlines()]
    assert [r["batch"] for r in rows] == [1, 3] and all(r["decode_tok_s"] > 0 and r["ttft_ms"] > 0 for r in rows)
    assert "pages of 16 tokens" in out.stderr
