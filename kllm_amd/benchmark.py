"""Measuring the engine: prefill and decode throughput with random weights
and synthetic token ids, and what a step must read or compute at least.

The reference's bench (cmd/bench/main.go:48-131) times prefills and
single-token forwards of one sequence with the host clock and synthetic ids
``(i*37+11) % vocab``; here steps are bracketed by device synchronisation,
batches are given, and every figure comes with its roofline.
"""

from __future__ import annotations

import time
from typing import Dict, List

import torch

from .engine import Engine, EngineOptions, StepEntry, TokenRef

# Published peaks of MI355X.
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float16": 2.5e15, "fp8": 5.0e15, "float32": 157.3e12}

TINYLLAMA_1_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 22,
    "hidden_size": 2048, "num_attention_heads": 32, "num_key_value_heads": 4, "head_dim": 64,
    "intermediate_size": 5632, "vocab_size": 32000, "rope_theta": 10000.0,
    "max_position_embeddings": 2048, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
    "hidden_act": "silu",
}


# The other sizes that the baseline names (Llama-2 7B: all heads keep keys; Llama-3 8B: groups
# of four, a vocabulary of 128,256).
LLAMA2_7B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 32,
    "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 32, "head_dim": 128,
    "intermediate_size": 11008, "vocab_size": 32000, "rope_theta": 10000.0,
    "max_position_embeddings": 4096, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
    "hidden_act": "silu",
}
LLAMA3_8B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 32,
    "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "intermediate_size": 14336, "vocab_size": 128256, "rope_theta": 500000.0,
    "max_position_embeddings": 8192, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
    "hidden_act": "silu",
}
PRESETS = {"tinyllama-1.1b": TINYLLAMA_1_1B, "llama2-7b": LLAMA2_7B, "llama3-8b": LLAMA3_8B}


def synthetic_ids(n: int, vocab: int, salt: int = 0) -> List[int]:
    """The reference's synthetic prompt (cmd/bench/main.go:61-64), salted per request."""
    return [((i + salt * 101) * 37 + 11) % vocab for i in range(n)]


def _sync():
    torch.cuda.synchronize()


def measure_prefill(engine: Engine, tokens: int, reps: int = 3, warmup: int = 1):
    """Milliseconds of one whole prompt of ``tokens`` ids in one step (best of reps)."""
    vocab = engine.vocab_size
    best = None
    for r in range(warmup + reps):
        ids = synthetic_ids(tokens, vocab, r)
        _sync()
        t0 = time.perf_counter()
        engine.step([StepEntry(("prefill", r), ids, [tokens - 1])])
        _sync()
        ms = (time.perf_counter() - t0) * 1e3
        engine.release(("prefill", r))
        if r >= warmup:
            best = ms if best is None else min(best, ms)
    return best


def fill_context(engine: Engine, batch: int, context: int, chunk: int = 2048, tag="decode"):
    """``batch`` live requests of ``context`` tokens each, prefilled through
    the step function.  Returns their ids and a first token for each."""
    vocab = engine.vocab_size
    rids = [(tag, i) for i in range(batch)]
    for i, rid in enumerate(rids):
        ids = synthetic_ids(context, vocab, i)
        for a in range(0, context, chunk):
            engine.step([StepEntry(rid, ids[a:a + chunk], [])])
    return rids, [synthetic_ids(1, vocab, 7 + i)[0] for i in range(batch)]


class DecodeLoop:
    """Greedy decoding of a fixed batch, each step fed with the ids of the one before.
    Where the engine can queue a step ahead (as its scheduler does), the ids go from step
    to step on the device and are read on the host one step late; every step's ids are
    read."""

    def __init__(self, engine: Engine, rids, first_tokens):
        self.engine, self.rids, self.toks = engine, list(rids), list(first_tokens)
        # steady decoding is what is timed: the batch's graph is recorded in the warm-up
        self._graph_after, engine.options.graph_after_steps = engine.options.graph_after_steps, 1
        self.zeros = [0.0] * len(self.rids)
        self.ahead = engine.can_sample_ahead([StepEntry(r, [t], [0]) for r, t in zip(self.rids, self.toks)])

    def run(self, k: int):
        eng, rids, zeros = self.engine, self.rids, self.zeros
        before = None
        for _ in range(k):
            if not self.ahead:
                self.toks = eng.step_sample([StepEntry(r, [t], [0]) for r, t in zip(rids, self.toks)], zeros, zeros)
                continue
            ids = self.toks if before is None else [TokenRef(before, i) for i in range(len(rids))]
            handle = eng.step_sample_ahead([StepEntry(r, [t], [0]) for r, t in zip(rids, ids)], zeros, zeros)
            if before is not None:
                before.tokens()
            before = handle
        if before is not None:
            self.toks = before.tokens()

    def timed(self, k: int) -> float:
        """Milliseconds per step over k steps, bracketed by device synchronisation."""
        _sync()
        t0 = time.perf_counter()
        self.run(k)
        _sync()
        return (time.perf_counter() - t0) * 1e3 / k

    def release(self):
        for r in self.rids:
            self.engine.release(r)
        self.engine.options.graph_after_steps = self._graph_after


def measure_decode(engine: Engine, batch: int, context_end: int, steps: int, warmup: int):
    """Decode ``warmup`` untimed and then ``steps`` timed steps of ``batch``
    requests, ending at ``context_end`` tokens each; greedy sampling on the
    device, each step's tokens fed into the next.  Returns (ms per step, mean
    context length during the timed steps)."""
    start = context_end - steps - warmup
    if start < 1:
        raise ValueError("context too short for the steps asked for")
    rids, toks = fill_context(engine, batch, start)
    loop = DecodeLoop(engine, rids, toks)
    loop.run(warmup)
    ms = loop.timed(steps)
    loop.release()
    return ms, context_end - steps / 2.0


def measure_decode_run(engine: Engine, batch: int, prompt_len: int = 512, total_len: int = 2048,
                       segment: int = 32, points=(512, 1280, 2047)):
    """The whole run the metric names: ``batch`` requests with prompts of
    ``prompt_len`` tokens decoded until each holds ``total_len``.  Steps are
    timed in segments of ``segment`` (a device synchronisation between them).
    Returns {"mean_tok_s": over the run, "at": {T: tok/s of the segment that
    holds context length T}, "steps": ..., "ms_per_step": mean}."""
    rids, toks = fill_context(engine, batch, prompt_len, chunk=prompt_len)
    loop = DecodeLoop(engine, rids, toks)
    loop.run(4)                                   # graphs recorded, caches warm; context prompt_len + 4
    segments, ctx = [], prompt_len + 4            # (first context length, steps, ms per step)
    while ctx < total_len:
        k = min(segment, total_len - ctx)
        segments.append((ctx, k, loop.timed(k)))
        ctx += k
    loop.release()
    total_ms = sum(k * ms for _, k, ms in segments)
    steps = sum(k for _, k, _ in segments)
    at = {}
    for T in points:
        holding = [sg for sg in segments if sg[0] <= T < sg[0] + sg[1]]
        sg = holding[0] if holding else (segments[0] if T < segments[0][0] else segments[-1])
        at[T] = round(batch * 1e3 / sg[2], 1)
    return {"mean_tok_s": round(batch * steps * 1e3 / total_ms, 1), "at": at, "steps": steps,
            "ms_per_step": round(total_ms / steps, 4)}


def measure_prefill_chunks(engine: Engine, tokens: int, chunk: int, reps: int = 3, warmup: int = 1):
    """Milliseconds for one prompt of ``tokens`` ids fed in portions of
    ``chunk`` tokens, one step each (best of reps); the last token's logits
    are asked for."""
    vocab = engine.vocab_size
    best = None
    for r in range(warmup + reps):
        ids = synthetic_ids(tokens, vocab, r)
        _sync()
        t0 = time.perf_counter()
        for a in range(0, tokens, chunk):
            part = ids[a:a + chunk]
            engine.step([StepEntry(("chunks", r), part, [len(part) - 1] if a + chunk >= tokens else [])])
        _sync()
        ms = (time.perf_counter() - t0) * 1e3
        engine.release(("chunks", r))
        if r >= warmup:
            best = ms if best is None else min(best, ms)
    return best


def measure_mixed(engine: Engine, requests: int = 32, min_prompt: int = 128, max_prompt: int = 2048,
                  new_tokens: int = 64, chunk: int = 512, seed: int = 0):
    """A serving workload for the 7B sizes: ``requests``
    prompts with lengths uniform in [min_prompt, max_prompt] (seeded, ids
    uniform in the vocabulary, as the reference's load generator draws them:
    cmd/loadgen/main.go:98-103), all submitted at once to the scheduler, which
    prefills in portions of ``chunk`` tokens beside the decode tokens of the
    requests already running; each generates ``new_tokens``.  Returns totals
    and rates over the wall time of the whole run."""
    import random

    from .engine.scheduler import Scheduler
    rng = random.Random(seed)
    vocab = engine.vocab_size
    prompts = [[rng.randrange(vocab) for _ in range(rng.randint(min_prompt, max_prompt))] for _ in range(requests)]
    sched = Scheduler(engine, max_batch=requests, max_step_tokens=chunk + requests, chunk_size=chunk)
    # a short run first, so that kernels are loaded and the decode graphs recorded
    warm = Scheduler(engine, max_batch=requests, max_step_tokens=chunk + requests, chunk_size=chunk)
    for p in prompts[:requests]:
        warm.submit(p[:min_prompt], 4)
    warm.run_until_done()
    for p in prompts:
        sched.submit(p, new_tokens)
    _sync()
    t0 = time.perf_counter()
    results = sched.run_until_done()
    _sync()
    wall = time.perf_counter() - t0
    errors = [r.error for r in results.values() if r.error]
    if errors:
        raise RuntimeError(f"{len(errors)} requests failed: {errors[0]}")
    prompt_tokens = sum(len(p) for p in prompts)
    generated = sum(len(r.tokens) for r in results.values())
    return {"requests": requests, "prompt_tokens": prompt_tokens, "generated_tokens": generated,
            "wall_s": round(wall, 4), "steps": sched.stats["steps"],
            "prompt_tok_s": round(prompt_tokens / wall, 1), "generated_tok_s": round(generated / wall, 1),
            "total_tok_s": round((prompt_tokens + generated) / wall, 1),
            "preemptions": sched.stats["preemptions"]}


def _attempt(pts, name, fn):
    try:
        fn()
    except Exception as e:                      # the headline figures stand without this point
        pts[name + "_error"] = f"{type(e).__name__}: {e}"[:200]


def same_engine_points(engine: Engine) -> Dict[str, float]:
    """Further workloads on the headline engine, as flat name -> number entries for the
    headline line's ``points`` (the reference's bench puts everything it measures into its one
    JSON object: cmd/bench/main.go:37-46): the 2,048-token prompt in portions of 512 and the
    decode run from 512 to 2,048 tokens at batch 8.  A point that fails leaves
    ``<name>_error``."""
    pts: Dict[str, float] = {}

    def run():
        ms = measure_prefill_chunks(engine, 2048, 512, reps=3, warmup=1)
        pts["prefill_chunks_512_ms"] = round(ms, 3)
        res = measure_decode_run(engine, 8, prompt_len=512, total_len=2048)
        pts["decode_run_b8_mean"] = res["mean_tok_s"]
        for T, v in res["at"].items():
            pts[f"decode_run_b8_T{T}"] = v
    _attempt(pts, "same_engine", run)
    return pts


def other_engine_points(cfg_small: dict, dtype: str, gemm: str = "hip", page_size: int = 16) -> Dict[str, float]:
    """The other configurations that the baseline names, each on an engine of its own (the
    caller has released the headline engine: the larger models need its memory): the float32
    path at the headline sizes ``cfg_small``, Llama-3-8B sizes at batch 64 with contexts of
    4,096, and the mixed serving workload at Llama-2-7B sizes through the scheduler."""
    import gc
    pts: Dict[str, float] = {}

    def attempt(name, fn):
        _attempt(pts, name, fn)

    def other(cfg, dt, max_tokens, max_requests, max_len, fn):
        eng = make_engine(cfg, dt, max_tokens=max_tokens, max_requests=max_requests, max_model_len=max_len,
                          gemm=gemm, page_size=page_size)
        try:
            fn(eng)
        finally:
            del eng
            gc.collect()
            torch.cuda.empty_cache()

    def fp32(eng):
        ms, ctx = measure_decode(eng, 8, 2048, 32, 8)
        pts["fp32_decode_b8"] = round(8e3 / ms, 1)
        pts["fp32_decode_b8_hbm_frac"] = round(eng.step_read_bytes([int(ctx)] * 8) / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
        pms = measure_prefill(eng, 2048)
        pts["fp32_prefill_ms"] = round(pms, 3)
        pts["fp32_prefill_frac"] = round(eng.model.step_flops(2048, 2048 * 2049 / 2.0, 1) / (pms * 1e-3)
                                         / PEAK_FLOPS["float32"], 4)
    if dtype != "float32":
        attempt("fp32", lambda: other(cfg_small, "float32", 8 * 2048 + 4096, 8, 2048 + 64, fp32))

    def llama3(eng):
        ms, ctx = measure_decode(eng, 64, 4096, 16, 4)
        pts["llama3_8b_b64_ctx4096_ms"] = round(ms, 3)
        pts["llama3_8b_b64_ctx4096_tok_s"] = round(64e3 / ms, 1)
        pts["llama3_8b_b64_ctx4096_hbm_frac"] = round(eng.step_read_bytes([int(ctx)] * 64) / (ms * 1e-3) / 1e9
                                                      / PEAK_HBM_GBS, 4)
    attempt("llama3_8b_b64_ctx4096", lambda: other(LLAMA3_8B, dtype, 64 * 4096 + 4096, 64, 4096 + 64, llama3))

    def llama2(eng):
        res = measure_mixed(eng, 32, 128, 2048, 64, 512)
        pts["llama2_7b_mixed_wall_s"] = res["wall_s"]
        pts["llama2_7b_mixed_prompt_tok_s"] = res["prompt_tok_s"]
        pts["llama2_7b_mixed_generated_tok_s"] = res["generated_tok_s"]
    attempt("llama2_7b_mixed", lambda: other(LLAMA2_7B, dtype, 32 * (2048 + 64 + page_size), 64, 2048 + 128, llama2))
    return pts


def make_engine(cfg: dict, dtype: str, max_tokens: int, seed: int = 0, **opts) -> Engine:
    options = EngineOptions(dtype=dtype, max_tokens=max_tokens, max_requests=max(64, opts.pop("max_requests", 64)),
                            **opts)
    return Engine.from_random(cfg, seed, options)


# ----------------------------------------------------------------------------- the box's own peaks

_calibration = {}


def calibrate(device=None) -> Dict[str, float]:
    """What this box reaches with nothing in the way: GB/s (read + written) of a plain
    copy kernel over 1 GiB, GB/s of a read-only stream over the same (what a decode step's
    kernels do), and TFLOP/s of a loop of independent MFMAs in registers, for
    bfloat16 and float32 operands.  Figures are quoted against the published peaks and
    against these."""
    if _calibration:
        return _calibration
    from . import kernels as K
    dev = device or torch.device("cuda", torch.cuda.current_device())
    n = 1 << 28
    src = torch.empty(n, dtype=torch.float32, device=dev).fill_(1.0)
    dst = torch.empty_like(src)
    K.calibrate_copy(dst, src)
    best = min(_event_ms(lambda: K.calibrate_copy(dst, src)) for _ in range(5))
    _calibration["copy_GBs"] = round(2 * n * 4 / (best * 1e-3) / 1e9, 1)
    rsink = torch.zeros(K.calibrate_read_workgroups(), dtype=torch.float32, device=dev)
    K.calibrate_read(src, rsink)
    best = min(_event_ms(lambda: K.calibrate_read(src, rsink)) for _ in range(5))
    _calibration["read_GBs"] = round(n * 4 / (best * 1e-3) / 1e9, 1)
    del src, dst
    sink = torch.zeros(64, dtype=torch.float32, device=dev)
    for name, code in (("bfloat16", K.DT_BF16), ("float32", K.DT_F32)):
        iters = 4096 if code == K.DT_BF16 else 1024
        flops = K.calibrate_mfma(code, iters, sink)
        best = min(_event_ms(lambda: K.calibrate_mfma(code, iters, sink)) for _ in range(5))
        _calibration[f"mfma_{name}_TFLOPs"] = round(flops / (best * 1e-3) / 1e12, 1)
    return _calibration


def _event_ms(fn, reps: int = 1) -> float:
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) / reps


# ----------------------------------------------------------------------------- one kernel at a time

def bench_kernel(name: str, shape, dtype: str = "bfloat16", reps: int = 50, warmup: int = 5):
    """Time one kernel alone at one shape with device events: the counterpart of the
    reference's te_bench_matmul (backend/shim.h:88-92, backend/model.cu:800-863), for every
    hot kernel.  ``shape`` is a tuple of ints whose meaning depends on the kernel:

      gemm          n, m, k      x [n, k] . w [m, k]^T, the kernel and split of K the engine picks
      gemm_swiglu   n, f, k      gate and up products with the gate in the epilogue
      attn_prefill  tokens, H, KV, hd     one prompt of that many tokens, no cached keys
      attn_decode   batch, context, H, KV, hd
      add_rmsnorm   n, d
      copy          bytes

    Returns a dict with microseconds (mean over reps), the bytes or flops the kernel must
    move or do, GB/s or TFLOP/s, and the fraction of the published and of the measured peak."""
    from . import kernels as K
    from .parts import linear as L
    td = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    elem = 2 if td == torch.bfloat16 else 4
    dev = torch.device("cuda", torch.cuda.current_device())
    shape = tuple(int(v) for v in shape)
    rnd = lambda *s: (torch.randn(*s, device=dev) * 0.05).to(td)
    flops = nbytes = 0
    note = ""
    if name == "gemm":
        n, m, k = shape
        x, w = rnd(n, k), rnd(m, k)
        algo, nsplit = L.choose(td, n, m, k, {})
        y = torch.empty(nsplit, n, m, dtype=torch.float32, device=dev)
        fn = lambda: K.gemm(x, w, y, algo, nsplit)
        flops, nbytes = 2.0 * n * m * k, (n * k + m * k) * elem + nsplit * n * m * 4
        note = f"algorithm {algo}, {nsplit} slices of K"
    elif name == "gemm_swiglu":
        n, f, k = shape
        x, w, h = rnd(n, k), rnd(2 * f, k), torch.empty(n, f, dtype=td, device=dev)
        fn = lambda: K.gemm_swiglu(x, w, h)
        flops, nbytes = 4.0 * n * f * k, (n * k + 2 * f * k + n * f) * elem
    elif name in ("attn_prefill", "attn_decode"):
        if name == "attn_prefill":
            tokens, H, KV, hd = shape
            batch, ctx, new = 1, tokens, tokens
        else:
            batch, ctx, H, KV, hd = shape
            new = 1
        ps = 16
        pages_per = -(-ctx // ps)
        cache = rnd(batch * pages_per, 2, KV, ps * hd)
        bt = torch.arange(batch * pages_per, dtype=torch.int32, device=dev).view(batch, pages_per)
        q, out = rnd(batch * new, H * hd), torch.empty(batch * new, H * hd, dtype=td, device=dev)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
        scale = hd ** -0.5
        if name == "attn_prefill":
            tiles = i32([[t, 0] for t in range(0, tokens, K.PREFILL_QUERY_BLOCK)])
            starts, pos = i32([0, tokens]), i32([0])
            fn = lambda: K.attn_prefill(q, out, cache, tiles, tiles.shape[0], starts, pos, bt, ps, H, KV, hd, 0, scale)
            flops = 4.0 * H * hd * tokens * (tokens + 1) / 2
            nbytes = (2 * tokens * H * hd + 2 * tokens * KV * hd) * elem
        else:
            posn, sot = i32([ctx - 1] * batch), i32(list(range(batch)))
            ns = K.attn_decode_slices(batch, KV, H, hd, td, ctx)
            part = torch.empty(batch * H * ns * (hd + 2), dtype=torch.float32, device=dev)
            fn = lambda: K.attn_decode(q, out, part, cache, posn, sot, bt, ps, H, KV, hd, 0, scale, ns)
            flops = 4.0 * batch * H * hd * ctx
            nbytes = batch * ctx * 2 * KV * hd * elem
            note = f"{ns} slices"
    elif name == "add_rmsnorm":
        n, d = shape
        x, delta, w = torch.randn(n, d, device=dev), torch.randn(n, d, device=dev), torch.ones(d, device=dev)
        out = torch.empty(n, d, dtype=td, device=dev)
        fn = lambda: K.add_rmsnorm(x, delta=delta, weight=w, out=out, eps=1e-5)
        nbytes = n * d * (4 + 4 + 4 + elem)
    elif name == "copy":
        (count,) = shape
        src = torch.empty(count // 4, dtype=torch.float32, device=dev).fill_(1.0)
        dst = torch.empty_like(src)
        fn = lambda: K.calibrate_copy(dst, src)
        nbytes = 2 * (count // 4) * 4
    else:
        raise ValueError(f"no kernel bench named {name!r} (gemm, gemm_swiglu, attn_prefill, attn_decode, "
                         f"add_rmsnorm, copy)")
    for _ in range(warmup):
        fn()
    us = _event_ms(fn, reps) * 1e3
    cal = calibrate(dev)
    res = {"kernel": name, "shape": list(shape), "dtype": dtype, "us": round(us, 2), "note": note}
    if flops:
        t = flops / (us * 1e-6) / 1e12
        res.update(TFLOPs=round(t, 1), frac_of_peak=round(t * 1e12 / PEAK_FLOPS[dtype], 4),
                   frac_of_measured=round(t / cal[f"mfma_{dtype}_TFLOPs"], 4))
    if nbytes:
        g = nbytes / (us * 1e-6) / 1e9
        res.update(GBs=round(g, 1), frac_of_hbm=round(g / PEAK_HBM_GBS, 4),
                   frac_of_measured_copy=round(g / cal["copy_GBs"], 4))
    return res
