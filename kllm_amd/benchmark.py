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


def sizes(cfg: dict) -> Dict[str, int]:
    H, d = cfg["num_attention_heads"], cfg["hidden_size"]
    hd = cfg.get("head_dim") or d // H
    KV = cfg.get("num_key_value_heads") or H
    return dict(L=cfg["num_hidden_layers"], d=d, H=H, KV=KV, hd=hd, qd=H * hd, kvd=KV * hd,
                f=cfg["intermediate_size"], V=cfg["vocab_size"])


def layer_matrix_elements(cfg: dict) -> int:
    s = sizes(cfg)
    return s["d"] * (s["qd"] + 2 * s["kvd"]) + s["qd"] * s["d"] + 3 * s["d"] * s["f"]


def decode_step_bytes(cfg: dict, batch: int, context: int, elem: int) -> int:
    """Bytes a decode step has to read: every weight it uses once (layer
    matrices, output matrix, norm vectors in 32-bit, one embedding row per
    request) and the keys and values of the live requests."""
    s = sizes(cfg)
    weights = (s["L"] * layer_matrix_elements(cfg) + s["V"] * s["d"] + batch * s["d"]) * elem
    vectors = (2 * s["L"] + 1) * s["d"] * 4
    cache = batch * context * s["L"] * 2 * s["kvd"] * elem
    return weights + vectors + cache


def prefill_flops(cfg: dict, tokens: int, logit_rows: int = 1) -> float:
    """Multiply-adds times two of one whole prompt: the layer matrices for
    every token, causal attention (scores and values), the output matrix for
    the wanted rows."""
    s = sizes(cfg)
    gemm = 2.0 * tokens * s["L"] * layer_matrix_elements(cfg)
    attn = 4.0 * s["L"] * s["H"] * s["hd"] * tokens * (tokens + 1) / 2.0
    head = 2.0 * logit_rows * s["d"] * s["V"]
    return gemm + attn + head


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


def measure_decode(engine: Engine, batch: int, context_end: int, steps: int, warmup: int):
    """Decode ``warmup`` untimed and then ``steps`` timed steps of ``batch``
    requests, ending at ``context_end`` tokens each; greedy sampling on the
    device, each step's tokens fed into the next.  Returns (ms per step, mean
    context length during the timed steps)."""
    start = context_end - steps - warmup
    if start < 1:
        raise ValueError("context too short for the steps asked for")
    rids, toks = fill_context(engine, batch, start)
    zeros = [0.0] * batch
    ahead = engine.can_sample_ahead([StepEntry(r, [t], [0]) for r, t in zip(rids, toks)])

    def run(k):
        """k steps, each fed with the ids of the one before.  Where the engine can queue a
        step ahead (as its scheduler does), the ids go from step to step on the device and
        are read on the host one step late; every step's ids are read."""
        nonlocal toks
        before = None
        for _ in range(k):
            if not ahead:
                toks = engine.step_sample([StepEntry(r, [t], [0]) for r, t in zip(rids, toks)], zeros, zeros)
                continue
            ids = toks if before is None else [TokenRef(before, i) for i in range(batch)]
            handle = engine.step_sample_ahead([StepEntry(r, [t], [0]) for r, t in zip(rids, ids)], zeros, zeros)
            if before is not None:
                before.tokens()
            before = handle
        if before is not None:
            toks = before.tokens()
    run(warmup)
    _sync()
    t0 = time.perf_counter()
    run(steps)
    _sync()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    for r in rids:
        engine.release(r)
    mean_ctx = context_end - steps / 2.0
    return ms, mean_ctx


def make_engine(cfg: dict, dtype: str, max_tokens: int, seed: int = 0, **opts) -> Engine:
    options = EngineOptions(dtype=dtype, max_tokens=max_tokens, max_requests=max(64, opts.pop("max_requests", 64)),
                            **opts)
    return Engine.from_random(cfg, seed, options)
