"""Tiny configurations and helpers shared by the tests.

A and B are the two tiny Llama configurations that differ in every size and
option: layers, width, heads and groups (GQA / MQA), head size, feed-forward
width, vocabulary, rotary base, context, eps, tying.  C is multi-head
(KV = H) with a head size that is not hidden/heads, a width and a vocabulary
that are not powers of two.  D has sizes the fast kernels refuse (they must
fall back, never give a wrong result).  E has many heads and room for long
prompts.  F has few heads of 128 and room for long prompts.  R is the reference's own tiny model
(tools/make_test_model.py:47-100).
"""

import json
import os

import torch

import plain_llama as P


def _cfg(**kw):
    base = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu"}
    base.update(kw)
    return base


CONFIGS = {
    "A": _cfg(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
              head_dim=16, intermediate_size=176, vocab_size=256, rope_theta=10000.0,
              max_position_embeddings=128, rms_norm_eps=1e-5, tie_word_embeddings=False),
    "B": _cfg(num_hidden_layers=3, hidden_size=96, num_attention_heads=3, num_key_value_heads=1,
              head_dim=32, intermediate_size=256, vocab_size=320, rope_theta=500000.0,
              max_position_embeddings=256, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "C": _cfg(num_hidden_layers=1, hidden_size=88, num_attention_heads=5, num_key_value_heads=5,
              head_dim=48, intermediate_size=120, vocab_size=131, rope_theta=1000.0,
              max_position_embeddings=512, rms_norm_eps=1e-4, tie_word_embeddings=False),
    # sizes the fast kernels do not take: a width that is no multiple of 8, a head size
    # with no prompt kernel, an odd vocabulary, no num_key_value_heads key (defaults to heads)
    "D": _cfg(num_hidden_layers=2, hidden_size=100, num_attention_heads=5, head_dim=80,
              intermediate_size=172, vocab_size=257, rope_theta=20000.0,
              max_position_embeddings=64, rms_norm_eps=1e-3, tie_word_embeddings=True),
    # many heads and a long context: prompts of this model fill the GPU with query blocks
    "E": _cfg(num_hidden_layers=1, hidden_size=64, num_attention_heads=16, num_key_value_heads=4,
              head_dim=32, intermediate_size=96, vocab_size=96, rope_theta=10000.0,
              max_position_embeddings=4096, rms_norm_eps=1e-5, tie_word_embeddings=False),
    # few heads of 128 and a long context: portions of a prompt far into it share out a block's
    # keys over several workgroups
    "F": _cfg(num_hidden_layers=2, hidden_size=72, num_attention_heads=3, num_key_value_heads=1,
              head_dim=128, intermediate_size=80, vocab_size=101, rope_theta=100000.0,
              max_position_embeddings=4096, rms_norm_eps=1e-5, tie_word_embeddings=True),
    "R": _cfg(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2,
              head_dim=16, intermediate_size=128, vocab_size=512, rope_theta=10000.0,
              max_position_embeddings=256, rms_norm_eps=1e-6, tie_word_embeddings=False,
              bos_token_id=1, eos_token_id=2),
}

# The reference's own test prompts for its tiny model (tools/prompts_tiny.txt:1-5).
REFERENCE_PROMPTS = [
    [1, 17, 42, 100, 7],
    [1, 300, 5, 250, 33, 90, 411],
    [1, 9],
    [1, 507, 3, 44, 205, 66, 137, 8, 259, 10, 311, 12],
    [1, 128, 256, 384, 500, 461, 320, 77, 15],
]


def write_model(out_dir, cfg, seed, store="float32", weights=None, std=0.05, norm_std=0.1):
    """A model folder written with the safetensors library (not with the
    package's own writer).  Weights are wider than a checkpoint's usual 0.02 so
    that attention and the norms matter in the logits."""
    from safetensors.torch import save_file
    w = weights if weights is not None else P.random_weights(cfg, seed, std=std, norm_std=norm_std)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[store]
    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.to(dt).contiguous() for k, v in w.items()},
              os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    return out_dir


def read_weights(model_dir, as_stored_in=None):
    """The folder's weights as float32 CPU tensors; with as_stored_in="bfloat16"
    every matrix is rounded to bfloat16 first, as a bfloat16 engine keeps it
    (vectors stay in 32-bit)."""
    from safetensors.torch import load_file
    w = load_file(os.path.join(model_dir, "model.safetensors"))
    out = {}
    for k, v in w.items():
        v = v.float()
        if as_stored_in == "bfloat16" and v.dim() > 1:
            v = v.to(torch.bfloat16).float()
        out[k] = v
    return out


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()


# Tolerances on logits (absolute).  float32: the reference's own bound on
# logits is 1e-3 and on hidden states 1e-4 (engine/e2e/e2e_test.go:21-24);
# ours is a hundred times tighter (measured on these configurations: at most
# 7e-7, the same as the plain float32 implementation is from float64).
# bfloat16: eight mantissa bits on activations of size ~1.  Measured against the
# plain implementation in float64 over the 48 random traces of
# test_gpu_random_traces.py (30,291 positions of these configurations, every
# way of cutting): mean 5.6e-3, 99.9 % below 1.3e-2, at most 1.76e-2 (a whole
# prompt of configuration B), and the same figures to three digits whether the
# RMS norm runs as a kernel of its own or is folded into the products around it
# (rows times the norm's weight rounded to bfloat16 before the row scale instead
# of after it: mean 5.615e-3 against 5.624e-3, 99.9 % 1.325e-2 against 1.343e-2,
# the same maximum).  The bound is that of the random traces.
TOL = {"float32": 1e-5, "bfloat16": 3e-2}

# The same at the layer sizes of TinyLlama 1.1B, Llama-3 8B and Llama-2 7B
# (tests/test_gpu_sizes.py; weights N(0, 0.02), logits of size 1 to 6), fixed by
# measurement on an MI355X over all ways of cutting: float32 at most 2.0e-5
# (width 2048) and 4.0e-5 (width 4096) from the plain implementation in float32
# -- the reference holds 1e-3 on logits at this size (engine/e2e/e2e_test.go:23);
# bfloat16 at most 4.3e-2 (width 2048) and 6.6e-2 (width 4096).  TOL_SIZES_STORED
# is against the plain implementation rounding to bfloat16 wherever the engine
# stores an activation: measured at most 3.9e-2.
TOL_SIZES = {"float32": 1e-4, "bfloat16": 1e-1}
TOL_SIZES_STORED = 6e-2
