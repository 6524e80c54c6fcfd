"""What a step must read and compute at least, as the model's parts report it, against the
closed form of the Llama layer written out here (the measurement's rooflines rest on it)."""

import torch

import tiny
from kllm_amd.config import config_from_dict, resolve_architecture
from kllm_amd.engine.model import Model
from kllm_amd.parts import Runtime
from kllm_amd.weights import random_weights


def build(cfg, dtype):
    raw = dict(cfg)
    spec = resolve_architecture(raw).build(config_from_dict(raw))
    model = Model(spec, Runtime(device=torch.device("cpu"), dtype=dtype))
    model.bind(random_weights(model.weight_specs(), 1, dtype, "cpu"))
    return model


def closed_form(cfg):
    H, d = cfg["num_attention_heads"], cfg["hidden_size"]
    hd = cfg.get("head_dim") or d // H
    KV = cfg.get("num_key_value_heads") or H
    f, V, L = cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    layer = d * (H * hd + 2 * KV * hd) + H * hd * d + 3 * d * f
    return dict(H=H, d=d, hd=hd, KV=KV, f=f, V=V, L=L, layer=layer)


def test_bytes_and_flops_of_a_step_follow_the_parts():
    for name in ("A", "B", "C"):
        cfg = tiny.CONFIGS[name]
        s = closed_form(cfg)
        for dtype, elem in ((torch.float32, 4), (torch.bfloat16, 2)):
            model = build(cfg, dtype)
            for tokens in (1, 5):
                # every layer matrix and the output matrix once, one embedding row per token, the
                # norms' vectors in 32-bit; a tied output matrix is the embedding's table, read whole
                table = s["V"] * s["d"] * elem
                rows = tokens * s["d"] * elem
                want = s["L"] * s["layer"] * elem + (2 * s["L"] + 1) * s["d"] * 4
                want += table if cfg.get("tie_word_embeddings") else table + rows
                assert model.step_read_bytes(tokens) == want, (name, dtype, tokens)
            T = 37
            keys = T * (T + 1) / 2.0
            want = 2.0 * T * s["L"] * s["layer"] + 4.0 * s["L"] * s["H"] * s["hd"] * keys + 2.0 * 3 * s["d"] * s["V"]
            assert model.step_flops(T, keys, 3) == want, (name, dtype)


def test_a_layer_run_twice_is_read_once_and_computed_twice():
    from kllm_amd.parts import Run
    cfg = tiny.CONFIGS["A"]
    s = closed_form(cfg)
    model = build(cfg, torch.float32)
    once_bytes, once_flops = model.step_read_bytes(1), model.step_flops(1, 10.0, 1)
    model.schedule = [Run(0), Run(1), Run(1)]
    assert model.step_read_bytes(1) == once_bytes
    extra = 2.0 * s["layer"] + 4.0 * s["H"] * s["hd"] * 10.0
    assert model.step_flops(1, 10.0, 1) == once_flops + extra
