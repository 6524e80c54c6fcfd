"""Random-weights mode: a model folder from a configuration and a seed.

Distributions follow the reference's test-model generator
(tools/make_test_model.py:59-80): matrices and embedding tables are
``std * N(0, 1)``, norm weights ``1 + norm_std * N(0, 1)``.  Each tensor is
drawn from a generator seeded by (seed, tensor name), so a tensor's values do
not depend on which other tensors the model has or in which order they are
made.
"""

from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterable

import torch

from ..config.base import ModelConfig
from ..parts.spec import WeightSpec
from .loader import merge_specs, target_dtype
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def random_tensor(spec: WeightSpec, seed: int, dtype: torch.dtype, std=0.02, norm_std=0.02,
                  device="cpu") -> torch.Tensor:
    """The seeded value of one tensor.  Values are drawn in float32 on the CPU
    (so they are the same everywhere) and then rounded to ``dtype``."""
    g = torch.Generator(device="cpu").manual_seed(_tensor_seed(seed, spec.name))
    if spec.role == "table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    r = torch.randn(spec.shape, generator=g, dtype=torch.float32)
    if spec.role == "vector":
        r = 1.0 + norm_std * r
    else:
        r = std * r
    return r.to(device).to(dtype)


def random_weights(specs: Iterable[WeightSpec], seed: int, compute_dtype: torch.dtype,
                   device="cpu", std=0.02, norm_std=0.02) -> Dict[str, torch.Tensor]:
    """``name -> tensor`` for every wanted tensor, in the dtype its role asks
    for, without touching the disk."""
    return {s.name: random_tensor(s, seed, target_dtype(s.role, compute_dtype), std, norm_std,
                                  device)
            for s in merge_specs(specs)}


def write_random_model(out_dir: str, config, seed: int, dtype: str = "float32",
                       std=0.02, norm_std=0.02) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a typed
    configuration or a config.json dict) with seeded random weights stored as
    ``dtype`` ("float32" or "bfloat16").  Returns ``out_dir``."""
    from ..config.registry import config_from_dict, resolve_architecture
    from ..engine.model import collect_weight_specs

    if isinstance(config, ModelConfig):
        raw = config.to_dict()
    else:
        raw = dict(config)
    cfg = config_from_dict(raw, where="config")
    store = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    spec = resolve_architecture(raw).build(cfg)
    specs = collect_weight_specs(spec)
    tensors = {}
    for s in specs:
        t = random_tensor(s, seed, torch.float32, std, norm_std)
        tensors[s.name] = t.to(torch.int32) if s.role == "table" else t.to(store)
    os.makedirs(out_dir, exist_ok=True)
    raw_out = cfg.to_dict()
    raw_out["torch_dtype"] = dtype
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw_out, f, indent=2)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed})
    return out_dir
