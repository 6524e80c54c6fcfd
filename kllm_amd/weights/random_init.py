"""Random-weights mode: a model folder, or tensors in memory, from a
configuration and a seed.

Distributions follow the reference's test-model generator
(tools/make_test_model.py:59-80): matrices and embedding tables are
``std * z``, norm weights ``1 + norm_std * z`` with z of mean 0 and variance 1.

The generator is counter-based: element i of a tensor is a function of (seed,
tensor name, i) alone, made of 32-bit integer mixing and one exact
integer-to-float conversion, with no transcendental function.  A tensor's
values therefore do not depend on which other tensors the model has, on the
order in which they are made, on how the work is cut into pieces, or on
whether the CPU or the GPU computes them: the engine draws a model of any
size directly in device memory, and a test can draw the same tensors on the
CPU for the plain implementation.  z is the sum of eight uniform 16-bit
numbers, centred and scaled to variance 1 (within 4.9 standard deviations;
close to normal, which is all that random test weights need).
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

_M32 = 0xFFFFFFFF
_CHUNK = 1 << 22        # elements drawn at a time (bounds the temporaries)


def _tensor_key(seed: int, name: str):
    """Two 32-bit words that stand for (seed, tensor name)."""
    h = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    return int.from_bytes(h[:4], "little"), int.from_bytes(h[4:8], "little")


def _mul32(x: torch.Tensor, c: int) -> torch.Tensor:
    """(x * c) mod 2^32 for int64 tensors holding 32-bit values, without ever
    leaving 63 bits (so that no device's overflow behaviour matters)."""
    lo = (x & 0xFFFF) * c
    hi = (((x >> 16) * c) & 0xFFFF) << 16
    return (lo + hi) & _M32


def _mix32(x: torch.Tensor) -> torch.Tensor:
    """A 32-bit finalizer of the multiply-xorshift kind (two multiplications,
    three shifts): every input bit reaches every output bit."""
    x = x ^ (x >> 16)
    x = _mul32(x, 0x7FEB352D)
    x = x ^ (x >> 15)
    x = _mul32(x, 0x846CA68B)
    return x ^ (x >> 16)


def unit_variates(seed: int, name: str, start: int, count: int, device="cpu") -> torch.Tensor:
    """z[start : start + count] of the tensor ``name`` as float32 on ``device``."""
    k0, k1 = _tensor_key(seed, name)
    i = torch.arange(start, start + count, dtype=torch.int64, device=device)
    state = _mix32((i & _M32) ^ k0)
    state = _mix32(state ^ k1 ^ _mul32((i >> 32) & _M32, 0x9E3779B1))
    total = torch.zeros_like(state)
    for j in range(4):
        u = _mix32((state + ((j + 1) * 0x9E3779B9 & _M32)) & _M32)
        total += (u & 0xFFFF) + (u >> 16)
    # eight uniforms on {0..65535}: mean 8 * 32767.5, variance 8 * (65536^2 - 1) / 12
    z = (total - 262140).to(torch.float32)
    return z * (1.0 / 53509.61)             # sqrt(8 * (65536^2 - 1) / 12) = 53509.61...


def random_tensor(spec: WeightSpec, seed: int, dtype: torch.dtype, std=0.02, norm_std=0.02,
                  device="cpu") -> torch.Tensor:
    """The seeded value of one tensor, computed on ``device`` in float32 and
    rounded to ``dtype`` there."""
    if spec.role == "table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    numel = 1
    for d in spec.shape:
        numel *= int(d)
    out = torch.empty(numel, dtype=dtype, device=device)
    for a in range(0, numel, _CHUNK):
        n = min(_CHUNK, numel - a)
        z = unit_variates(seed, spec.name, a, n, device)
        out[a:a + n] = (1.0 + norm_std * z if spec.role == "vector" else std * z).to(dtype)
    return out.view(*spec.shape)


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
