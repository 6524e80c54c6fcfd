"""Weights by tensor name.

The model says which tensors it wants (``WeightSpec``: name, shape, role); the
loader looks each up in the checkpoint and moves it to the device.  Everything
that is wrong is reported at once in a single ``WeightError``: tensors the
model wants and the checkpoint lacks, tensors the checkpoint has and the model
does not know, and tensors whose shape differs.  The reference checks element
counts only and one tensor at a time (backend/model.cu:510-519, :873-892);
here the full shape is checked.

What is kept in which dtype:

* role "matrix" (projection matrices, embedding tables): the engine's compute
  dtype.  In a bfloat16 engine a matrix stored as BF16 is taken as it is and
  one stored as F32 or F16 is rounded to nearest even once, at load; in a
  float32 engine every matrix is widened to float32.
* role "vector" (norm weights and other per-channel parameters): float32
  always; widening BF16 or F16 is exact, and a vector stored in 32-bit stays so.
* role "table": integer tables, int32.

The reference uploads F32 only and refuses every other dtype
(engine/engine.go:140-141).
"""

from __future__ import annotations

import fnmatch
from typing import Dict, Iterable, List, Sequence

import torch

from ..parts.spec import WeightSpec
from .safetensors_io import Checkpoint

# Buffers that old exports carry and no model reads.
DEFAULT_IGNORED = ("*.rotary_emb.inv_freq", "*.attention.masked_bias", "*.attn.bias")

_FLOAT_FILE_DTYPES = ("F64", "F32", "F16", "BF16")
_INT_FILE_DTYPES = ("I64", "I32", "I16", "I8", "U8")


class WeightError(ValueError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected``,
    ``wrong_shape`` ((name, found, wanted) triples) and ``wrong_dtype`` hold
    the details that the message lists."""

    def __init__(self, where, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"{where}: the checkpoint does not fit the model"]

        def some(items, fmt):
            shown = [fmt(i) for i in items[:12]]
            if len(items) > 12:
                shown.append(f"... and {len(items) - 12} more")
            return shown

        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}):")
            lines += ["    " + s for s in some(self.missing, str)]
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}):")
            lines += ["    " + s for s in some(self.unexpected, str)]
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}):")
            lines += ["    " + s for s in some(
                self.wrong_shape,
                lambda t: f"{t[0]}: checkpoint has {list(t[1])}, model wants {list(t[2])}")]
        if self.wrong_dtype:
            lines.append(f"  wrong dtypes ({len(self.wrong_dtype)}):")
            lines += ["    " + s for s in some(
                self.wrong_dtype, lambda t: f"{t[0]}: {t[1]} cannot be used as a {t[2]}")]
        super().__init__("\n".join(lines))


def merge_specs(specs: Iterable[WeightSpec]) -> List[WeightSpec]:
    """Two parts may want the same tensor (a head tied to the embedding); the
    wishes must then agree."""
    seen: Dict[str, WeightSpec] = {}
    for s in specs:
        if s.name in seen:
            if seen[s.name].shape != tuple(s.shape) or seen[s.name].role != s.role:
                raise ValueError(
                    f"tensor {s.name!r} is wanted twice with different shapes or roles: "
                    f"{seen[s.name]} and {s}")
        else:
            seen[s.name] = WeightSpec(s.name, tuple(s.shape), s.role)
    return list(seen.values())


def target_dtype(role: str, compute_dtype: torch.dtype) -> torch.dtype:
    if role == "matrix":
        return compute_dtype
    if role == "vector":
        return torch.float32
    if role == "table":
        return torch.int32
    raise ValueError(f"unknown weight role {role!r}")


def check_checkpoint(ckpt: Checkpoint, specs: Sequence[WeightSpec], where: str,
                     ignored: Sequence[str] = DEFAULT_IGNORED,
                     optional: Sequence[str] = ()):
    """Raise one WeightError for everything that does not fit."""
    wanted = {s.name: s for s in specs}
    missing = [n for n in wanted if n not in ckpt.entries]
    unexpected = [
        n for n in ckpt.names()
        if n not in wanted and n not in optional
        and not any(fnmatch.fnmatchcase(n, pat) for pat in ignored)]
    wrong_shape, wrong_dtype = [], []
    for n, s in wanted.items():
        e = ckpt.entries.get(n)
        if e is None:
            continue
        if tuple(e.shape) != tuple(s.shape):
            wrong_shape.append((n, tuple(e.shape), tuple(s.shape)))
        ok = _INT_FILE_DTYPES if s.role == "table" else _FLOAT_FILE_DTYPES
        if e.dtype not in ok:
            wrong_dtype.append((n, e.dtype, s.role))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(where, sorted(missing), unexpected, wrong_shape, wrong_dtype)


def load_weights(path: str, specs: Iterable[WeightSpec], compute_dtype: torch.dtype,
                 device, ignored: Sequence[str] = DEFAULT_IGNORED,
                 optional: Sequence[str] = ()) -> Dict[str, torch.Tensor]:
    """Read every wanted tensor from the model folder (or file) ``path`` and
    return ``name -> tensor`` on ``device`` in the dtype its role asks for."""
    specs = merge_specs(specs)
    out: Dict[str, torch.Tensor] = {}
    with Checkpoint(path) as ckpt:
        check_checkpoint(ckpt, specs, path, ignored, optional)
        for s in specs:
            src = ckpt.read(s.name)
            dst = target_dtype(s.role, compute_dtype)
            if src.dtype == dst:
                t = src.to(device, copy=True)
            elif src.dtype in (torch.float64,) and dst != torch.float64:
                t = src.to(dst).to(device)
            else:
                # Move first, convert on the device: float -> bfloat16 rounds to
                # nearest even, widening is exact.
                t = src.to(device).to(dst)
            out[s.name] = t.contiguous()
    return out
