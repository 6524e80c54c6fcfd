"""The small per-step arrays that cross from the host to the device.

Everything a step needs besides weights and cache -- token ids, positions,
which span a token belongs to, span offsets, state slots, the rows whose
logits are wanted, one block table per cache group, the sampling parameters,
and the index lists that parts ask for (how a mixer tiles the spans) -- is packed into one int32 buffer and sent with a single copy
(the reference sends five, backend/model.cu:1048-1054).  The layout is fixed
by (tokens, spans, wanted rows, pages per table), so a recorded HIP graph
finds every array at the same address on every replay.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from ..parts.base import StepContext


def _pad4(n: int) -> int:
    return (n + 3) // 4 * 4   # sections start 16-byte aligned


@dataclass(frozen=True)
class ControlLayout:
    n: int                 # tokens
    spans: int
    rows: int              # wanted logit rows
    pages: tuple           # table width per cache group
    samples: int = 0       # rows of sampling parameters (temperature, uniform)
    lists: tuple = ()      # (name, count) of the index lists that parts asked for
    refs: int = 0          # tokens that may take their id from the step sampled last (0 or n)

    def sections(self):
        s = [("token_ids", self.n), ("positions", self.n), ("span_of_token", self.n),
             ("span_start", self.spans + 1), ("span_pos", self.spans), ("slots", self.spans),
             ("logit_rows", max(self.rows, 1))]
        s += [(f"table{g}", self.spans * m) for g, m in enumerate(self.pages)]
        s += [("temperature", self.samples), ("uniform", self.samples), ("token_from", self.samples)]
        s += [("token_ref", self.refs)]
        s += [("list:" + name, count) for name, count in self.lists]
        return s

    def offsets(self):
        out, at = {}, 0
        for name, count in self.sections():
            out[name] = (at, count)
            at += _pad4(max(count, 1))
        return out, at

    @property
    def total(self) -> int:
        return self.offsets()[1]


def layout_for(lens: Sequence[int], rows: int, pages: tuple, samples: int = 0, lists=None,
               refs: bool = False) -> ControlLayout:
    """``lists``: name -> list of ints, the parts' index lists for these spans
    (only their lengths enter the layout).  ``refs``: the step has tokens whose ids are taken
    from the step sampled last (any step, not only one of single decode tokens, whose
    ``token_from`` has one entry per sample)."""
    sizes = tuple((name, len(v)) for name, v in (lists or {}).items())
    return ControlLayout(sum(lens), len(lens), rows, tuple(pages), samples, sizes, sum(lens) if refs else 0)


def fill(host: np.ndarray, layout: ControlLayout, tokens: Sequence[Sequence[int]],
         pos0: Sequence[int], slots: Sequence[int], rows: Sequence[int],
         tables: Sequence[Sequence[Sequence[int]]], temperatures=None, uniforms=None,
         token_from=None, lists=None, token_ref=None):
    """Write one step into ``host`` (int32).  ``tables[g][s]`` is span s's
    table in group g.  ``token_from[t] >= 0`` (sampled steps only) says that
    token t's id is not ``tokens`` but the id the last sampled step left on
    the device at that index; ``token_ref`` says the same per token for a layout with
    ``refs``."""
    offs, _ = layout.offsets()

    def sec(name):
        a, c = offs[name]
        return host[a:a + c]
    tok, posv, sot = sec("token_ids"), sec("positions"), sec("span_of_token")
    starts, at = [0], 0
    for s, t in enumerate(tokens):
        b = at + len(t)
        tok[at:b] = np.asarray(t, dtype=np.int32)
        posv[at:b] = np.arange(pos0[s], pos0[s] + len(t), dtype=np.int32)
        sot[at:b] = s
        at = b
        starts.append(at)
    sec("span_start")[:] = starts
    sec("span_pos")[:] = pos0
    sec("slots")[:] = slots
    if layout.rows:
        sec("logit_rows")[:] = rows
    for g, width in enumerate(layout.pages):
        bt = sec(f"table{g}").reshape(layout.spans, width)
        bt.fill(-1)
        for s, t in enumerate(tables[g]):
            bt[s, :len(t)] = t
    lists = lists or {}
    for name, count in layout.lists:
        values = lists.get(name)
        if values is None or len(values) != count:
            raise ValueError(f"control layout does not fit the step's list {name!r}")
        if count:
            sec("list:" + name)[:] = np.asarray(values, dtype=np.int32)
    if layout.samples:
        sec("temperature").view(np.float32)[:] = np.asarray(temperatures, dtype=np.float32)
        sec("uniform").view(np.float32)[:] = np.asarray(uniforms, dtype=np.float32)
        sec("token_from")[:] = -1 if token_from is None else np.asarray(token_from, dtype=np.int32)
    if layout.refs:
        sec("token_ref")[:] = -1 if token_ref is None else np.asarray(token_ref, dtype=np.int32)
    return starts


def context(dev: torch.Tensor, layout: ControlLayout, runtime, starts, pos0, lens) -> StepContext:
    """The step context whose arrays are views of the device copy ``dev``."""
    offs, _ = layout.offsets()

    def sec(name):
        a, c = offs[name]
        return dev[a:a + c]
    return StepContext(
        n=layout.n, n_spans=layout.spans,
        token_ids=sec("token_ids"), positions=sec("positions"), span_of_token=sec("span_of_token"),
        span_start=sec("span_start"), span_pos=sec("span_pos"), slots=sec("slots"),
        logit_rows=sec("logit_rows") if layout.rows else None,
        h_span_start=list(starts), h_span_pos=list(pos0), h_span_len=list(lens),
        block_tables=[sec(f"table{g}").view(layout.spans, m) for g, m in enumerate(layout.pages)],
        runtime=runtime, max_span_len=max(lens), all_decode=all(l == 1 for l in lens),
        lists={name: sec("list:" + name) for name, _ in layout.lists},
        token_from=(sec("token_ref") if layout.refs
                    else sec("token_from") if layout.samples and layout.samples == layout.n else None))


def sampling_views(dev: torch.Tensor, layout: ControlLayout):
    offs, _ = layout.offsets()
    (a, c), (b, _) = offs["temperature"], offs["uniform"]
    return dev[a:a + c].view(torch.float32), dev[b:b + c].view(torch.float32)
