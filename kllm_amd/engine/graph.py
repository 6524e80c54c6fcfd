"""Decode steps as HIP graphs.

A decode step of a small model is hundreds of short kernels; launched one by
one from the host they cost more than they run (the reference names launch
overhead as its bound at small scale and graphs as the fix it did not build:
docs/JOURNAL.md:90-101).  A batch of B single tokens is therefore recorded
once -- forward pass and sampling -- and replayed: per step the host fills one
control buffer, copies it, launches the graph and reads B token ids back.

What makes a step replayable: every array a kernel reads lives at a fixed
address (the control buffer's layout depends only on B and on the width of the
block tables, which grows in powers of two), scratch tensors come from a
workspace that belongs to the recording and is never resized, and no launch
dimension depends on a context length.  A recording is made after the same
step has run once eagerly, so the eager run is also its warm-up.  Nothing in a
recording clears memory with a memset node.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import List, Sequence

import torch

from .. import kernels as K
from ..parts.base import Workspace
from . import control


def _bucket(pages: int) -> int:
    b = 8
    while b < pages:
        b *= 2
    return b


class _Recording:
    def __init__(self, engine, batch: int, caps: tuple):
        self.layout = control.layout_for([1] * batch, batch, caps, samples=batch)
        self.control = torch.zeros(self.layout.total, dtype=torch.int32, device=engine.device)
        self.tokens = torch.zeros(batch, dtype=torch.int32, device=engine.device)
        self.workspace = Workspace(engine.device)
        self.graph = None
        self.replays = 0


class DecodeGraphs:
    MAX_RECORDINGS = 64

    def __init__(self, engine):
        self.engine = engine
        self.recordings: "OrderedDict[tuple, _Recording]" = OrderedDict()
        self.captures = 0

    def _run(self, rec: _Recording, lens, pos0):
        eng = self.engine
        starts = list(range(rec.layout.n + 1))
        ctx = control.context(rec.control, rec.layout, eng.runtime, starts, pos0, lens)
        ctx.workspace = rec.workspace
        logits = eng.model.run(ctx, eng._cache_views(ctx))
        temps, uniforms = control.sampling_views(rec.control, rec.layout)
        K.sample(rec.tokens, logits, temps, uniforms)

    def decode(self, entries, temperatures: Sequence[float], uniforms: Sequence[float]) -> List[int]:
        """One token for every entry (each entry is a single decode token)."""
        eng = self.engine
        eng._validate(entries)
        opened, reserved = eng._reserve(entries)
        try:
            rcs, lens, rows, tables = eng._describe(entries)
            batch = len(entries)
            caps = tuple(_bucket(max(len(t) for t in tg)) for tg in tables)
            key = (batch, caps)
            rec = self.recordings.get(key)
            if rec is None:
                rec = _Recording(eng, batch, caps)
                self.recordings[key] = rec
                while len(self.recordings) > self.MAX_RECORDINGS:
                    self.recordings.popitem(last=False)
            else:
                self.recordings.move_to_end(key)
            host = eng._staging(rec.layout.total)
            pos0 = [rc.length for rc in rcs]
            control.fill(host.numpy(), rec.layout, [e.tokens for e in entries], pos0,
                         [rc.slot for rc in rcs], rows, tables, temperatures, uniforms)
            eng._send(host, rec.control, rec.layout.total)
            if rec.graph is None:
                self._run(rec, lens, pos0)              # the step itself, and the warm-up
                out = rec.tokens.tolist()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, capture_error_mode="thread_local"):
                    self._run(rec, lens, pos0)          # recorded, not executed
                rec.graph = graph
                self.captures += 1
            else:
                rec.graph.replay()
                rec.replays += 1
                out = rec.tokens.tolist()
        except Exception:
            eng._undo(opened, reserved)
            raise
        eng._commit(entries)
        return out
