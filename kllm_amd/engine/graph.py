"""Decode steps as HIP graphs.

A decode step of a small model is hundreds of short kernels; launched one by
one from the host they cost more than they run (the reference names launch
overhead as its bound at small scale and graphs as the fix it did not build:
docs/JOURNAL.md:90-101).  A batch of B single tokens is therefore recorded
once -- forward pass and sampling -- and replayed: per step the host fills one
control buffer, copies it, launches the graph and reads B token ids back.

The ids need not be read back before the next step is queued.  A step's ids
stay in ``engine``-wide device memory where the next step's embedding finds
them (an entry names its token as a ``TokenRef`` to the previous step's
result), and the copy to the host is queued between the two graphs; the caller
takes the ids from the ``SampledTokens`` handle when it wants them.  Queued
one step ahead, the device does not wait for the host between steps.

What makes a step replayable: every array a kernel reads lives at a fixed
address (the control buffer's layout depends only on B and on the width of the
block tables, which grows in powers of two), scratch tensors come from a
workspace that belongs to the recording and is never resized, and no launch
dimension depends on a context length.  A recording is made after the same
step has run once eagerly, so the eager run is also its warm-up.  Nothing in a
recording clears memory with a memset node.
"""

from __future__ import annotations

import gc
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


class SampledTokens:
    """The token ids of a sampled step, on their way to the host."""

    def __init__(self, host: torch.Tensor, event: torch.cuda.Event, count: int, logits=None, recording=None):
        self._host, self._event, self.count = host, event, count
        self._ids = None
        self._logits, self._recording = logits, recording
        self._use = recording.uses if recording is not None else 0

    @property
    def logits(self):
        """The step's float32 logits [count, vocab] on the device, what was sampled from.  They
        lie in the recording's own buffer and hold until a step of the same batch size and
        table width is queued again; asked for after that, this raises instead of handing out
        the later step's numbers (clone them before queuing on if they are to be kept)."""
        if self._recording is not None and self._recording.uses != self._use:
            raise RuntimeError("the logits of this step have been overwritten: a step of the same shape was "
                               "queued since; read (or clone) them before queuing the next step")
        return self._logits

    def ready(self) -> bool:
        return self._ids is not None or self._event.query()

    def tokens(self) -> List[int]:
        """Waits for the step and returns its ids."""
        if self._ids is None:
            self._event.synchronize()
            self._ids = self._host[:self.count].tolist()
            self._host = None
        return self._ids


class ReservedStep:
    """A step whose entries are checked and whose pages are reserved, on its way to
    ``Engine._run``: the entries' ids as arrays, where their ids come from on the device
    (or None), and what ``Engine._reserve`` and ``Engine._describe`` returned."""
    __slots__ = ("arrays", "token_ref", "opened", "reserved", "described")

    def __init__(self, arrays, token_ref, opened, reserved, described):
        self.arrays, self.token_ref = arrays, token_ref
        self.opened, self.reserved, self.described = opened, reserved, described


class TokenRef:
    """In place of a token id in a step's entry: "what ``source`` chose at
    ``index``", for a source that is the step sampled last."""
    __slots__ = ("source", "index")

    def __init__(self, source: SampledTokens, index: int):
        self.source, self.index = source, int(index)


class _Recording:
    def __init__(self, engine, batch: int, caps: tuple):
        # the parts' index lists depend on the spans only: the same on every replay
        self.lists = engine.model.step_lists(list(range(batch + 1)), [1] * batch)
        self.layout = control.layout_for([1] * batch, batch, caps, samples=batch, lists=self.lists)
        self.control = torch.zeros(self.layout.total, dtype=torch.int32, device=engine.device)
        self.workspace = Workspace(engine.device)
        self.graph = None
        self.replays = 0
        self.uses = 0            # runs of the step, direct or replayed: each overwrites ``logits``
        self.logits = None


class DecodeGraphs:
    MAX_RECORDINGS = 64

    def __init__(self, engine):
        self.engine = engine
        self.recordings: "OrderedDict[tuple, _Recording]" = OrderedDict()
        self.captures = 0
        # Every recording samples into the same place, so that the next step, whichever
        # recording it is, finds the ids there.
        self.sampled = torch.zeros(max(engine.options.max_graph_batch, 1), dtype=torch.int32,
                                   device=engine.device)
        self.last: "SampledTokens | None" = None
        self.seen: "OrderedDict[tuple, int]" = OrderedDict()   # times a shape was asked for before it had a recording
        self._host_ring = [torch.empty(self.sampled.numel(), dtype=torch.int32, pin_memory=True)
                           for _ in range(4)]
        self._host_owner = [None] * len(self._host_ring)   # the handle that reads from each
        self._host_next = 0

    def _run(self, rec: _Recording, lens, pos0):
        eng = self.engine
        starts = list(range(rec.layout.n + 1))
        ctx = control.context(rec.control, rec.layout, eng.runtime, starts, pos0, lens)
        ctx.workspace = rec.workspace
        ctx.sampled = self.sampled
        with K.stream_scope(record=eng.records_launches):   # the capture's stream while recording a graph
            logits = eng.model.run(ctx, eng._cache_views(ctx))
            rec.logits = logits
            temps, uniforms = control.sampling_views(rec.control, rec.layout)
            K.sample(self.sampled[:rec.layout.n], logits, temps, uniforms)

    def decode(self, entries, temperatures: Sequence[float], uniforms: Sequence[float],
               wait_for_uses: bool = False):
        """One token for every entry (each entry is a single decode token, given
        as an id or as a TokenRef to the step sampled last).  Returns at once;
        the ids are read from the handle.  ``wait_for_uses``: a shape without a recording
        that was asked for fewer than ``EngineOptions.graph_after_steps`` times is counted and
        left to the caller: a ``ReservedStep`` is returned, the entries checked and their pages
        reserved, which the caller runs (``Engine._run``) or undoes.  Recording costs two runs of
        the step and the instantiation, which a shape that comes by a few times (a batch that
        shrinks as its requests end) never earns back."""
        eng = self.engine
        token_from, tokens = [], []
        for e in entries:
            t = e.tokens[0]
            if isinstance(t, TokenRef):
                if t.source is not self.last or not 0 <= t.index < t.source.count:
                    raise ValueError("a TokenRef must name a token of the step that was sampled last")
                token_from.append(t.index)
                tokens.append([0])
            else:
                token_from.append(-1)
                tokens.append([int(t)])
        arrays = eng._validate(entries)
        opened, reserved = eng._reserve(entries)
        try:
            described = rcs, lens, rows, tables = eng._describe(entries)
            batch = len(entries)
            caps = tuple(_bucket(max(len(t) for t in tg)) for tg in tables)
            key = (batch, caps)
            rec = self.recordings.get(key)
            if rec is None and wait_for_uses:
                uses = self.seen.get(key, 0) + 1
                if uses < eng.options.graph_after_steps:
                    self.seen[key] = uses
                    self.seen.move_to_end(key)
                    while len(self.seen) > 4 * self.MAX_RECORDINGS:
                        self.seen.popitem(last=False)
                    # (what was checked and reserved goes with the step, not back)
                    return ReservedStep(arrays, token_from if max(token_from) >= 0 else None, opened, reserved, described)
                self.seen.pop(key, None)
            if rec is None:
                rec = _Recording(eng, batch, caps)
                self.recordings[key] = rec
                while len(self.recordings) > self.MAX_RECORDINGS:
                    self.recordings.popitem(last=False)
            else:
                self.recordings.move_to_end(key)
            host = eng._staging(rec.layout.total)
            pos0 = [rc.length for rc in rcs]
            control.fill(host.numpy(), rec.layout, tokens, pos0, [rc.slot for rc in rcs], rows, tables,
                         temperatures, uniforms, token_from, lists=rec.lists)
            eng._send(host, rec.control, rec.layout.total)
            rec.uses += 1
            if rec.graph is None:
                self._run(rec, lens, pos0)              # the step itself, and the warm-up
                out = self._read_back(batch, rec)
                out.tokens()                            # before the capture's second run of the kernels
                graph = torch.cuda.CUDAGraph()
                # No collection of garbage while recording: it may destroy the recordings of an
                # engine that is no longer used, which HIP refuses on a thread that records, and
                # the error leaves a destructor and ends the process.
                collecting = gc.isenabled()
                gc.disable()
                try:
                    with torch.cuda.graph(graph, capture_error_mode="thread_local"):
                        self._run(rec, lens, pos0)      # recorded, not executed
                finally:
                    if collecting:
                        gc.enable()
                rec.graph = graph
                self.captures += 1
            else:
                rec.graph.replay()
                rec.replays += 1
                out = self._read_back(batch, rec)
        except Exception:
            eng._undo(opened, reserved)
            raise
        eng._commit(entries)
        self.last = out
        return out

    def handle(self, count: int, logits) -> SampledTokens:
        """The handle of a sampled step that was not one of this class's recordings (its
        ``count`` ids lie in ``sampled``): the copy to the host queued behind it, and the step
        remembered as the one sampled last."""
        out = self._read_back(count, None, logits)
        if count:
            self.last = out
        return out

    def _read_back(self, batch: int, rec, logits=None) -> SampledTokens:
        """Queue the copy of the sampled ids to the host behind the step."""
        i = self._host_next
        self._host_next = (i + 1) % len(self._host_ring)
        if self._host_owner[i] is not None:
            self._host_owner[i].tokens()                # an old handle nobody has read yet: read it now
        host = self._host_ring[i]
        if batch:
            host[:batch].copy_(self.sampled[:batch], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        self._host_owner[i] = SampledTokens(host, event, batch, rec.logits if rec is not None else logits, rec)
        return self._host_owner[i]
