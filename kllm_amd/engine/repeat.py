"""Layers that are alike are walked through once a step.

A step whose launches are recorded as commands (``kllm_amd.kernels.stream_scope`` with
``record``) spends most of its host time in the parts: every layer checks its shapes, asks
for its scratch buffers and writes its half dozen commands.  Layers with the same
description issue the same commands, each with the addresses of its own tensors.  So, for
every kind of layer in the running order, the first run of a step is recorded as ever, the
second is recorded too and compared with it word by word: each word that differs, or that
points into a tensor of the first run's layer, must be the address of the tensor that the
second run's layer holds under the same name (same attribute path, same offset into it).
If that explains the second run completely, the runs after it are not walked through any
more: their commands are the first run's with the addresses of their own tensors.  If
anything does not fit (a part launched past the recording, a word that no tensor explains,
scratch buffers that alternate between layers, a buffer that grew), the step goes on as if
this module were not there.

What a layer's tensors are is found by looking: every tensor reachable from the block (its
parts, their attributes, lists and dicts in them), from the norm of the next layer where the
block is handed one, and the tensors of the run's cache view.  A part that *replaces* a
tensor after ``bind`` (tensors that appear later are found) calls
``Runtime.tensors_changed()``.

Nothing here knows a part, a kernel or an architecture.
"""

from __future__ import annotations

import copy
import dataclasses
from bisect import bisect_right
from typing import Any, Dict, List, Optional

import numpy as np
import torch

from .. import kernels as K
from ..parts.base import Part, Runtime, Workspace
from ..parts.spec import LayerSpec, PartSpec


def _alike(obj) -> Any:
    """A hashable that is equal for two descriptions that differ in tensor names only."""
    if isinstance(obj, PartSpec):
        return ("part", obj.kind, tuple(sorted((k, _alike(v)) for k, v in obj.params.items() if k != "names")))
    if isinstance(obj, LayerSpec):
        return ("layer",) + tuple(_alike(getattr(obj, f.name)) for f in dataclasses.fields(obj))
    if isinstance(obj, dict):
        return ("dict",) + tuple(sorted((str(k), _alike(v)) for k, v in obj.items()))
    if isinstance(obj, (list, tuple)):
        return ("seq",) + tuple(_alike(v) for v in obj)
    if obj is None or isinstance(obj, (bool, int, float, str)):
        return obj
    return ("object", id(obj))               # equal to itself only


_OPAQUE = (Runtime, Workspace, PartSpec, LayerSpec, type, torch.dtype, torch.device)


def _walk(obj, path, parts, tensors, seen, depth=0):
    """Every part and tensor reachable from ``obj``: path -> part, path -> tensor."""
    if isinstance(obj, torch.Tensor):
        tensors[path] = obj
        return
    if obj is None or isinstance(obj, (bool, int, float, str, bytes)) or isinstance(obj, _OPAQUE) or depth > 8:
        return
    if isinstance(obj, (list, tuple)):
        for j, v in enumerate(obj):
            _walk(v, path + (j,), parts, tensors, seen, depth + 1)
        return
    if isinstance(obj, dict):
        for k, v in obj.items():
            _walk(v, path + (repr(k),), parts, tensors, seen, depth + 1)
        return
    if callable(obj) and not isinstance(obj, Part):
        return
    if id(obj) in seen or not hasattr(obj, "__dict__"):
        return
    seen.add(id(obj))
    if isinstance(obj, Part):
        parts[path] = obj
    for k, v in vars(obj).items():
        _walk(v, path + (k,), parts, tensors, seen, depth + 1)


def _extent(t: torch.Tensor) -> int:
    if t.numel() == 0:
        return 0
    return (sum((n - 1) * s for n, s in zip(t.shape, t.stride())) + 1) * t.element_size()


class _Names:
    """What one run of the schedule may name: its parts and its tensors by path, and the
    tensors' addresses in order."""

    def __init__(self, block, next_norm):
        self.parts: Dict[tuple, Part] = {}
        self.tensors: Dict[tuple, torch.Tensor] = {}
        seen = set()
        _walk(block, ("b",), self.parts, self.tensors, seen)
        if next_norm is not None:
            _walk(next_norm, ("n",), self.parts, self.tensors, seen)     # (nothing new if the layer follows itself)
        self.path_of = {id(p): path for path, p in reversed(list(self.parts.items()))}
        self.address = {path: t.data_ptr() for path, t in self.tensors.items() if t.numel()}
        spans = sorted((a, a + _extent(self.tensors[path]), path) for path, a in self.address.items())
        self.starts = [s[0] for s in spans]
        self.spans = spans
        self.lo = spans[0][0] if spans else 0
        self.hi = max(s[1] for s in spans) if spans else 0

    def find(self, word: int):
        """(path, offset) of the tensor that ``word`` points into, or None."""
        if not self.lo <= word < self.hi:
            return None
        j = bisect_right(self.starts, word)
        while j > 0:                     # (a view and the tensor it is cut from may both be held)
            j -= 1
            a, end, path = self.spans[j]
            if a <= word < end:
                return path, word - a
        return None


def _view_tensors(view) -> Dict[tuple, torch.Tensor]:
    if view is None:
        return {}
    return {("c", k): v for k, v in vars(view).items() if isinstance(v, torch.Tensor) and v.numel()}


class _Unnamed(Exception):
    pass


def _shape(obj, names: _Names):
    """What a block was given or gave back, as a hashable: tensors by address and layout, parts
    by their path among the run's parts (a part that the run cannot name fits nothing)."""
    if isinstance(obj, torch.Tensor):
        return ("t", obj.data_ptr(), tuple(obj.shape), tuple(obj.stride()), obj.dtype)
    if obj is None or isinstance(obj, (bool, int, float, str)):
        return obj
    if isinstance(obj, _OPAQUE):
        raise _Unnamed()
    if isinstance(obj, Part):
        path = names.path_of.get(id(obj))
        if path is None:
            raise _Unnamed()
        return ("p", path)
    if isinstance(obj, (list, tuple)):
        return (type(obj).__name__,) + tuple(_shape(v, names) for v in obj)
    if isinstance(obj, dict):
        return ("d",) + tuple((repr(k), _shape(v, names)) for k, v in obj.items())
    if hasattr(obj, "__dict__"):
        return (type(obj).__name__,) + tuple((k, _shape(v, names)) for k, v in vars(obj).items())
    raise _Unnamed()


def _moved(obj, src: _Names, dst: _Names):
    """``obj`` (made by a run with the parts ``src``) as the run with the parts ``dst`` would
    have made it: the same tensors and numbers, that run's parts."""
    if obj is None or isinstance(obj, (torch.Tensor, bool, int, float, str)):
        return obj
    if isinstance(obj, Part):
        return dst.parts[src.path_of[id(obj)]]
    if isinstance(obj, tuple):
        return tuple(_moved(v, src, dst) for v in obj)
    if isinstance(obj, list):
        return [_moved(v, src, dst) for v in obj]
    if isinstance(obj, dict):
        return {k: _moved(v, src, dst) for k, v in obj.items()}
    out = copy.copy(obj)
    for k, v in vars(obj).items():
        setattr(out, k, _moved(v, src, dst))
    return out


class _Template:
    """A kind of run in one step: the first one's commands, and (once the second one has been
    compared) which of their words are whose tensor's address."""

    def __init__(self, index, run, given, gave, given_shape, gave_shape):
        self.index, self.run = index, run
        self.given, self.gave = given, gave
        self.given_shape, self.gave_shape = given_shape, gave_shape
        self.ready = self.dead = False
        self.chains = False           # the second run was given what the first gave
        self.words = None             # the commands as 64-bit words
        self.at = None                # indices of the words that are addresses
        self.paths: List[tuple] = []  # whose
        self.offsets = None           # and how far into it
        self.repeats = 0


class LayerRepeater:
    """For one model: which runs of the schedule are alike, and what each may name."""

    def __init__(self, model):
        self.model = model
        spec = model.spec
        alike = [_alike(layer) for layer in spec.layers]
        keys = []
        for i, run in enumerate(model.schedule):
            nxt = model.schedule[i + 1].layer if i + 1 < len(model.schedule) else None
            block = model.blocks[run.layer]
            takes = getattr(block, "takes_next_norm", False) and nxt is not None
            cache = model.cache_plan.runs[i]
            keys.append((alike[run.layer], alike[nxt] if takes else None,
                         None if cache is None else (cache[0], cache[2])))
        count: Dict[Any, int] = {}
        for k in keys:
            count[k] = count.get(k, 0) + 1
        self.keys = [k if count[k] >= 3 else None for k in keys]      # two are walked through anyway
        self.worthwhile = any(k is not None for k in self.keys)
        self._names: Dict[int, _Names] = {}
        self._epoch = None
        self.last = None

    def names(self, i) -> _Names:
        epoch = self.model.runtime.tensor_epoch
        if epoch != self._epoch:
            self._names, self._epoch = {}, epoch
        got = self._names.get(i)
        if got is None:
            model = self.model
            block = model.blocks[model.schedule[i].layer]
            nxt = None
            if getattr(block, "takes_next_norm", False) and i + 1 < len(model.schedule):
                after = model.blocks[model.schedule[i + 1].layer]
                nxt = after.first_norm() if hasattr(after, "first_norm") else None
            got = self._names[i] = _Names(block, nxt)
        return got

    def forget(self, i):
        self._names.pop(i, None)

    def step(self, ctx, cache_views) -> Optional["_StepRepeater"]:
        """The repeater of one step, or None where it cannot help (nothing is recorded, or
        the residual stream is tapped layer by layer)."""
        if not self.worthwhile or ctx.taps is not None or not K.recording():
            return None
        self.last = _StepRepeater(self, ctx, cache_views)      # (kept for whoever asks why a step was walked through)
        return self.last


class _StepRepeater:
    def __init__(self, owner: LayerRepeater, ctx, cache_views):
        self.owner, self.ctx, self.views = owner, ctx, cache_views
        self.workspace = ctx.workspace or ctx.runtime.workspace
        self.generation = self.workspace.generation
        self.templates: Dict[Any, _Template] = {}
        self.off = False
        self.stale = None        # (template, index): x and pending are the template's, standing for that run's
        self.repeated = 0
        self.why: List[str] = []  # what ended the repeating, of the step or of a kind of run

    # -- what the model's loop calls
    def run(self, i, x, pending, call):
        """Run i of the schedule: ``call(i, x, pending)`` walks through it; returns what it
        returns, (x, pending), by that call or from the commands of a run like it."""
        key = None if self.off else self.owner.keys[i]
        if key is None:
            x, pending = self.current(x, pending)
            return call(i, x, pending)
        key = (key, type(pending).__name__)
        t = self.templates.get(key)
        if t is not None and t.ready and not t.dead:
            # (the run before this one was of the same kind, and what it gave is what the
            # kind's first run was given: nothing to look at)
            chained = (self.stale is not None and self.stale[0] is t and t.chains
                       and x is t.gave[0] and pending is t.gave[1])
            if not chained:
                x, pending = self.current(x, pending)
            if self._repeat(t, i, x, pending, chained):
                return t.gave
        x, pending = self.current(x, pending)
        if t is not None and (t.ready or t.dead):
            return call(i, x, pending)
        names = self.owner.names(i)
        try:
            given_shape = _shape((x, pending), names)
        except _Unnamed:
            return call(i, x, pending)
        with K.copy_recorded() as copied:
            out = call(i, x, pending)
        if copied.run is None or not copied.whole or self.workspace.generation != self.generation:
            self.off = True              # launches past the recording, or buffers that moved: no more of this
            self.why.append(f"run {i}: " + ("a scratch buffer grew" if self.workspace.generation != self.generation
                                            else "something was launched past the recording"))
            return out
        try:
            gave_shape = _shape(out, names)
        except _Unnamed:
            self.templates[key] = t = t or _Template(i, copied.run, None, None, None, None)
            t.dead = True
            self.why.append(f"run {i}: it gave something that holds a part of another layer, or an object without attributes")
            return out
        if t is None:
            self.templates[key] = _Template(i, copied.run, (x, pending), out, given_shape, gave_shape)
        else:
            self._learn(t, i, copied.run, (x, pending), given_shape, gave_shape)
        return out

    def current(self, x, pending):
        """(x, pending) for code that looks into them: what the last run would have given had
        it been walked through."""
        if self.stale is not None:
            t, i = self.stale
            self.stale = None
            x, pending = _moved((x, pending), self.owner.names(t.index), self.owner.names(i))
        return x, pending

    # -- the second run of a kind
    def _learn(self, t: _Template, j, run, given, given_shape, gave_shape):
        a, b = t.run, run
        if (given_shape != t.given_shape or gave_shape != t.gave_shape or len(a.data) != len(b.data)
                or a.names != b.names or a.patches != b.patches or len(a.data) % 8):
            t.dead = True
            self.why.append(f"runs {t.index} and {j}: " + (
                "they were given other buffers" if given_shape != t.given_shape else
                "they gave other buffers" if gave_shape != t.gave_shape else "they launched other kernels"))
            return
        wa = np.frombuffer(bytes(a.data), dtype=np.uint64)
        wb = np.frombuffer(bytes(b.data), dtype=np.uint64)
        for attempt in range(2):
            na, nb = self.owner.names(t.index), self.owner.names(j)
            found = self._explain(wa, wb, na, nb, self.views[t.index], self.views[j])
            if found is not None:
                break
            if attempt == 0:             # tensors that a part made since its names were looked up
                self.owner.forget(t.index)
                self.owner.forget(j)
        if found is None:
            t.dead = True
            self.why.append(f"runs {t.index} and {j}: their commands differ in a word that no tensor of the layers explains")
            return
        t.words = wa
        t.at = np.array([f[0] for f in found], dtype=np.int64)
        t.paths = [f[1] for f in found]
        t.offsets = np.array([f[2] for f in found], dtype=np.uint64)
        t.chains = given[0] is t.gave[0] and given[1] is t.gave[1]
        t.ready = True

    @staticmethod
    def _explain(wa, wb, na: _Names, nb: _Names, view_a, view_b):
        ca, cb = _view_tensors(view_a), _view_tensors(view_b)
        if set(ca) != set(cb):
            return None
        cache_spans = [(t.data_ptr(), t.data_ptr() + _extent(t), path) for path, t in ca.items()]
        near = (wa != wb) | ((wa >= np.uint64(na.lo)) & (wa < np.uint64(na.hi)))
        found = []
        for idx in np.nonzero(near)[0].tolist():
            word, other = int(wa[idx]), int(wb[idx])
            hit = na.find(word)
            if hit is not None:
                path, off = hit
                if nb.address.get(path, -1) + off != other:
                    return None
                found.append((idx, path, off))
                continue
            for lo, hi, path in cache_spans:
                if lo <= word < hi:
                    if cb[path].data_ptr() + (word - lo) != other:
                        return None
                    found.append((idx, path, word - lo))
                    break
            else:
                if word != other:
                    return None          # a difference that no tensor of the two layers explains
        return found

    # -- every further run
    def _repeat(self, t: _Template, i, x, pending, chained) -> bool:
        if self.workspace.generation != self.generation:
            self.off = True              # a run of another kind made a scratch buffer grow: the first run's addresses are gone
            self.why.append(f"run {i}: a scratch buffer grew")
            return False
        names = self.owner.names(i)
        if names.parts.keys() != self.owner.names(t.index).parts.keys():
            return False
        if not chained:
            try:
                if _shape((x, pending), names) != t.given_shape:
                    return False
            except _Unnamed:
                return False
        view = self.views[i]
        values = []
        for path in t.paths:
            if path[0] == "c":
                tensor = getattr(view, path[1], None)
                if not isinstance(tensor, torch.Tensor):
                    return False
                values.append(tensor.data_ptr())
            else:
                address = names.address.get(path)
                if address is None:              # a tensor that this layer makes when it is first walked through:
                    self.owner.forget(i)         # walked through now, looked up again the next time
                    return False
                values.append(address)
        words = t.words.copy()
        if values:
            words[t.at] = np.array(values, dtype=np.uint64) + t.offsets
        K.add_recorded(words.tobytes(), t.run.names, t.run.patches)
        self.stale = (t, i)
        self.repeated += 1
        return True
