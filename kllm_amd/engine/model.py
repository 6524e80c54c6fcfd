"""A model: parts instantiated from a ModelSpec, bound to weights, and run over
one step's tokens.

The model owns no request state.  It says what its runs need kept between
steps (``cache_plan``), the engine allocates that and hands a view per run to
``run``.  The order of the runs is the spec's ``schedule``; nothing here
assumes that it is 0..L-1.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from .. import kernels as K
from ..parts.base import Runtime, call_part, make_part
from ..parts.spec import CacheNeed, ModelSpec, PartSpec, WeightSpec


@dataclass
class CacheGroupPlan:
    """Runs with the same needs: ``entries`` of them keep a cache of their own."""
    need: CacheNeed
    entries: int = 0


@dataclass
class CachePlan:
    groups: List[CacheGroupPlan] = field(default_factory=list)
    # per run of the schedule: (group, entry, writes) or None for a mixer without cache
    runs: List[Optional[Tuple[int, int, bool]]] = field(default_factory=list)


class Model:
    def __init__(self, spec: ModelSpec, runtime: Runtime):
        self.spec = spec
        self.runtime = runtime
        self.embedding = make_part("embedding", spec.embedding, runtime)
        self.blocks = [
            make_part("block", PartSpec(layer.block, layer=layer, **layer.block_params), runtime)
            for layer in spec.layers]
        self.final_norm = make_part("norm", spec.final_norm, runtime)
        self.head = make_part("head", spec.head, runtime)
        self.schedule = list(spec.schedule)
        self.cache_plan = self._plan_cache()
        self._list_providers = None
        self._value_providers = None
        self._repeater = None          # set by ``repeat_layers``
        self.runs_repeated = 0         # runs of the schedule that were not walked through

    # ------------------------------------------------------------------ cache plan
    def _plan_cache(self) -> CachePlan:
        plan = CachePlan()
        keys: Dict[tuple, int] = {}
        for i, run in enumerate(self.schedule):
            if not 0 <= run.layer < len(self.blocks):
                raise ValueError(f"schedule entry {i} names layer {run.layer}, the model has "
                                 f"{len(self.blocks)}")
            need = self.blocks[run.layer].cache_need()
            if need is None:
                if run.cache_of is not None:
                    raise ValueError(f"schedule entry {i}: its mixer keeps no cache to share")
                plan.runs.append(None)
                continue
            if run.cache_of is not None:
                j = run.cache_of
                if not 0 <= j < i or plan.runs[j] is None or not plan.runs[j][2]:
                    raise ValueError(
                        f"schedule entry {i} reads the cache of entry {j}, which must be an "
                        f"earlier entry that writes one")
                other = self.blocks[self.schedule[j].layer].cache_need()
                if other.group_key() != need.group_key():
                    raise ValueError(f"schedule entry {i} cannot read the cache of entry {j}: "
                                     f"{need} does not fit {other}")
                g, e, _ = plan.runs[j]
                plan.runs.append((g, e, False))
                continue
            key = need.group_key()
            if key not in keys:
                keys[key] = len(plan.groups)
                plan.groups.append(CacheGroupPlan(need))
            g = keys[key]
            plan.runs.append((g, plan.groups[g].entries, True))
            plan.groups[g].entries += 1
        return plan

    # ------------------------------------------------------------------ weights
    def parts(self):
        return [self.embedding, *self.blocks, self.final_norm, self.head]

    def weight_specs(self) -> List[WeightSpec]:
        return [s for p in self.parts() for s in p.weight_specs()]

    def bind(self, weights: Dict[str, torch.Tensor]) -> None:
        for p in self.parts():
            p.bind(weights)
        self.runtime.tensors_changed()

    def all_parts(self):
        """Every part of the model, those inside arrangements and the shared ones included."""
        out, todo = [], self.parts() + [p for _, p in self.runtime.shared.values()]
        while todo:
            p = todo.pop(0)
            if any(p is q for q in out):
                continue
            out.append(p)
            todo.extend(p.children())
        return out

    def step_lists(self, starts, lens) -> Dict[str, list]:
        """The index lists that the model's parts want for a step with these spans:
        "<key>.<name>" -> list of ints, one set per key."""
        if self._list_providers is None:
            seen = {}
            for p in self.all_parts():
                key = getattr(p, "step_lists_key", None)
                if key is not None and key not in seen:
                    seen[key] = p
            self._list_providers = seen
        out = {}
        for key, part in self._list_providers.items():
            for name, values in part.step_lists(list(starts), list(lens)).items():
                out[f"{key}.{name}"] = values
        return out

    def step_values(self, starts, lens, positions) -> Dict[str, int]:
        """The host-side numbers that the model's parts want of a step's positions:
        "<key>.<name>" -> int."""
        if self._value_providers is None:
            seen = {}
            for p in self.all_parts():
                key = getattr(p, "step_values_key", None)
                if key is not None and key not in seen:
                    seen[key] = p
            self._value_providers = seen
        out = {}
        for key, part in self._value_providers.items():
            for name, value in part.step_values(list(starts), list(lens), list(positions)).items():
                out[f"{key}.{name}"] = int(value)
        return out

    def repeat_layers(self, on: bool = True) -> None:
        """Whether runs of layers that are alike share the host's work within a step (see
        ``repeat.LayerRepeater``); only a model whose steps are ``repeatable`` takes it."""
        from .repeat import LayerRepeater
        self._repeater = LayerRepeater(self) if on and self.repeatable else None

    @property
    def repeatable(self) -> bool:
        """Whether a step of this model can be run again from its recorded commands: every part
        records its launches, and what it launches depends on the step's shape alone (and on
        values it names through ``step_values``)."""
        return self.graph_safe and all(getattr(p, "records_launches", False) for p in self.all_parts())

    @property
    def graph_safe(self) -> bool:
        """Whether a step of this model can be recorded in a HIP graph."""
        shared = [p for _, p in self.runtime.shared.values()]
        return all(p.graph_safe for p in self.parts() + shared)

    def weight_bytes(self) -> int:
        """Bytes of distinct weight tensors the parts hold after bind."""
        seen = {}

        def visit(obj):
            for v in vars(obj).values():
                if isinstance(v, torch.Tensor):
                    seen[v.data_ptr()] = v.numel() * v.element_size()
                elif hasattr(v, "weight_specs") and hasattr(v, "bind"):
                    visit(v)
        for p in self.parts():
            visit(p)
        return sum(seen.values())

    def step_read_bytes(self, tokens: int) -> int:
        """Bytes of weights that a step of ``tokens`` tokens has to read: every tensor the
        scheduled parts use, once (a tensor that two parts share counts once, at the larger
        of what they read), as the parts themselves say."""
        seen: Dict[int, int] = {}
        used = [self.embedding, self.final_norm, self.head] + [self.blocks[r.layer] for r in self.schedule]
        used += [p for _, p in self.runtime.shared.values()]
        for part in used:
            for ptr, nbytes in part.read_bytes(tokens).items():
                seen[ptr] = max(seen.get(ptr, 0), nbytes)
        return sum(seen.values())

    def step_flops(self, tokens: int, keys_read: float, logit_rows: int = 1) -> float:
        """Floating-point operations of a step of ``tokens`` tokens that read ``keys_read``
        cached positions all together in every run, with logits at ``logit_rows`` rows."""
        return (sum(self.blocks[r.layer].flops(tokens, keys_read) for r in self.schedule)
                + self.head.flops(logit_rows))

    # ------------------------------------------------------------------ one step
    def run(self, ctx, cache_views) -> Optional[torch.Tensor]:
        """Run the step's tokens through every scheduled layer.  Returns
        float32 logits [R, vocab] for ``ctx.logit_rows`` (None if no row is
        wanted)."""
        shared = [p for _, p in self.runtime.shared.values()]
        for p in shared:
            if hasattr(p, "prepare"):
                call_part(p, p.prepare, ctx)
        x = call_part(self.embedding, self.embedding.forward, ctx, ctx.token_ids)
        for p in shared:
            if hasattr(p, "on_embedding"):
                call_part(p, p.on_embedding, ctx, x)
        if ctx.taps is not None:
            K.flush_recorded()                    # the copies below are torch's: behind what was recorded
            ctx.taps.append(x.clone())
        def walk_through(i, x, pending):
            block = self.blocks[self.schedule[i].layer]
            if getattr(block, "takes_next_norm", False):
                # the norm that will take this layer's output: the next layer's first, if it names
                # one, and the final norm behind the last layer
                if i + 1 < len(self.schedule):
                    nxt = self.blocks[self.schedule[i + 1].layer]
                    first = nxt.first_norm() if hasattr(nxt, "first_norm") else None
                else:
                    first = self.final_norm
                return call_part(block, block.forward, ctx, x, pending, cache_views[i], next_norm=first)
            return call_part(block, block.forward, ctx, x, pending, cache_views[i])

        pending = None
        # runs whose layers are alike are walked through twice a step, the others' commands
        # are those of the first with their own tensors' addresses
        repeater = self._repeater.step(ctx, cache_views) if self._repeater is not None else None
        for i in range(len(self.schedule)):
            if repeater is not None:
                x, pending = repeater.run(i, x, pending, walk_through)
                if i + 1 == len(self.schedule):
                    x, pending = repeater.current(x, pending)
                    self.runs_repeated += repeater.repeated
                continue
            x, pending = walk_through(i, x, pending)
            if ctx.taps is not None:
                if pending is not None:
                    call_part(self.final_norm, self.final_norm.add, ctx, x, pending)
                    pending = None
                K.flush_recorded()
                ctx.taps.append(x.clone())
        if ctx.taps is not None:
            tap = call_part(self.final_norm, self.final_norm.forward, ctx, x, delta=pending, tag="xn_tap")
            K.flush_recorded()
            ctx.taps.append(tap.clone())
            pending = None
        if ctx.logit_rows is None or ctx.logit_rows.numel() == 0:
            return None
        xn = call_part(self.final_norm, self.final_norm.forward, ctx, x, delta=pending, rows=ctx.logit_rows,
                       tag="xn_rows")
        return call_part(self.head, self.head.forward, ctx, xn)


def collect_weight_specs(spec: ModelSpec) -> List[WeightSpec]:
    """Every tensor a model of this spec wants, without touching a device."""
    from ..weights.loader import merge_specs
    rt = Runtime(device=torch.device("cpu"), dtype=torch.float32)
    return merge_specs(Model(spec, rt).weight_specs())
