"""The engine: a model on the GPU, its cache, and the one step function.

``Engine.step`` takes a batch of (request, its next tokens) -- portions of
prompts beside single decoded tokens, cut anywhere -- runs exactly those
tokens as one batch against the cache that earlier steps left, and returns
the logits at the wanted places.  It is the counterpart of the reference's
``te_forward_batch`` (backend/model.cu:995-1195) together with the host
protocol around it, reserve -> forward -> commit (engine/engine.go:160-185).
The device side knows nothing about requests: positions and block tables are
passed every step (backend/shim.h:106-113).
"""

from __future__ import annotations

from collections import OrderedDict
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from .. import kernels as K
from ..cache import CacheManager, GroupSpec, OutOfPages
from ..cache.manager import window_pages
from ..config import ModelConfig, config_from_dict, load_config, resolve_architecture
from ..parts.base import PagedCacheView, Runtime, StateCacheView, StepContext
from ..weights import load_weights, random_weights
from . import control
from .graph import DecodeGraphs, SampledTokens, TokenRef, _bucket as table_bucket
from .model import Model

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "bfloat16": torch.bfloat16,
           "bf16": torch.bfloat16}


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


class StepError(ValueError):
    """A step that cannot be run as asked (bad token id, unknown request...)."""


@dataclass
class EngineOptions:
    """Sizes of the engine, apart from the model's own.  The reference's
    Options (engine/engine.go:16-33) have one bound, MaxSeq, for both a
    request's length and a step's tokens; here they are separate."""
    device: int = 0
    dtype: str = "bfloat16"               # "bfloat16" or "float32"
    page_size: int = 16                   # tokens per page (reference default: 16)
    max_tokens: Optional[int] = None      # cache capacity in tokens (per group)
    num_pages: Optional[int] = None       # ... or directly in pages
    memory_bytes: Optional[int] = None    # ... and never more than fits into this many bytes
    max_step_tokens: Optional[int] = None  # most tokens one request brings in one step (None: any)
    max_requests: int = 64                # live requests (state slots)
    max_model_len: Optional[int] = None   # longest request; default max_position_embeddings
    gemm: str = "hip"                     # "hip" or "library" (vendor GEMM for large prompts)
    attention: str = "auto"               # "auto" or "generic"
    graphs: bool = True                   # replay decode steps as HIP graphs
    max_graph_batch: int = 256            # largest decode batch that is recorded as a graph
    graph_after_steps: int = 8            # a batch shape is recorded the n-th time it is queued ahead (before: as any step)
    poison_freed_pages: bool = False      # debugging: fill pages with NaN when they are given back
    extra: Dict[str, object] = field(default_factory=dict)

    def torch_dtype(self) -> torch.dtype:
        try:
            return _DTYPES[self.dtype]
        except KeyError:
            raise ValueError(f"dtype {self.dtype!r} is not one of {sorted(_DTYPES)}") from None


@dataclass
class StepEntry:
    """One request's part of a step: its next tokens and the places among
    them whose logits are wanted."""
    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class _StepPlan:
    """A step's recorded launches, the logits they leave, and what must still hold for the
    addresses in them: the scratch buffers and the control buffer not replaced since."""
    commands: object
    logits: Optional[torch.Tensor]
    generation: int
    control: int


class Engine:
    MAX_STEP_PLANS = 256

    def __init__(self, config: ModelConfig, raw_config: dict, weights_from, options: EngineOptions):
        if not torch.cuda.is_available():
            raise RuntimeError("kllm_amd runs on a GPU only; torch sees none")
        from .. import kernels
        kernels.library()  # fail now, and loudly, if the kernels are missing
        self.kernels = kernels
        self.options = options
        self.config = config
        self.device = torch.device("cuda", options.device)
        torch.cuda.set_device(self.device)
        self.dtype = options.torch_dtype()
        rt_options = {"gemm": options.gemm, "attention": options.attention}
        rt_options.update(options.extra)
        self.runtime = Runtime(device=self.device, dtype=self.dtype, options=rt_options)
        arch = resolve_architecture(raw_config)
        self.spec = arch.build(config)
        self.model = Model(self.spec, self.runtime)
        self.vocab_size = self.spec.vocab_size
        specs = self.model.weight_specs()
        weights = weights_from(specs, self.spec)
        self.model.bind(weights)
        del weights
        self.max_model_len = options.max_model_len or self.spec.max_positions
        self._alloc_cache()
        self._pinned: List[torch.Tensor] = []
        self._pinned_events: List[Optional[torch.cuda.Event]] = []
        self._pinned_next = 0
        self._control = None
        self.steps_run = 0
        self.tokens_run = 0
        # A step's launches go to the library as one buffer of commands, not one by one
        # (EngineOptions.extra["launch_one_by_one"] keeps the old way, for comparison).
        self.records_launches = not options.extra.get("launch_one_by_one")
        # ... and a step whose shape (tokens per request, wanted rows, table widths) has been seen
        # runs again from the commands recorded then, without going through the parts: what a
        # part launches may depend on the shape alone and on the values it names
        # (Part.step_values), which is also what recording a decode step as a HIP graph asks.
        self._repeat_steps = (self.records_launches and self.model.repeatable
                              and not options.extra.get("no_repeated_steps"))
        self._plans: "OrderedDict[tuple, _StepPlan]" = OrderedDict()
        self.steps_repeated = 0
        # ... and within a step that is walked through, layers that are alike share the walk
        # (extra["no_repeated_layers"] switches that off, for comparison).
        self.model.repeat_layers(self.records_launches and not options.extra.get("no_repeated_layers"))
        self._graphs = DecodeGraphs(self)
        # What a scheduler should know of the kernels: a step's tokens are the rows of every
        # product, and those work on tiles of this many rows.
        self.step_row_multiple = K.GEMM_TILE_ROWS

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_dir(cls, model_dir: str, options: EngineOptions = None) -> "Engine":
        """Load ``model_dir`` (config.json + safetensors); the architecture
        named in config.json chooses the model."""
        from ..config.base import read_config_json
        options = options or EngineOptions()
        raw = read_config_json(model_dir)
        config = config_from_dict(raw, where=f"{model_dir}/config.json")
        dtype, device = options.torch_dtype(), torch.device("cuda", options.device)

        def weights_from(specs, spec):
            return load_weights(model_dir, specs, dtype, device, optional=spec.optional_tensors)
        return cls(config, raw, weights_from, options)

    @classmethod
    def from_random(cls, config, seed: int, options: EngineOptions = None, std=0.02,
                    norm_std=0.02) -> "Engine":
        """Seeded random weights for ``config`` (typed or a config.json dict),
        made in memory; the values equal those ``write_random_model`` stores."""
        options = options or EngineOptions()
        raw = config.to_dict() if isinstance(config, ModelConfig) else dict(config)
        typed = config_from_dict(raw, where="config")
        dtype, device = options.torch_dtype(), torch.device("cuda", options.device)

        def weights_from(specs, spec):
            return random_weights(specs, seed, dtype, device, std, norm_std)
        return cls(typed, raw, weights_from, options)

    # ------------------------------------------------------------------ cache
    def _alloc_cache(self):
        """Pools and device tensors of every cache group.

        Capacity rule: the pool holds ``num_pages`` pages (or ``max_tokens``
        tokens; by default four longest requests, engine/engine.go:30-32), but
        never more than fit into ``memory_bytes`` beside the state slots -- the
        reference's lesson that a pool must be sized from the model's
        dimensions under a byte budget, not by a fixed count
        (docs/JOURNAL.md:364-367, tools/modal_lab.py:232-240).  A group whose
        layers read only a window of keys gets no more pages than
        ``max_requests`` requests can hold at one time."""
        o = self.options
        plan = self.model.cache_plan
        if o.page_size <= 0:
            raise ValueError(f"page_size {o.page_size} must be positive")
        for part in self.model.all_parts():
            part.check_cache(o.page_size)
        if o.num_pages is not None:
            asked = int(o.num_pages)
        else:
            tokens = o.max_tokens
            if tokens is None:
                tokens = 4 * (self.max_model_len or 2048)
            asked = -(-int(tokens) // o.page_size)
        paged = [(g, gp) for g, gp in enumerate(plan.groups) if gp.need.kind == "paged"]
        for g, gp in enumerate(plan.groups):
            if gp.need.kind not in ("paged", "state"):
                raise ValueError(f"unknown cache kind {gp.need.kind!r}")
        def dtype_of(need, default):
            if need.dtype is None:
                return default
            dt = getattr(torch, str(need.dtype), None)
            if not isinstance(dt, torch.dtype):
                raise ValueError(f"cache dtype {need.dtype!r} is no torch dtype")
            return dt

        def size_of(dt):
            return torch.empty((), dtype=dt).element_size()
        state_bytes = sum(gp.entries * o.max_requests * _numel(gp.need.state_shape)
                          * size_of(dtype_of(gp.need, torch.float32))
                          for gp in plan.groups if gp.need.kind == "state")
        page_bytes = {g: gp.entries * gp.need.kv_heads * o.page_size * (gp.need.head_dim + gp.need.value_width)
                      * size_of(dtype_of(gp.need, self.dtype)) for g, gp in paged}
        step = o.max_step_tokens or self.max_model_len or 0
        want = {}
        for g, gp in paged:
            want[g] = asked
            if gp.need.window > 0 and self.max_model_len:
                per_request = window_pages(self.max_model_len, step, o.page_size, gp.need.window)
                want[g] = min(asked, o.max_requests * per_request)
        if o.memory_bytes is not None and paged:
            budget = int(o.memory_bytes) - state_bytes
            # shrink all groups by the same factor until they fit
            need = sum(want[g] * page_bytes[g] for g, _ in paged)
            if need > budget:
                scale = max(budget, 0) / need
                want = {g: int(want[g] * scale) for g in want}
            if min(want.values()) < 1:
                raise ValueError(
                    f"memory_bytes={o.memory_bytes} leaves no room for a cache page in every group "
                    f"(a page of each group takes {sum(page_bytes.values())} bytes, state slots "
                    f"{state_bytes})")
        self.num_pages = max(want.values()) if want else 0
        groups, self._paged_group_of, self.kv, self.state = [], {}, {}, {}
        self._capacity = []
        for g, gp in enumerate(plan.groups):
            need = gp.need
            if need.kind == "paged":
                self._paged_group_of[g] = len(groups)
                groups.append(GroupSpec(f"group{g}", o.page_size, want[g], need.window))
                if need.value_width == need.head_dim:
                    shape = (2, need.kv_heads, o.page_size * need.head_dim)
                else:       # keys and values of different widths (or no values): the mixer lays a page out
                    shape = (need.kv_heads * o.page_size * (need.head_dim + need.value_width),)
                self.kv[g] = torch.zeros(gp.entries, want[g], *shape, dtype=dtype_of(need, self.dtype),
                                         device=self.device)
                self._capacity.append(
                    f"group{g}: {gp.entries} layers, {need.kv_heads} KV heads of {need.head_dim}"
                    + (f" (values of {need.value_width})" if need.value_width != need.head_dim else "")
                    + (f", window {need.window}" if need.window else "")
                    + f": {want[g]} pages of {o.page_size} tokens = {want[g] * o.page_size} tokens, "
                    f"{want[g] * page_bytes[g] / 2**20:.1f} MiB"
                    + (f" (asked for {asked} pages)" if want[g] != asked else ""))
            else:
                self.state[g] = torch.zeros(gp.entries, o.max_requests, *need.state_shape,
                                            dtype=dtype_of(need, torch.float32), device=self.device)
                self._capacity.append(
                    f"group{g}: {gp.entries} layers with state {tuple(need.state_shape)} in {o.max_requests} slots, "
                    f"{self.state[g].numel() * self.state[g].element_size() / 2**20:.1f} MiB")
        self.cache = CacheManager(groups, o.max_requests)

    def capacity_report(self) -> str:
        """What the cache was sized to, one line per group: for printing at start."""
        head = f"cache: {self.cache_bytes() / 2**20:.1f} MiB"
        if self.options.memory_bytes is not None:
            head += f" of a budget of {self.options.memory_bytes / 2**20:.1f} MiB"
        return "\n".join([head] + ["  " + line for line in self._capacity])

    def cache_read_bytes(self, contexts: Sequence[int]) -> int:
        """Bytes of cache that a decode step of requests holding ``contexts`` tokens has to
        read: per paged group and run, each request's keys and values (its window of them)."""
        total = 0
        for g, gp in enumerate(self.model.cache_plan.groups):
            if gp.need.kind != "paged":
                continue
            per_token = gp.need.kv_heads * (gp.need.head_dim + gp.need.value_width) * self.kv[g].element_size()
            readers = sum(1 for r in self.model.cache_plan.runs if r is not None and r[0] == g)
            for c in contexts:
                total += readers * per_token * (min(c, gp.need.window) if gp.need.window else c)
        return total

    def step_read_bytes(self, contexts: Sequence[int]) -> int:
        """What a decode step of these requests must read at least: every weight it uses once
        and the cache of the live requests."""
        return self.model.step_read_bytes(len(contexts)) + self.cache_read_bytes(contexts)

    def cache_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in list(self.kv.values()) + list(self.state.values()))

    def _poison(self, per_group_pages):
        for g, mg in self._paged_group_of.items():
            ids = [p for p in per_group_pages[mg] if p >= 0]
            if ids:
                idx = torch.tensor(ids, dtype=torch.long, device=self.device)
                kv = self.kv[g]
                kv[:, idx] = float("nan") if kv.is_floating_point() else torch.iinfo(kv.dtype).min

    # ------------------------------------------------------------------ requests
    def open(self, request_id: Hashable):
        return self.cache.open(request_id)

    def release(self, request_id: Hashable):
        """The request is over; what it holds is given back."""
        if self.options.poison_freed_pages:
            held = [list(t) for t in self.cache.get(request_id).tables]
            self.cache.release(request_id)
            self._poison(held)
        else:
            self.cache.release(request_id)

    def length(self, request_id: Hashable) -> int:
        return self.cache.get(request_id).length

    # ------------------------------------------------------------------ the step
    def _staging(self, n_ints: int) -> torch.Tensor:
        """A pinned host buffer; a small ring, so that filling the next step
        does not wait for the copy of the last one."""
        ring = 4
        if len(self._pinned) < ring:
            self._pinned.append(torch.empty(max(n_ints, 4096), dtype=torch.int32, pin_memory=True))
            self._pinned_events.append(None)
            i = len(self._pinned) - 1
        else:
            i = self._pinned_next
            self._pinned_next = (i + 1) % ring
            if self._pinned_events[i] is not None:
                self._pinned_events[i].synchronize()
            if self._pinned[i].numel() < n_ints:
                self._pinned[i] = torch.empty(n_ints, dtype=torch.int32, pin_memory=True)
        self._staging_index = i
        return self._pinned[i]

    def _send(self, host: torch.Tensor, dev: torch.Tensor, total: int):
        dev[:total].copy_(host[:total], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._pinned_events[self._staging_index] = ev

    def _validate(self, entries: Sequence[StepEntry], allow_refs: bool = True):
        """Checks the entries and returns each one's token ids as an array (a
        TokenRef stands as 0).  Plain ids are converted once, here, and the
        arrays go on into the control buffer."""
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        arrays = []
        for e in entries:
            if e.request_id in seen:
                raise StepError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            try:
                toks = np.asarray(e.tokens, dtype=np.int64)          # plain ids: one pass
            except (TypeError, ValueError):
                if not all(isinstance(t, (int, np.integer, TokenRef)) for t in e.tokens):
                    raise StepError(f"request {e.request_id!r}: token ids must be integers") from None
                if not allow_refs:
                    raise StepError("a TokenRef can only stand in a batch of single decode tokens "
                                    "that is sampled") from None
                toks = np.asarray([0 if isinstance(t, TokenRef) else t for t in e.tokens], dtype=np.int64)
            if toks.ndim != 1 or toks.size == 0:
                raise StepError(f"request {e.request_id!r}: a step needs at least one token")
            if toks.min() < 0 or toks.max() >= self.vocab_size:
                bad = int(toks[(toks < 0) | (toks >= self.vocab_size)][0])
                raise StepError(f"request {e.request_id!r}: token id {bad} is outside "
                                f"[0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < toks.size:
                    raise StepError(f"request {e.request_id!r}: wanted place {w} is outside its "
                                    f"{toks.size} tokens")
            arrays.append(toks)
        return arrays

    def _reserve(self, entries: Sequence[StepEntry]):
        """Room for every entry's tokens, or nothing taken.  Returns what to
        undo if the step fails."""
        opened, reserved = [], []
        try:
            for e in entries:
                if e.request_id not in self.cache:
                    self.cache.open(e.request_id)
                    opened.append(e.request_id)
                rc = self.cache.get(e.request_id)
                if self.max_model_len is not None and rc.length + len(e.tokens) > self.max_model_len:
                    raise StepError(
                        f"request {e.request_id!r} would reach {rc.length + len(e.tokens)} tokens, "
                        f"the longest allowed is {self.max_model_len}")
                if self.options.max_step_tokens and len(e.tokens) > self.options.max_step_tokens:
                    raise StepError(
                        f"request {e.request_id!r} brings {len(e.tokens)} tokens in one step, the engine "
                        f"was sized for {self.options.max_step_tokens} (EngineOptions.max_step_tokens)")
                self.cache.reserve(e.request_id, len(e.tokens))
                reserved.append(e.request_id)
        except Exception:
            self._undo(opened, reserved)
            raise
        return opened, reserved

    def _undo(self, opened, reserved):
        for rid in reserved:
            self.cache.cancel(rid)
        for rid in opened:
            self.cache.release(rid)

    def _commit(self, entries: Sequence[StepEntry]):
        before = None
        if self.options.poison_freed_pages:
            before = {e.request_id: [list(t) for t in self.cache.get(e.request_id).tables]
                      for e in entries}
        for e in entries:
            self.cache.commit(e.request_id, len(e.tokens))
        if before is not None:
            for e in entries:
                now = self.cache.get(e.request_id).tables
                self._poison([[p for p, q in zip(b, a) if p >= 0 and q < 0]
                              for b, a in zip(before[e.request_id], now)])
        self.steps_run += 1
        self.tokens_run += sum(len(e.tokens) for e in entries)

    def _describe(self, entries: Sequence[StepEntry]):
        rcs = [self.cache.get(e.request_id) for e in entries]
        lens = [len(e.tokens) for e in entries]
        starts = [0]
        for l in lens:
            starts.append(starts[-1] + l)
        rows = [starts[s] + int(w) for s, e in enumerate(entries) for w in e.want]
        n_groups = len(self.cache.groups)
        tables = [[rc.tables[g] for rc in rcs] for g in range(n_groups)]
        return rcs, lens, rows, tables

    def step(self, entries: Sequence[StepEntry], taps: Optional[list] = None):
        """Run one batch.  Returns float32 logits [wanted, vocab] on the
        device, in the order of the entries and of their ``want`` lists, or
        None if nothing is wanted.  Raises OutOfPages (and changes nothing) if
        the cache cannot hold the step's tokens."""
        return self._run(entries, self._validate(entries, allow_refs=False), taps, None)

    def _run(self, entries, arrays, taps, sampling, reserved=None):
        """The step itself.  ``sampling``: None, or (temperatures, uniforms, token_ref) for a
        step whose wanted places are sampled on the device into the place where the next
        step's embedding finds the ids (``token_ref[t] >= 0``: token t's id is what the step
        sampled last left there at that index).  ``reserved``: a ``ReservedStep`` whose pages
        are reserved already."""
        opened, reserved_ids = (reserved.opened, reserved.reserved) if reserved is not None else self._reserve(entries)
        try:
            rcs, lens, rows, tables = reserved.described if reserved is not None else self._describe(entries)
            # table widths in powers of two, as recorded steps have them: few distinct layouts
            pages = tuple(table_bucket(max(len(t) for t in tg)) for tg in tables)
            span_starts = [0]
            for l in lens:
                span_starts.append(span_starts[-1] + l)
            lists = self.model.step_lists(span_starts, lens)
            if sampling is None:
                layout = control.layout_for(lens, len(rows), pages, lists=lists)
                temps = unis = token_ref = None
            else:
                temps, unis, token_ref = sampling
                layout = control.layout_for(lens, len(rows), pages, samples=len(rows), lists=lists,
                                            refs=token_ref is not None)
            total = layout.total
            host = self._staging(total)
            pos0 = [rc.length for rc in rcs]
            starts = control.fill(host.numpy(), layout, arrays, pos0,
                                  [rc.slot for rc in rcs], rows, tables, temps, unis, lists=lists,
                                  token_ref=token_ref)
            if self._control is None or self._control.numel() < total:
                self._control = torch.empty(max(total, 4096), dtype=torch.int32, device=self.device)
            self._send(host, self._control, total)
            values = self.model.step_values(span_starts, lens, pos0)
            key = (layout, tuple(lens)) if self._repeat_steps and taps is None else None
            plan = self._plans.get(key) if key is not None else None
            workspace = self.runtime.workspace
            if plan is not None and plan.generation == workspace.generation and plan.control == self._control.data_ptr():
                # a step of this shape ran before: its launches again, in one call, with this
                # step's values in place of that step's
                self._plans.move_to_end(key)
                plan.commands.run(values, torch.cuda.current_stream().cuda_stream)
                logits = plan.logits
                self.steps_repeated += 1
            else:
                ctx = control.context(self._control, layout, self.runtime, starts, pos0, lens)
                ctx.taps = taps
                ctx.values = {k: self.kernels.StepValue(v, k) for k, v in values.items()}
                if sampling is not None:
                    ctx.sampled = self._graphs.sampled
                generation = workspace.generation
                with self.kernels.stream_scope(record=self.records_launches, keep=key is not None) as scope:
                    logits = self.model.run(ctx, self._cache_views(ctx))
                    if sampling is not None and rows:
                        t_dev, u_dev = control.sampling_views(self._control, layout)
                        self.kernels.sample(self._graphs.sampled[:len(rows)], logits, t_dev, u_dev)
                commands = scope.plan() if key is not None and generation == workspace.generation else None
                if commands is not None:          # (a step that grew its scratch buffers is kept the next time)
                    self._plans[key] = _StepPlan(commands, logits, workspace.generation, self._control.data_ptr())
                    while len(self._plans) > self.MAX_STEP_PLANS:
                        self._plans.popitem(last=False)
        except Exception:
            self._undo(opened, reserved_ids)
            raise
        self._commit(entries)
        return logits

    def can_sample_ahead(self, entries: Sequence[StepEntry]) -> bool:
        """Whether these entries are replayed as a HIP graph: single decode
        tokens of a model whose parts can be."""
        return (self.options.graphs and self.model.graph_safe
                and 0 < len(entries) <= self.options.max_graph_batch
                and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries))

    def can_queue_ahead(self, entries: Sequence[StepEntry]) -> bool:
        """Whether ``step_sample_ahead`` takes these entries: any step whose wanted places
        (one token sampled for each) fit the place where sampled ids are kept."""
        return 0 < len(entries) and sum(len(e.want) for e in entries) <= self._graphs.sampled.numel()

    def step_sample_ahead(self, entries: Sequence[StepEntry], temperatures, uniforms) -> SampledTokens:
        """Queue a step whose wanted places are sampled on the device and return
        without waiting for it.  The sampled ids are read from the handle, in the
        order of the wanted places; the *next* step may be queued before that, with
        ``TokenRef(handle, i)`` as the only token of an entry in place of the id.
        Batches of single decode tokens are replayed as HIP graphs, any other step
        (portions of prompts beside decode tokens) runs from its recorded commands."""
        count = sum(len(e.want) for e in entries)
        if len(temperatures) != count or len(uniforms) != count:
            raise StepError(f"{count} places are wanted, {len(temperatures)} temperatures and "
                            f"{len(uniforms)} uniforms were given")
        if self.can_sample_ahead(entries):
            # (a shape that was not seen often enough yet runs as any other step does: from its
            # recorded commands, which costs the host a little more and no recording)
            out = self._graphs.decode(entries, temperatures, uniforms, wait_for_uses=self.can_queue_ahead(entries))
            if isinstance(out, SampledTokens):
                return out
            logits = self._run(entries, out.arrays, None, (list(temperatures), list(uniforms), out.token_ref),
                               reserved=out)
            return self._graphs.handle(count, logits)
        if not self.can_queue_ahead(entries):
            raise StepError(f"a step queued ahead samples at most {self._graphs.sampled.numel()} tokens")
        arrays = self._validate(entries, allow_refs=True)
        token_ref = None
        if any(isinstance(t, TokenRef) for e in entries for t in e.tokens):
            token_ref = []
            for e in entries:
                if len(e.tokens) > 1 and any(isinstance(t, TokenRef) for t in e.tokens):
                    raise StepError("a TokenRef stands alone in its entry (one decode token)")
                for t in e.tokens:
                    if isinstance(t, TokenRef):
                        last = self._graphs.last
                        if t.source is not last or not 0 <= t.index < t.source.count:
                            raise StepError("a TokenRef must name a token of the step that was sampled last")
                        token_ref.append(t.index)
                    else:
                        token_ref.append(-1)
        logits = self._run(entries, arrays, None, (list(temperatures), list(uniforms), token_ref))
        return self._graphs.handle(count, logits)

    def step_sample(self, entries: Sequence[StepEntry], temperatures, uniforms) -> List[int]:
        """A step whose wanted places are sampled on the device: one token per
        wanted place, as host ints.  Batches of single decode tokens are
        replayed as a HIP graph (forward pass and sampling in one launch)."""
        if self.can_sample_ahead(entries):
            return self.step_sample_ahead(entries, temperatures, uniforms).tokens()
        if any(isinstance(t, TokenRef) for e in entries for t in e.tokens):
            return self.step_sample_ahead(entries, temperatures, uniforms).tokens()
        logits = self.step(entries)
        if logits is None:
            return []
        return self.sample(logits, temperatures, uniforms)

    def _cache_views(self, ctx: StepContext):
        views = []
        for entry in self.model.cache_plan.runs:
            if entry is None:
                views.append(None)
                continue
            g, e, writes = entry
            if g in self.kv:
                views.append(PagedCacheView(self.kv[g][e], ctx.block_tables[self._paged_group_of[g]],
                                            self.options.page_size, writes))
            else:
                views.append(StateCacheView(self.state[g][e], ctx.slots, writes))
        return views

    # ------------------------------------------------------------------ sampling
    @property
    def eos_token_ids(self):
        return tuple(self.spec.eos_token_ids)

    def sample(self, logits, temperatures, uniforms) -> List[int]:
        """One token per row of logits (greedy where the temperature is 0)."""
        from ..sampling import DeviceSampler
        if getattr(self, "_sampler", None) is None:
            self._sampler = DeviceSampler(self.device)
        return self._sampler.sample(logits, temperatures, uniforms)

    # ------------------------------------------------------------------ generation
    def generate(self, prompts, max_new_tokens: int, temperature: float = 0.0, seed: int = 0,
                 max_step_tokens: Optional[int] = None, max_batch: Optional[int] = None):
        """Generate for each prompt (a list of token ids) up to
        ``max_new_tokens`` tokens, stopping at an end-of-sequence id; all
        prompts are scheduled together, as many at a time as ``max_batch``
        says (default: all of them, up to the engine's number of requests).
        Returns one list of ids per prompt.
        The reference's Generate runs one prompt, greedily
        (engine/engine.go:192-213)."""
        from .scheduler import Scheduler
        single = bool(prompts) and isinstance(prompts[0], int)
        if single:
            prompts = [prompts]
        if max_batch is None:
            max_batch = max(1, min(len(prompts), self.options.max_requests))
        sched = Scheduler(self, max_batch=max_batch, max_step_tokens=max_step_tokens)
        ids = [sched.submit(list(p), max_new_tokens, temperature=temperature, seed=seed + i)
               for i, p in enumerate(prompts)]
        results = sched.run_until_done()
        out = [results[i].tokens for i in ids]
        for i in ids:
            if results[i].error:
                raise RuntimeError(f"prompt {i}: {results[i].error}")
        return out[0] if single else out
