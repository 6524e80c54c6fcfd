"""What every part is: the interfaces, the registry of part kinds, and the
step context that parts are called with.

A part is built from a ``PartSpec`` (its kind, its tensor-name prefix and its
sizes and constants), says which tensors it wants (``weight_specs``), is bound
to them once (``bind``) and is then called once per step.  A part sees the
step only through ``StepContext``: token positions, which span a token belongs
to, block tables, state slots.  It does not see the model, the other layers or
the requests.

Categories and their call interface (x is the float32 residual stream
[n, hidden]; xn a normalised activation [n, hidden] in the compute dtype;
a *delta* is a float32 tensor [n, hidden] or [nsplit, n, hidden] of partial
sums to be added to x):

  norm          forward(ctx, x, delta=None, rows=None) -> xn
                  adds delta into x first (fused); with ``rows`` it reads only
                  those rows and leaves x alone
                add(ctx, x, delta)            x += delta, nothing else
  position      prepare(ctx)                  once per step, before any layer
                on_embedding(ctx, x)          optional: acts on the embedded
                                              tokens (additive encodings)
                tables(ctx) -> (cos, sin)     optional: rotation tables
                                              [n, rotary_dim/2] that a mixer
                                              applies to queries and keys;
                                              ``rotary_dim`` (default: the
                                              head) and ``interleaved`` (pairs
                                              (2j, 2j+1) instead of
                                              (j, j + rotary_dim/2)) say how
  mixer         cache_need() -> CacheNeed | None
                forward(ctx, xn, cache) -> delta
                  ``cache`` is a PagedCacheView or StateCacheView (or None)
  feed_forward  forward(ctx, xn) -> delta
  block         forward(ctx, x, pending, cache) -> (x, pending)
                  ``pending`` is a delta not yet added to x (or None)
  embedding     forward(ctx, token_ids) -> x
  head          forward(ctx, xn_rows) -> float32 logits [rows, vocab]
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Tuple

import torch

from .spec import CacheNeed, PartSpec, WeightSpec

CATEGORIES = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")
_REGISTRY: Dict[Tuple[str, str], type] = {}


def register_part(category: str, kind: str, cls: type = None):
    """Register ``cls`` as the part ``kind`` of ``category``; usable as a decorator."""
    if category not in CATEGORIES:
        raise ValueError(f"unknown part category {category!r} (one of {CATEGORIES})")

    def deco(c):
        _REGISTRY[(category, kind)] = c
        c.category = category
        c.kind = kind
        return c

    return deco(cls) if cls is not None else deco


def unregister_part(category: str, kind: str):
    _REGISTRY.pop((category, kind), None)


def registered_parts(category: str = None):
    return sorted(k for k in _REGISTRY if category is None or k[0] == category)


def make_part(category: str, spec: PartSpec, runtime: "Runtime"):
    try:
        cls = _REGISTRY[(category, spec.kind)]
    except KeyError:
        kinds = [k[1] for k in registered_parts(category)]
        raise ValueError(
            f"no {category} part of kind {spec.kind!r} is registered (registered: {kinds})") from None
    return cls(spec, runtime)


class Workspace:
    """Scratch tensors that live across steps.  ``get`` returns a view of a
    buffer kept per tag and grown when a larger one is asked for, so that a
    step allocates nothing once sizes have been seen (a HIP graph needs that)."""

    def __init__(self, device):
        self.device = device
        self.generation = 0          # grows when a buffer is replaced: addresses handed out before may be gone
        self._bufs: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}
        self._views: Dict[Tuple[str, tuple, torch.dtype], torch.Tensor] = {}   # handed out before

    def get(self, tag: str, shape, dtype) -> torch.Tensor:
        shape = tuple(shape)
        view = self._views.get((tag, shape, dtype))
        if view is not None:
            return view
        numel = 1
        for s in shape:
            numel *= int(s)
        key = (tag, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < numel:
            if buf is not None:
                from .. import kernels as K
                K.flush_recorded()   # launches recorded with the old buffer's address run before it goes
                self.generation += 1
            buf = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self._bufs[key] = buf
            for k in [k for k in self._views if k[0] == tag and k[2] == dtype]:   # views of the old buffer
                del self._views[k]
        view = buf[:numel].view(*shape)
        if len(self._views) < 4096:
            self._views[(tag, shape, dtype)] = view
        return view

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._bufs.values())


@dataclass
class Runtime:
    """What parts need to know about the engine they run in."""
    device: torch.device
    dtype: torch.dtype                      # compute/storage dtype: float32 or bfloat16
    workspace: Workspace = None
    options: Dict[str, Any] = field(default_factory=dict)
    shared: Dict[int, Any] = field(default_factory=dict)   # parts used by several layers
    tensor_epoch: int = 0                   # grows when parts may hold other tensors than before

    def __post_init__(self):
        if self.workspace is None:
            self.workspace = Workspace(self.device)

    def tensors_changed(self):
        """A part that puts another tensor in the place of one it holds, other than in
        ``bind``, says so here: addresses that were looked up before are looked up again."""
        self.tensor_epoch += 1

    def shared_part(self, category: str, spec: PartSpec):
        """The one instance of a part that several layers name with the same
        PartSpec object (a position encoding, for instance)."""
        key = id(spec)
        if key not in self.shared:
            self.shared[key] = (spec, make_part(category, spec, self))
        return self.shared[key][1]


@dataclass
class PagedCacheView:
    """One run's keys and values: ``pages`` is [num_pages, 2, kv_heads,
    page_size*head_dim] (keys [slot][hd], values [hd][slot] inside a page);
    ``block_table`` [spans, max_pages] int32 maps a span's logical page to a
    physical one.  ``write`` is False for a run that reads another run's cache."""
    pages: torch.Tensor
    block_table: torch.Tensor
    page_size: int
    write: bool = True


@dataclass
class StateCacheView:
    """One run's per-request state: ``state`` is [num_slots, *shape] float32,
    ``slots`` [spans] int32 gives each span's slot."""
    state: torch.Tensor
    slots: torch.Tensor
    write: bool = True


@dataclass
class ResidualSink:
    """An offer to a sub-layer that ends in a matrix product: add your output to the
    residual stream ``x`` yourself, in the product's epilogue, and leave what the norm
    behind the addition needs (``norm`` has ``weight`` and ``eps`` of an RMS norm).  A part
    that takes the offer (it declares ``fills_sink = True`` and gets ``sink=`` in forward)
    returns a ``Normed`` instead of its output; it may decline and return its output."""
    x: torch.Tensor
    norm: "Part"


@dataclass
class Normed:
    """An RMS norm that its consumer performs, as a residual product leaves it: ``x`` is
    the residual stream [n, d] (it already holds the sub-layer's output), ``ss`` [n, parts
    rounded up to 4] the partial sums of squares of its rows, ``norm`` the norm part it
    stands for (weight and eps).  A consumer whose kernel normalises while it stages its
    input takes ``kernel_input()``; one whose kernel scales its sums by the row takes
    ``scaled_rows()`` where the producer also left ``xw``, the rows of x times the norm's
    weight in the compute dtype; any other calls ``materialize``, which runs the norm."""
    x: torch.Tensor
    ss: torch.Tensor
    parts: int
    norm: "Part"
    xw: Optional[torch.Tensor] = None

    @property
    def rows(self) -> int:
        return self.x.shape[0]

    def kernel_input(self):
        from .. import kernels as K
        return K.NormedInput(self.x, self.norm.weight, self.ss, self.parts, self.norm.eps)

    def scaled_rows(self):
        from .. import kernels as K
        return K.ScaledRows(self.xw, self.ss, self.parts, self.norm.eps)

    def materialize(self, ctx):
        return self.norm.forward(ctx, self.x, delta=self)


@dataclass
class StepContext:
    """One step's batch as the parts see it.  All index tensors are int32 on
    the device; the ``h_`` lists are their host copies.

    A *span* is one request's tokens of this step: ``span_len[s]`` tokens at
    absolute positions ``span_pos[s] ...``; they sit at rows
    ``span_start[s] .. span_start[s+1]`` of every [n, ...] activation."""
    n: int
    n_spans: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    span_of_token: torch.Tensor
    span_start: torch.Tensor              # [n_spans + 1]
    span_pos: torch.Tensor                # [n_spans]
    slots: torch.Tensor                   # [n_spans] state slot of each span's request
    logit_rows: Optional[torch.Tensor]    # [R] rows whose logits are wanted
    h_span_start: List[int]
    h_span_pos: List[int]
    h_span_len: List[int]
    block_tables: List[torch.Tensor]      # per cache group [n_spans, max_pages]
    runtime: Runtime = None
    max_span_len: int = 0
    all_decode: bool = False              # every span is a single token
    scratch: Dict[Any, Any] = field(default_factory=dict)   # per-step values of parts
    taps: Optional[List[torch.Tensor]] = None               # residual-stream captures
    workspace: Optional["Workspace"] = None                 # scratch of this step (default: the runtime's)
    # Index lists that parts asked for through ``Part.step_lists``: "<key>.<name>" -> int32
    # tensor on the device (as long as the host list was, possibly empty).
    lists: Dict[str, torch.Tensor] = field(default_factory=dict)
    # Numbers that parts asked for through ``Part.step_values``: "<key>.<name>" -> int, worked
    # out on the host from the step's positions.
    values: Dict[str, int] = field(default_factory=dict)
    # Token ids that never reached the host: token t with token_from[t] >= 0 is
    # sampled[token_from[t]], what the last sampled step chose (both or neither are set).
    token_from: Optional[torch.Tensor] = None
    sampled: Optional[torch.Tensor] = None

    def buf(self, tag, shape, dtype):
        return (self.workspace or self.runtime.workspace).get(tag, shape, dtype)


def call_part(part, fn, *args, **kwargs):
    """Call ``fn`` (a method of ``part``) so that its work reaches the stream in program order:
    as it is for a part that records its launches, otherwise with the recorded launches run
    first and recording switched off inside."""
    from .. import kernels as K
    if getattr(part, "records_launches", False) or not K.recording():
        return fn(*args, **kwargs)
    with K.direct_launches():
        return fn(*args, **kwargs)


class Part:
    """Base of all parts."""
    category = None
    kind = None
    # True if the part's forward only launches kernels on the current stream with
    # addresses and sizes that depend on nothing but the batch's shape: such a
    # part can be recorded in a HIP graph.  A part that reads device values on
    # the host, or loops over host-side span data, leaves this False.
    graph_safe = False
    # A part whose kernels want index lists that depend on how the step's tokens are cut
    # into spans (which tokens are decode tokens, where tiles of queries begin) names a
    # key here and builds the lists on the host in ``step_lists``; the engine packs them
    # into the step's one control buffer and the part finds them as
    # ``ctx.lists["<key>.<name>"]``.  Parts with the same key share one set of lists.  The
    # lists may depend on nothing but ``starts`` and ``lens`` (a recorded step replays them).
    step_lists_key: Optional[str] = None
    step_values_key: Optional[str] = None      # the same for ``step_values`` (see there)
    # A mixer or feed-forward whose first product can normalise its input while staging it
    # declares ``takes_normed`` and may then get a ``Normed`` as its input; one whose
    # last product can add itself to the residual stream declares ``fills_sink`` and then
    # gets ``sink=ResidualSink`` (see those classes).  A norm that others may fuse this way
    # declares ``fusable`` (it has ``weight`` and ``eps`` of an RMS norm).
    takes_normed = False
    fills_sink = False
    fusable = False
    # True if everything the part gives to the stream goes through the package's kernel wrappers
    # (``kllm_amd.kernels``), which can record a step's launches and hand them to the library in
    # one call.  A part that uses torch operations or launches by other ways leaves this False:
    # it is then called with what was recorded already run, and its own launches made at once.
    records_launches = False

    def __init__(self, spec: PartSpec, runtime: Runtime):
        self.spec = spec
        self.runtime = runtime
        self.prefix = spec.prefix

    def param(self, key, default=...):
        if key in self.spec.params:
            return self.spec.params[key]
        if default is ...:
            raise ValueError(f"{self.category} part {self.kind!r} needs parameter {key!r}")
        return default

    def tensor_name(self, local: str) -> str:
        names = self.spec.params.get("names") or {}
        if local in names:
            return names[local]
        return f"{self.prefix}.{local}" if self.prefix else local

    def weight_specs(self) -> List[WeightSpec]:
        return []

    def bind(self, weights: Dict[str, torch.Tensor]) -> None:
        """Take the tensors named by weight_specs out of ``weights``."""

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def check_cache(self, page_size: int) -> None:
        """Raise ValueError if this part's kernels do not take a cache with pages of
        ``page_size`` tokens; the engine asks every part before it allocates."""

    def step_values(self, starts: List[int], lens: List[int], positions: List[int]) -> Dict[str, int]:
        """name -> int for a step whose span s covers rows ``starts[s] .. starts[s] + lens[s]`` at
        positions ``positions[s] ...``: what the part's launches need to know of the step's
        positions on the host (a count that chooses a kernel, a bound of a loop).  The part
        finds them as ``ctx.values["<step_values_key>.<name>"]`` and hands them to the kernel
        wrappers as they are; a step that is run again from its recorded commands gets the new
        step's values in their place.  Everything else of a part's launches may depend on
        ``starts`` and ``lens`` only.  Only called when ``step_values_key`` is set; parts with
        the same key share one set of values."""
        return {}

    def children(self) -> List["Part"]:
        """Parts this part is made of (an arrangement's norms, mixer, feed-forward)."""
        return []

    # ---- what a step costs at least (for rooflines; measurement code asks the model, which asks its parts)
    def tensors(self) -> List[torch.Tensor]:
        """The tensors this part itself holds after ``bind`` (its children's excluded)."""
        return [v for v in vars(self).values() if isinstance(v, torch.Tensor)]

    def read_bytes(self, tokens: int) -> Dict[int, int]:
        """address -> bytes of its tensors that a step of ``tokens`` tokens has to read: all of
        each by default (a table that is only gathered from overrides this)."""
        return {t.data_ptr(): t.numel() * t.element_size() for t in self.tensors()}

    def flops(self, tokens: int, keys_read: float = 0.0) -> float:
        """Floating-point operations of ``tokens`` tokens through this part, the tokens reading
        ``keys_read`` cached positions all together (a mixer adds its scores and values): two
        per element of every matrix it holds and token, by default."""
        return 2.0 * tokens * sum(t.numel() for t in self.tensors() if t.dim() == 2)

    def step_lists(self, starts: List[int], lens: List[int]) -> Dict[str, List[int]]:
        """name -> list of ints for a step whose span s covers rows
        ``starts[s] .. starts[s] + lens[s]``; only called when ``step_lists_key`` is set."""
        return {}
