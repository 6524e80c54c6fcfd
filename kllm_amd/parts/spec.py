"""The data a model is described with: parts, layers and their running order.

A model is nothing but this description.  ``PartSpec`` names a registered
part kind and gives it every size and constant it needs; ``LayerSpec`` puts a
mixer, a feed-forward and their norms into an arrangement; ``ModelSpec.schedule``
lists the layers in the order they run.  The same layer may be listed twice
(it then keeps a cache of its own for each run), and a run may read the cache
that an earlier run wrote instead of writing one.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class WeightSpec:
    """One tensor a part wants from the checkpoint.

    role "matrix": held in the engine's compute dtype (bfloat16 or float32);
    role "vector": small per-channel parameters, always held in float32;
    role "table":  integer tables, held as int32."""
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer needs kept between steps.

    kind "paged": keys and values per token, in pages; ``window`` > 0 means
    only the last ``window`` positions are ever read, so pages behind it are
    given back.  A token's entry is, per KV head, a key of ``head_dim`` and a
    value of ``value_dim`` elements (default: as wide as the key; 0: no value,
    one vector per token).  With equal widths a page is handed to the mixer as
    [2, kv_heads, page_size * head_dim]; otherwise as a flat run of
    kv_heads * page_size * (head_dim + value_dim) elements that the mixer lays
    out itself.  kind "state": one fixed-size tensor per request
    (``state_shape``), held in a slot.  ``dtype`` names the element type
    ("float32", "bfloat16", "int32", ...); the default is the engine's compute
    dtype for pages and float32 for state."""
    kind: str = "paged"
    kv_heads: int = 0
    head_dim: int = 0
    window: int = 0
    state_shape: Tuple[int, ...] = ()
    value_dim: Optional[int] = None
    dtype: Optional[str] = None

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else int(self.value_dim)

    def group_key(self):
        if self.kind == "paged":
            return ("paged", self.kv_heads, self.head_dim, self.window, self.value_width, self.dtype)
        return ("state", self.dtype) + tuple(self.state_shape)


class PartSpec:
    """A registered part kind plus its parameters.  ``prefix`` is the start of
    the part's tensor names in the checkpoint; the part adds its own suffixes
    (which ``params['names']`` may override)."""

    def __init__(self, kind: str, prefix: str = "", **params: Any):
        self.kind = kind
        self.prefix = prefix
        self.params = dict(params)

    def __repr__(self):
        return f"PartSpec({self.kind!r}, prefix={self.prefix!r}, {self.params})"


@dataclass
class LayerSpec:
    """One layer: an arrangement (block kind) of two norms, a mixer and a
    feed-forward.  Each layer chooses its own parts."""
    mixer: PartSpec
    feed_forward: PartSpec
    norm_mixer: PartSpec
    norm_feed_forward: PartSpec
    block: str = "pre_norm"
    block_params: Dict[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class Run:
    """One entry of the running order: run ``layer``; ``cache_of`` is None for
    a cache of its own, or the index of an earlier entry of the schedule whose
    cache this run reads (it then writes none)."""
    layer: int
    cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[Run]
    final_norm: PartSpec
    head: PartSpec
    vocab_size: int = 0
    hidden_size: int = 0
    eos_token_ids: Tuple[int, ...] = ()
    max_positions: Optional[int] = None
    optional_tensors: Tuple[str, ...] = ()   # may be in the checkpoint, are not read
