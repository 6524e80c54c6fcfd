"""Rotary position encoding, half-split pairing.

For pair (j, j + head_dim/2) of every head: angle = pos * theta^(-2j/head_dim),
computed in double; a' = a cos - b sin, b' = b cos + a sin
(backend/model.cu:170-184).  Keys are rotated before they are cached
(:1093-1100), so the cache never needs re-encoding.

Parameters: ``head_dim``, ``theta``.  No tensors.  ``prepare`` computes the
step's cos/sin tables once; every mixer that shares this part reads them.
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, register_part


@register_part("position", "rotary")
class RotaryEncoding(Part):
    graph_safe = True
    records_launches = True


    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.head_dim = int(self.param("head_dim"))
        self.theta = float(self.param("theta"))
        if self.head_dim % 2:
            raise ValueError(f"rotary: head_dim {self.head_dim} must be even")

    def prepare(self, ctx):
        half = self.head_dim // 2
        cos = ctx.buf(f"rope.cos.{id(self)}", (ctx.n, half), torch.float32)
        sin = ctx.buf(f"rope.sin.{id(self)}", (ctx.n, half), torch.float32)
        K.rope_tables(cos, sin, ctx.positions[:ctx.n], self.head_dim, self.theta)
        ctx.scratch[("rotary", id(self))] = (cos, sin)

    def tables(self, ctx):
        return ctx.scratch[("rotary", id(self))]
