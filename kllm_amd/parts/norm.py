"""RMSNorm, alone or fused with the residual add that precedes it.

out = x * rsqrt(mean(x^2) + eps) * w, all in 32-bit; eps is added to the mean
inside the root and the weight multiplies after normalisation
(backend/model.cu:101-122; fused with the add: :144-165).

Parameters: ``size`` (channels), ``eps``.  Tensor: ``<prefix>.weight`` [size].
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, register_part
from .spec import WeightSpec


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    graph_safe = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.size = int(self.param("size"))
        self.eps = float(self.param("eps"))
        self.weight = None

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("weight"), (self.size,), "vector")]

    def bind(self, weights):
        self.weight = weights[self.tensor_name("weight")]

    def forward(self, ctx, x, delta=None, rows=None, tag="xn"):
        """Normalised rows in the compute dtype.  ``delta`` is added into x
        first (and x is updated) unless ``rows`` selects rows to read."""
        n = rows.numel() if rows is not None else x.shape[0]
        out = ctx.buf(tag, (n, self.size), self.runtime.dtype)
        K.add_rmsnorm(x, delta=delta, weight=self.weight, out=out, rows=rows, eps=self.eps)
        return out

    def add(self, ctx, x, delta):
        K.add_rmsnorm(x, delta=delta, write_x=True)
        return x
