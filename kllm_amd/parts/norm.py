"""RMSNorm, alone or fused with the residual add that precedes it.

out = x * rsqrt(mean(x^2) + eps) * w, all in 32-bit; eps is added to the mean
inside the root and the weight multiplies after normalisation
(backend/model.cu:101-122; fused with the add: :144-165).

Parameters: ``size`` (channels), ``eps``.  Tensor: ``<prefix>.weight`` [size].
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Normed, Part, register_part
from .spec import WeightSpec


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    graph_safe = True
    records_launches = True
    fusable = True     # a product's epilogue may do the addition, its consumer the row scale

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.size = int(self.param("size"))
        self.eps = float(self.param("eps"))
        self.weight = None

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("weight"), (self.size,), "vector")]

    def bind(self, weights):
        self.weight = weights[self.tensor_name("weight")]

    def forward(self, ctx, x, delta=None, rows=None, tag="xn", normed_ok=False):
        """Normalised rows in the compute dtype.  ``delta`` is added into x
        first (and x is updated) unless ``rows`` selects rows to read.  A
        ``delta`` that is a ``Normed`` says that x already holds the sum: it
        is handed on to a consumer that takes it (``normed_ok``), or the rows
        of x are normalised here."""
        if isinstance(delta, Normed):
            if delta.norm is not self:
                raise ValueError("norm: the residual product was made for another norm")
            if normed_ok and rows is None:
                return delta
            delta = None
        n = rows.numel() if rows is not None else x.shape[0]
        out = ctx.buf(tag, (n, self.size), self.runtime.dtype)
        K.add_rmsnorm(x, delta=delta, weight=self.weight, out=out, rows=rows, eps=self.eps)
        return out

    def add(self, ctx, x, delta):
        if not isinstance(delta, Normed):        # a Normed's sum is in x already
            K.add_rmsnorm(x, delta=delta, write_x=True)
        return x
