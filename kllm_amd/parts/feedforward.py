"""Gated feed-forward: down(act(gate(x)) * up(x)), no biases
(backend/model.cu:1112-1115; SiLU: :477-483).

Parameters: ``hidden``, ``intermediate``, ``activation`` ("silu"; also
"gelu_tanh": every kernel with a gate takes the activation as an argument).  Tensors:
``<prefix>.{gate,up,down}_proj.weight``.  Gate and up are kept as one matrix
[2*intermediate, hidden] (gate rows first).
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Normed, Part, register_part
from .linear import linear, linear_into, tiled_copy
from .spec import WeightSpec


@register_part("feed_forward", "gated_mlp")
class GatedFeedForward(Part):
    graph_safe = True
    records_launches = True
    takes_normed = True     # the gate and up products of a decode batch apply the norm's row scale
    fills_sink = True       # the down projection of a decode batch adds itself to the residual stream

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = int(self.param("hidden"))
        self.intermediate = int(self.param("intermediate"))
        act = self.param("activation", "silu")
        if act not in K.ACTIVATIONS:
            raise ValueError(f"gated_mlp: activation {act!r} is not built (one of {sorted(K.ACTIVATIONS)})")
        self.act = K.ACTIVATIONS[act]
        self.w_gu = None
        self.w_down = None
        self._tiled = {}

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("gate_proj.weight"), (self.intermediate, self.hidden)),
                WeightSpec(self.tensor_name("up_proj.weight"), (self.intermediate, self.hidden)),
                WeightSpec(self.tensor_name("down_proj.weight"), (self.hidden, self.intermediate))]

    def bind(self, weights):
        self.w_gu = torch.cat([weights[self.tensor_name("gate_proj.weight")],
                               weights[self.tensor_name("up_proj.weight")]], dim=0).contiguous()
        self.w_down = weights[self.tensor_name("down_proj.weight")]
        # second copies for decode batches, in the order that kernel reads them
        self._tiled = {"gu": tiled_copy(self.runtime, self.w_gu, K.LINEAR_SWIGLU),
                       "down": tiled_copy(self.runtime, self.w_down, K.LINEAR_PARTS)}

    def _gate_in_tiles(self, n, dtype):
        """Decode batches whose gate runs in the tiled product's epilogue: more than 32 rows
        where the tiles of 64 gate columns give three fifths of the CUs a workgroup, more
        than 16 where they give seven eighths (measured against the product in slices of K and
        a separate gate, in us: 64 rows, intermediate 14,336 x 4,096: 59 / 83; 11,008: 56 / 68;
        5,632 x 2,048: 30 / 23; 32 rows: 58 / 66; 54 / 53; 17 rows, 14,336: 57 / 61)."""
        if dtype != torch.bfloat16 or n <= 16:
            return False
        tiles, cus = -(-self.intermediate // 64), K.device_cus()
        return (n > 32 and 5 * tiles >= 3 * cus) or 8 * tiles >= 7 * cus

    def forward(self, ctx, xn, sink=None):
        dtype, opts = self.runtime.dtype, self.runtime.options
        n = xn.rows if isinstance(xn, Normed) else xn.shape[0]
        gemv = K.gemv_fits(n, 2 * self.intermediate, self.hidden, dtype) and not opts.get("no_fused_gemv")
        if gemv and isinstance(xn, Normed) and xn.xw is not None:
            gemv = False       # the producer was the decode-batch kernel: its consumer is, too
        tiles = (K.fused_linear_tiles(n, 2 * self.intermediate, self.hidden)
                 if dtype == torch.bfloat16 and n <= K.FUSED_SWIGLU_BEST_ROWS else 0)
        fused = not gemv and tiles > 0 and not opts.get("no_fused_linear")
        if isinstance(xn, Normed):     # the small-batch kernel below normalises while it stages its input,
            # the decode-batch kernel scales its sums by the row
            xn = (xn.kernel_input() if gemv and n <= K.normed_max_rows()
                  else xn.scaled_rows() if fused and xn.xw is not None else xn.materialize(ctx))
        h = ctx.buf("ffn.h", (n, self.intermediate), dtype)
        if gemv:
            K.gemv_swiglu(xn, self.w_gu, h, self.act)   # few tokens: both products and the gate in one launch
        elif fused:
            # a decode batch: the same on the matrix cores
            K.fused_linear(self._tiled.get("gu") or self.w_gu, h, K.LINEAR_SWIGLU, x=xn, act=self.act,
                           tiles_per_wg=tiles)
        elif ((n > 128 or self._gate_in_tiles(n, dtype))
              and self.runtime.options.get("gemm") != "library"
              and self.hidden % (8 if xn.dtype == torch.bfloat16 else 4) == 0):
            # prompts: the gate in the product's epilogue (up to 128 rows the product with K
            # in slices and a separate gate is faster: the epilogue cannot split K), and decode
            # batches against wide feed-forwards
            K.gemm_swiglu(xn, self.w_gu, h, self.act)
        else:
            gu = linear(ctx, xn, self.w_gu, "ffn.gu")
            K.silu_mul(gu, h, self.act)
        if sink is not None:
            normed = linear_into(ctx, h, self.w_down, sink, "ffn.down", w_tiled=self._tiled.get("down"))
            if normed is not None:
                return normed
        return linear(ctx, h, self.w_down, "ffn.down")
