"""Token embedding and output head.

Embedding: x[t, :] = E[id_t, :], no scaling (backend/model.cu:89-95,
:1056-1060).  Head: logits = xn . W^T in float32 for the wanted rows
(:1185-1188).  The head names its own tensor; a tied head simply names the
embedding's table (the reference resolves tying offline by copying it:
tools/convert_hf.py:81-82).
"""

from __future__ import annotations

import torch

from .. import kernels as K
from .base import Part, register_part
from .linear import linear, tiled_copy
from .spec import WeightSpec


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.vocab = int(self.param("vocab"))
        self.hidden = int(self.param("hidden"))
        self.table = None

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("weight"), (self.vocab, self.hidden))]

    def bind(self, weights):
        self.table = weights[self.tensor_name("weight")]

    def read_bytes(self, tokens):
        return {self.table.data_ptr(): tokens * self.hidden * self.table.element_size()}   # one row per token

    def flops(self, tokens, keys_read=0.0):
        return 0.0

    def forward(self, ctx, token_ids):
        x = ctx.buf("x", (ctx.n, self.hidden), torch.float32)
        if ctx.sampled is not None and ctx.token_from is not None:
            K.embed(x, self.table, token_ids, ctx.token_from, ctx.sampled)
        else:
            K.embed(x, self.table, token_ids)
        return x


@register_part("head", "linear_head")
class LinearHead(Part):
    graph_safe = True
    records_launches = True

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.vocab = int(self.param("vocab"))
        self.hidden = int(self.param("hidden"))
        self.weight = None

    def weight_specs(self):
        return [WeightSpec(self.tensor_name("weight"), (self.vocab, self.hidden))]

    def bind(self, weights):
        self.weight = weights[self.tensor_name("weight")]
        self._tiled = {"w": tiled_copy(self.runtime, self.weight, K.LINEAR_PARTS)}   # for decode batches

    def forward(self, ctx, xn_rows):
        return linear(ctx, xn_rows, self.weight, "logits", split=False, w_tiled=self._tiled.get("w"))
