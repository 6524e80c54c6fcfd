"""Causal self-attention over a paged cache, with grouped KV heads.

q, k, v projections without bias; rotary on q and k before the keys are
cached; for the token at position p, head h reads KV head h // (H/KV) and keys
[0, p] (or the last ``window`` of them); scores times 1/sqrt(head_dim),
softmax in 32-bit, values, output projection
(backend/model.cu:1090-1104, :343-408, :224-225).

Parameters: ``hidden``, ``heads``, ``kv_heads``, ``head_dim``, ``window``
(0: all keys), ``position`` (a PartSpec or None), ``own_kv`` (False: the run
reads keys and values that another run cached and has no k/v projections).
Tensors: ``<prefix>.{q,k,v,o}_proj.weight``.  The three input projections are
kept as one matrix so that a step reads one weight for them.
"""

from __future__ import annotations

import math

import torch

from .. import kernels as K
from .base import Normed, Part, register_part
from .linear import linear, linear_into, tiled_copy
from .spec import CacheNeed, WeightSpec


@register_part("mixer", "attention")
class CausalSelfAttention(Part):
    graph_safe = True
    records_launches = True
    takes_normed = True     # the q, k, v product of a decode batch applies the norm's row scale itself
    fills_sink = True       # the output projection of a decode batch adds itself to the residual stream
    # How the attention kernels want a step's spans listed: the tokens of spans of at most
    # SHORT_SPAN tokens one by one (for the kernel that cuts a token's keys into slices),
    # longer spans in blocks of QUERY_BLOCK tokens (for the prompt kernel).
    step_lists_key = "attention.spans"
    SHORT_SPAN = 4
    QUERY_BLOCK = K.PREFILL_QUERY_BLOCK

    def step_lists(self, starts, lens):
        short, blocks = [], []
        for s, n in enumerate(lens):
            a = starts[s]
            if n <= self.SHORT_SPAN:
                short.extend(range(a, a + n))
            else:
                for t in range(a, a + n, self.QUERY_BLOCK):
                    blocks += [t, s]
        return {"short": short, "blocks": blocks}

    def step_values(self, starts, lens, positions):
        """How many keys the step's query blocks read, all together and the longest block
        alone: a whole prompt's blocks read more and more, a portion far into its context reads
        many in every block, and the prompt kernel is chosen by that."""
        total = longest = 0
        for pos, n in zip(positions, lens):
            if n <= self.SHORT_SPAN:
                continue
            for first in range(0, n, self.QUERY_BLOCK):
                last = pos + min(first + self.QUERY_BLOCK, n)          # keys [0, last) are before the block's end
                keys = min(last, self.window + self.QUERY_BLOCK) if self.window else last
                total += keys
                longest = max(longest, keys)
        return {"keys_total": total, "keys_longest": longest}

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = int(self.param("hidden"))
        self.heads = int(self.param("heads"))
        self.kv_heads = int(self.param("kv_heads"))
        self.head_dim = int(self.param("head_dim"))
        self.window = int(self.param("window", 0) or 0)
        self.step_values_key = f"attention.keys.window{self.window}"     # layers with the same window read alike
        self.own_kv = bool(self.param("own_kv", True))
        if self.heads % self.kv_heads:
            raise ValueError(f"attention: {self.heads} heads are not a multiple of {self.kv_heads} KV heads")
        if self.head_dim % 2 or self.head_dim > 256:
            raise ValueError(f"attention: head_dim {self.head_dim} must be even and at most 256")
        pos = self.param("position", None)
        self.position = runtime.shared_part("position", pos) if pos is not None else None
        # How the position part wants a head rotated (default: the whole head, halves paired, which
        # is what the fused epilogues of the small-batch products do; anything else goes through
        # the separate rotate-and-append kernel, which takes the pairing as arguments).
        rotates = self.position is not None and hasattr(self.position, "tables")
        self.rotary_dim = int(getattr(self.position, "rotary_dim", self.head_dim)) if rotates else self.head_dim
        self.interleaved = bool(getattr(self.position, "interleaved", False)) if rotates else False
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError(f"attention: rotary dimension {self.rotary_dim} of a head of {self.head_dim}")
        self.plain_rotation = self.rotary_dim == self.head_dim and not self.interleaved
        self.scale = 1.0 / math.sqrt(self.head_dim)
        self.q_dim = self.heads * self.head_dim
        self.kv_dim = self.kv_heads * self.head_dim
        self.w_in = None
        self.w_o = None
        self._tiled = {}

    def weight_specs(self):
        specs = [WeightSpec(self.tensor_name("q_proj.weight"), (self.q_dim, self.hidden))]
        if self.own_kv:
            specs += [WeightSpec(self.tensor_name("k_proj.weight"), (self.kv_dim, self.hidden)),
                      WeightSpec(self.tensor_name("v_proj.weight"), (self.kv_dim, self.hidden))]
        specs.append(WeightSpec(self.tensor_name("o_proj.weight"), (self.hidden, self.q_dim)))
        return specs

    def bind(self, weights):
        names = ["q_proj.weight"] + (["k_proj.weight", "v_proj.weight"] if self.own_kv else [])
        mats = [weights[self.tensor_name(n)] for n in names]
        self.w_in = torch.cat(mats, dim=0).contiguous() if len(mats) > 1 else mats[0]
        self.w_o = weights[self.tensor_name("o_proj.weight")]
        # second copies for decode batches, in the order that kernel reads them (not tensors of
        # the part in the sense of read_bytes: a step reads one copy or the other)
        self._tiled = {}
        if self.plain_rotation:
            heads = K.Rope(None, None, True if self.own_kv else None, None, None, None, 0, self.heads, self.kv_heads,
                           self.head_dim)
            self._tiled["in"] = tiled_copy(self.runtime, self.w_in, K.LINEAR_ROPE, heads)
        self._tiled["o"] = tiled_copy(self.runtime, self.w_o, K.LINEAR_PARTS)

    def cache_need(self):
        return CacheNeed("paged", kv_heads=self.kv_heads, head_dim=self.head_dim, window=self.window)

    def flops(self, tokens, keys_read=0.0):
        # the projections, and per key read a score and a value product for every head
        return super().flops(tokens) + 4.0 * self.heads * self.head_dim * keys_read

    def check_cache(self, page_size):
        # The kernel that takes every size walks a chunk of up to 256 keys at a time, whole
        # pages of them; the faster kernels are chosen per step where the sizes fit them.
        if not 1 <= page_size <= K.GENERIC_MAX_PAGE_SIZE:
            raise ValueError(f"attention: pages of {page_size} tokens are not built "
                             f"(1 to {K.GENERIC_MAX_PAGE_SIZE})")

    def _fused_tiles(self, n):
        """Tiles per workgroup of the decode-batch kernel for the input projections of n
        tokens, or 0 where it is not taken."""
        if (self.runtime.dtype != torch.bfloat16 or n > K.FUSED_ROPE_BEST_ROWS or not self.plain_rotation
                or self.runtime.options.get("no_fused_linear")):
            return 0
        return K.fused_linear_tiles(n, self.w_in.shape[0], self.hidden)

    def forward(self, ctx, xn, cache, sink=None):
        dtype = self.runtime.dtype
        if isinstance(xn, Normed):
            n = xn.rows
            opts = self.runtime.options
            gemv = (K.gemv_fits(n, self.w_in.shape[0], self.hidden, dtype) and n <= K.normed_max_rows()
                    and not opts.get("no_fused_gemv") and self.plain_rotation and xn.xw is None)
            scaled = (not gemv and xn.xw is not None and self._fused_tiles(n) > 0)
            # the small-batch kernel below normalises while it stages its input, the decode-batch
            # kernel scales its sums by the row
            xn = xn.kernel_input() if gemv else xn.scaled_rows() if scaled else xn.materialize(ctx)
        n = xn.shape[0]
        writes = self.own_kv
        if writes != bool(cache.write):
            raise ValueError("attention: a run must write its cache exactly when it has k/v projections")
        q = ctx.buf("attn.q", (n, self.q_dim), dtype)
        cos = sin = None
        if self.position is not None and hasattr(self.position, "tables"):
            cos, sin = self.position.tables(ctx)
        plain_rotation = self.plain_rotation
        pages = cache.pages if writes else None
        opts = self.runtime.options
        if (K.gemv_fits(n, self.w_in.shape[0], self.hidden, dtype) and not opts.get("no_fused_gemv") and plain_rotation
                and not isinstance(xn, K.ScaledRows)):
            # few tokens: projections, rotation and append in one launch
            K.gemv_rope_append(xn, self.w_in, q, cos, sin, pages, ctx.positions, ctx.span_of_token,
                               cache.block_table, cache.page_size, self.heads, self.kv_heads,
                               self.head_dim)
        elif self._fused_tiles(n) > 0:
            # a decode batch: the same on the matrix cores
            K.fused_linear(self._tiled.get("in") or self.w_in, q, K.LINEAR_ROPE, x=xn,
                           tiles_per_wg=self._fused_tiles(n),
                           rope=K.Rope(cos, sin, pages, ctx.positions, ctx.span_of_token, cache.block_table,
                                       cache.page_size, self.heads, self.kv_heads, self.head_dim))
        else:
            qkv = linear(ctx, xn, self.w_in, "attn.qkv")
            K.rope_append(qkv, q, cos, sin, pages, ctx.positions, ctx.span_of_token,
                          cache.block_table, cache.page_size, self.heads, self.kv_heads,
                          self.head_dim, self.rotary_dim, self.interleaved)
        out = ctx.buf("attn.out", (n, self.q_dim), dtype)
        self.attend(ctx, q, out, cache)
        if sink is not None:
            normed = linear_into(ctx, out, self.w_o, sink, "attn.proj", w_tiled=self._tiled.get("o"))
            if normed is not None:
                return normed
        return linear(ctx, out, self.w_o, "attn.proj")

    def attend(self, ctx, q, out, cache):
        """Choose the attention kernels by the spans' lengths: tokens of short
        spans (decode tokens) go to the kernel that splits a token's keys over
        many waves, longer spans to the prompt kernel in blocks of 128 queries
        (both on the matrix cores, in bfloat16 or with 32-bit operands); sizes
        those kernels do not take go to the kernel that takes every size."""
        mode = self.runtime.options.get("attention", "auto")
        if q.dtype == torch.bfloat16:
            fast = cache.page_size % 16 == 0 and self.head_dim in K.DECODE_HEAD_DIMS
            prompt_ok = self.head_dim in K.PREFILL_HEAD_DIMS
        else:
            fast = prompt_ok = K.attn_f32_fits(self.head_dim, cache.page_size)
        fast = fast and mode != "generic"
        if not fast:
            K.attn_generic(q, out, cache.pages, ctx.positions, ctx.span_of_token, cache.block_table,
                           cache.page_size, self.heads, self.kv_heads, self.head_dim, self.window,
                           self.scale)
            return
        n = q.shape[0]
        short = ctx.lists.get("attention.spans.short")
        blocks = ctx.lists.get("attention.spans.blocks")
        n_short = short.numel() if short is not None else 0
        n_blocks = blocks.numel() // 2 if blocks is not None else 0
        if n_short + n_blocks == 0 or (n_blocks and not prompt_ok):   # a context built by hand may carry no lists
            self._decode(ctx, q, out, cache, None, n)   # token by token
            return
        if n_short:
            self._decode(ctx, q, out, cache, None if n_short == n else short, n_short)
        if n_blocks:
            total, longest = self._keys_read(ctx)
            part = None
            slices = (1 if self.runtime.options.get("no_attention_slices")
                      else K.attn_prefill_slices(n_blocks, self.heads, self.head_dim, q.dtype))
            if slices > 1:     # few blocks of a large head: their keys in slices over workgroups, merged in the same call
                part = ctx.buf("attn.block_part", (n * self.heads * slices * (self.head_dim + 2),), torch.float32)
            K.attn_prefill(q, out, cache.pages, blocks, n_blocks, ctx.span_start,
                           ctx.span_pos, cache.block_table, cache.page_size, self.heads,
                           self.kv_heads, self.head_dim, self.window, self.scale, total, longest, part=part,
                           nslices=slices)

    def _keys_read(self, ctx):
        """The step's key counts (see ``step_values``), as the engine worked them out for this
        step, or from the host's copies of the spans for a context built by hand."""
        v, key = ctx.values, self.step_values_key
        if key + ".keys_total" in v:
            return v[key + ".keys_total"], v[key + ".keys_longest"]
        own = self.step_values(ctx.h_span_start, ctx.h_span_len, ctx.h_span_pos)
        return own["keys_total"], own["keys_longest"]

    def _decode(self, ctx, q, out, cache, token_list, count):
        n = q.shape[0]
        # The block table's width bounds the keys of the step's longest request.  It is rounded up
        # to a power of two of pages (from 8), as recorded steps round theirs: a step then cuts
        # the keys alike, and gives the same sums bit for bit, whether it runs directly or as
        # a replayed recording with a wider table.
        pages = 8
        while pages < cache.block_table.shape[1]:
            pages *= 2
        max_keys = pages * cache.page_size
        if self.window:
            max_keys = min(max_keys, self.window + cache.page_size)
        nslices = K.attn_decode_slices(count, self.kv_heads, self.heads, self.head_dim, q.dtype, max_keys)
        part = ctx.buf("attn.part", (n * self.heads * nslices * (self.head_dim + 2),), torch.float32)
        K.attn_decode(q, out, part, cache.pages, ctx.positions, ctx.span_of_token, cache.block_table,
                      cache.page_size, self.heads, self.kv_heads, self.head_dim, self.window,
                      self.scale, nslices, token_list, count)
