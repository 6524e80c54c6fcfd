"""Arrangements of a layer's parts.

``pre_norm``: a = h + Mixer(Norm1(h)); h' = a + FeedForward(Norm2(a))
(backend/model.cu:1083-1117).  As in the reference, a sub-layer's output is
not added to the residual stream by a pass of its own: it travels as
``pending`` into the next norm, which adds it while it normalises (:1084,
:1105, :1117).  For decode batches even that launch goes: where the parts
allow it, a sub-layer's last product adds its sums to the stream in its
epilogue (``ResidualSink``) and the next sub-layer's first product applies the
norm's row scale to its own sums (``Normed``).
"""

from __future__ import annotations

from .base import Part, ResidualSink, call_part, make_part, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Part):
    records_launches = True     # the arrangement itself launches nothing; its parts are called each in its own way

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        layer = self.param("layer")
        self.norm_mixer = make_part("norm", layer.norm_mixer, runtime)
        self.mixer = make_part("mixer", layer.mixer, runtime)
        self.norm_ff = make_part("norm", layer.norm_feed_forward, runtime)
        self.feed_forward = make_part("feed_forward", layer.feed_forward, runtime)

    def parts(self):
        return [self.norm_mixer, self.mixer, self.norm_ff, self.feed_forward]

    def children(self):
        return self.parts()

    @property
    def graph_safe(self):
        return all(p.graph_safe for p in self.parts())

    def weight_specs(self):
        return [s for p in self.parts() for s in p.weight_specs()]

    def bind(self, weights):
        for p in self.parts():
            p.bind(weights)

    def cache_need(self):
        return self.mixer.cache_need()

    def read_bytes(self, tokens):
        out = {}
        for p in self.parts():
            out.update(p.read_bytes(tokens))
        return out

    def flops(self, tokens, keys_read=0.0):
        return sum(p.flops(tokens, keys_read) for p in self.parts())

    takes_next_norm = True

    def first_norm(self):
        """The norm that takes what the layer before this one leaves pending."""
        return self.norm_mixer

    @staticmethod
    def _normed_ok(ctx, norm, consumer):
        return {"normed_ok": True} if (norm.fusable and consumer.takes_normed and ctx.taps is None) else {}

    @staticmethod
    def _sink(ctx, x, producer, norm):
        if norm is None or not (producer.fills_sink and norm.fusable) or ctx.taps is not None:
            return {}
        return {"sink": ResidualSink(x, norm)}

    def forward(self, ctx, x, pending, cache, next_norm=None):
        """``next_norm``: the norm that will take this layer's pending output
        (the next layer's first norm), if the caller knows it; the feed-forward
        may then add its output to x itself."""
        xn = call_part(self.norm_mixer, self.norm_mixer.forward, ctx, x, delta=pending,
                       **self._normed_ok(ctx, self.norm_mixer, self.mixer))
        delta = call_part(self.mixer, self.mixer.forward, ctx, xn, cache, **self._sink(ctx, x, self.mixer, self.norm_ff))
        xn = call_part(self.norm_ff, self.norm_ff.forward, ctx, x, delta=delta,
                       **self._normed_ok(ctx, self.norm_ff, self.feed_forward))
        pending = call_part(self.feed_forward, self.feed_forward.forward, ctx, xn,
                            **self._sink(ctx, x, self.feed_forward, next_norm))
        return x, pending
