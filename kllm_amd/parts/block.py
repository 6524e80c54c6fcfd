"""Arrangements of a layer's parts.

``pre_norm``: a = h + Mixer(Norm1(h)); h' = a + FeedForward(Norm2(a))
(backend/model.cu:1083-1117).  As in the reference, a sub-layer's output is
not added to the residual stream by a pass of its own: it travels as
``pending`` into the next norm, which adds it while it normalises (:1084,
:1105, :1117).
"""

from __future__ import annotations

from .base import Part, make_part, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Part):
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

    def forward(self, ctx, x, pending, cache):
        xn = self.norm_mixer.forward(ctx, x, delta=pending)
        delta = self.mixer.forward(ctx, xn, cache)
        xn = self.norm_ff.forward(ctx, x, delta=delta)
        pending = self.feed_forward.forward(ctx, xn)
        return x, pending
