"""The arrangement of a layer's parts around the residual stream.

``pre_norm``: x += mixer(norm(x)); x += feed_forward(norm(x)) (models/qwen3.py:254-287).  The residual
stream x is float32.  A branch's output is never added by a kernel of its own: it goes into a
``ResidualSink`` (parts/residual.py), and either the norm that reads x next adds it in the pass in which it
norms (the sum is made in 32-bit and written back to x), or the branch's last product does both.  So the
block gets its first norm's output from whoever ran before it, and returns the output of the norm that comes
after it.
"""
from __future__ import annotations

from .base import cache_needs, register_part
from .residual import ResidualSink, run_branch


@register_part("block", "pre_norm")
class PreNormBlock:
    def __init__(self, spec, builder):
        self.mixer_norm = builder.build(spec.parts["mixer_norm"])
        self.mixer = builder.build(spec.parts["mixer"])
        self.feed_forward_norm = builder.build(spec.parts["feed_forward_norm"])
        self.feed_forward = builder.build(spec.parts["feed_forward"])

    @property
    def capturable(self) -> bool:
        return all(getattr(p, "capturable", False) for p in (self.mixer_norm, self.mixer, self.feed_forward_norm,
                                                              self.feed_forward))

    @staticmethod
    def cache_needs(spec):
        return cache_needs(spec.parts["mixer"])

    @property
    def entry_norm(self):
        return self.mixer_norm

    def forward(self, x, h, ctx, sink):
        h = run_branch(self.mixer, h, ctx, ResidualSink(x, self.feed_forward_norm))
        return run_branch(self.feed_forward, h, ctx, sink)
