"""The arrangement of a layer's parts around the residual stream.

``pre_norm``: x += mixer(norm(x)); x += feed_forward(norm(x)) (models/qwen3.py:254-287).  The residual
stream x is float32; a branch's output is not added at once but handed on as ``pending``, and the next
norm adds it in the same pass in which it norms (the sum is made in 32-bit and written back to x).
A branch may hand its output on as float32 planes [P, n, width] of partial sums if ``ctx.planes_ok`` says
that the norm which reads it adds them up; a part that ignores the flag returns [n, width] as ever.
"""
from __future__ import annotations

from .base import cache_needs, register_part


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
    def takes_planes(self) -> bool:
        """Whether ``pending`` may come as float32 planes [P, n, width] (the first norm adds them up)."""
        return bool(getattr(self.mixer_norm, "takes_planes", False))

    def forward(self, x, pending, ctx):
        h = self.mixer_norm(x, delta=pending, update=pending is not None)
        ctx.planes_ok = bool(getattr(self.feed_forward_norm, "takes_planes", False))
        a = self.mixer.forward(h, ctx)
        h = self.feed_forward_norm(x, delta=a, update=True)
        ctx.planes_ok = ctx.next_takes_planes
        out = self.feed_forward.forward(h, ctx)
        ctx.planes_ok = False
        return x, out
