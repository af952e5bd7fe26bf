"""Position encodings that act on q and k as a rotation of pairs.

``rotary``: inv_i = 1 / theta^(2i / rotary_dim), angle = position * inv_i, both in 32-bit
(engine/input_prep.cpp:17-30); pairs are (i, i + rotary_dim/2) for "half_split", the reference's
interleave=false (kernels/rope.cpp:38-48), or (2i, 2i + 1) for "interleaved"; dims beyond rotary_dim
pass unchanged.  ``none`` rotates nothing.

A position part hands the mixer cos/sin rows for the step's tokens, as the reference feeds its graph
(models/qwen3.py:226-227); they are made once per step and shared by all layers that use the same
part settings.
"""
from __future__ import annotations

import numpy as np
import torch

from ..kernels import ops
from .base import register_part

PAIRINGS = {"half_split": 0, "interleaved": 1}


@register_part("position", "rotary")
class Rotary:
    capturable = True

    def __init__(self, spec, builder):
        self.rotary_dim = int(spec.params["rotary_dim"])
        self.theta = float(spec.params["theta"])
        self.pairing = str(spec.params.get("pairing", "half_split"))
        if self.pairing not in PAIRINGS:
            raise ValueError(f"rotary pairing {self.pairing!r} is not one of {sorted(PAIRINGS)}")
        if self.rotary_dim <= 0 or self.rotary_dim % 2:
            raise ValueError(f"rotary_dim = {self.rotary_dim} must be positive and even")
        half = self.rotary_dim // 2
        i = np.arange(half, dtype=np.float32)
        inv = np.float32(1.0) / np.power(np.float32(self.theta), np.float32(2.0) * i / np.float32(self.rotary_dim))
        self.inv_freq = torch.from_numpy(inv.astype(np.float32)).to(builder.device)
        self._key = ("rotary", self.rotary_dim, self.theta)

    def tables(self, ctx):
        if self._key not in ctx.memo:
            ctx.memo[self._key] = ops.rope_table(ctx.positions, self.inv_freq)
        return ctx.memo[self._key]


@register_part("position", "none")
class NoPosition:
    capturable = True
    rotary_dim, pairing = 0, "half_split"

    def __init__(self, spec, builder):
        pass

    def tables(self, ctx):
        return None
