"""The gated feed-forward: down( silu(gate(h)) * up(h) ), silu(z) = z / (1 + exp(-z)), with gate and up
joined into one [2I, H] product (models/qwen3.py:276-287; kernels/elementwise.cpp:529-583)."""
from __future__ import annotations

from .base import register_part
from .linear import Linear


@register_part("feed_forward", "gated_silu")
class GatedSiluFeedForward:
    capturable = True

    def __init__(self, spec, builder):
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        bias = lambda name: builder.tensor(spec, name) if name in spec.tensors else None
        self.gate_up = Linear(builder.tensor(spec, "gate_up"), bias("gate_up_bias"))
        self.down = Linear(builder.tensor(spec, "down"), bias("down_bias"))
        if self.gate_up.weight.shape != (2 * self.inter, self.hidden) or self.down.weight.shape != (self.hidden, self.inter):
            raise ValueError(f"feed-forward: weights {tuple(self.gate_up.weight.shape)}, {tuple(self.down.weight.shape)} "
                             f"do not fit hidden {self.hidden}, intermediate {self.inter}")

    takes_sink = True

    def forward(self, h, ctx, sink=None):
        return self.down(self.gate_up.gated(h), sink=sink)
