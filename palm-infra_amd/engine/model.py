"""A decoder built from a description: embedding, layers in their run order, final norm, head.

This replaces the reference's graph builder and executor for the one path a request takes
(models/qwen3.py:171-251, graph/execute.cpp:244-833): the description is walked directly, every part
launches its kernels, and nothing is serialised.  The model knows no architecture by name.
"""
from __future__ import annotations

import torch

from ..config.spec import ModelSpec
from ..parts import Builder, ResidualSink, cache_needs


class DecoderModel:
    def __init__(self, spec: ModelSpec, weights, dtype: torch.dtype, device):
        self.spec, self.dtype, self.device = spec, dtype, torch.device(device)
        builder = Builder(weights, dtype, device)
        self.embedding = builder.build(spec.embedding)
        self.layers = [builder.build(layer) for layer in spec.layers]
        self.final_norm = builder.build(spec.final_norm)
        self.head = builder.build(spec.head)
        self.order = spec.order
        self.weights = weights

    @property
    def capturable(self) -> bool:
        """Whether a decode step of this model may be recorded into a HIP graph: every part says of itself
        that it launches the same kernels whatever the step holds (a part that plans on the host does not)."""
        parts = [self.embedding, *self.layers, self.final_norm, self.head]
        return all(getattr(p, "capturable", False) for p in parts)

    def cache_plan(self):
        """For each entry of the run order: what it keeps per sequence, and whose cache it reads."""
        needs, shares = [], []
        for call in self.order:
            if call.cache_of is None:
                needs.append(cache_needs(self.spec.layers[call.layer]))
                shares.append(None)
            else:
                needs.append([])
                shares.append(call.cache_of)
        return needs, shares

    def forward(self, ctx, cache, want_rows: torch.Tensor | None) -> torch.Tensor:
        """Run the step's tokens through all layers; logits (float32) at the rows ``want_rows`` of the
        packed tokens (all rows if None)."""
        x = self.embedding.forward(ctx.token_ids)
        if not self.order:
            return self.head.forward(self.final_norm(x, rows=want_rows))
        # a layer gets its first norm's output and returns the output of the norm after it: the next layer's
        # first norm, at the end the final norm over the wanted rows
        h = self.layers[self.order[0].layer].entry_norm(x)
        for i, call in enumerate(self.order):
            ctx.layer_cache = cache.layer_caches[i]
            if i + 1 < len(self.order):
                sink = ResidualSink(x, self.layers[self.order[i + 1].layer].entry_norm)
            else:
                sink = ResidualSink(x, self.final_norm, rows=want_rows)
            h = self.layers[call.layer].forward(x, h, ctx, sink)
        ctx.layer_cache = None
        return self.head.forward(h)
