"""The two ends of a decoder: token ids -> residual stream, and final hidden rows -> logits."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import register_part
from .linear import Linear


@register_part("embedding", "token_table")
class TokenEmbedding:
    capturable = True

    """x[t, :] = E[id_t, :] widened to float32 (engine/engine.cpp:332-357).  Unlike the reference, an id
    outside the table is not mapped to row 0: the step refuses it before anything runs."""

    def __init__(self, spec, builder):
        self.table = builder.tensor(spec, "table")
        self.vocab, self.hidden = int(spec.params["vocab_size"]), int(spec.params["hidden_size"])
        if self.table.shape != (self.vocab, self.hidden):
            raise ValueError(f"embedding table {tuple(self.table.shape)} is not [{self.vocab}, {self.hidden}]")

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return ops.embed(self.table, token_ids)


@register_part("head", "linear")
class LinearHead:
    capturable = True

    """logits = h W^T in float32; W is lm_head.weight, or the embedding table when the head is tied
    (models/qwen3.py:89-95, 162-165; engine/engine.cpp:403-485)."""

    def __init__(self, spec, builder):
        self.linear = Linear(builder.tensor(spec, "weight"))
        self.vocab = int(spec.params["vocab_size"])
        if self.linear.weight.shape != (self.vocab, int(spec.params["hidden_size"])):
            raise ValueError(f"head weight {tuple(self.linear.weight.shape)} does not fit")

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.linear(h, out_dtype=torch.float32)
