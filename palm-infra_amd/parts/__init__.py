"""The parts that layers are put together from: norms, position encodings, mixers, feed-forwards,
blocks, and the embedding and head at the two ends."""
from .base import (CATEGORIES, Builder, StepContext, cache_needs, context_ints, make_context, part_class, register_part)
from . import norm, position, attention, feedforward, block, embedding  # noqa: F401  (registers the kinds)
from .linear import Linear
from .residual import Prenormed, ResidualSink, as_tensor, run_branch

__all__ = ["CATEGORIES", "Builder", "StepContext", "cache_needs", "context_ints", "make_context", "part_class", "register_part", "Linear"]
