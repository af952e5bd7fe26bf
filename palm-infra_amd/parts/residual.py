"""How a branch's output reaches the residual stream and its next reader.

A block hands each branch (mixer, feed-forward) a ``ResidualSink``: the residual stream x and the norm that
reads x next.  The plain way to use it is ``sink.finish(delta)``: the norm adds the branch output to x and
norms the sum, one kernel.  A branch whose last step is a ``Linear`` can pass the sink on to it
(``linear(o, sink=sink)``); for a step of few rows the product then does the add and the norm's elementwise
part itself and returns ``Prenormed`` rows, and the norm's kernel is not needed at all.

``Prenormed`` rows are x * w in the activation type, still lacking the row factor 1 / sqrt(mean(x^2) + eps),
together with the pieces of each row's sum of squares.  A ``Linear`` takes them as they are (a product of
rows times a factor is the factor times the product); anything else calls ``materialize()``.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import ops


@dataclass
class Prenormed:
    values: torch.Tensor     # [n, width], activation type: x * w
    ss: torch.Tensor         # [n, pieces] float32: the pieces of each row's sum of squares
    eps: float

    @property
    def shape(self):
        return self.values.shape

    @property
    def dtype(self):
        return self.values.dtype

    def materialize(self) -> torch.Tensor:
        return ops.scale_rows(self.values, self.ss, self.eps)


def as_tensor(h) -> torch.Tensor:
    """The normed rows as a plain tensor, whatever form they came in."""
    return h.materialize() if isinstance(h, Prenormed) else h


class ResidualSink:
    """x: the float32 residual stream [n, width], updated in place; norm: the part that reads it next;
    rows: the rows that reader wants (None: all, and x is updated)."""

    def __init__(self, x: torch.Tensor, norm, rows: torch.Tensor | None = None):
        self.x, self.norm, self.rows = x, norm, rows

    @property
    def takes_planes(self) -> bool:
        return bool(getattr(self.norm, "takes_planes", False))

    @property
    def foldable(self) -> bool:
        """Whether a product may do the add and this norm's elementwise part itself: a norm of the form
        x * f(row) * weight with f from the mean square (it says so), over all rows."""
        return self.rows is None and bool(getattr(self.norm, "folds_into_products", False))

    def finish(self, delta: torch.Tensor) -> torch.Tensor:
        if self.rows is None:
            return self.norm(self.x, delta=delta, update=True)
        return self.norm(self.x, delta=delta, rows=self.rows)


def run_branch(part, h, ctx, sink: ResidualSink):
    """part.forward on normed rows h, its output added to the residual stream and normed for the next reader.
    A part that says ``takes_sink`` gets the sink (and h as it is); any other part gets a plain tensor and its
    output goes through ``sink.finish``."""
    if getattr(part, "takes_sink", False):
        return part.forward(h, ctx, sink=sink)
    return sink.finish(part.forward(as_tensor(h), ctx))
