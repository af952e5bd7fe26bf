"""RMSNorm: y = x * (1 / sqrt(mean(x^2) + eps)) * w, statistics in 32-bit (kernels/norm.cpp:13-31).
The residual add that precedes a norm in a block is fused into the same pass
(engine/cuda_ops.cu:140-170 has the same fusion)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import register_part


@register_part("norm", "rms")
class RMSNorm:
    capturable = True      # launches the same kernels whatever the step holds: may be recorded into a HIP graph
    takes_planes = True    # ``delta`` may be float32 planes [P, n, width], added one after the other
    folds_into_products = True   # y = x * f(row) * weight, f = 1 / sqrt(mean(x^2) + eps): see parts/residual.py

    def __init__(self, spec, builder):
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.weight = builder.tensor(spec, "weight")
        self.dtype = builder.dtype
        if self.weight.shape != (self.width,):
            raise ValueError(f"RMSNorm of width {self.width} got a weight of shape {tuple(self.weight.shape)}")

    def __call__(self, x: torch.Tensor, delta: torch.Tensor | None = None, update: bool = False,
                 rows: torch.Tensor | None = None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, out_dtype or self.dtype, delta=delta, update_x=update, rows=rows)
