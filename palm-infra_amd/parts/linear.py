"""y = x W^T for a weight in the checkpoint's [out, in] layout: the one place that picks the kernel.

  float32 run, or a 32-bit weight under bfloat16 activations   the exact FMA kernel
  bfloat16 x bfloat16, up to 16 rows (decode)                   the matrix-core kernel for thin products
  bfloat16 x bfloat16, 17 to 256 rows (decode batches, short    the kernel that brings both operands through rings in
  prompts)                                                      LDS, where it beats the others (ops.mid_pays); where
                                                                it does not serve (K no multiple of 64, few weight
                                                                rows), up to 128 rows, the kernel that shares the
                                                                rows through LDS, a strip of weights in each wave's
                                                                registers
  bfloat16 x bfloat16, many rows (prompts)                      the BLAS library, as the reference's GPU path
                                                                does for its products (engine/cuda_matmul.cu:245-260)

A bias (none of Qwen3's projections has one) is added by a pass of its own to the product's 32-bit result, which
then comes whole (no planes, no norm folded in) and is rounded once, after the add: correct for any part that needs
it, at the price of two launches.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .residual import Prenormed

# Up to this many rows the kernel that streams the weight past one block of 16 rows serves; from 17 to 256 rows the
# kernel with rings in LDS where it pays (ops.mid_pays); else, up to 128 rows, the kernel that shares the rows through
# LDS, where it has blocks enough to fill the chip (ops.wide_pays), and for every product with a float32 result; else
# the library.
THIN_ROWS = 16


class Linear:
    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None = None):
        if weight.dim() != 2:
            raise ValueError(f"a linear weight must be [out, in], got {tuple(weight.shape)}")
        self.weight = weight
        self.out_features, self.in_features = weight.shape
        if bias is not None and (bias.shape != (self.out_features,) or bias.dtype != torch.float32):
            raise ValueError(f"a linear bias must be float32 [{self.out_features}], got {bias.dtype} {tuple(bias.shape)}")
        self.bias = bias

    def __call__(self, x, out_dtype: torch.dtype | None = None, planes_ok: bool = False, sink=None):
        """x: rows [n, in], or ``Prenormed`` rows (their row factor is applied to the result).

        ``planes_ok``: the caller hands the result to a reader that adds float32 planes [P, n, out] (a norm's
        ``delta``, the q/k/v of qk_norm_rope_store); a thin product with few weight rows may then come as such
        planes, each the sum over one range of the inner size.

        ``sink`` (a ``ResidualSink``): the product is a branch's output; what comes back is what the sink's
        norm makes of the residual stream after the add, as a tensor or as ``Prenormed`` rows."""
        if sink is not None:
            return self._into(x, sink)
        if self.bias is not None:
            rows = x.values if isinstance(x, Prenormed) else x
            out_dtype = out_dtype or rows.dtype
            y = ops.add_bias(self._product(x, torch.float32, False), self.bias)         # added where the sum still is 32-bit
            if out_dtype == torch.float32:
                return y
            out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
            ops.convert_into(y, out)
            return out
        return self._product(x, out_dtype, planes_ok)

    def _product(self, x, out_dtype, planes_ok):
        w = self.weight
        if isinstance(x, Prenormed):
            if self._folds(x.values):
                return ops.linear_thin(x.values, w, out_dtype or x.dtype, planes_ok=planes_ok, row_ss=x.ss, row_eps=x.eps)
            x = x.materialize()
        out_dtype = out_dtype or x.dtype
        if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
            rows = x.shape[0]
            if x.is_contiguous() and ops.mid_pays(rows, self.out_features, self.in_features, planes_ok=planes_ok, out_dtype=out_dtype):
                return ops.linear_mid(x, w, out_dtype, planes_ok=planes_ok)
            if (rows <= THIN_ROWS or out_dtype != torch.bfloat16
                    or (ops.thin_serves(x, w) and ops.wide_pays(rows, self.out_features, self.in_features, planes_ok=planes_ok))):
                return ops.linear_thin(x, w, out_dtype, planes_ok=planes_ok)
            return ops.linear_library(x, w)
        return ops.linear_exact(x, w, out_dtype)

    def _folds(self, rows: torch.Tensor) -> bool:
        """Whether the kernel that folds a norm into the product serves these rows."""
        return rows.shape[0] <= ops.THIN_TOKENS and ops.thin_serves(rows, self.weight)

    def _into(self, x, sink):
        rows = x.values if isinstance(x, Prenormed) else x
        if (self.bias is None and sink.foldable and self._folds(rows) and sink.x.shape == (rows.shape[0], self.out_features)
                and rows.dtype == torch.bfloat16 and ops.fold_pays(rows.shape[0], self.out_features, self.in_features)):
            ss_in, eps_in = (x.ss, x.eps) if isinstance(x, Prenormed) else (None, 0.0)
            values, ss = ops.linear_thin_into_residual(rows, self.weight, sink.x, sink.norm.weight, row_ss=ss_in, row_eps=eps_in)
            return Prenormed(values, ss, sink.norm.eps)
        return sink.finish(self(x, planes_ok=sink.takes_planes))

    def gated(self, x) -> torch.Tensor:
        """silu(x G^T) * (x U^T) for a weight that is [G rows | U rows]: in one kernel when the product is thin,
        else the product and then the activation."""
        if self.bias is not None:
            return ops.swiglu(self(x))
        if isinstance(x, Prenormed):
            if self._folds(x.values):
                return ops.linear_thin(x.values, self.weight, x.dtype, gated=True, row_ss=x.ss, row_eps=x.eps)
            x = x.materialize()
        if (x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and x.is_contiguous()
                and ops.mid_pays(x.shape[0], self.out_features, self.in_features, gated=True)):
            return ops.linear_mid(x, self.weight, x.dtype, gated=True)
        if ops.thin_serves(x, self.weight) and (
                x.shape[0] <= THIN_ROWS or ops.wide_pays(x.shape[0], self.out_features, self.in_features, gated=True)):
            return ops.linear_thin(x, self.weight, x.dtype, gated=True)
        return ops.swiglu(self(x))
