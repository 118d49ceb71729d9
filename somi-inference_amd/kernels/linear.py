"""Chooses the matrix-product kernel for a linear layer by dtype and shape."""

from __future__ import annotations

import torch

from . import ops


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
           out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x @ weight.T (+ bias).  float32 always takes the plain FMA kernel (the true 32-bit path)."""
    return ops.linear_plain(x, weight, bias, out_dtype)
