"""Chooses the matrix-product kernel for a linear layer by dtype and shape."""

from __future__ import annotations

import torch

from . import ops

SKINNY_MAX_ROWS = 64   # what the skinny MFMA kernel takes
SKINNY_ROWS = 64       # up to here it beats the library product at 7B layer sizes (measured inside decode steps
                       # of 64 requests: gate_up with the gate fused in 80 us against 90 + 5, down 55 against 60)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
           out_dtype: torch.dtype | None = None, bias_lowp: torch.Tensor | None = None) -> torch.Tensor:
    """x @ weight.T (+ bias).

    float32 always takes the plain FMA kernel (the true 32-bit path).  bfloat16 with few rows takes the
    hand-written skinny MFMA kernel; with many rows the product is a plain library GEMM, as it is in the
    reference (nn.Linear / F.linear), with float32 outputs (logits) produced 64 rows at a time by the
    skinny kernel so that they are never rounded to bfloat16.  The library product is also what runs inside
    captured decode steps of more than SKINNY_ROWS requests; tests replay such graphs against eager steps.
    """
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        return ops.linear_plain(x, weight, bias, out_dtype)
    m, k = x.shape
    if k % 8 != 0 or x.data_ptr() % 16 or weight.data_ptr() % 16:
        return ops.linear_plain(x, weight, bias, out_dtype)
    if m <= SKINNY_ROWS:
        return ops.linear_skinny(x, weight, bias, out_dtype)
    if out_dtype == torch.float32:
        return torch.cat([ops.linear_skinny(x[at:at + SKINNY_MAX_ROWS], weight, bias, out_dtype)
                          for at in range(0, m, SKINNY_MAX_ROWS)])
    if bias is not None and bias_lowp is None:
        bias_lowp = bias.to(x.dtype)
    return torch.nn.functional.linear(x, weight, bias_lowp)
