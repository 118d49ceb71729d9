"""Chooses the matrix-product kernel for a linear layer by dtype and shape."""

from __future__ import annotations

import torch

from . import ops

SKINNY_MAX_ROWS = 64   # what the skinny MFMA kernel takes
SKINNY_ROWS = 64       # up to here the few-rows kernels run; beyond, the many-rows kernel (ops.linear_big)


LONG_K = 8192            # a K that the split-K kernel cuts into eight pieces of sixteen chunks
FEW_COLUMNS_PER_UNIT = 32     # up to this many columns per compute unit the few-rows kernel has two workgroups a unit at most
MANY_COLUMNS_PER_UNIT = 64    # from this many on its workgroups come in several rounds, each reading all of x again


def _mid_is_faster(m: int, n: int, k: int) -> bool:
    """From 17 rows on, the kernel that shares x inside a workgroup and splits K over workgroups wins where K is
    long and the columns are few for the device (7B down projection on 256 units: 26 + 5 us against 38 at 32 rows,
    34 + 5 against 53 at 64) and where there are very many columns (gate_up: steps of 20 to 32 requests 1.7 %
    shorter, 58 + 8 us against 79 at 64 rows).  Measured inside decode steps at 7B layer sizes; the bounds on the
    columns go with the device's compute units."""
    if m <= 16:
        return False
    units = ops.compute_units()
    return (k >= LONG_K and n <= FEW_COLUMNS_PER_UNIT * units) or n >= MANY_COLUMNS_PER_UNIT * units


def linear_swiglu(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """silu(x @ gate.T) * (x @ up.T) for bfloat16 rows; weight: [2 I, K], gate and up rows interleaved in blocks
    of 16."""
    m, k = x.shape
    if m > SKINNY_ROWS:
        return ops.linear_big(x, weight, swiglu=True)
    if _mid_is_faster(m, weight.shape[0], k):
        return ops.linear_mid(x, weight, swiglu=True)
    return ops.linear_skinny_swiglu(x, weight)


def linear_residual(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, h: torch.Tensor,
                    next_norm_weight: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor | None]:
    """h += x @ weight.T (+ bias) in place, by the kernel that :func:`linear` would take for the sizes; see
    :func:`ops.linear_residual`.  More than 64 rows take the many-rows kernel, which shares a tile's K among workgroups
    where its tiles are few (o and down of 65 to some hundred rows; passes of the few-rows kernel over 64 rows each
    measured the same inside decode steps of 128 requests, 10.70 against 10.72 ms)."""
    m, n = x.shape[0], weight.shape[0]
    if m > ops.FUSED_MAX_ROWS:
        return ops.linear_big_residual(x, weight, bias, h, next_norm_weight)
    mid = _mid_is_faster(m, n, x.shape[1])
    return ops.linear_residual(x, weight, bias, h, next_norm_weight, mid=mid)


def linear_scaled(x: torch.Tensor, eps: float, stats: torch.Tensor, weight: torch.Tensor,
                  bias: torch.Tensor | None = None, swiglu: bool = False) -> torch.Tensor:
    """The product of rows that are still to be normed, by the kernel that :func:`linear` would take for the
    sizes; see :func:`ops.linear_scaled`."""
    if x.shape[0] > ops.FUSED_MAX_ROWS:
        return ops.linear_big(x, weight, bias, swiglu=swiglu, eps=eps, stats=stats)
    mid = _mid_is_faster(x.shape[0], weight.shape[0], x.shape[1])
    return ops.linear_scaled(x, eps, stats, weight, bias, swiglu, mid=mid)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
           out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """x @ weight.T (+ bias).

    float32 always takes the plain FMA kernel (the true 32-bit path).  bfloat16 with few rows takes the
    hand-written few-rows MFMA kernels, with more rows the many-rows MFMA kernel (256-row tiles), whose float32
    form writes the logits of many rows without rounding them to bfloat16 (rows of an input it does not take go
    through the few-rows kernel 64 at a time).  Operands the MFMA kernels do not take (K no multiple of 8, unaligned) run the plain
    kernel.
    """
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        return ops.linear_plain(x, weight, bias, out_dtype)
    m, k = x.shape
    if k % 8 != 0 or x.data_ptr() % 16 or weight.data_ptr() % 16:
        return ops.linear_plain(x, weight, bias, out_dtype)
    if m <= SKINNY_ROWS:
        if _mid_is_faster(m, weight.shape[0], k):
            return ops.linear_mid(x, weight, bias, out_dtype)
        return ops.linear_skinny(x, weight, bias, out_dtype)
    if out_dtype == x.dtype and ops.big_supported(x, weight):
        return ops.linear_big(x, weight, bias)
    if out_dtype == torch.float32 and ops.big_supported(x, weight):
        # logits of more than 64 rows: one pass over the output matrix instead of one per 64 rows (7B head at 256 rows:
        # four passes of 290 us)
        return ops.linear_big_f32(x, weight, bias)
    if out_dtype == torch.float32:
        return torch.cat([ops.linear_skinny(x[at:at + SKINNY_MAX_ROWS], weight, bias, out_dtype)
                          for at in range(0, m, SKINNY_MAX_ROWS)])
    return ops.linear_plain(x, weight, bias, out_dtype)
