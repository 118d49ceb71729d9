"""A linear layer's weights and its product, shared by the parts that project.

Reference: the ``nn.Linear`` modules of somi_inference/models/qwen2.py:221-222,
268-271: ``y = x . W^T + b`` with W stored ``[out, in]``.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage


class NormedRows:
    """Rows of the residual stream that are still to be normed: what a block hands to a mixer or a feed-forward
    that says it ``takes_normed_rows``, when the product that last added to the stream has left what the norm
    needs: ``weighted`` = bfloat16(norm weight * h) and ``stats``, the rows' sums of squares in partial sums.
    A :class:`Projection` called with it computes ``norm(h) . W^T`` in one kernel (the product of ``weighted``,
    scaled per row); ``materialize()`` gives the normed rows themselves."""

    def __init__(self, h: torch.Tensor, weighted: torch.Tensor, stats: torch.Tensor, norm) -> None:
        self.h, self.weighted, self.stats, self.norm = h, weighted, stats, norm
        self.shape = h.shape

    def materialize(self) -> torch.Tensor:
        return self.norm.forward(self.h)


class DeferredProduct:
    """``x . W^T (+ b)`` that has not been computed: what a mixer or a feed-forward may return for its last
    projection, so that the residual stream can add it to its float32 rows in the kernel that computes it."""

    def __init__(self, projection: "Projection", x: torch.Tensor) -> None:
        self.projection, self.x = projection, x
        self.shape = (x.shape[0], projection.out_features)

    def materialize(self) -> torch.Tensor:
        return self.projection(self.x)

    def add_to(self, h: torch.Tensor, next_norm=None) -> "NormedRows | None":
        """h += the product, in place.  With the norm that follows, returns its rows, still to be normed."""
        weight = next_norm.weight if next_norm is not None else None
        with stage(self.projection.label):
            stats, weighted = linear_kernels.linear_residual(self.x, self.projection.weight, self.projection.bias, h, weight)
        return NormedRows(h, weighted, stats, next_norm) if next_norm is not None else None


class Projection:
    """``[out, in]`` weight (compute dtype) and optional float32 bias, fused from one or more
    checkpoint tensors that share their input (q/k/v, gate/up) by stacking their rows."""

    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None = None, label: str = "projection") -> None:
        self.weight = weight
        self.bias = bias
        self.label = label                 # the name of its stage where stages are timed
        self.out_features, self.in_features = weight.shape

    def flops(self, rows: int) -> float:
        return 2.0 * rows * self.out_features * self.in_features

    @classmethod
    def stacked(cls, weights: list[torch.Tensor], biases: list[torch.Tensor] | None = None,
                label: str = "projection") -> "Projection":
        weight = weights[0] if len(weights) == 1 else torch.cat(weights, dim=0).contiguous()
        bias = None
        if biases:
            bias = biases[0] if len(biases) == 1 else torch.cat(biases, dim=0).contiguous()
        return cls(weight, bias, label)

    def __call__(self, x: "torch.Tensor | NormedRows", out_dtype: torch.dtype | None = None) -> torch.Tensor:
        with stage(self.label):
            if isinstance(x, NormedRows):
                if out_dtype in (None, torch.bfloat16) and self.fusable(x.h.shape[0]):
                    return linear_kernels.linear_scaled(x.weighted, x.norm.eps, x.stats, self.weight, self.bias)
                x = x.materialize()
            return linear_kernels.linear(x, self.weight, self.bias, out_dtype)

    def fusable(self, rows: int) -> bool:
        """The kernels that fuse this product with the norm before it, or with the add into the stream after it, take
        it."""
        return (self.weight.dtype == torch.bfloat16 and rows > 0 and self.in_features % 8 == 0
                and self.weight.data_ptr() % 16 == 0)

    def deferred(self, x: torch.Tensor) -> "torch.Tensor | DeferredProduct":
        """The product, or a promise of it where the residual stream can compute and add it in one kernel (any number
        of bfloat16 rows: the few-rows kernels, or the many-rows kernel, which shares a tile's K where tiles are few)."""
        if x.dtype == torch.bfloat16 and x.data_ptr() % 16 == 0 and self.fusable(x.shape[0]):
            return DeferredProduct(self, x)
        return self(x)
