"""A linear layer's weights and its product, shared by the parts that project.

Reference: the ``nn.Linear`` modules of somi_inference/models/qwen2.py:221-222,
268-271: ``y = x . W^T + b`` with W stored ``[out, in]``.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels


class Projection:
    """``[out, in]`` weight (compute dtype) and optional float32 bias, fused from one or more
    checkpoint tensors that share their input (q/k/v, gate/up) by stacking their rows."""

    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None = None) -> None:
        self.weight = weight
        self.bias = bias
        self.out_features, self.in_features = weight.shape
        # the library GEMM used for many rows wants the bias in the compute dtype (exact for a
        # bias that came from a bfloat16 checkpoint)
        self.bias_lowp = bias.to(weight.dtype) if bias is not None and weight.dtype != torch.float32 else None

    @classmethod
    def stacked(cls, weights: list[torch.Tensor], biases: list[torch.Tensor] | None = None) -> "Projection":
        weight = weights[0] if len(weights) == 1 else torch.cat(weights, dim=0).contiguous()
        bias = None
        if biases:
            bias = biases[0] if len(biases) == 1 else torch.cat(biases, dim=0).contiguous()
        return cls(weight, bias)

    def __call__(self, x: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
        return linear_kernels.linear(x, self.weight, self.bias, out_dtype, self.bias_lowp)
