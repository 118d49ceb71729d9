"""Position encodings.  Reference: somi_inference/models/qwen2.py:65-113."""

from __future__ import annotations

import torch

from .base import Fetch, PositionEncoding, Runtime


class RotaryPosition(PositionEncoding):
    """Rotate-half rotary embedding: element i of a head pairs with i + rotary_dim/2
    (qwen2.py:95-99) and the pair is turned by the angle p * theta^(-2j/rotary_dim)
    (qwen2.py:76-79).  No table over positions is kept (the reference bounds the
    sequence length by its table, qwen2.py:72-81): the angle is computed from the
    position in float32 by the kernel that also writes k into its cache page."""
    graph_safe = True

    def __init__(self, prefix: str, head_dim: int, theta: float, rotary_dim: int | None = None) -> None:
        super().__init__(prefix)
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.rotary_dim = int(rotary_dim if rotary_dim is not None else head_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and within head_dim {self.head_dim}")
        self.inv_freq: torch.Tensor | None = None

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        self.inv_freq = (1.0 / (self.theta ** exponents)).to(runtime.device)

    def rotation_table(self) -> tuple[torch.Tensor, int]:
        return self.inv_freq, self.rotary_dim


class NoPosition(PositionEncoding):
    """No position information (attention is then invariant to a shift of all positions)."""
    graph_safe = True

    def __init__(self, prefix: str = "") -> None:
        super().__init__(prefix)
