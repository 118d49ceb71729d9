"""The residual stream of one step: float32 rows plus one pending, not yet added, delta.

The reference adds a sub-layer's output to the hidden state in the model dtype
(somi_inference/models/qwen2.py:333-339).  Here the sum is always float32, and
an add is deferred until the next norm so that one kernel does both
(``h += delta; x = norm(h)``).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Norm


class ResidualStream:
    def __init__(self, h: torch.Tensor) -> None:
        assert h.dtype == torch.float32 and h.dim() == 2
        self.h = h
        self._pending: torch.Tensor | None = None

    def add(self, delta: torch.Tensor) -> None:
        """Queue ``h += delta``."""
        self.settle()
        self._pending = delta

    def normed(self, norm: Norm) -> torch.Tensor:
        """norm(h) after any queued add."""
        if self._pending is not None:
            delta, self._pending = self._pending, None
            return norm.add_forward(self.h, delta)
        return norm.forward(self.h)

    def settle(self) -> torch.Tensor:
        """Apply a queued add and return the float32 rows."""
        if self._pending is not None:
            ops.residual_add(self.h, self._pending)
            self._pending = None
        return self.h
