"""The residual stream of one step: float32 rows plus one pending, not yet added, delta.

The reference adds a sub-layer's output to the hidden state in the model dtype
(somi_inference/models/qwen2.py:333-339).  Here the sum is always float32, and
an add is deferred until the next norm so that one kernel does both
(``h += delta; x = norm(h)``).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.stages import stage
from .base import Norm
from .linear import DeferredProduct, NormedRows


class ResidualStream:
    """For a few bfloat16 rows (decode steps) neither the add nor the norm is a kernel of its own: a part's
    last projection may arrive as a :class:`DeferredProduct`; ``normed(norm, lazy=True)`` then has it computed
    straight into ``h`` by a kernel that also leaves what the norm needs, and hands out :class:`NormedRows`,
    which the next projection scales while it multiplies."""

    def __init__(self, h: torch.Tensor) -> None:
        assert h.dtype == torch.float32 and h.dim() == 2
        self.h = h
        self._pending: torch.Tensor | DeferredProduct | None = None

    def add(self, delta: "torch.Tensor | DeferredProduct") -> None:
        """Queue ``h += delta``."""
        self.settle()
        self._pending = delta

    def normed(self, norm: Norm, lazy: bool = False) -> "torch.Tensor | NormedRows":
        """norm(h) after any queued add.  ``lazy``: the caller's consumer takes :class:`NormedRows`."""
        if isinstance(self._pending, DeferredProduct):
            pending, self._pending = self._pending, None
            if lazy and getattr(norm, "fusable", False):
                return pending.add_to(self.h, norm)
            pending.add_to(self.h)
        with stage("residual add, norm"):
            if self._pending is not None:
                delta, self._pending = self._pending, None
                return norm.add_forward(self.h, delta)
            return norm.forward(self.h)

    def settle(self) -> torch.Tensor:
        """Apply a queued add and return the float32 rows."""
        if isinstance(self._pending, DeferredProduct):
            self._pending.add_to(self.h)
        elif self._pending is not None:
            with stage("residual add, norm"):
                ops.residual_add(self.h, self._pending)
        self._pending = None
        return self.h
