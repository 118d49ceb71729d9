"""Dense SwiGLU feed-forward.  Reference: somi_inference/models/qwen2.py:209-229."""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..kernels.stages import stage
from ..weights.spec import MATRIX, WeightSpec
from .base import FeedForward, Fetch, Runtime
from .linear import NormedRows, Projection


class SwiGLU(FeedForward):
    """y = down(silu(gate(x)) * up(x)), no biases.  gate and up are stacked into one
    ``[2I, H]`` matrix, gate rows first, as the reference merges them at load
    (somi_inference/models/qwen2_adapter.py:183-190, 244-248; qwen2.py:228 chunks the result)."""
    graph_safe = True
    takes_normed_rows = True

    ROLES = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int,
                 names: dict[str, str] | None = None) -> None:
        """``names``: what the checkpoint calls this part's matrices, role -> name under the prefix.  Roles:
        ``gate``, ``up``, ``down`` (defaults ``gate_proj``, ``up_proj``, ``down_proj``), and ``gate_up`` for a
        checkpoint that stores gate and up as one ``[2I, H]`` matrix, gate rows first."""
        super().__init__(prefix)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        unknown = set(names or {}) - set(self.ROLES) - {"gate_up"}
        if unknown:
            raise ValueError(f"{prefix}: unknown tensor roles {sorted(unknown)}; known: {sorted(self.ROLES)} and 'gate_up'")
        self.names = {**self.ROLES, **(names or {})}

    def weight_specs(self) -> list[WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        down = WeightSpec(self.name(f"{self.names['down']}.weight"), (h, i), MATRIX)
        if "gate_up" in self.names:
            return [WeightSpec(self.name(f"{self.names['gate_up']}.weight"), (2 * i, h), MATRIX), down]
        return [WeightSpec(self.name(f"{self.names['gate']}.weight"), (i, h), MATRIX),
                WeightSpec(self.name(f"{self.names['up']}.weight"), (i, h), MATRIX), down]

    INTERLEAVE = 16       # rows per block when gate and up are interleaved for the fused kernel

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        if "gate_up" in self.names:
            gate, up = fetch(self.name(f"{self.names['gate_up']}.weight")).chunk(2, dim=0)
        else:
            gate, up = (fetch(self.name(f"{self.names[role]}.weight")) for role in ("gate", "up"))
        # The layout of the merged matrix is private.  In bfloat16 the rows are interleaved in blocks of 16
        # (gate 0..15, up 0..15, gate 16..31, ...), so that the decode kernel has gate and up of the same
        # columns in one workgroup and applies the gate in its epilogue.
        self.interleaved = (runtime.dtype == torch.bfloat16 and self.intermediate_size % self.INTERLEAVE == 0
                            and self.hidden_size % 8 == 0)
        if self.interleaved:
            b, h = self.INTERLEAVE, self.hidden_size
            merged = torch.stack([gate.view(-1, b, h), up.view(-1, b, h)], dim=1).reshape(-1, h).contiguous()
            self.gate_up = Projection(merged, label="gate_up")
        else:
            self.gate_up = Projection.stacked([gate, up], label="gate_up")
        self.down = Projection(fetch(self.name(f"{self.names['down']}.weight")), label="down")

    def flops(self, tokens: int, attended: int) -> float:
        return self.gate_up.flops(tokens) + self.down.flops(tokens)

    def forward(self, x, step=None):
        if isinstance(x, NormedRows):
            if self.interleaved and self.gate_up.fusable(x.h.shape[0]):
                # norm, gate_up and SiLU . up in one kernel
                with stage(self.gate_up.label):
                    gated = linear_kernels.linear_scaled(x.weighted, x.norm.eps, x.stats, self.gate_up.weight, swiglu=True)
                return self.down.deferred(gated)
            x = x.materialize()
        if not self.interleaved:
            projected = self.gate_up(x)
            with stage("activation"):
                return self.down.deferred(ops.silu_mul(projected))
        if x.data_ptr() % 16 == 0:
            with stage(self.gate_up.label):
                return self.down.deferred(linear_kernels.linear_swiglu(x, self.gate_up.weight))
        projected = self.gate_up(x)
        with stage("activation"):
            return self.down.deferred(ops.silu_mul(projected, block=self.INTERLEAVE))
