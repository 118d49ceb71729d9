"""Interfaces of the parts a layer is put together from.

A part is built from its own sizes and constants only; it does not know which
model, which layer index or which configuration it belongs to.  Every part

* declares the tensors it needs (``weight_specs``) under the name prefix it was
  given, and receives them through ``load(fetch, runtime)``;
* runs on the flat token batch of one step.  Token ``t`` of the batch belongs
  to entry ``step.token_entry[t]`` (a request's portion) and sits at
  ``step.positions[t]`` of its request.

The kinds of part:

``Norm``            ``forward(h) -> x``: float32 residual rows in, compute-dtype rows out.
``PositionEncoding`` hooks a mixer (or the embedding) calls with explicit positions.
``Mixer``           ``forward(x, step, cache) -> y``: mixes tokens of one request; declares the
                    cache it needs through ``cache_spec()``.
``FeedForward``     ``forward(x, step) -> y``: token-wise.
``Block``           arrangement of norms, mixer and feed-forward around the residual stream.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable

import torch

from ..weights.spec import WeightSpec


@dataclass(frozen=True)
class PartSpec:
    """Names a part kind and carries its sizes and constants."""

    kind: str
    params: dict[str, Any] = field(default_factory=dict)

    def with_params(self, **more: Any) -> "PartSpec":
        merged = dict(self.params)
        merged.update(more)
        return PartSpec(self.kind, merged)


@dataclass(frozen=True)
class Runtime:
    """Where and in which precision the parts compute."""

    dtype: torch.dtype           # torch.bfloat16, or torch.float32 for the true 32-bit path
    device: torch.device

    @property
    def exact32(self) -> bool:
        return self.dtype == torch.float32


# ---------------------------------------------------------------- cache needs
@dataclass(frozen=True)
class PagedKVSpec:
    """Keys and values of every past token, in pages.  ``window``: how many keys
    (the current one included) stay visible; None = all."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class FixedStateSpec:
    """State of fixed size per request (``shape`` per slot), zeroed when a request starts."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """What one run of a layer sees of the cache: the tensors of its call site.

    ``group`` indexes ``step.paged`` (paged) — the block table and slot mapping
    of the layer's group.  ``writes`` is False for a layer that reads the cache
    another layer wrote.
    """

    spec: PagedKVSpec | FixedStateSpec
    group: int
    k: torch.Tensor | None = None        # [pages, kv_heads, page_size, head_dim]
    v: torch.Tensor | None = None        # [pages, kv_heads, head_dim, page_size]
    state: torch.Tensor | None = None    # [slots, *shape]
    writes: bool = True


Fetch = Callable[[str], torch.Tensor]


class Part:
    """Base of all parts: weights in, nothing else assumed.

    ``graph_safe``: the part's forward only launches work on the current stream and reads the step
    through its device arrays, never through host-side values that change from step to step.  The
    runner captures decode steps as HIP graphs only if every part of the model says so.
    """

    graph_safe = False

    def __init__(self, prefix: str = "") -> None:
        self.prefix = prefix

    def name(self, suffix: str) -> str:
        return f"{self.prefix}.{suffix}" if self.prefix else suffix

    def weight_specs(self) -> list[WeightSpec]:
        return []

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        self.runtime = runtime


class Norm(Part):
    def forward(self, h: torch.Tensor) -> torch.Tensor:
        """h: [N, H] float32 residual rows -> [N, H] in the compute dtype."""
        raise NotImplementedError

    def add_forward(self, h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        """h += delta (in place, float32), then ``forward(h)``.  Parts with a fused kernel override it."""
        from ..kernels import ops
        ops.residual_add(h, delta)
        return self.forward(h)


class PositionEncoding(Part):
    def rotation_table(self) -> tuple[torch.Tensor, int] | None:
        """(inv_freq [rotary_dim/2] float32 on the device, rotary_dim) when the encoding is a
        rotation of q and k by position-proportional angles, which the attention kernels fuse
        with the cache write; None otherwise."""
        return None

    def encode_qk(self, qkv: torch.Tensor, step: Any, nq: int, nkv: int, head_dim: int) -> None:
        """Encode positions into the q and k heads of ``qkv`` in place (used when no
        rotation table is offered).  Default: nothing."""

    def encode_embeddings(self, h: torch.Tensor, step: Any) -> None:
        """Encode positions into the embedded tokens in place.  Default: nothing."""


class Mixer(Part):
    def cache_spec(self) -> PagedKVSpec | FixedStateSpec | None:
        return None

    takes_normed_rows = False      # True: x may arrive as parts.linear.NormedRows (rows still to be normed)
    portion_granule = 1            # a prompt portion that does not end its prompt holds a multiple of this many tokens

    def forward(self, x: torch.Tensor, step: Any, cache: LayerCache | None) -> torch.Tensor:
        """x: [N, H] compute dtype -> [N, H] compute dtype, or a parts.linear.DeferredProduct of that shape
        (the part's last projection, left for the residual stream to compute and add in one kernel)."""
        raise NotImplementedError


class FeedForward(Part):
    takes_normed_rows = False

    def forward(self, x: torch.Tensor, step: Any) -> torch.Tensor:
        """x: [N, H] -> [N, H], or a DeferredProduct, as for a mixer."""
        raise NotImplementedError


class Block(Part):
    """Arrangement of the parts of one layer around the residual stream."""

    mixer: Mixer

    def parts(self) -> list[Part]:
        raise NotImplementedError

    def weight_specs(self) -> list[WeightSpec]:
        specs: list[WeightSpec] = []
        for part in self.parts():
            specs.extend(part.weight_specs())
        return specs

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        self.runtime = runtime
        for part in self.parts():
            part.load(fetch, runtime)

    def forward(self, stream: Any, step: Any, cache: LayerCache | None) -> None:
        raise NotImplementedError
