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
PAGE = "page"       # stands in a page tensor's shape where the tokens of a page go


@dataclass(frozen=True)
class PageTensor:
    """One tensor of a paged cache: what a page of it holds.  ``shape`` is the shape of one page with PAGE in
    the place of the page's tokens, e.g. ``(kv_heads, PAGE, head_dim)``; ``dtype`` None means the engine's."""

    name: str
    shape: tuple
    dtype: torch.dtype | None = None

    def __post_init__(self) -> None:
        if list(self.shape).count(PAGE) != 1:
            raise ValueError(f"page tensor {self.name!r}: its shape {self.shape} must hold PAGE exactly once")

    def page_shape(self, page_size: int) -> tuple[int, ...]:
        return tuple(int(page_size) if dim == PAGE else int(dim) for dim in self.shape)

    def elements_per_token(self) -> int:
        count = 1
        for dim in self.shape:
            if dim != PAGE:
                count *= int(dim)
        return count


@dataclass(frozen=True)
class PagedSpec:
    """Something kept for every past token, in pages: the tensors a page holds, how many of the latest tokens
    stay visible (``window``, the current one included; None = all), and the page size the mixer's kernels want
    (None = the engine's).  Layers whose window and page size agree share one pool of pages and one block table
    per request; each layer run has its own tensors."""

    tensors: tuple[PageTensor, ...]
    window: int | None = None
    page_size: int | None = None

    def __post_init__(self) -> None:
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError(f"a paged cache needs at least one tensor and distinct names, got {names}")
        if self.page_size is not None and self.page_size < 1:
            raise ValueError(f"page size {self.page_size} must be >= 1")


class PagedKVSpec(PagedSpec):
    """Keys and values of every past token: K ``[pages, kv_heads, page, head_dim]`` and V transposed inside a
    page, ``[pages, kv_heads, head_dim, page]`` (consecutive positions of one channel are adjacent: the operand
    layout of the weights-times-values product)."""

    def __init__(self, num_kv_heads: int, head_dim: int, window: int | None = None, page_size: int | None = None) -> None:
        super().__init__((PageTensor("k", (int(num_kv_heads), PAGE, int(head_dim))),
                          PageTensor("v", (int(num_kv_heads), int(head_dim), PAGE))), window, page_size)
        object.__setattr__(self, "num_kv_heads", int(num_kv_heads))
        object.__setattr__(self, "head_dim", int(head_dim))


@dataclass(frozen=True)
class FixedStateSpec:
    """State of fixed size per request (``shape`` per slot), zeroed when a request starts."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class LayerCache:
    """What one run of a layer sees of the cache: the tensors of its call site.

    ``group`` indexes ``step.paged`` (paged) — the block table and slot mapping of the layer's group, whose pages
    hold ``page_size`` tokens.  ``tensors[name]`` is ``[pages, *page shape]`` for each tensor of the spec.
    ``writes`` is False for a layer that reads the cache another layer wrote.
    """

    spec: PagedSpec | FixedStateSpec
    group: int
    tensors: dict[str, torch.Tensor] = field(default_factory=dict)
    state: torch.Tensor | None = None    # [slots, *shape]
    writes: bool = True
    page_size: int = 0

    @property
    def k(self) -> torch.Tensor | None:      # [pages, kv_heads, page_size, head_dim]
        return self.tensors.get("k")

    @property
    def v(self) -> torch.Tensor | None:      # [pages, kv_heads, head_dim, page_size]
        return self.tensors.get("v")


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

    def flops(self, tokens: int, attended: int) -> float:
        """Floating-point operations of the part's matrix products in a step of ``tokens`` tokens that see
        ``attended`` (token, key) pairs in all (a windowed mixer sees fewer: an upper bound then).  What a
        measurement divides by the step's time; element-wise work is not counted."""
        return 0.0


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
    def cache_spec(self) -> PagedSpec | FixedStateSpec | None:
        return None

    takes_normed_rows = False      # True: x may arrive as parts.linear.NormedRows (rows still to be normed)
    portion_granule = 1            # a prompt portion that does not end its prompt holds a multiple of this many tokens
    entry_split = None             # an int: ``step.split(entry_split)`` lists the entries longer than this many tokens
                                   # and the tokens of the others, for mixers that serve the two with different kernels

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

    def flops(self, tokens: int, attended: int) -> float:
        return sum(part.flops(tokens, attended) for part in self.parts())

    def forward(self, stream: Any, step: Any, cache: LayerCache | None) -> None:
        raise NotImplementedError
