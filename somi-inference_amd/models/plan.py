"""A model as data: which parts every layer has and in which order layers run.

An architecture's plan builder turns its typed configuration into a
:class:`ModelPlan`; :class:`~somi_inference_amd.models.decoder.DecoderModel`
builds and runs any plan.  Layers may differ in every part; ``order`` may name
a layer twice (its weights are shared, each run has its own cache), and
``cache_from`` lets a run read the cache that an earlier run wrote.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.base import PartSpec
from ..parts.registry import build_part
from ..weights.spec import WeightSpec


@dataclass(frozen=True)
class LayerSpec:
    prefix: str                      # tensor-name prefix of the layer, e.g. "model.layers.3"
    block: PartSpec                  # arrangement kind; its params name the layer's parts


@dataclass(frozen=True)
class ModelPlan:
    embedding: PartSpec
    embedding_prefix: str
    layers: tuple[LayerSpec, ...]
    final_norm: PartSpec
    final_norm_prefix: str
    head: PartSpec
    head_prefix: str
    order: tuple[int, ...] = ()                      # run order over ``layers``; empty = each once, in order
    cache_from: dict[int, int] = field(default_factory=dict)   # run index -> earlier run index whose cache it reads
    ignore_weights: tuple[str, ...] = ()             # glob patterns of tensors a checkpoint may carry unused
    vocab_size: int = 0
    embedding_position: PartSpec | None = None       # a position encoding applied to the embedded tokens
    embedding_position_prefix: str = ""
    max_positions: int | None = None                 # longest sequence the position encoding covers; None = no bound

    def run_order(self) -> tuple[int, ...]:
        return self.order if self.order else tuple(range(len(self.layers)))

    def __post_init__(self) -> None:
        order = self.run_order()
        for index in order:
            if not 0 <= index < len(self.layers):
                raise ValueError(f"order names layer {index}, but the plan has {len(self.layers)} layers")
        for run, source in self.cache_from.items():
            if not (0 <= source < run < len(order)):
                raise ValueError(f"cache_from[{run}] = {source}: a run may only read the cache of an earlier run")


def collect_weight_specs(plan: ModelPlan) -> list[WeightSpec]:
    """Every tensor the plan's parts declare, each name once (no device needed)."""
    specs: list[WeightSpec] = []
    specs += build_part("embedding", plan.embedding, prefix=plan.embedding_prefix).weight_specs()
    if plan.embedding_position is not None:
        specs += build_part("position", plan.embedding_position, prefix=plan.embedding_position_prefix).weight_specs()
    for layer in plan.layers:
        specs += build_part("block", layer.block, prefix=layer.prefix).weight_specs()
    specs += build_part("norm", plan.final_norm, prefix=plan.final_norm_prefix).weight_specs()
    specs += build_part("head", plan.head, prefix=plan.head_prefix).weight_specs()
    seen: dict[str, WeightSpec] = {}
    for spec in specs:
        if spec.name in seen and seen[spec.name] != spec:
            raise ValueError(f"tensor {spec.name!r} is declared twice with different shapes or roles")
        seen[spec.name] = spec
    return list(seen.values())
