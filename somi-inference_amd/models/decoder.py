"""Builds and runs any :class:`ModelPlan`: embedding, layers in plan order, final norm, head.

Reference: somi_inference/models/qwen2.py:342-386 (embedding, N layers, final
norm) and somi_inference/models/qwen2_adapter.py:60-62, 95, 146 (head applied to
the selected rows only).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.stages import stage
from ..parts.base import FixedStateSpec, LayerCache, PagedSpec, Runtime
from ..parts.registry import build_part
from ..parts.residual import ResidualStream
from ..weights.loader import WeightFetcher, check_weights
from ..weights.source import WeightSource
from ..weights.spec import WeightSpec
from .plan import ModelPlan


class DecoderModel:
    def __init__(self, plan: ModelPlan, runtime: Runtime) -> None:
        self.plan = plan
        self.runtime = runtime
        self.embedding = build_part("embedding", plan.embedding, prefix=plan.embedding_prefix)
        self.embedding_position = None
        if plan.embedding_position is not None:
            self.embedding_position = build_part("position", plan.embedding_position,
                                                 prefix=plan.embedding_position_prefix)
        self.layers = [build_part("block", layer.block, prefix=layer.prefix) for layer in plan.layers]
        self.final_norm = build_part("norm", plan.final_norm, prefix=plan.final_norm_prefix)
        self.head = build_part("head", plan.head, prefix=plan.head_prefix)
        self.order = plan.run_order()
        self.vocab_size = plan.vocab_size or getattr(self.head, "vocab_size")
        self.loaded = False

    # ------------------------------------------------------------------ weights
    def weight_specs(self) -> list[WeightSpec]:
        specs: dict[str, WeightSpec] = {}
        for part in self._top_level_parts():
            for spec in part.weight_specs():
                specs[spec.name] = spec
        return list(specs.values())

    def _top_level_parts(self) -> list:
        parts = [self.embedding, *self.layers, self.final_norm, self.head]
        if self.embedding_position is not None:
            parts.insert(1, self.embedding_position)
        return parts

    def load(self, source: WeightSource) -> None:
        """Check the source against the declared tensors (one error for everything), then place them."""
        specs = self.weight_specs()
        check_weights(specs, source, self.plan.ignore_weights)
        fetch = WeightFetcher(specs, source, self.runtime.dtype, self.runtime.device)
        self.embedding.load(fetch, self.runtime)
        if self.embedding_position is not None:
            self.embedding_position.load(fetch, self.runtime)
        for layer in self.layers:
            layer.load(fetch, self.runtime)
        self.final_norm.load(fetch, self.runtime)
        self.head.load(fetch, self.runtime)
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding)
        self.loaded = True

    def graph_safe(self) -> bool:
        """True when every part says that its forward only launches work on the current stream from
        device-side arrays of the step (so a step can be captured once and replayed)."""
        parts = [self.embedding, self.final_norm, self.head]
        if self.embedding_position is not None:
            parts.append(self.embedding_position)
        for layer in self.layers:
            parts.append(layer)
            parts.extend(layer.parts())
        return all(getattr(part, "graph_safe", False) for part in parts)

    def portion_granule(self) -> int:
        """The least common multiple of what the mixers ask of the scheduler's prompt portions."""
        import math
        return math.lcm(*[int(getattr(layer.mixer, "portion_granule", 1)) for layer in self.layers] or [1])

    def entry_splits(self) -> list[int]:
        """The entry lengths at which some mixer wants a step's entries cut into long and short ones."""
        return sorted({int(layer.mixer.entry_split) for layer in self.layers
                       if getattr(layer.mixer, "entry_split", None) is not None})

    # -------------------------------------------------------------------- cache
    def cache_needs(self) -> list[PagedSpec | FixedStateSpec | int | None]:
        """For each run of a layer: the cache its mixer needs, the index of the earlier
        run whose cache it reads, or None."""
        needs: list[PagedSpec | FixedStateSpec | int | None] = []
        for run, index in enumerate(self.order):
            if run in self.plan.cache_from:
                needs.append(self.plan.cache_from[run])
            else:
                needs.append(self.layers[index].mixer.cache_spec())
        return needs

    # ------------------------------------------------------------------ forward
    def forward(self, step, caches: list[LayerCache | None]) -> torch.Tensor:
        """Run the step's tokens; float32 logits ``[len(step.logit_rows), vocab]``."""
        if not self.loaded:
            raise RuntimeError("model weights are not loaded")
        with stage("embedding"):
            h = self.embedding.forward(step.token_ids)
            if self.embedding_position is not None:
                self.embedding_position.encode_embeddings(h, step)
        stream = ResidualStream(h)
        for run, index in enumerate(self.order):
            self.layers[index].forward(stream, step, caches[run])
        h = stream.settle()
        if step.num_logit_rows == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=h.device)
        with stage("final norm"):
            rows = self.final_norm.forward(ops.gather_rows(h, step.logit_rows))
        with stage("head"):
            return self.head.forward(rows)

    # ------------------------------------------------------------- what a step costs
    def step_flops(self, tokens: int, attended: int, logit_rows: int) -> float:
        """Floating-point operations of the matrix products of a step of ``tokens`` tokens that see ``attended``
        (token, key) pairs in all and want ``logit_rows`` logits: every run of every layer, and the head."""
        return (sum(self.layers[index].flops(tokens, attended) for index in self.order)
                + self.head.flops(logit_rows))

    def step_weight_bytes(self) -> int:
        """Bytes of the weights that a step reads whole, from what the parts declare: every tensor but the
        embedding's, of which a step gathers one row a token (unless the head is tied to it and multiplies by it)."""
        from ..weights.loader import device_dtype
        gathered = set() if getattr(self.head, "tied", False) else {spec.name for spec in self.embedding.weight_specs()}
        total = 0
        for spec in self.weight_specs():
            if spec.name in gathered:
                continue
            count = 1
            for size in spec.shape:
                count *= size
            total += count * torch.empty((), dtype=device_dtype(spec.role, self.runtime.dtype)).element_size()
        return total
