"""The step function: runs one batch of (request, its next tokens) from the cache.

The reference has two functions, ``prefill`` for one whole prompt and ``decode``
for one token of each of B requests (somi_inference/models/base.py:17-56,
somi_inference/models/qwen2_adapter.py:64-146), each bracketed by
``allocate_slots`` before and ``advance_tokens`` after the forward.  Here there
is one: a step holds any mix of prompt portions and single decoded tokens, runs
exactly the tokens it is given against what earlier steps left in the cache,
and returns float32 logits at the wanted places only.
"""

from __future__ import annotations

from typing import Hashable

import torch

from ..cache.manager import CacheManager
from ..cache.pool import OutOfPages
from ..models.decoder import DecoderModel
from .batch import StepBatch, StepEntry, build_step


class StepError(ValueError):
    """A step's entries break the step function's contract."""


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager) -> None:
        self.model = model
        self.cache = cache
        self.device = model.runtime.device
        self.vocab_size = model.vocab_size
        self.steps_run = 0

    # ------------------------------------------------------------ request life
    def begin(self, request_id: Hashable) -> None:
        self.cache.register(request_id)

    def end(self, request_id: Hashable) -> None:
        self.cache.free(request_id)

    # -------------------------------------------------------------------- step
    def _validate(self, entries: list[StepEntry]) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        for entry in entries:
            if entry.request_id in seen:
                raise StepError(f"request {entry.request_id!r} appears twice in one step")
            seen.add(entry.request_id)
            if not self.cache.has(entry.request_id):
                raise StepError(f"request {entry.request_id!r} is not live (begin() it first)")
            if len(entry.tokens) < 1:
                raise StepError(f"request {entry.request_id!r}: an entry holds at least one token")
            for token in entry.tokens:
                # the reference's embedding lookup raises on out-of-range ids
                # (tests/models/test_qwen2_error_handling.py:42-86)
                if not 0 <= int(token) < self.vocab_size:
                    raise StepError(f"request {entry.request_id!r}: token id {token} is outside [0, {self.vocab_size})")
            for w in entry.want:
                if not 0 <= int(w) < len(entry.tokens):
                    raise StepError(f"request {entry.request_id!r}: wanted place {w} is outside its {len(entry.tokens)} tokens")

    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Run the entries as one batch; float32 logits ``[sum(len(want)), vocab]`` in entry order.

        Raises :class:`OutOfPages` before anything changes if the pages for
        all entries are not free.
        """
        self._validate(entries)
        portions = [(e.request_id, len(e.tokens)) for e in entries]
        if not self.cache.can_reserve(portions):
            raise OutOfPages(f"the step needs more pages than are free ({self.cache.free_pages()} free)")
        for request_id, count in portions:
            self.cache.reserve(request_id, count)
        batch = build_step(entries, self.cache, self.device)
        logits = self.model.forward(batch, self.cache.layer_caches)
        for request_id, count in portions:
            self.cache.commit(request_id, count)
        self.steps_run += 1
        return logits
