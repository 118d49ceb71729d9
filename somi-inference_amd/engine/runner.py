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
from .batch import StaticStep, StepBatch, StepEntry, build_step


class StepError(ValueError):
    """A step's entries break the step function's contract."""


class _DecodeGraph:
    """One captured decode step: its static arrays, the HIP graph and the logits it writes."""

    def __init__(self, static: StaticStep, graph: torch.cuda.CUDAGraph, logits: torch.Tensor) -> None:
        self.static, self.graph, self.logits = static, graph, logits


TABLE_WIDTH_FLOOR = 16


def table_width(pages: int) -> int:
    """The width of a captured step's block table that holds ``pages`` pages: the next power of two, at least
    TABLE_WIDTH_FLOOR, so that a graph serves until a request has doubled its pages."""
    width = TABLE_WIDTH_FLOOR
    while width < pages:
        width *= 2
    return width


def graph_rows(entries: int) -> int:
    """How many rows the captured step for this many single-token entries has: the next power of two up to
    16, then the next multiple of 16 (the row tile of the matrix products, which cost the same for 17 as for 32
    rows), so that a batch that shrinks request by request replays a handful of graphs instead of capturing
    one per size.  The rows beyond the entries are padding."""
    if entries <= 16:
        rows = 1
        while rows < entries:
            rows *= 2
        return rows
    return (entries + 15) // 16 * 16


class ModelRunner:
    accepts_device_tokens = True      # step() may take its tokens from a device tensor the host has not read

    def __init__(self, model: DecoderModel, cache: CacheManager, *, decode_graphs: bool = True) -> None:
        self.model = model
        self.cache = cache
        self.device = model.runtime.device
        self.vocab_size = model.vocab_size
        self.entry_splits = tuple(model.entry_splits())     # lengths at which mixers want a step's entries cut in two
        self.steps_run = 0
        # Steps of single decoded tokens are bound by kernel launches, so they are captured once per
        # shape as a HIP graph and replayed.  Only for models whose parts all launch on the stream
        # without looking at host-side values of the step.
        self.decode_graphs = bool(decode_graphs) and model.graph_safe()
        self._graphs: dict[tuple, _DecodeGraph] = {}
        self.graph_replays = 0

    # ------------------------------------------------------------ request life
    def begin(self, request_id: Hashable) -> None:
        self.cache.register(request_id)

    def end(self, request_id: Hashable) -> None:
        self.cache.free(request_id)

    # -------------------------------------------------------------------- step
    def _validate(self, entries: list[StepEntry], device_tokens: torch.Tensor | None = None) -> None:
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
                if device_tokens is None and not 0 <= int(token) < self.vocab_size:
                    raise StepError(f"request {entry.request_id!r}: token id {token} is outside [0, {self.vocab_size})")
            for w in entry.want:
                if not 0 <= int(w) < len(entry.tokens):
                    raise StepError(f"request {entry.request_id!r}: wanted place {w} is outside its {len(entry.tokens)} tokens")
        if device_tokens is not None:
            if any(len(entry.tokens) != 1 for entry in entries):
                raise StepError("tokens that are still on the device stand for entries of one token each")
            if (device_tokens.dtype != torch.int32 or device_tokens.device != self.device
                    or tuple(device_tokens.shape) != (len(entries),)):
                raise StepError(f"device tokens must be {len(entries)} int32 values on {self.device}")

    def step(self, entries: list[StepEntry], device_tokens: torch.Tensor | None = None) -> torch.Tensor:
        """Run the entries as one batch; float32 logits ``[sum(len(want)), vocab]`` in entry order.

        Raises :class:`OutOfPages` before anything changes if the pages for
        all entries are not free.  If the forward pass raises, the pages the step
        reserved are given back and the requests' token counts stay as they were.

        ``device_tokens``: the entries' (single) tokens as an int32 tensor that is still on the device,
        typically what the sampler drew from the previous step's logits and the host has not read yet;
        the ids in ``entries`` are then placeholders.  The step is laid out and launched without waiting
        for the device, so the host works on step n + 1 while the device runs step n.
        """
        self._validate(entries, device_tokens)
        portions = [(e.request_id, len(e.tokens)) for e in entries]
        if not self.cache.can_reserve(portions):
            raise OutOfPages(f"the step needs more pages than are free ({self.cache.free_pages()} free)")
        for request_id, count in portions:
            self.cache.reserve(request_id, count)
        try:
            if self.decode_graphs and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
                logits = self._decode_with_graph(entries, device_tokens)
            else:
                batch = build_step(entries, self.cache, self.device, self.entry_splits)
                if device_tokens is not None:
                    batch.token_ids.copy_(device_tokens)
                logits = self.model.forward(batch, self.cache.layer_caches)
        except BaseException:
            # nothing of the step counts: the pages it took go back, the requests stand where they stood
            for request_id, _ in portions:
                self.cache.rollback(request_id)
            raise
        for request_id, count in portions:
            self.cache.commit(request_id, count)
        self.steps_run += 1
        return logits

    # ------------------------------------------------------------- HIP graphs
    def _capture(self, entries: list[StepEntry], rows: int, widths: list[int],
                 device_tokens: torch.Tensor | None = None) -> _DecodeGraph:
        """Capture the decode step of ``rows`` rows and these table widths, laid out for ``entries`` (none: all
        rows are padding, which is how graphs are captured ahead of any request)."""
        static = StaticStep(entries, self.cache, self.device, widths, pad_to=rows, entry_splits=self.entry_splits)
        if device_tokens is not None:
            static.batch.token_ids[:len(entries)].copy_(device_tokens)
        # once outside a capture: lazy initialisation (library handles, first allocations) must
        # not happen while the stream is being recorded; the step's writes are simply redone
        self.model.forward(static.batch, self.cache.layer_caches)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(static.batch, self.cache.layer_caches)
        held = self._graphs[(rows, tuple(widths))] = _DecodeGraph(static, graph, logits)
        return held

    def capture_decode_graphs(self, max_entries: int, max_context: int) -> int:
        """Capture ahead of time the decode graphs that up to ``max_entries`` requests with contexts of up to
        ``max_context`` tokens will replay (every row count of :func:`graph_rows`, every power-of-two table
        width), so that serving does not stop to capture when a batch changes its size or outgrows its
        tables.  Returns how many graphs were captured."""
        if not self.decode_graphs or max_entries < 1:
            return 0
        sizes = [group.page_size for group in self.cache.groups]
        # the contexts at which some group's table doubles, and the widths of all groups at each of them
        contexts = {max(1, max_context)}
        for size in sizes:
            width = TABLE_WIDTH_FLOOR
            while width * size < max_context:
                contexts.add(width * size)
                width *= 2
        shapes = sorted({tuple(table_width((c + s - 1) // s) for s in sizes) for c in contexts})
        captured = 0
        for rows in sorted({graph_rows(n) for n in range(1, max_entries + 1)}):
            for per_group in shapes:
                if (rows, per_group) not in self._graphs:
                    self._capture([], rows, list(per_group))
                    captured += 1
        return captured

    def _decode_with_graph(self, entries: list[StepEntry], device_tokens: torch.Tensor | None = None) -> torch.Tensor:
        """Replay (or first capture) the graph for this many single-token entries.

        The block tables of a captured step have a fixed width, the next power of two of pages that
        holds the longest request, so a graph serves until a request outgrows it; its rows are
        ``graph_rows(entries)``, the ones beyond the entries being padding.  The returned logits
        are the graph's own output tensor: they are overwritten by the next replay of the same graph.
        """
        widths = []
        for g in range(len(self.cache.groups)):
            widths.append(table_width(max(len(self.cache.page_list(g, e.request_id)) for e in entries)))
        real, rows = len(entries), graph_rows(len(entries))
        key = (rows, tuple(widths))
        held = self._graphs.get(key)
        if held is None:
            held = self._capture(entries, rows, widths, device_tokens)
        else:
            held.static.update(entries, self.cache)
            if device_tokens is not None:
                held.static.batch.token_ids[:real].copy_(device_tokens)   # on the stream, after the arrays' own copy
        held.graph.replay()
        self.graph_replays += 1
        return held.logits[:real]
