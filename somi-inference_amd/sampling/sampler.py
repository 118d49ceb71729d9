"""Turns float32 logits into next-token ids on the GPU.

Reference: ``Sampler.sample`` (somi_inference/core/sampler.py:31-55): clone,
repetition penalty, temperature, top-k, top-p, then argmax (temperature 0) or a
draw from the float32 softmax (:159-176).  The order and every rule are kept.
Penalty, top-k, top-p, the temperature scaling, the softmax and the pick run in
HIP kernels (top-k and top-p by a radix search for the cut value, without a sort).
The draw is by inverse CDF from the request's own counter-based uniform number
instead of ``torch.multinomial`` on the global generator, so the distribution is
the reference's and the stream is the request's own.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.stages import stage
from .params import SamplingParams
from .rng import uniform


class PendingTokens:
    """Sampled token ids that are on their way to the host: ``device`` can feed the next step at once,
    ``tolist()`` waits for the copy (and only for it, not for work launched since)."""

    def __init__(self, device: torch.Tensor, host: torch.Tensor, copied: torch.cuda.Event) -> None:
        self.device, self._host, self._copied = device, host, copied

    def tolist(self) -> list[int]:
        self._copied.synchronize()
        return self._host.tolist()


class Sampler:
    RING = 4      # host buffers per batch size: a result must be read before that many later ones are drawn

    def __init__(self) -> None:
        self._greedy_inputs: dict[tuple[int, torch.device], torch.Tensor] = {}
        self._host_rings: dict[tuple[str, int, torch.dtype], tuple[list[torch.Tensor], list, list[int]]] = {}

    def _host_buffer(self, purpose: str, size: int, dtype: torch.dtype) -> tuple[torch.Tensor, list, int]:
        """Pinned host memory, a few buffers per purpose and size in turn: copies to and from it do not wait for
        the device.  Returns (buffer, events, turn): the caller records ``events[turn]`` after the copy it
        starts on the buffer; a buffer is handed out again only once that copy has finished."""
        ring, events, turn = self._host_rings.setdefault(
            (purpose, size, dtype), ([torch.empty(size, dtype=dtype).pin_memory() for _ in range(self.RING)],
                                     [None] * self.RING, [0]))
        turn[0] = (turn[0] + 1) % self.RING
        if events[turn[0]] is not None:
            events[turn[0]].synchronize()
        return ring[turn[0]], events, turn[0]

    def _staged(self, values: list, dtype: torch.dtype, device: torch.device) -> torch.Tensor:
        """``values`` on the device through pinned memory (buffers come in power-of-two sizes, so that a few serve
        every length)."""
        capacity = 64
        while capacity < len(values):
            capacity *= 2
        staged, events, turn = self._host_buffer("in", capacity, dtype)
        staged[:len(values)].copy_(torch.tensor(values, dtype=dtype))
        on_device = staged.to(device, non_blocking=True)
        events[turn] = torch.cuda.Event()
        events[turn].record()
        return on_device[:len(values)]

    def _row_inputs(self, plist: list[SamplingParams], seeds: list[int], counters: list[int],
                    device: torch.device) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """Temperatures, uniform draws, top-p values and penalties of the rows on the device, in one transfer (none
        for all-greedy rows, which read neither of the last three)."""
        rows = len(plist)
        if all(p.temperature == 0.0 and p.repetition_penalty == 1.0 for p in plist):
            held = self._greedy_inputs.get((rows, device))
            if held is None:
                held = self._greedy_inputs[(rows, device)] = torch.zeros(4 * rows, dtype=torch.float32, device=device)
        else:
            held = self._staged([p.temperature for p in plist] + [uniform(s, c) for s, c in zip(seeds, counters)]
                                + [p.top_p for p in plist] + [p.repetition_penalty for p in plist],
                                torch.float32, device)
        return held[:rows], held[rows:2 * rows], held[2 * rows:3 * rows], held[3 * rows:]

    def sample(self, logits: torch.Tensor, params: SamplingParams | list[SamplingParams],
               token_histories: list[list[int]] | None = None,
               seeds: list[int] | None = None, counters: list[int] | None = None) -> list[int]:
        """One token per row of ``logits`` ([rows, vocab] float32 on the GPU).

        ``token_histories``: per row, the ids the repetition penalty looks at (sampler.py:80-102).
        ``seeds`` / ``counters``: per row, the request's seed and how many tokens it has drawn.
        """
        if logits.dim() == 2 and logits.shape[0] == 0:
            return []
        return self.sample_async(logits, params, token_histories, seeds, counters).tolist()

    def sample_async(self, logits: torch.Tensor, params: SamplingParams | list[SamplingParams],
                     token_histories: list[list[int]] | None = None,
                     seeds: list[int] | None = None, counters: list[int] | None = None) -> PendingTokens:
        """The same, without waiting: the ids stay on the device and their copy to the host is under way."""
        if logits.dim() != 2:
            raise ValueError(f"logits must be 2D, got shape {tuple(logits.shape)}")
        rows, vocab = logits.shape
        plist = [params] * rows if isinstance(params, SamplingParams) else list(params)
        if len(plist) != rows:
            raise ValueError("Length of params must match batch size")
        histories = token_histories if token_histories is not None else [[] for _ in range(rows)]
        if len(histories) != rows:
            raise ValueError("Length of token_histories must match batch size")
        seeds = seeds if seeds is not None else [0] * rows
        counters = counters if counters is not None else [0] * rows
        if rows == 0:
            raise ValueError("nothing to sample")

        with stage("sampling"):
            return self._draw(logits, plist, histories, seeds, counters, rows)

    def _draw(self, logits, plist, histories, seeds, counters, rows) -> PendingTokens:
        needs_copy = any(p.repetition_penalty != 1.0 and h for p, h in zip(plist, histories)) or any(
            p.temperature > 0.0 and (p.top_k != -1 or p.top_p != 1.0) for p in plist)
        work = logits.clone() if needs_copy else logits
        if work.dtype != torch.float32:
            work = work.float()
        work = work.contiguous()

        temperature, draws, top_p, penalties = self._row_inputs(plist, seeds, counters, work.device)
        filters = any(p.temperature > 0.0 and (p.top_k != -1 or p.top_p != 1.0) for p in plist)
        # the rows' integers in one transfer: top-k values, then where each row's penalised ids start, then the ids
        offsets, ids, most = [0], [], 0
        for p, history in zip(plist, histories):
            if p.repetition_penalty != 1.0 and history:
                distinct = set(history)
                ids.extend(distinct)
                most = max(most, len(distinct))
            offsets.append(len(ids))
        if filters or most:
            ints = self._staged([p.top_k for p in plist] + offsets + ids, torch.int32, work.device)
            if most:
                ops.repetition_penalty_rows(work, ints[rows:2 * rows + 1], ints[2 * rows + 1:], penalties, most)
            if filters:
                ops.sample_filter(work, temperature, ints[:rows], top_p)
        picked = ops.sample(work, temperature, draws)
        host, events, turn = self._host_buffer("out", rows, torch.int32)
        host.copy_(picked, non_blocking=True)
        copied = events[turn] = torch.cuda.Event()
        copied.record()
        return PendingTokens(picked, host, copied)
