"""Turns float32 logits into next-token ids on the GPU.

Reference: ``Sampler.sample`` (somi_inference/core/sampler.py:31-55): clone,
repetition penalty, temperature, top-k, top-p, then argmax (temperature 0) or a
draw from the float32 softmax (:159-176).  The order and every rule are kept.
Penalty, the temperature scaling, the softmax and the pick run in HIP kernels;
the top-k and top-p masks use the library's ``topk``/``sort`` on the device.
The draw is by inverse CDF from the request's own counter-based uniform number
instead of ``torch.multinomial`` on the global generator, so the distribution is
the reference's and the stream is the request's own.
"""

from __future__ import annotations

import torch

from ..kernels import ops
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
        self._host_rings: dict[tuple[int, torch.dtype], tuple[list[torch.Tensor], list[int]]] = {}

    def _host_buffer(self, size: int, dtype: torch.dtype) -> torch.Tensor:
        """Pinned host memory, a few buffers per size in turn: copies to and from it do not wait for the device."""
        ring, turn = self._host_rings.setdefault(
            (size, dtype), ([torch.empty(size, dtype=dtype).pin_memory() for _ in range(self.RING)], [0]))
        turn[0] = (turn[0] + 1) % self.RING
        return ring[turn[0]]

    def _pick_inputs(self, plist: list[SamplingParams], seeds: list[int], counters: list[int],
                     device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
        """Temperatures and uniform draws of the rows on the device, in one transfer (none for all-greedy rows)."""
        rows = len(plist)
        if all(p.temperature == 0.0 for p in plist):
            held = self._greedy_inputs.get((rows, device))
            if held is None:
                held = self._greedy_inputs[(rows, device)] = torch.zeros(2 * rows, dtype=torch.float32, device=device)
        else:
            staged = self._host_buffer(2 * rows, torch.float32)
            staged.copy_(torch.tensor([p.temperature for p in plist] + [uniform(s, c) for s, c in zip(seeds, counters)],
                                      dtype=torch.float32))
            held = staged.to(device, non_blocking=True)
        return held[:rows], held[rows:]

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

        needs_copy = any(p.repetition_penalty != 1.0 and h for p, h in zip(plist, histories)) or any(
            p.temperature > 0.0 and (p.top_k != -1 or p.top_p != 1.0) for p in plist)
        work = logits.clone() if needs_copy else logits
        if work.dtype != torch.float32:
            work = work.float()
        work = work.contiguous()

        for row, (p, history) in enumerate(zip(plist, histories)):
            if p.repetition_penalty != 1.0 and history:
                ids = torch.tensor(sorted(set(int(t) for t in history)), dtype=torch.int32, device=work.device)
                ops.repetition_penalty(work[row], ids, p.repetition_penalty)
        for row, p in enumerate(plist):
            if p.temperature == 0.0:
                continue                    # greedy ignores top-k / top-p (sampler.py:123, 142)
            if p.top_k != -1:
                keep = torch.topk(work[row], k=min(p.top_k, vocab)).indices
                masked = torch.full_like(work[row], float("-inf"))
                masked[keep] = work[row][keep]
                work[row] = masked
            if p.top_p != 1.0:
                ordered, order = torch.sort(work[row] / p.temperature, descending=True)
                cumulative = torch.cumsum(torch.softmax(ordered, dim=-1, dtype=torch.float32), dim=-1)
                remove = cumulative > p.top_p
                remove[1:] = remove[:-1].clone()     # the entry that crosses p stays (sampler.py:151-153)
                remove[0] = False
                work[row, order[remove]] = float("-inf")

        temperature, draws = self._pick_inputs(plist, seeds, counters, work.device)
        picked = ops.sample(work, temperature, draws)
        host = self._host_buffer(rows, torch.int32)
        host.copy_(picked, non_blocking=True)
        copied = torch.cuda.Event()
        copied.record()
        return PendingTokens(picked, host, copied)
