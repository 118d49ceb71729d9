"""Continuous-batching scheduler with a token budget and prompt portions.

Reference: ``Scheduler`` (somi_inference/core/continuous_batching.py:46-120):
three queues (waiting FIFO, running, finished), first come first served with
head-of-line blocking, at most ``max_concurrent`` running, finished requests
give their pages back before new ones are admitted.  The reference admits a
request only if the pages of its whole life fit (``ceil((prompt + max_new - 1) /
block_size)``, :64-67) and then runs the whole prompt at once.

Here a step has a budget of tokens.  Running requests that decode come first
(one token each), then running requests with prompt left, then new admissions;
a prompt is cut into portions of at most ``chunk`` tokens, or what is left of
the budget.  Pages are taken portion by portion, so they can run out:

* a request whose whole life can never fit the pool is refused when it is added;
* a new request is admitted only if the pages of its first portion are free
  (the head of the queue blocks those behind it);
* if a running request cannot get the pages for its next token(s), the most
  recently admitted running request is preempted: its pages are given back, it
  returns to the head of the waiting queue and is recomputed from its first
  token later (prompt and the tokens it already produced).  The oldest running
  request is never starved, because the admission check above guarantees that
  it fits the pool alone.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..cache.manager import CacheManager
from .request import Request, RequestStatus


class SchedulerError(ValueError):
    """A request cannot be accepted."""


@dataclass
class ScheduledPortion:
    request: Request
    start: int                    # index of the portion's first token in request.all_tokens
    tokens: list[int]
    samples: bool                 # the portion reaches the request's last token: its last logits are sampled


@dataclass
class SchedulerOutput:
    portions: list[ScheduledPortion] = field(default_factory=list)
    admitted: list[Request] = field(default_factory=list)
    preempted: list[Request] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(len(p.tokens) for p in self.portions)


class Scheduler:
    def __init__(self, cache: CacheManager, *, max_concurrent: int, max_num_batched_tokens: int,
                 chunk: int | None = None, vocab_size: int | None = None, max_positions: int | None = None,
                 granule: int = 1) -> None:
        """``vocab_size``: token ids must lie below it (None: not checked here).  ``max_positions``: the longest
        sequence the model's position encoding covers (None: unbounded).  ``granule``: a prompt portion that
        does not end its prompt holds a multiple of this many tokens (a mixer that works on blocks of tokens
        says so through ``portion_granule``)."""
        if max_concurrent < 1 or max_num_batched_tokens < 1:
            raise SchedulerError("max_concurrent and max_num_batched_tokens must be >= 1")
        if granule < 1 or granule > max_num_batched_tokens:
            raise SchedulerError(f"the portion granule {granule} must lie in [1, max_num_batched_tokens = "
                                 f"{max_num_batched_tokens}]")
        self.cache = cache
        self.max_concurrent = int(max_concurrent)
        self.max_num_batched_tokens = int(max_num_batched_tokens)
        self.granule = int(granule)
        self.chunk = int(min(chunk or max_num_batched_tokens, max_num_batched_tokens))
        if self.chunk < self.granule:
            raise SchedulerError(f"portions of at most {self.chunk} tokens cannot hold the granule of {self.granule}")
        self.chunk -= self.chunk % self.granule
        self.vocab_size = int(vocab_size) if vocab_size is not None else None
        self.max_positions = int(max_positions) if max_positions is not None else None
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []          # in admission order
        self.finished: list[Request] = []
        self.preemptions = 0                      # how often a running request had to give its pages back

    # -------------------------------------------------------------- requests
    def check_request(self, request: Request) -> None:
        """Raises :class:`SchedulerError` if the request can never run; changes nothing."""
        if not self.cache.holds(request.max_cached_tokens):
            pages = (request.max_cached_tokens + self.cache.block_size - 1) // self.cache.block_size
            raise SchedulerError(
                f"request {request.request_id!r} needs {pages} pages for {request.max_cached_tokens} tokens "
                f"(prompt {len(request.prompt_tokens)} + max_new_tokens {request.max_new_tokens} - 1), "
                f"the cache has {self.cache.num_blocks}")
        if self.max_positions is not None and request.max_cached_tokens > self.max_positions:
            # the reference's rotary table ends at max_position_embeddings and a lookup beyond it fails
            # (somi_inference/models/qwen2.py:72-81, 89-90)
            raise SchedulerError(
                f"request {request.request_id!r} reaches position {request.max_cached_tokens - 1} "
                f"(prompt {len(request.prompt_tokens)} + max_new_tokens {request.max_new_tokens} - 1 tokens), beyond "
                f"the model's max_position_embeddings = {self.max_positions}")
        if self.vocab_size is not None:
            for token in request.prompt_tokens:
                if not 0 <= int(token) < self.vocab_size:
                    raise SchedulerError(f"request {request.request_id!r}: token id {token} is outside "
                                         f"[0, {self.vocab_size})")

    def add_request(self, request: Request) -> None:
        self.check_request(request)
        request.status = RequestStatus.WAITING
        self.waiting.append(request)

    def abort(self, request: Request) -> None:
        """Take a request out wherever it stands and give back what it holds (no-op for one that is finished
        or unknown)."""
        if request in self.running:
            self.running.remove(request)
        else:
            try:
                self.waiting.remove(request)
            except ValueError:
                pass
        if self.cache.has(request.request_id):
            self.cache.free(request.request_id)
        if request.status is not RequestStatus.FINISHED:
            request.status = RequestStatus.FINISHED
            request.finish_reason = "aborted"

    def has_unfinished(self) -> bool:
        return bool(self.waiting) or bool(self.running)

    def drain_finished(self) -> list[Request]:
        done, self.finished = self.finished, []
        return done

    def finish(self, request: Request, reason: str) -> None:
        """Retire a running request now: its pages and state slot are free for the next step."""
        request.status = RequestStatus.FINISHED
        request.finish_reason = reason
        self.running.remove(request)
        self.cache.free(request.request_id)
        self.finished.append(request)

    # ------------------------------------------------------------- scheduling
    def _preempt_newest(self, output: SchedulerOutput) -> Request:
        victim = self.running.pop()
        self.cache.free(victim.request_id)
        victim.status = RequestStatus.WAITING
        victim.num_computed = 0
        victim.num_preemptions += 1
        self.preemptions += 1
        self.waiting.appendleft(victim)
        output.preempted.append(victim)
        output.portions = [p for p in output.portions if p.request is not victim]
        return victim

    def _whole(self, request: Request, count: int) -> int:
        """``count`` cut down to a multiple of the granule, unless it ends what the request has pending."""
        if self.granule == 1 or count >= request.num_pending:
            return count
        return count - count % self.granule

    def _fit(self, request: Request, want: int, taken: list[int]) -> tuple[int, list[int]]:
        """Largest portion <= want whose pages are free after what this step already took, and the pages it
        takes in each group."""
        free = [f - t for f, t in zip(self.cache.free_pages(), taken)]
        count = self._whole(request, want)
        while count > 0:
            need = self.cache.pages_needed(request.request_id, count)
            if all(n <= f for n, f in zip(need, free)):
                return count, need
            # shrink to the end of the last page that still fits
            count = self._whole(request, min(count - 1, self.cache.tokens_within(request.request_id, free)))
        return 0, [0] * len(free)

    def schedule(self) -> SchedulerOutput:
        output = SchedulerOutput()
        budget = self.max_num_batched_tokens
        taken = [0] * len(self.cache.groups)

        def take(request: Request, count: int, need: list[int]) -> None:
            nonlocal budget
            for g, n in enumerate(need):
                taken[g] += n
            start = request.num_computed
            output.portions.append(ScheduledPortion(request, start, request.tokens[start:start + count],
                                                    samples=start + count == request.num_tokens))
            budget -= count

        # 1. running requests: those that decode first, then those with prompt left
        order = [r for r in self.running if r.num_pending == 1] + [r for r in self.running if r.num_pending > 1]
        for request in order:
            if request.status is not RequestStatus.RUNNING or budget <= 0:
                continue                     # preempted in this step, or nothing left to give
            want = self._whole(request, min(request.num_pending, self.chunk, budget))
            if want == 0:
                continue                     # what is left of the budget does not hold a granule: next step
            while True:
                count, need = self._fit(request, want, taken)
                if count > 0:
                    take(request, count, need)
                    break
                if self.running[-1] is request and len(self.running) == 1:
                    raise SchedulerError(
                        f"request {request.request_id!r} cannot get a page although it runs alone")
                victim = self._preempt_newest(output)
                # what the victim had taken in this step is free again: recount
                budget = self.max_num_batched_tokens - output.num_tokens
                for g in range(len(taken)):
                    taken[g] = 0
                for portion in output.portions:
                    for g, n in enumerate(self.cache.pages_needed(portion.request.request_id, len(portion.tokens))):
                        taken[g] += n
                if victim is request:
                    break

        # 2. admissions, first come first served; the head of the queue blocks the rest
        while self.waiting and len(self.running) < self.max_concurrent and budget > 0 and not output.preempted:
            request = self.waiting[0]
            want = self._whole(request, min(request.num_pending, self.chunk, budget))
            if want == 0:
                break
            self.cache.register(request.request_id)
            count, need = self._fit(request, want, taken)
            if count < want:
                self.cache.free(request.request_id)     # the pages of its first portion are not free: wait
                break
            self.waiting.popleft()
            request.status = RequestStatus.RUNNING
            self.running.append(request)
            output.admitted.append(request)
            take(request, count, need)
        return output
