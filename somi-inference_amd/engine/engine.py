"""The generation loop: schedule, run one step, sample, finish and free.

Reference: ``ContinuousBatchingEngine`` (somi_inference/core/continuous_batching.py:123-205):
each iteration injects the arrivals of that step, schedules, frees what finished,
prefills the admitted requests one by one and decodes the running ones as a batch;
after every sampled token a request finishes on EOS (which is kept in its output)
or when it has ``max_new_tokens`` (:150-158).  Here one model step serves the whole
mixed batch, and a finished request's pages are free for the very next step.
"""

from __future__ import annotations

import contextlib
import gc
from collections import deque
from dataclasses import dataclass

from ..sampling.sampler import Sampler
from .batch import StepEntry
from .request import Request, RequestStatus
from .scheduler import ScheduledPortion, Scheduler, SchedulerOutput

UNREAD = -1       # stands in a request's output for a token that is drawn but not yet read from the device


@contextlib.contextmanager
def full_collections_deferred():
    """While requests are stepped, Python's collections of its oldest generation are put off until the block ends.
    Such a collection walks every tracked object; with a couple of hundred requests of thousands of token ids it
    takes 30 to 50 ms, several decode steps during which the device waits for its next launch (192 requests at 7B
    sizes: one step in five took 50 ms instead of 17).  The young generations, which take what a step allocates,
    are collected as ever."""
    young, middle, old = gc.get_threshold()
    gc.set_threshold(young, middle, 1 << 30)
    try:
        yield
    finally:
        gc.set_threshold(young, middle, old)


@dataclass
class _UnreadStep:
    """The sampled portions of a launched step whose tokens the host has not read yet."""
    portions: list[ScheduledPortion]
    places: list[int]             # index of each portion's stand-in in its request's output_tokens
    tokens: object                # sampling.PendingTokens


class Engine:
    def __init__(self, runner, scheduler: Scheduler, sampler: Sampler, eos_token_id: int | None) -> None:
        self.runner = runner
        self.scheduler = scheduler
        self.sampler = sampler
        self.eos_token_id = -1 if eos_token_id is None else int(eos_token_id)   # -1: nothing ends a request early
        self.num_steps = 0
        self.last_output: SchedulerOutput | None = None
        # Running ahead: while only decoding requests run, step n + 1 is launched with step n's tokens
        # still on the device, and step n's tokens are read (and checked for EOS) while n + 1 runs.  A
        # request that turns out to have ended at n has then run one token too far; that token is dropped.
        self.run_ahead = bool(getattr(runner, "accepts_device_tokens", False)) and hasattr(sampler, "sample_async")
        self.steps_run_ahead = 0
        self._unread: _UnreadStep | None = None

    def add_request(self, request: Request) -> None:
        self.scheduler.add_request(request)

    def _check_finished(self, request: Request, token: int, count: int | None = None) -> None:
        """``count``: how many tokens the request has with this one (its output may already hold a stand-in
        for a later one)."""
        count = len(request.output_tokens) if count is None else count
        if token == self.eos_token_id:
            self.scheduler.finish(request, "eos")
        elif count >= request.max_new_tokens:
            self.scheduler.finish(request, "length")

    def _can_run_ahead(self) -> bool:
        """The next step is known without the unread tokens' values: the same requests, one token each, nobody
        waiting, nobody at its last token, no sampling rule that reads the history, pages free for all."""
        unread, scheduler = self._unread, self.scheduler
        if unread is None or scheduler.waiting or len(scheduler.running) > scheduler.max_num_batched_tokens:
            return False
        if [p.request for p in unread.portions] != scheduler.running:
            return False
        for request in scheduler.running:
            if (request.num_pending != 1 or request.sampling_params.repetition_penalty != 1.0
                    or len(request.output_tokens) >= request.max_new_tokens):
                return False
        return scheduler.cache.can_reserve([(r.request_id, 1) for r in scheduler.running])

    def _read_unread(self) -> None:
        """Read the tokens of the step that is still unread, put them in place and retire what ended."""
        unread, self._unread = self._unread, None
        if unread is None:
            return
        for portion, place, token in zip(unread.portions, unread.places, unread.tokens.tolist()):
            request = portion.request
            if request.status is RequestStatus.FINISHED:
                continue                         # ended a step earlier: this was the token too far
            request.output_tokens[place] = int(token)
            self._check_finished(request, int(token), place + 1)
            if request.status is RequestStatus.FINISHED:
                del request.output_tokens[place + 1:]      # the stand-in of a step launched since

    def step(self) -> list[Request]:
        """One scheduling decision and one model step; returns the requests that finished in it."""
        ahead = self._can_run_ahead()
        if not ahead:
            self._read_unread()
        output = self.scheduler.schedule()
        self.last_output = output
        self.num_steps += 1
        if not output.portions:
            self._read_unread()
            return self.scheduler.drain_finished()
        entries = [StepEntry(p.request.request_id, [max(t, 0) for t in p.tokens], [len(p.tokens) - 1] if p.samples else [])
                   for p in output.portions]
        if ahead:
            assert [p.request for p in output.portions] == [p.request for p in self._unread.portions]
            logits = self.runner.step(entries, device_tokens=self._unread.tokens.device)
            self.steps_run_ahead += 1
        else:
            logits = self.runner.step(entries)
        sampled = [p for p in output.portions if p.samples]
        for portion in output.portions:
            portion.request.num_computed += len(portion.tokens)
        if sampled:
            draw = self.sampler.sample_async if self.run_ahead else self.sampler.sample
            tokens = draw(
                logits,
                [p.request.sampling_params for p in sampled],
                token_histories=[p.request.tokens for p in sampled],
                seeds=[p.request.seed for p in sampled],
                counters=[len(p.request.output_tokens) for p in sampled],
            )
            if self.run_ahead:
                older, self._unread = self._unread, None
                places = []
                for portion in sampled:
                    places.append(len(portion.request.output_tokens))
                    portion.request.output_tokens.append(UNREAD)
                newest = _UnreadStep(sampled, places, tokens)
                self._unread = older
                self._read_unread()              # the step before, while this one runs
                self._unread = newest
            else:
                for portion, token in zip(sampled, tokens):
                    portion.request.output_tokens.append(int(token))
                    self._check_finished(portion.request, int(token))
        elif ahead:
            self._read_unread()
        return self.scheduler.drain_finished()

    def run(self, requests: deque[tuple[int, Request]] | None = None) -> list[Request]:
        """Run until every request has finished; ``requests`` holds (arrival_step, request) in
        arrival order, as the reference's ``run`` takes them (continuous_batching.py:179-205).
        Returns the requests in the order they finished.  A request that can never run (too long for the pool
        or the model, a token id outside the vocabulary) raises before anything is queued; if a step raises,
        the call's requests are aborted and what they held is free again, so the next call starts clean."""
        requests = requests if requests is not None else deque()
        mine = [request for _, request in requests]
        for request in mine:
            self.scheduler.check_request(request)      # all of them before any is queued: a refusal leaves nothing behind
        finished: list[Request] = []
        self.scheduler.drain_finished()
        step = 0
        try:
            with full_collections_deferred():
                while requests or self.scheduler.has_unfinished():
                    while requests and requests[0][0] <= step:
                        self.add_request(requests.popleft()[1])
                    finished.extend(self.step())
                    step += 1
                self._read_unread()
        except BaseException:
            self.abort(mine)
            raise
        finished.extend(self.scheduler.drain_finished())
        return finished

    def abort(self, requests: list[Request]) -> None:
        """Take these requests out of the queues and give back their pages and state slots, whatever state a
        failed step left them in.  Tokens of a launched step that the host has not read yet are read first, so
        that a request which is not among ``requests`` (queued earlier through ``add_request`` and still
        running) keeps its real token instead of a stand-in; if they cannot be read (the device failed), every
        request that holds a stand-in is aborted too."""
        requests = list(requests)
        pending = self._unread
        try:
            self._read_unread()
        except Exception:
            self._unread = None
            for portion in pending.portions:
                if portion.request not in requests:
                    requests.append(portion.request)
        for request in requests:
            if request.status is not RequestStatus.FINISHED and request.output_tokens \
                    and request.output_tokens[-1] == UNREAD:
                request.output_tokens.pop()
            self.scheduler.abort(request)
        self.scheduler.drain_finished()
