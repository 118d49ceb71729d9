"""The generation loop: schedule, run one step, sample, finish and free.

Reference: ``ContinuousBatchingEngine`` (somi_inference/core/continuous_batching.py:123-205):
each iteration injects the arrivals of that step, schedules, frees what finished,
prefills the admitted requests one by one and decodes the running ones as a batch;
after every sampled token a request finishes on EOS (which is kept in its output)
or when it has ``max_new_tokens`` (:150-158).  Here one model step serves the whole
mixed batch, and a finished request's pages are free for the very next step.
"""

from __future__ import annotations

from collections import deque

from ..sampling.sampler import Sampler
from .batch import StepEntry
from .request import Request, RequestStatus
from .scheduler import Scheduler, SchedulerOutput


class Engine:
    def __init__(self, runner, scheduler: Scheduler, sampler: Sampler, eos_token_id: int | None) -> None:
        self.runner = runner
        self.scheduler = scheduler
        self.sampler = sampler
        self.eos_token_id = -1 if eos_token_id is None else int(eos_token_id)   # -1: nothing ends a request early
        self.num_steps = 0
        self.last_output: SchedulerOutput | None = None

    def add_request(self, request: Request) -> None:
        self.scheduler.add_request(request)

    def _check_finished(self, request: Request, token: int) -> None:
        if token == self.eos_token_id:
            self.scheduler.finish(request, "eos")
        elif len(request.output_tokens) >= request.max_new_tokens:
            self.scheduler.finish(request, "length")

    def step(self) -> list[Request]:
        """One scheduling decision and one model step; returns the requests that finished in it."""
        output = self.scheduler.schedule()
        self.last_output = output
        self.num_steps += 1
        if not output.portions:
            return self.scheduler.drain_finished()
        entries = [StepEntry(p.request.request_id, p.tokens, [len(p.tokens) - 1] if p.samples else [])
                   for p in output.portions]
        logits = self.runner.step(entries)
        sampled = [p for p in output.portions if p.samples]
        for portion in output.portions:
            portion.request.num_computed += len(portion.tokens)
        if sampled:
            tokens = self.sampler.sample(
                logits,
                [p.request.sampling_params for p in sampled],
                token_histories=[p.request.all_tokens for p in sampled],
                seeds=[p.request.seed for p in sampled],
                counters=[len(p.request.output_tokens) for p in sampled],
            )
            for portion, token in zip(sampled, tokens):
                portion.request.output_tokens.append(int(token))
                self._check_finished(portion.request, int(token))
        return self.scheduler.drain_finished()

    def run(self, requests: deque[tuple[int, Request]] | None = None) -> list[Request]:
        """Run until every request has finished; ``requests`` holds (arrival_step, request) in
        arrival order, as the reference's ``run`` takes them (continuous_batching.py:179-205).
        Returns the requests in the order they finished."""
        requests = requests if requests is not None else deque()
        finished: list[Request] = []
        self.scheduler.drain_finished()
        step = 0
        while requests or self.scheduler.has_unfinished():
            while requests and requests[0][0] <= step:
                self.add_request(requests.popleft()[1])
            finished.extend(self.step())
            step += 1
        return finished
