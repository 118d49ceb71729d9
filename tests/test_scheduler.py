"""The scheduler's decisions and the generation loop, with a scripted model (no GPU).

Scenarios follow the reference's tests/core/test_continuous_batching.py (mock runner with scripted
tokens, :35-75): admission order, a full pool blocks admission, finishing frees before admitting,
max_concurrent, EOS at the first token, per-request parameters and histories.
"""

from collections import deque

import pytest
import torch

from somi_inference_amd.cache import CacheManager
from somi_inference_amd.engine import Engine, Request, RequestStatus, Scheduler, SchedulerError
from somi_inference_amd.engine.engine import UNREAD
from somi_inference_amd.parts import PagedKVSpec
from somi_inference_amd.sampling import SamplingParams


def make_cache(num_blocks=8, block_size=4, max_requests=8):
    return CacheManager([PagedKVSpec(1, 8)], block_size=block_size, num_blocks=num_blocks,
                        max_requests=max_requests, dtype=torch.float32, device="cpu", allocate_tensors=False)


class ScriptedRunner:
    """Stands in for the model step: does the cache bookkeeping and records what it was given."""

    def __init__(self, cache):
        self.cache = cache
        self.calls = []

    def step(self, entries):
        self.calls.append([(e.request_id, list(e.tokens), list(e.want)) for e in entries])
        for e in entries:
            self.cache.reserve(e.request_id, len(e.tokens))
        for e in entries:
            self.cache.commit(e.request_id, len(e.tokens))
        self.cache.check_invariants()
        return torch.zeros((sum(len(e.want) for e in entries), 4))


class ScriptedSampler:
    """Returns the next scripted token of each request (keyed by its seed, which tests set to its id)."""

    def __init__(self, scripts):
        self.scripts = {k: list(v) for k, v in scripts.items()}
        self.seen = []
        self.draws = []

    def sample(self, logits, params, token_histories=None, seeds=None, counters=None):
        self.seen.append((list(params), [list(h) for h in token_histories], list(counters)))
        assert logits.shape[0] == len(params)
        self.draws.extend(zip(seeds, counters))
        return [self.scripts[s][c] for s, c in zip(seeds, counters)]


def request(rid, prompt_len, max_new, **kw):
    return Request(rid, list(range(100, 100 + prompt_len)), max_new, seed=rid, **kw)


def make_engine(cache, scripts, *, max_concurrent=4, budget=64, chunk=None, eos=None):
    scheduler = Scheduler(cache, max_concurrent=max_concurrent, max_num_batched_tokens=budget, chunk=chunk)
    runner, sampler = ScriptedRunner(cache), ScriptedSampler(scripts)
    return Engine(runner, scheduler, sampler, eos), scheduler, runner, sampler


def test_three_new_tokens_are_one_prompt_step_and_two_decodes_and_the_pool_is_empty_after():
    # /root/reference/tests/core/test_continuous_batching.py:231-261
    cache = make_cache()
    engine, _, runner, _ = make_engine(cache, {0: [7, 8, 9]})
    done = engine.run(deque([(0, request(0, 5, 3))]))
    assert [r.output_tokens for r in done] == [[7, 8, 9]] and done[0].finish_reason == "length"
    assert runner.calls == [[(0, [100, 101, 102, 103, 104], [4])], [(0, [7], [0])], [(0, [8], [0])]]
    assert cache.free_pages() == [8] and not cache.live_requests()


def test_eos_at_the_first_token_ends_without_decoding_and_is_kept():
    # /root/reference/tests/core/test_continuous_batching.py:263-281
    cache = make_cache()
    engine, _, runner, _ = make_engine(cache, {0: [2, 5]}, eos=2)
    done = engine.run(deque([(0, request(0, 3, 4))]))
    assert done[0].output_tokens == [2] and done[0].finish_reason == "eos" and len(runner.calls) == 1
    assert done[0].status == RequestStatus.FINISHED


def test_prompt_is_cut_into_portions_under_the_token_budget_beside_decodes():
    cache = make_cache(num_blocks=16)
    engine, _, runner, _ = make_engine(cache, {0: [1, 2, 3, 4], 1: [5, 6]}, budget=8, chunk=7)
    done = engine.run(deque([(0, request(0, 3, 4)), (1, request(1, 17, 2))]))
    assert {r.request_id: r.output_tokens for r in done} == {0: [1, 2, 3, 4], 1: [5, 6]}
    sizes = [[(rid, len(tokens), want) for rid, tokens, want in call] for call in runner.calls]
    # step 0: request 0's whole prompt; step 1: 0 decodes, 1 gets its first portion of 7 (chunk);
    # step 2: decode + 7 more; step 3: decode first, then the last 3 prompt tokens, whose last logits are sampled
    assert sizes[0] == [(0, 3, [2])]
    assert sizes[1] == [(0, 1, [0]), (1, 7, [])]
    assert sizes[2] == [(0, 1, [0]), (1, 7, [])]
    assert sizes[3] == [(0, 1, [0]), (1, 3, [2])]
    assert all(sum(n for _, n, _ in call) <= 8 for call in sizes)
    assert sizes[4] == [(1, 1, [0])]


def test_first_come_first_served_and_max_concurrent():
    # /root/reference/tests/core/test_continuous_batching.py:120-156, 209-225
    cache = make_cache(num_blocks=32)
    engine, scheduler, runner, _ = make_engine(cache, {i: [1] * 3 for i in range(4)}, max_concurrent=2)
    for i in range(4):
        engine.add_request(request(i, 2, 3))
    engine.step()
    assert [r.request_id for r in scheduler.running] == [0, 1] and [r.request_id for r in scheduler.waiting] == [2, 3]
    done = engine.run()
    assert sorted(r.request_id for r in done) == [0, 1, 2, 3]
    assert max(len(call) for call in runner.calls) == 2


def test_head_of_queue_blocks_those_behind_it_when_its_pages_are_not_free():
    # /root/reference/tests/core/test_continuous_batching.py:158-207
    cache = make_cache(num_blocks=4, block_size=4)
    engine, scheduler, _, _ = make_engine(cache, {0: [1] * 6, 1: [1] * 2, 2: [1] * 2})
    engine.add_request(request(0, 10, 6))     # 3 pages now, a 4th later
    engine.add_request(request(1, 8, 2))      # first portion needs 2 pages: does not fit beside request 0
    engine.add_request(request(2, 2, 2))      # would fit, but must not overtake
    engine.step()
    assert [r.request_id for r in scheduler.running] == [0]
    assert [r.request_id for r in scheduler.waiting] == [1, 2]
    done = engine.run()
    assert [r.request_id for r in done] == [0, 1, 2]
    assert cache.free_pages() == [4]


def test_request_that_can_never_fit_is_refused_when_added():
    cache = make_cache(num_blocks=2, block_size=4)
    engine, _, _, _ = make_engine(cache, {})
    with pytest.raises(SchedulerError, match="needs 3 pages"):
        engine.add_request(request(0, 8, 2))
    engine.add_request(request(1, 8, 1))       # 8 cached tokens at most: fits exactly


def test_when_pages_run_out_the_newest_request_is_preempted_and_recomputed():
    cache = make_cache(num_blocks=4, block_size=4)
    scripts = {0: list(range(10, 20)), 1: list(range(30, 40))}
    engine, scheduler, runner, sampler = make_engine(cache, scripts)
    engine.add_request(request(0, 6, 7))       # grows to 12 tokens = 3 pages
    engine.add_request(request(1, 6, 6))       # 2 pages each at first; both want a third at the same step
    done = engine.run()
    assert {r.request_id: r.output_tokens for r in done} == {0: scripts[0][:7], 1: scripts[1][:6]}
    victim = next(r for r in done if r.request_id == 1)
    assert victim.num_preemptions >= 1
    # the recomputation feeds prompt and the tokens made so far in one portion and samples at its end
    recompute = [call for call in runner.calls for rid, tokens, want in call
                 if rid == 1 and len(tokens) > 6]
    assert recompute, "request 1 was never recomputed"
    assert cache.free_pages() == [4] and not cache.live_requests()
    # a request's random stream goes on where it stopped: every counter 0..5 is drawn exactly once
    assert [c for s, c in sampler.draws if s == 1] == list(range(6))
    assert [c for s, c in sampler.draws if s == 0] == list(range(7))
    assert all(r.finish_reason == "length" for r in done)


def test_oldest_request_is_never_the_victim():
    cache = make_cache(num_blocks=3, block_size=4)
    engine, scheduler, _, _ = make_engine(cache, {0: [1] * 8, 1: [1] * 8})
    engine.add_request(request(0, 4, 8))
    engine.add_request(request(1, 4, 4))
    done = engine.run()
    assert next(r for r in done if r.request_id == 0).num_preemptions == 0
    assert sorted(r.request_id for r in done) == [0, 1]


def test_sampler_sees_each_requests_parameters_history_and_counter():
    # /root/reference/tests/core/test_continuous_batching.py:304-362
    cache = make_cache(num_blocks=16)
    engine, _, _, sampler = make_engine(cache, {0: [50, 51], 1: [60, 61]})
    a = request(0, 3, 2, sampling_params=SamplingParams(temperature=0.0))
    b = request(1, 2, 2, sampling_params=SamplingParams(temperature=0.8, top_k=5))
    engine.run(deque([(0, a), (0, b)]))
    params, histories, counters = sampler.seen[0]
    assert [p.temperature for p in params] == [0.0, 0.8] and counters == [0, 0]
    assert histories == [[100, 101, 102], [100, 101]]            # the prompt alone at the first token (model_runner.py:36)
    params, histories, counters = sampler.seen[1]
    assert histories == [[100, 101, 102, 50], [100, 101, 60]] and counters == [1, 1]   # prompt + outputs (continuous_batching.py:167)


def test_finished_requests_do_not_leak_into_the_next_run():
    # /root/reference/tests/core/test_continuous_batching.py:283-302
    cache = make_cache()
    engine, _, _, _ = make_engine(cache, {0: [1], 1: [2]})
    assert [r.request_id for r in engine.run(deque([(0, request(0, 2, 1))]))] == [0]
    assert [r.request_id for r in engine.run(deque([(0, request(1, 2, 1))]))] == [1]


def test_arrivals_are_injected_by_step():
    cache = make_cache(num_blocks=16)
    engine, _, runner, _ = make_engine(cache, {0: [1] * 4, 1: [2] * 2})
    engine.run(deque([(0, request(0, 2, 4)), (2, request(1, 2, 2))]))
    assert [rid for rid, _, _ in runner.calls[0]] == [0] and [rid for rid, _, _ in runner.calls[1]] == [0]
    assert [rid for rid, _, _ in runner.calls[2]] == [0, 1]


def test_bad_requests_are_refused():
    with pytest.raises(ValueError, match="max_new_tokens"):     # asserted by the reference (continuous_batching.py:34)
        Request(0, [1], 0)
    with pytest.raises(ValueError, match="prompt"):
        Request(0, [], 1)
    for bad in (dict(temperature=-1.0), dict(top_k=0), dict(top_p=0.0), dict(top_p=1.5), dict(repetition_penalty=0.0)):
        with pytest.raises(ValueError):                           # reference: sampler.py:20-25
            SamplingParams(**bad)


class LateTokens:
    """Stands in for tokens that are still on the device: they may be handed on, but reading them is counted."""

    def __init__(self, values, log):
        self.device, self._log = list(values), log

    def tolist(self):
        self._log.append("read")
        return list(self.device)


class AheadRunner(ScriptedRunner):
    accepts_device_tokens = True

    def step(self, entries, device_tokens=None):
        if device_tokens is not None:
            assert all(e.tokens == [0] for e in entries) and len(device_tokens) == len(entries)
            for e, token in zip(entries, device_tokens):
                e.tokens = [token]
            self.log.append("launch ahead")
        else:
            self.log.append("launch")
        return super().step(entries)


class AheadSampler(ScriptedSampler):
    def sample_async(self, logits, params, token_histories=None, seeds=None, counters=None):
        return LateTokens(self.sample(logits, params, token_histories, seeds, counters), self.log)


def ahead_engine(cache, scripts, *, ahead, eos=None, max_concurrent=4):
    scheduler = Scheduler(cache, max_concurrent=max_concurrent, max_num_batched_tokens=64)
    runner, sampler = AheadRunner(cache), AheadSampler(scripts)
    runner.log = sampler.log = []
    engine = Engine(runner, scheduler, sampler, eos)
    assert engine.run_ahead
    engine.run_ahead = ahead
    return engine, runner


@pytest.mark.parametrize("eos", [None, 33])
def test_running_ahead_launches_the_next_step_before_reading_and_changes_no_token(eos):
    """Two decoding requests of different lengths and a late arrival.  Running ahead, a decode step is
    launched before the tokens of the step before are read; it falls back to reading first whenever a
    request is at its last token, one is waiting or one has ended.  The model sees the same tokens at the
    same places as without it, except that a request that ends on EOS has run one token too far."""
    scripts = {0: [30, 31, 32, 33, 34, 35, 36], 1: [40, 41, 42, 43], 2: [50, 51, 52]}

    def run(ahead):
        cache = make_cache(num_blocks=16)
        engine, runner = ahead_engine(cache, scripts, ahead=ahead, eos=eos)
        arrivals = deque([(0, request(0, 5, 7)), (0, request(1, 3, 4)), (4, request(2, 6, 3))])
        done = engine.run(arrivals)
        assert cache.free_pages() == [16] and not cache.live_requests()
        return {r.request_id: (r.output_tokens, r.finish_reason) for r in done}, runner, engine

    want, plain_runner, plain = run(False)
    got, runner, engine = run(True)
    assert got == want and plain.steps_run_ahead == 0 and engine.steps_run_ahead >= 2
    assert all(UNREAD not in tokens for tokens, _ in got.values())
    if eos is None:
        assert runner.calls == plain_runner.calls
        assert got[0] == ([30, 31, 32, 33, 34, 35, 36], "length")
    else:
        assert got[0] == ([30, 31, 32, 33], "eos")
        # the model was given every token it is given without running ahead, at the same place
        given = {(rid, tuple(tokens)) for call in runner.calls for rid, tokens, _ in call}
        assert {(rid, tuple(tokens)) for call in plain_runner.calls for rid, tokens, _ in call} <= given
    log = runner.log
    first = log.index("launch ahead")
    assert log[first - 1] != "read" and log[first + 1] == "read"      # launched first, the older step read after


def test_running_ahead_is_left_alone_when_a_sampling_rule_reads_the_history():
    cache = make_cache(num_blocks=16)
    engine, runner = ahead_engine(cache, {0: [30, 31, 32, 33]}, ahead=True)
    done = engine.run(deque([(0, request(0, 5, 4, sampling_params=SamplingParams(repetition_penalty=1.3)))]))
    assert done[0].output_tokens == [30, 31, 32, 33] and engine.steps_run_ahead == 0
    assert "launch ahead" not in runner.log


def test_a_refused_request_leaves_nothing_behind_for_the_next_call():
    """A list whose second request can never fit is refused before the first is queued, so the next call runs
    its own requests only."""
    cache = make_cache(num_blocks=4, block_size=4)
    engine, scheduler, _, _ = make_engine(cache, {0: [1, 2], 1: [3], 2: [4, 5]})
    with pytest.raises(SchedulerError, match="pages"):
        engine.run(deque([(0, request(0, 3, 2)), (0, request(1, 30, 1))]))
    assert not scheduler.waiting and not scheduler.running and cache.free_pages() == [4]
    done = engine.run(deque([(0, request(2, 3, 2))]))
    assert [(r.request_id, r.output_tokens) for r in done] == [(2, [4, 5])]


def test_token_ids_and_positions_are_checked_before_anything_is_queued():
    cache = make_cache(num_blocks=16)
    scheduler = Scheduler(cache, max_concurrent=4, max_num_batched_tokens=64, vocab_size=50, max_positions=12)
    engine = Engine(ScriptedRunner(cache), scheduler, ScriptedSampler({0: [1, 2], 1: [3, 4, 5]}), None)
    good = Request(0, [1, 2, 3], 2, seed=0)
    with pytest.raises(SchedulerError, match=r"token id 50 is outside \[0, 50\)"):
        engine.run(deque([(0, good), (0, Request(1, [4, 50], 1, seed=1))]))
    with pytest.raises(SchedulerError, match="max_position_embeddings = 12"):
        engine.run(deque([(0, Request(1, list(range(10)), 4, seed=1))]))       # 13 cached tokens
    assert not scheduler.waiting and not scheduler.running and not cache.live_requests()
    done = engine.run(deque([(0, good), (0, Request(1, list(range(10)), 3, seed=1))]))   # 12 tokens: the last position
    assert sorted(r.request_id for r in done) == [0, 1]


class FailingRunner(ScriptedRunner):
    """Raises in a chosen step after it has reserved pages, as a kernel that refuses its arguments would."""

    def __init__(self, cache, fail_at):
        super().__init__(cache)
        self.fail_at = fail_at

    def step(self, entries):
        if len(self.calls) == self.fail_at:
            self.fail_at = -1
            for e in entries:
                self.cache.reserve(e.request_id, len(e.tokens))
            raise RuntimeError("the step failed")
        return super().step(entries)


def test_a_step_that_raises_aborts_the_calls_requests_and_the_next_call_runs():
    cache = make_cache(num_blocks=8, block_size=4)
    scheduler = Scheduler(cache, max_concurrent=4, max_num_batched_tokens=64)
    runner = FailingRunner(cache, fail_at=2)
    engine = Engine(runner, scheduler, ScriptedSampler({0: [1] * 6, 1: [2] * 6, 2: [7, 8]}), None)
    first, second = request(0, 5, 6), request(1, 6, 6)
    with pytest.raises(RuntimeError, match="the step failed"):
        engine.run(deque([(0, first), (0, second)]))
    assert first.finish_reason == second.finish_reason == "aborted"
    assert not scheduler.waiting and not scheduler.running and not cache.live_requests()
    assert cache.free_pages() == [8]
    cache.check_invariants()
    done = engine.run(deque([(0, request(2, 3, 2))]))
    assert [(r.request_id, r.output_tokens) for r in done] == [(2, [7, 8])]


def test_a_bystander_keeps_its_tokens_when_another_calls_step_raises_while_running_ahead():
    """A request queued earlier through add_request decodes beside the request of a run() call.  The step that
    raises was launched ahead of reading the step before, so both requests hold a stand-in for an unread token.
    The call's request is aborted; the bystander gets its real token, is fed that token (not a stand-in) in its
    next step and ends with exactly its scripted tokens."""
    scripts = {0: [30, 31, 32, 33, 34, 35, 36, 37], 1: [40, 41, 42, 43, 44, 45]}

    class FailingAhead(AheadRunner):
        fail_at = 4

        def step(self, entries, device_tokens=None):
            if len(self.calls) == self.fail_at and device_tokens is not None:
                self.fail_at = -1
                raise RuntimeError("the step failed")
            return super().step(entries, device_tokens)

    cache = make_cache(num_blocks=16)
    scheduler = Scheduler(cache, max_concurrent=4, max_num_batched_tokens=64)
    runner, sampler = FailingAhead(cache), AheadSampler(scripts)
    runner.log = sampler.log = []
    engine = Engine(runner, scheduler, sampler, None)
    bystander, mine = request(0, 5, 8), request(1, 3, 6)
    engine.add_request(bystander)
    with pytest.raises(RuntimeError, match="the step failed"):
        engine.run(deque([(0, mine)]))
    assert engine.steps_run_ahead >= 1, "the failing step was not one launched ahead"
    assert mine.finish_reason == "aborted" and UNREAD not in mine.output_tokens
    assert bystander.status is not RequestStatus.FINISHED and scheduler.running == [bystander]
    assert UNREAD not in bystander.output_tokens
    assert bystander.output_tokens == scripts[0][:len(bystander.output_tokens)] and bystander.output_tokens
    done = engine.run()
    assert [(r.request_id, r.output_tokens, r.finish_reason) for r in done] == [(0, scripts[0], "length")]
    fed = [tokens for call in runner.calls for rid, tokens, _ in call if rid == 0]
    assert all(t >= 0 for tokens in fed for t in tokens)
    assert [tokens[0] for tokens in fed[1:]] == scripts[0][:7]
    assert cache.free_pages() == [16] and not cache.live_requests()


def test_portions_come_in_multiples_of_the_granule_except_the_one_that_ends_the_prompt():
    cache = make_cache(num_blocks=32)
    scheduler = Scheduler(cache, max_concurrent=4, max_num_batched_tokens=11, chunk=10, granule=4)
    runner = ScriptedRunner(cache)
    engine = Engine(runner, scheduler, ScriptedSampler({0: [1, 2, 3], 1: [5, 6]}), None)
    done = engine.run(deque([(0, request(0, 3, 3)), (1, request(1, 18, 2))]))
    assert {r.request_id: r.output_tokens for r in done} == {0: [1, 2, 3], 1: [5, 6]}
    portions = [n for call in runner.calls for rid, tokens, _ in call if rid == 1 for n in [len(tokens)]]
    # chunk 10 becomes 8; beside a decoding request 10 tokens of budget are left: 8 again; the rest ends the prompt
    assert portions[:3] == [8, 8, 2] and all(n == 1 for n in portions[3:])
    with pytest.raises(SchedulerError, match="granule"):
        Scheduler(cache, max_concurrent=1, max_num_batched_tokens=8, chunk=3, granule=4)


def test_full_collections_wait_while_requests_are_stepped_and_come_back_after():
    import gc
    before = gc.get_threshold()
    seen = []

    class Watching(ScriptedRunner):
        def step(self, entries):
            seen.append(gc.get_threshold())
            if len(seen) == 3 and self.fail:
                raise RuntimeError("a step that fails")
            return super().step(entries)

    cache = make_cache()
    scheduler = Scheduler(cache, max_concurrent=4, max_num_batched_tokens=64)
    runner = Watching(cache)
    runner.fail = False
    engine = Engine(runner, scheduler, ScriptedSampler({0: [7, 8, 9]}), None)
    engine.run(deque([(0, request(0, 5, 3))]))
    assert seen and all(t[:2] == before[:2] and t[2] > 1_000_000 for t in seen)
    assert gc.get_threshold() == before
    runner.fail = True
    del seen[:]
    with pytest.raises(RuntimeError, match="a step that fails"):
        engine.run(deque([(0, request(0, 5, 3))]))
    assert gc.get_threshold() == before and not cache.live_requests()
