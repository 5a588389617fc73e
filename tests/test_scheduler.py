"""The scheduler's decisions, and the engine loop over a runner and a sampler that need no GPU.

The fake runner keeps real cache books (a KVCacheManager without pools) and returns logits whose
argmax is a known function of the request, as the reference's mock model does with a fixed
argmax of 3 (test/test_engine/test_engine.cpp:11-80)."""
import types

import pytest
import torch

from nanoinfer_amd.cache.block_manager import OutOfPages
from nanoinfer_amd.cache.manager import KVCacheManager
from nanoinfer_amd.engine.llm import Engine
from nanoinfer_amd.engine.scheduler import EngineConfig, RequestRefused, RequestState, Scheduler
from nanoinfer_amd.parts.base import CacheNeed, KVNeed
from nanoinfer_amd.sampling.params import SamplingParams

VOCAB = 50


class FakeRunner:
    """Books like the real runner; logits put the mass on (last token + 1) % VOCAB."""

    def __init__(self, page_size=4, num_pages=16, max_requests=8, max_positions=1000, eos=()):
        self.cache = KVCacheManager({0: CacheNeed(kv=KVNeed(1, 16))}, page_size, num_pages, max_requests)
        self.device = torch.device("cpu")
        self.vocab_size = VOCAB
        self.max_positions = max_positions
        self.eos_token_ids = tuple(eos)
        self._done = {}
        self.steps = []          # [(request, n_tokens, wants)] of every step, for the assertions

    def release(self, request):
        if request in self._done:
            del self._done[request]
            self.cache.release(request)

    def step(self, entries, end=()):
        totals = [(e.request, self._done.get(e.request, 0) + len(e.tokens)) for e in entries]
        if not self.cache.can_reserve_all(totals):
            raise OutOfPages("fake runner: the scheduler planned more than the cache holds")
        rows = []
        for e, (_, total) in zip(entries, totals):
            assert self.cache.reserve(e.request, total)
            self._done[e.request] = total
            for w in e.want:
                row = torch.zeros(VOCAB)
                row[(int(e.tokens[w]) + 1) % VOCAB] = 5.0
                rows.append(row)
        self.steps.append([(e.request, len(e.tokens), list(e.want)) for e in entries])
        self.cache.check()
        return torch.stack(rows) if rows else None


class ArgmaxSampler:
    def sample(self, logits, params, generated, counters, greedy=None):
        assert len(params) == len(generated) == len(counters) == logits.shape[0]
        return logits.argmax(dim=-1).tolist()


def make_engine(**kw):
    runner_kw = {k: kw.pop(k) for k in list(kw) if k in ("page_size", "num_pages", "max_requests", "max_positions", "eos")}
    runner = FakeRunner(**runner_kw)
    cfg = EngineConfig(block_size=runner.cache.page_size, num_cache_blocks=runner.cache.num_pages, **kw)
    return Engine(config=cfg, runner=runner, sampler=ArgmaxSampler()), runner


def test_first_token_comes_with_the_last_prompt_portion():
    # test/test_engine/test_engine.cpp:121-143: prefill yields the first token in the same step
    eng, runner = make_engine()
    rid = eng.add_request([7, 8, 9], max_new_tokens=3, params=SamplingParams.greedy())
    assert eng.get_request(rid).state == RequestState.WAITING
    assert eng.step() == []
    r = eng.get_request(rid)
    assert r.generated == [10] and r.num_computed == 3 and r.state == RequestState.RUNNING
    assert runner.steps[0] == [(rid, 3, [2])]
    eng.step()                                     # one token per decode step (test_engine.cpp:145-163)
    assert r.generated == [10, 11] and runner.steps[1] == [(rid, 1, [0])]
    done = eng.step()
    assert [d.request_id for d in done] == [rid] and r.generated == [10, 11, 12] and r.finish_reason == "length"
    assert not eng.has_work() and not runner.cache.live_requests()        # pages and slot are back
    # the last sampled token is never fed: 1 prompt step + 2 decode steps for 3 tokens
    assert len(runner.steps) == 3


def test_running_first_then_fcfs_fill():
    # test/test_engine/test_scheduler.cpp:78-117
    eng, runner = make_engine(max_batch_size=2, num_pages=64)
    a = eng.add_request([1, 2], 4)
    b = eng.add_request([3], 4)
    c = eng.add_request([4], 4)
    for r in (a, b, c):
        eng.get_request(r).params = SamplingParams.greedy()
    eng.step()
    assert [x[0] for x in runner.steps[0]] == [a, b]          # the batch cap keeps c waiting
    eng.step()
    assert [x[0] for x in runner.steps[1]] == [a, b]          # running requests come first, every step
    assert eng.scheduler.stats()["num_waiting"] == 1
    eng.run()
    assert [eng.get_request(r).finish_reason for r in (a, b, c)] == ["length"] * 3
    first_c = next(i for i, s in enumerate(runner.steps) if any(x[0] == c for x in s))
    assert first_c == 4                                       # c enters when a and b have finished (4 steps each)


def test_max_sequences_caps_running_requests():
    eng, runner = make_engine(max_sequences=1, num_pages=64)
    a, b = eng.add_request([1], 2), eng.add_request([2], 2)
    eng.step()
    assert eng.scheduler.stats()["num_running"] == 1 and eng.scheduler.stats()["num_waiting"] == 1
    eng.run()
    assert all(len(s) == 1 for s in runner.steps)


def test_token_budget_cuts_prompts_into_portions():
    eng, runner = make_engine(max_num_batched_tokens=8, prefill_chunk_size=6, num_pages=64)
    a = eng.add_request(list(range(1, 11)), 2)                # 10 prompt tokens
    b = eng.add_request(list(range(20, 25)), 2)               # 5 prompt tokens
    for r in (a, b):
        eng.get_request(r).params = SamplingParams.greedy()
    eng.step()
    assert runner.steps[0] == [(a, 6, []), (b, 2, [])]        # chunk cap 6, then what is left of the budget
    eng.step()
    # a's rest (4, sampling) and b's rest (3, sampling): both portions end at the prompt's last token
    assert runner.steps[1] == [(a, 4, [3]), (b, 3, [2])]
    eng.step()
    assert runner.steps[2] == [(a, 1, [0]), (b, 1, [0])]
    assert all(sum(n for _, n, _ in s) <= 8 for s in runner.steps)


def test_decode_tokens_go_before_prompt_portions():
    eng, runner = make_engine(max_num_batched_tokens=5, prefill_chunk_size=4, num_pages=64)
    a = eng.add_request(list(range(12)), 3)
    eng.step()                                                # a: 4 of 12
    b = eng.add_request([1], 3)
    eng.step()                                                # a: 4 more; b admitted with 1 token
    assert runner.steps[1] == [(a, 4, []), (b, 1, [0])]
    eng.step()                                                # b decodes first, a gets the rest of the budget
    assert runner.steps[2] == [(b, 1, [0]), (a, 4, [3])]


def test_stop_token_ends_a_request_and_is_kept():
    # src/engine/inference_request.cpp:61-73: the stop token is appended, then the request ends
    eng, runner = make_engine(eos=(12,), num_pages=64)
    rid = eng.add_request([9], 10, SamplingParams.greedy())
    eng.run()
    r = eng.get_request(rid)
    assert r.generated == [10, 11, 12] and r.finish_reason == "stop"


def test_requests_that_can_never_fit_are_refused():
    eng, runner = make_engine(page_size=4, num_pages=4, max_positions=1000)      # 16 tokens in all
    with pytest.raises(RequestRefused):
        eng.add_request(list(range(10)), 8)                   # 10 + 8 - 1 = 17 > 16
    eng.add_request(list(range(10)), 7)                       # 16 fits
    with pytest.raises(RequestRefused):
        eng.add_request([], 3)
    with pytest.raises(RequestRefused):
        eng.add_request([1], 0)
    with pytest.raises(ValueError):
        eng.add_request([VOCAB], 3)
    eng2, _ = make_engine(num_pages=64, max_positions=12)
    with pytest.raises(RequestRefused):
        eng2.add_request(list(range(10)), 4)                  # the model's positions end at 12
    eng3, _ = make_engine(num_pages=64, max_model_len=8)
    with pytest.raises(RequestRefused):
        eng3.add_request(list(range(8)), 2)


def test_waiting_request_waits_for_pages():
    eng, runner = make_engine(page_size=4, num_pages=4)       # 16 tokens
    a = eng.add_request(list(range(9)), 4, SamplingParams.greedy())    # 3 pages
    b = eng.add_request(list(range(7)), 2, SamplingParams.greedy())    # 2 pages: does not fit beside a
    eng.step()
    assert [x[0] for x in runner.steps[0]] == [a] and eng.get_request(b).state == RequestState.WAITING
    eng.run()
    assert eng.scheduler.num_preemptions == 0
    assert eng.get_request(b).generated == [7, 8] and eng.get_request(a).generated == [9, 10, 11, 12]


def test_running_out_of_pages_preempts_the_youngest():
    eng, runner = make_engine(page_size=4, num_pages=4, max_num_batched_tokens=64, admission_headroom=0)
    a = eng.add_request([1, 2, 3, 4, 5, 6, 7], 9, SamplingParams.greedy())   # 7 -> 15 tokens: ends in 4 pages
    b = eng.add_request([11, 12, 13, 14, 15, 16, 17], 9, SamplingParams.greedy())
    eng.step()                                                # both admitted: 2 pages each, pool full
    assert [x[0] for x in runner.steps[0]] == [a, b]
    eng.step()                                                # position 7 still lies in each one's second page
    assert eng.scheduler.num_preemptions == 0
    eng.step()                                                # position 8 needs a third page: b, the youngest, gives way
    rb = eng.get_request(b)
    assert eng.scheduler.num_preemptions == 1 and rb.preemptions == 1
    assert rb.state == RequestState.WAITING and rb.num_computed == 0 and eng.scheduler.waiting[0] is rb
    assert rb.generated == [18, 19] and [x[0] for x in runner.steps[2]] == [a]      # what b generated is kept
    assert not runner.cache.has(b)
    eng.run()
    ra = eng.get_request(a)
    assert ra.generated == list(range(8, 17)) and rb.generated == list(range(18, 27))
    assert ra.finish_reason == rb.finish_reason == "length"
    # b was recomputed from position 0 with its generated tokens as part of the prompt
    again = [s for s in runner.steps if any(x[0] == b and x[1] > 1 for x in s)]
    assert len(again) == 2 and again[1][0][1] == 9            # 7 prompt + 2 generated
    assert not runner.cache.live_requests() and runner.cache.free_pages() == 4


def test_a_newcomer_is_not_admitted_into_the_last_pages():
    """With headroom (the default: one page for every running request) the second request waits
    until the first is done instead of being admitted and preempted; a request alone may fill the
    pool; and fewer prompts are computed twice under random traffic."""
    eng, runner = make_engine(page_size=4, num_pages=4, max_num_batched_tokens=64)
    a = eng.add_request([1, 2, 3, 4, 5, 6, 7], 9, SamplingParams.greedy())
    b = eng.add_request([11, 12, 13, 14, 15, 16, 17], 9, SamplingParams.greedy())
    eng.step()
    assert [x[0] for x in runner.steps[0]] == [a] and eng.get_request(b).state == RequestState.WAITING
    eng.run()
    assert eng.scheduler.num_preemptions == 0
    assert eng.get_request(a).generated == list(range(8, 17)) and eng.get_request(b).generated == list(range(18, 27))
    # alone, a request takes every page
    eng, runner = make_engine(page_size=4, num_pages=4)
    c = eng.add_request(list(range(1, 14)), 4, SamplingParams.greedy())           # 13 + 3 = 16 tokens: the whole pool
    eng.run()
    assert eng.get_request(c).finish_reason == "length" and eng.scheduler.num_preemptions == 0
    # random traffic on a small pool: all finish either way, with headroom fewer are thrown out
    import random
    thrown = {}
    for headroom in (0, 1):
        rng = random.Random(5)
        eng, runner = make_engine(page_size=4, num_pages=24, max_requests=8, max_sequences=8, max_batch_size=8,
                                  max_num_batched_tokens=32, admission_headroom=headroom)
        want = {}
        for _ in range(60):
            if rng.random() < 0.5:
                prompt = [rng.randrange(VOCAB) for _ in range(rng.randint(4, 24))]
                n = rng.randint(8, 24)
                want[eng.add_request(prompt, n, SamplingParams.greedy())] = [(prompt[-1] + 1 + i) % VOCAB for i in range(n)]
            eng.step()
        eng.run()
        assert all(eng.get_request(r).generated == t for r, t in want.items())
        assert runner.cache.free_pages() == 24
        thrown[headroom] = eng.scheduler.num_preemptions
    assert thrown[1] < thrown[0], thrown


def test_engine_never_plans_more_than_fits():
    """Random traffic on a small pool: every step the runner can reserve what was planned (the
    fake runner raises otherwise), every request finishes with the right tokens."""
    import random
    rng = random.Random(0)
    eng, runner = make_engine(page_size=4, num_pages=12, max_requests=6, max_sequences=6, max_batch_size=4,
                              max_num_batched_tokens=16, prefill_chunk_size=8)
    want = {}
    for _ in range(40):
        for _ in range(rng.randint(0, 2)):
            prompt = [rng.randrange(VOCAB) for _ in range(rng.randint(1, 20))]
            n = rng.randint(1, 12)
            rid = eng.add_request(prompt, n, SamplingParams.greedy())
            want[rid] = [(prompt[-1] + 1 + i) % VOCAB for i in range(n)]
        eng.step()
    eng.run()
    for rid, tokens in want.items():
        assert eng.get_request(rid).generated == tokens
    assert runner.cache.free_pages() == 12 and eng.scheduler.stats()["num_finished"] == len(want)
    assert all(len(s) <= 4 and sum(n for _, n, _ in s) <= 16 for s in runner.steps)


# ---- runs of decode steps on one scheduling decision

class FakeRunnerWithRuns(FakeRunner):
    """A runner that can also decode several steps in a row, feeding every step's largest logit to the next."""

    def __init__(self, **kw):
        super().__init__(**kw)
        self.runs = []           # length of every run asked for

    def decode_run(self, entries, steps, pick=None):
        from nanoinfer_amd.engine.runner import StepEntry
        self.runs.append(steps)
        chosen = []
        tokens = [e.tokens[0] for e in entries]
        for k in range(steps):
            logits = self.step([StepEntry(e.request, [t], [0]) for e, t in zip(entries, tokens)])
            if pick is None:
                tokens = logits.argmax(dim=-1).tolist()
            else:
                out = torch.empty(len(entries), dtype=torch.int32)
                pick(k, logits, out)
                tokens = out.tolist()
            chosen.append(tokens)
        return chosen


def make_run_engine(**kw):
    runner_kw = {k: kw.pop(k) for k in list(kw) if k in ("page_size", "num_pages", "max_requests", "max_positions", "eos")}
    runner = FakeRunnerWithRuns(**runner_kw)
    cfg = EngineConfig(block_size=runner.cache.page_size, num_cache_blocks=runner.cache.num_pages, **kw)
    return Engine(config=cfg, runner=runner, sampler=ArgmaxSampler()), runner


def test_decode_runs_give_the_tokens_of_single_steps():
    outs = []
    for run in (1, 8):
        eng, runner = make_run_engine(max_decode_run=run, num_pages=32)
        a = eng.add_request([7, 8, 9], max_new_tokens=12, params=SamplingParams.greedy())
        b = eng.add_request([20], max_new_tokens=5, params=SamplingParams.greedy())
        eng.run()
        outs.append([(eng.get_request(r).generated, eng.get_request(r).finish_reason) for r in (a, b)])
        assert not runner.cache.live_requests()
        if run == 1:
            assert runner.runs == []
        else:
            # both decode together for 4 steps (the shorter request has 4 tokens left), then the longer alone: 7 = 7
            assert runner.runs == [4, 7]
    assert outs[0] == outs[1]
    assert outs[0][0] == (list(range(10, 22)), "length") and outs[0][1] == (list(range(21, 26)), "length")


def test_a_stop_token_inside_a_run_ends_the_request_there():
    eng, runner = make_run_engine(max_decode_run=8, eos=(13,), num_pages=32)
    a = eng.add_request([8, 9], max_new_tokens=20, params=SamplingParams.greedy())      # 10, 11, 12, 13: stop
    b = eng.add_request([19, 20], max_new_tokens=20, params=SamplingParams.greedy())
    eng.step()                                     # the prompts (a prompt of one token would start a run itself)
    finished = eng.step()                          # one run of 8 steps: a stops at its third
    ra, rb = eng.get_request(a), eng.get_request(b)
    assert [r.request_id for r in finished] == [a]
    assert ra.generated == [10, 11, 12, 13] and ra.finish_reason == "stop"      # the stop token is kept, nothing after it
    assert rb.generated == list(range(21, 30)) and rb.finish_reason is None
    assert set(runner.cache.live_requests()) == {b}
    eng.run()
    assert rb.generated == list(range(21, 41)) and not runner.cache.live_requests()


def test_what_keeps_a_decode_step_single():
    greedy = SamplingParams.greedy()
    # somebody who waits for a place keeps nothing single: the decision has just refused it, and nothing changes
    # before a request ends (max_sequences 1 keeps the second request out until the first has gone)
    eng, runner = make_run_engine(max_decode_run=8, max_sequences=1, num_pages=32)
    a = eng.add_request([1, 2], max_new_tokens=4, params=greedy)
    b = eng.add_request([3, 4], max_new_tokens=4, params=greedy)
    eng.run()
    assert runner.runs == [3, 3]
    assert eng.get_request(a).generated == [3, 4, 5, 6] and eng.get_request(b).generated == [5, 6, 7, 8]
    # a request that draws, or that has a repetition penalty
    for params in (SamplingParams(temperature=0.7, seed=1), SamplingParams(temperature=0.0, repetition_penalty=1.3)):
        eng, runner = make_run_engine(max_decode_run=8, num_pages=32)
        eng.add_request([1, 2], max_new_tokens=6, params=params)
        eng.run()
        assert runner.runs == []
    # unless the sampler can plan a request's choices ahead (it then keeps the tokens of a penalty itself)
    class PlanningSampler(ArgmaxSampler):
        def __init__(self):
            self.plans = []

        def plan(self, params, generated, steps):
            self.plans.append(([list(g) for g in generated], steps))
            return types.SimpleNamespace(launch=lambda i, logits, out: out.copy_(logits.argmax(dim=-1)))
    for params in (SamplingParams(temperature=0.7, seed=1), SamplingParams(temperature=0.0, repetition_penalty=1.3)):
        eng, runner = make_run_engine(max_decode_run=8, num_pages=32)
        eng.sampler = PlanningSampler()
        r = eng.add_request([1, 2], max_new_tokens=6, params=params)
        eng.run()
        assert runner.runs == [5] and eng.get_request(r).generated == [3, 4, 5, 6, 7, 8]
        assert eng.sampler.plans == [([[3]], 5)]
    # a prompt portion in the batch
    eng, runner = make_run_engine(max_decode_run=8, num_pages=32, max_num_batched_tokens=4)
    eng.add_request([1, 2], max_new_tokens=6, params=greedy)
    eng.step()
    eng.add_request(list(range(10)), max_new_tokens=2, params=greedy)
    eng.step()
    assert runner.runs == []                        # the step mixed a decode token with a prompt portion
    # pages: four tokens a page, five pages; one request of 3 + 14 tokens can run only as far as pages reach
    eng, runner = make_run_engine(max_decode_run=8, num_pages=5, page_size=4)
    r = eng.add_request([1, 2, 3], max_new_tokens=18, params=greedy)
    eng.run()
    assert eng.get_request(r).finish_reason == "length" and max(runner.runs) <= 8
    sched = eng.scheduler
    assert sched.config.max_decode_run == 8
    with pytest.raises(ValueError):
        EngineConfig(max_decode_run=0).validate()


def test_a_run_can_be_stopped_and_taken_up_again():
    """``stop`` (src/engine/engine.cpp: the flag that ``run`` looks at) ends the loop after the step under way;
    what the requests have generated by then is theirs, and another ``run`` finishes them."""
    eng, runner = make_engine(num_pages=32)
    rid = eng.add_request([1, 2, 3], max_new_tokens=10)
    steps = []
    plain_step = eng.step

    def step_then_stop():
        out = plain_step()
        steps.append(1)
        if len(steps) == 4:
            eng.stop()
        return out

    eng.step = step_then_stop
    assert eng.run() == [] and len(steps) == 4 and eng.has_work()
    assert eng.get_request_result(rid) == [4, 5, 6, 7]          # the prompt's step gave the first, three steps more
    assert eng.get_scheduler_stats()["num_running"] == 1 and eng.get_scheduler_stats()["num_finished"] == 0
    done = eng.run()
    assert [r.request_id for r in done] == [rid] and eng.get_request_result(rid) == list(range(4, 14))
    assert eng.get_scheduler_stats()["num_finished"] == 1 and not eng.has_work()


def test_decode_steps_bring_the_longest_context_first():
    """A step of single tokens is handed to the runner longest context first, whatever the order of arrival (the
    attention kernels pair the ends of that order on a compute unit); the tokens are each request's own."""
    eng, runner = make_engine(num_pages=64)
    short = eng.add_request([1, 2, 3], max_new_tokens=4)
    long = eng.add_request(list(range(10, 19)), max_new_tokens=4)
    middle = eng.add_request([30, 31, 32, 33, 34], max_new_tokens=4)
    eng.run()
    decode_steps = [st for st in runner.steps if all(n == 1 for _, n, _ in st)]
    assert decode_steps and all([r for r, _, _ in st] == [long, middle, short] for st in decode_steps)
    assert eng.get_request_result(short) == [4, 5, 6, 7] and eng.get_request_result(long) == [19, 20, 21, 22]
    assert eng.get_request_result(middle) == [35, 36, 37, 38]
