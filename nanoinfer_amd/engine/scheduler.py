"""Requests, and the scheduler that decides what each step runs.

Policy, after the reference's FCFS scheduler (src/engine/scheduler.cpp:51-119): requests that are
running come first in every step, then waiting requests are admitted in arrival order while the
caps allow.  Beyond the reference: a step has a token budget (``max_num_batched_tokens``); decode
tokens take one each, what is left is cut into prompt portions of at most ``prefill_chunk_size``
tokens, so a portion may be of any length down to one token; pages are taken portion by
portion, not for the whole prompt at admission (src/engine/engine.cpp:167-172 does the latter).

When pages run out (the reference fails the whole step there, src/engine/engine.cpp:403-404):
a waiting request simply waits (and is admitted only while ``admission_headroom`` pages stay free for
every request already running, so that it is not thrown out again at the next page edge); if a
*running* request cannot get pages for its next tokens, the youngest running request is preempted: its pages go back, its tokens so far (prompt and what it
generated) are kept, and it returns to the *front* of the waiting queue to be recomputed from
position 0 when room appears.  A request that could never fit (longer than the whole pool or the
model's positions) is refused when it is added.

The scheduler is host-only: it sees the cache manager's books, never the GPU.
"""
from __future__ import annotations

import enum
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence

from ..sampling.params import SamplingParams


class RequestState(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass(eq=False)
class Request:
    """Token-level state of one request (include/nanoinfer/engine/inference_request.h:32-169).
    Two requests are the same only if they are the same object (the queues look requests up by
    identity, never by comparing token lists)."""

    request_id: int
    prompt: List[int]
    max_new_tokens: int
    params: SamplingParams
    generated: List[int] = field(default_factory=list)
    num_computed: int = 0            # tokens whose keys and values are in the cache
    state: RequestState = RequestState.WAITING
    finish_reason: Optional[str] = None
    preemptions: int = 0
    arrival_time: float = field(default_factory=time.perf_counter)
    first_token_time: Optional[float] = None
    finish_time: Optional[float] = None

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.generated

    def tokens_from(self, start: int, count: int) -> List[int]:
        """``tokens[start:start + count]`` without putting prompt and generated tokens together first."""
        n = len(self.prompt)
        stop = start + count
        if stop <= n:
            return self.prompt[start:stop]
        if start >= n:
            return self.generated[start - n:stop - n]
        return self.prompt[start:] + self.generated[:stop - n]

    @property
    def num_tokens(self) -> int:
        return len(self.prompt) + len(self.generated)

    @property
    def remaining(self) -> int:
        """Tokens not yet in the cache; the last of them yields the next token's logits."""
        return self.num_tokens - self.num_computed

    def is_prefill(self) -> bool:
        return self.remaining > 1 or not self.generated

    def is_finished(self) -> bool:
        return self.state == RequestState.FINISHED


@dataclass
class EngineConfig:
    """Options of the engine; the first six carry the reference's names
    (include/nanoinfer/engine/engine.h:23-30) and, but for one, its defaults.  A prompt portion
    is as long as the step's token budget by default (the reference cuts at 512): on a GPU of
    256 compute units the matrix products of 512 rows leave most of them idle, and a prompt of
    2,048 tokens runs 1.6 times faster in one portion than in four."""

    max_batch_size: int = 32          # most sequences in one step
    max_sequences: int = 128          # most requests running at once
    prefill_chunk_size: int = 2048    # longest prompt portion of one request in one step
    block_size: int = 16              # tokens per cache page
    num_cache_blocks: int = 1024      # pages in the pool
    kv_cache_bytes: Optional[int] = None  # instead of num_cache_blocks: device memory for all key and value pools
    max_num_batched_tokens: int = 2048  # token budget of a step
    max_model_len: Optional[int] = None  # longest request (prompt + generated); None: what model and pool allow
    max_decode_run: int = 8           # decode steps run back to back on one scheduling decision (1: never more than one)
    admission_headroom: int = 1       # pages left free for every request already running when another is admitted
    one_weight_copy: bool = False     # keep every layer matrix once on the device (no re-tiled copy for decode steps: slower)
    graph_memory_bytes: Optional[int] = None  # device memory that recorded steps may hold together (None: the runner's default)
    dtype: str = "bfloat16"
    seed: int = 0

    def validate(self) -> None:
        for name in ("max_batch_size", "max_sequences", "prefill_chunk_size", "block_size", "num_cache_blocks",
                     "max_num_batched_tokens", "max_decode_run"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be at least 1, got {getattr(self, name)}")


@dataclass
class ScheduledItem:
    request: Request
    start: int          # index of the first token to run (== request.num_computed)
    count: int          # how many tokens to run
    samples: bool       # whether this portion ends at the request's last token (logits wanted there)


@dataclass
class ScheduledBatch:
    items: List[ScheduledItem] = field(default_factory=list)
    preempted: List[int] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(i.count for i in self.items)

    def __bool__(self) -> bool:
        return bool(self.items)


class RequestRefused(ValueError):
    pass


class Scheduler:
    def __init__(self, config: EngineConfig, cache, max_positions: int, eos_token_ids: Sequence[int] = ()):
        config.validate()
        self.config = config
        self.cache = cache
        self.eos_token_ids = frozenset(int(e) for e in eos_token_ids)
        limit = min(int(max_positions), cache.max_tokens_per_request())
        if config.max_model_len is not None:
            limit = min(limit, int(config.max_model_len))
        self.max_model_len = limit
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.requests: Dict[int, Request] = {}
        self._next_id = 0
        self.num_preemptions = 0
        self.num_finished = 0
        self.last_scheduled_tokens = 0

    # ---------------------------------------------------------------- admission
    def add_request(self, prompt: Sequence[int], max_new_tokens: int, params: Optional[SamplingParams] = None) -> int:
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise RequestRefused("a request needs at least one prompt token")
        if max_new_tokens < 1:
            raise RequestRefused(f"max_new_tokens must be at least 1, got {max_new_tokens}")
        # the last generated token is never fed back, so it needs no place in the cache
        need = len(prompt) + max_new_tokens - 1
        if need > self.max_model_len:
            raise RequestRefused(f"a prompt of {len(prompt)} tokens plus {max_new_tokens} new ones needs room for "
                                 f"{need} tokens; the limit is {self.max_model_len}")
        params = params or SamplingParams()
        params.validate()
        rid = self._next_id
        self._next_id += 1
        req = Request(rid, prompt, int(max_new_tokens), params)
        self.requests[rid] = req
        self.waiting.append(req)
        return rid

    # ---------------------------------------------------------------- one step's decision
    def _preempt(self, victim: Request, batch: ScheduledBatch) -> None:
        if self.cache.has(victim.request_id):
            self.release(victim)
        victim.num_computed = 0
        victim.state = RequestState.WAITING
        victim.preemptions += 1
        self.running.remove(victim)
        self.waiting.appendleft(victim)
        self.num_preemptions += 1
        batch.preempted.append(victim.request_id)

    def release(self, request: Request) -> None:
        """Hook for giving back what a request holds; the engine overrides it to tell the runner."""
        self.cache.release(request.request_id)

    def schedule(self) -> ScheduledBatch:
        cfg = self.config
        batch = ScheduledBatch()
        budget = cfg.max_num_batched_tokens
        plan = self.cache.plan()         # what this step will reserve, filled request by request

        def fits(req: Request, count: int) -> bool:
            return plan.fits(req.request_id, req.num_computed + count)

        def take(req: Request, count: int) -> None:
            nonlocal budget
            batch.items.append(ScheduledItem(req, req.num_computed, count, req.num_computed + count == req.num_tokens))
            plan.add(req.request_id, req.num_computed + count)
            budget -= count

        # 1. running requests, decode tokens before prompt portions, each group in admission order
        order = [r for r in self.running if r.remaining == 1] + [r for r in self.running if r.remaining > 1]
        for req in order:
            if req.state is not RequestState.RUNNING:      # preempted while making room for an earlier one
                continue
            if len(batch.items) >= cfg.max_batch_size or budget <= 0:
                break
            count = min(req.remaining, cfg.prefill_chunk_size, budget)
            while not fits(req, count):
                # the youngest running request that this step has not already planned for gives way;
                # that may be the request that does not fit itself
                in_batch = {id(i.request) for i in batch.items}
                victim = next(r for r in reversed(self.running) if id(r) not in in_batch)
                self._preempt(victim, batch)
                if victim is req:
                    break
            else:
                take(req, count)
        # 2. admit waiting requests first come first served
        while self.waiting and len(batch.items) < cfg.max_batch_size and len(self.running) < cfg.max_sequences \
                and budget > 0:
            req = self.waiting[0]
            count = min(req.remaining, cfg.prefill_chunk_size, budget)
            if not fits(req, count):
                break                          # strict FCFS: nobody overtakes the head of the queue
            # Those already running grow by a page now and then: a newcomer that takes the last pages is the
            # youngest, and would be preempted at the next page edge with its prompt computed for nothing.
            # It waits instead until the pool has a little room beside it (nobody running: it may fill the pool).
            if plan.free_after(req.request_id, req.num_computed + count) < cfg.admission_headroom * len(self.running):
                break
            self.waiting.popleft()
            req.state = RequestState.RUNNING
            self.running.append(req)
            take(req, count)
        self.last_scheduled_tokens = batch.num_tokens
        return batch

    def decode_run_length(self, batch: ScheduledBatch, draws: bool = False) -> int:
        """For how many steps in a row ``batch`` can be run again on this one decision (at most
        ``max_decode_run``; 1: only the step that was scheduled).  More than one only if a new
        decision could change nothing but by a request's end: the batch is every running request,
        one token each whose successor is wanted; nobody was preempted; every request decodes
        greedily without a repetition penalty (its next token is then the largest logit, which
        the runner can feed back without the host) unless ``draws`` says that the sampler can plan
        a request's choices ahead; each has that many tokens left to generate; and the pool has
        pages for all of them.  Requests may wait meanwhile: this decision has just refused the
        first of them for want of a place or of pages, and neither comes back before a request
        ends.  A request that meets its stop token within the run has run a few tokens too far:
        they are dropped, and whoever waits for its place gets it that many steps later."""
        steps = self.config.max_decode_run
        if steps <= 1 or not batch.items or batch.preempted or len(batch.items) != len(self.running):
            return 1
        for item in batch.items:
            req = item.request
            if item.count != 1 or not item.samples:
                return 1
            if not draws and (req.params.use_repetition_penalty() or not req.params.use_greedy()):
                return 1
            steps = min(steps, req.max_new_tokens - len(req.generated))
        while steps > 1 and not self.cache.can_reserve_all(
                [(i.request.request_id, i.request.num_computed + steps) for i in batch.items]):
            steps -= 1
        return max(steps, 1)

    # ---------------------------------------------------------------- after the step
    def commit(self, batch: ScheduledBatch, sampled: Dict[int, int]) -> List[Request]:
        """Record that the batch ran; ``sampled`` holds the next token of every item that
        ``samples``.  Returns the requests that finished (src/engine/inference_request.cpp:61-73:
        the stop token is appended before the check)."""
        finished: List[Request] = []
        now = time.perf_counter()
        for item in batch.items:
            req = item.request
            req.num_computed += item.count
            if not item.samples:
                continue
            token = int(sampled[req.request_id])
            req.generated.append(token)
            if req.first_token_time is None:
                req.first_token_time = now
            if token in self.eos_token_ids:
                req.finish_reason = "stop"
            elif len(req.generated) >= req.max_new_tokens:
                req.finish_reason = "length"
            if req.finish_reason is not None:
                req.state = RequestState.FINISHED
                req.finish_time = now
                self.running.remove(req)
                self.release(req)
                self.num_finished += 1
                finished.append(req)
        return finished

    # ---------------------------------------------------------------- queries
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def stats(self) -> Dict[str, int]:
        """src/engine/scheduler.cpp:134-148, plus tokens of the last step and preemptions."""
        return {"num_running": len(self.running), "num_waiting": len(self.waiting),
                "num_finished": self.num_finished, "total_requests": len(self.requests),
                "last_scheduled_tokens": self.last_scheduled_tokens, "num_preemptions": self.num_preemptions}

    def clear_finished(self) -> None:
        for rid in [r for r, q in self.requests.items() if q.is_finished()]:
            del self.requests[rid]
