"""The Python entry point: an engine with the reference's verbs.

``Engine(model*, EngineConfig)``, ``add_request(prompt, max_new_tokens, params)``, ``step()``,
``run()``, ``has_work()``, ``get_request(id)`` are the reference's
(include/nanoinfer/engine/engine.h:23-105, src/engine/engine.cpp:119-250); requests are given as
token ids, since the engine is driven below the tokenizer.  A step is: the scheduler picks the
batch, the runner executes it as one forward, the sampler turns the wanted logits into tokens,
the scheduler books the result.  ``generate`` wraps the loop for a list of prompts.
"""
from __future__ import annotations

import random
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

from ..sampling.params import SamplingParams
from .scheduler import EngineConfig, Request, ScheduledBatch, ScheduledItem, Scheduler


@dataclass
class GenerationResult:
    request_id: int
    prompt: List[int]
    tokens: List[int]
    finish_reason: str
    preemptions: int = 0
    time_to_first_token: Optional[float] = None
    total_time: Optional[float] = None


class Engine:
    """``Engine(model_dir, EngineConfig())``; or pass ``runner`` and ``sampler`` objects of your own
    (anything with the same methods), which is how the scheduler's decisions are tested without a GPU."""

    def __init__(self, model_dir: Optional[str] = None, config: Optional[EngineConfig] = None, runner=None,
                 sampler=None, ignore_eos: bool = False):
        self.config = config or EngineConfig()
        self.config.validate()
        if runner is None:
            if model_dir is None:
                raise ValueError("Engine needs a model folder or a runner")
            from .runner import ModelRunner
            runner = ModelRunner(model_dir, dtype=self.config.dtype, page_size=self.config.block_size,
                                 max_tokens=self.config.block_size * self.config.num_cache_blocks,
                                 max_requests=self.config.max_sequences, kv_cache_bytes=self.config.kv_cache_bytes,
                                 max_step_tokens=min(self.config.prefill_chunk_size, self.config.max_num_batched_tokens),
                                 one_weight_copy=self.config.one_weight_copy,
                                 graph_memory_bytes=self.config.graph_memory_bytes)
        if sampler is None:
            from ..sampling.sampler import Sampler
            sampler = Sampler(runner.device)
        self.runner = runner
        self.sampler = sampler
        eos = () if ignore_eos else tuple(getattr(runner, "eos_token_ids", ()) or ())
        self.scheduler = Scheduler(self.config, runner.cache, runner.max_positions, eos)
        self.scheduler.release = lambda req: runner.release(req.request_id)
        self._rng = random.Random(self.config.seed)
        self.num_steps = 0
        self._stop = False
        self.last_prompt_tokens = 0   # tokens of the last step that belonged to prompt portions

    # ---------------------------------------------------------------- requests
    def add_request(self, prompt: Sequence[int], max_new_tokens: int = 128,
                    params: Optional[SamplingParams] = None) -> int:
        params = params or SamplingParams()
        if params.seed < 0 and not params.use_greedy():
            # the reference draws from a clock-seeded generator (configurable_sampler.cpp:23-26);
            # here the draw comes from the engine's own seeded generator, fixed at admission
            params = SamplingParams(params.temperature, params.top_k, params.top_p, params.repetition_penalty,
                                    self._rng.getrandbits(62))
        vocab = getattr(self.runner, "vocab_size", None)
        if vocab is not None:
            for t in prompt:
                if not 0 <= int(t) < vocab:
                    raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        return self.scheduler.add_request(prompt, max_new_tokens, params)

    def get_request(self, request_id: int) -> Request:
        return self.scheduler.requests[request_id]

    def get_request_result(self, request_id: int) -> List[int]:
        """The tokens a request has generated so far (src/engine/engine.cpp: ``get_request_result`` gives their
        text; token ids in and out here, a tokenizer is the caller's)."""
        return list(self.get_request(request_id).generated)

    def get_scheduler_stats(self) -> Dict[str, int]:
        return self.scheduler.stats()

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def stop(self) -> None:
        """Make a ``run`` that is under way (on another thread, or from a callback between steps) return after
        the step it is in; the requests stay where they are and a later ``run`` or ``step`` goes on with them."""
        self._stop = True

    # ---------------------------------------------------------------- stepping
    def step(self) -> List[Request]:
        """One scheduling decision, one forward, one sampling call.  Returns the requests that
        finished in this step."""
        from .runner import StepEntry  # plain data; needs no GPU

        batch: ScheduledBatch = self.scheduler.schedule()
        if not batch:
            return []
        if len(batch.items) > 1 and all(i.count == 1 and i.samples for i in batch.items):
            # a decode step: longest context first (the order stays as the contexts grow together).  The attention
            # kernels give a compute unit the tokens b and B - 1 - b of an uncut batch, a long and a short one.
            batch.items.sort(key=lambda i: -i.start)
        entries = []
        sampling = []
        for item in batch.items:
            toks = item.request.tokens_from(item.start, item.count)
            entries.append(StepEntry(item.request.request_id, toks, [item.count - 1] if item.samples else []))
            if item.samples:
                sampling.append(item.request)
        self.last_prompt_tokens = sum(i.count for i in batch.items if i.count > 1 or not i.request.generated)
        run = 1
        if hasattr(self.runner, "decode_run"):
            run = self.scheduler.decode_run_length(batch, draws=hasattr(self.sampler, "plan"))
        if run > 1:
            return self._decode_run(batch, entries, run)
        logits = self.runner.step(entries)
        sampled: Dict[int, int] = {}
        if sampling:
            ids = self.sampler.sample(logits, [r.params for r in sampling], [r.generated for r in sampling],
                                      [len(r.generated) for r in sampling],
                                      greedy=getattr(self.runner, "greedy_tokens", None))
            sampled = {r.request_id: int(t) for r, t in zip(sampling, ids)}
        self.num_steps += 1
        return self.scheduler.commit(batch, sampled)

    def _decode_run(self, batch: ScheduledBatch, entries, run: int) -> List[Request]:
        """``run`` decode steps of the same batch on one scheduling decision: the runner
        feeds every step's tokens to the next by itself (the largest logits, or what the sampler's
        plan draws); the scheduler then books the steps one by one, and a request that stops on the
        way is finished there and its later tokens dropped."""
        requests = [item.request for item in batch.items]
        if all(r.params.use_greedy() and not r.params.use_repetition_penalty() for r in requests):
            chosen = self.runner.decode_run(entries, run)
        elif (getattr(self.runner, "takes_draw_tables", False) and hasattr(self.sampler, "draw_tables")
              and not any(r.params.use_repetition_penalty() for r in requests)):
            # the draw is part of the recorded step: nothing is launched between a step and the next
            tables = self.sampler.draw_tables([r.params for r in requests], [r.generated for r in requests], run)
            chosen = self.runner.decode_run(entries, run, draw=tables)
        else:
            plan = self.sampler.plan([r.params for r in requests], [r.generated for r in requests], run)
            chosen = self.runner.decode_run(entries, run, pick=plan.launch)
        column = {item.request.request_id: b for b, item in enumerate(batch.items)}
        finished: List[Request] = []
        live = list(batch.items)
        for k, tokens in enumerate(chosen):
            if not live:
                break
            sub = batch if k == 0 else ScheduledBatch(
                items=[ScheduledItem(i.request, i.request.num_computed, 1, True) for i in live])
            sampled = {i.request.request_id: int(tokens[column[i.request.request_id]]) for i in sub.items}
            finished.extend(self.scheduler.commit(sub, sampled))
            live = [i for i in sub.items if i.request.finish_reason is None]
            self.num_steps += 1
        self.scheduler.last_scheduled_tokens = sum(len(t) for t in chosen)
        return finished

    def run(self) -> List[Request]:
        """Step until nothing is left (src/engine/engine.cpp:191-198)."""
        finished: List[Request] = []
        self._stop = False
        while self.has_work() and not self._stop:
            finished.extend(self.step())
        return finished

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128,
                 params: Optional[SamplingParams] = None) -> List[GenerationResult]:
        """Generate for every prompt (lists of token ids) under continuous batching; results in
        the order of the prompts."""
        ids = [self.add_request(p, max_new_tokens, params) for p in prompts]
        self.run()
        out = []
        for rid in ids:
            r = self.get_request(rid)
            out.append(GenerationResult(
                rid, list(r.prompt), list(r.generated), r.finish_reason or "", r.preemptions,
                None if r.first_token_time is None else r.first_token_time - r.arrival_time,
                None if r.finish_time is None else r.finish_time - r.arrival_time))
        return out
