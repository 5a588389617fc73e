"""The sampler above the kernels: from logits and per-request options to one token per row.

Pipeline and fast path follow src/sampler/configurable_sampler.cpp:65-174 of the reference: when
every row is greedy one argmax kernel runs; otherwise one kernel per row does penalty ->
temperature -> top-k -> softmax -> top-p -> renormalise -> draw, and takes the argmax for rows
whose temperature is <= 0 (the reference fixes those up through the host afterwards).

Two things differ on purpose.  The uniform number of a draw comes from a counter-based generator
keyed by (seed, tokens generated so far), so a seeded request gives the same tokens whatever
else is in the batch; the reference passes the same seed at every step and so draws the same
number each time (src/sampler/configurable_sampler.cpp:282).  And a greedy row with a repetition
penalty gets the penalty, also when all rows are greedy.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .. import kernels as K
from .params import SamplingParams

_M64 = (1 << 64) - 1


def uniform_from_counter(seed: int, counter: int) -> float:
    """A number in (0, 1] from (seed, counter): a splitmix64 finaliser over the mixed pair."""
    x = (seed * 0x9E3779B97F4A7C15 + (counter + 1) * 0xD1B54A32D192ED03 + 0x2545F4914F6CDD1D) & _M64
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _M64
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _M64
    x ^= x >> 31
    return ((x >> 40) + 1) / float(1 << 24)


class Sampler:
    """``sample(logits, params, generated, counters) -> token ids`` on the GPU."""

    def __init__(self, device: Optional[torch.device] = None):
        self.device = device or K.require_gpu()

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               generated: Sequence[Sequence[int]], counters: Sequence[int], greedy=None) -> List[int]:
        """One token id per row of ``logits``.  ``greedy`` (optional) is a function from logits to
        the argmax of every row, for a caller that may hold them already."""
        R, V = logits.shape
        if not (len(params) == len(generated) == len(counters) == R):
            raise ValueError(f"{R} rows of logits need {R} parameter sets, token lists and counters")
        plain_greedy = all(p.use_greedy() and not p.use_repetition_penalty() for p in params)
        if plain_greedy:
            return greedy(logits) if greedy is not None else K.argmax(logits).tolist()
        pen_ids: List[int] = []
        pen_off = [0]
        for p, g in zip(params, generated):
            if p.use_repetition_penalty():
                pen_ids.extend(sorted(set(int(t) for t in g)))
            pen_off.append(len(pen_ids))
        dev = self.device
        f32, i32 = torch.float32, torch.int32
        temperature = torch.tensor([p.temperature for p in params], dtype=f32).to(dev)
        top_k = torch.tensor([p.top_k if p.use_top_k() else 0 for p in params], dtype=i32).to(dev)
        top_p = torch.tensor([p.top_p if p.use_top_p() else 1.0 for p in params], dtype=f32).to(dev)
        penalty = torch.tensor([p.repetition_penalty for p in params], dtype=f32).to(dev)
        uniform = torch.tensor([uniform_from_counter(max(p.seed, 0), c) for p, c in zip(params, counters)],
                               dtype=f32).to(dev)
        ids = torch.tensor(pen_ids if pen_ids else [0], dtype=i32).to(dev)
        off = torch.tensor(pen_off, dtype=i32).to(dev)
        work = torch.empty_like(logits)
        out = torch.empty(R, dtype=i32, device=dev)
        K.sample(logits, work, temperature, top_k, top_p, penalty, ids, off, uniform, out)
        return out.tolist()
