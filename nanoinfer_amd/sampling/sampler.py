"""The sampler above the kernels: from logits and per-request options to one token per row.

Pipeline and fast path follow src/sampler/configurable_sampler.cpp:65-174 of the reference: when
every row is greedy one argmax kernel runs; otherwise a chain of short kernels, in which several
workgroups share a row, does penalty -> temperature -> top-k -> softmax -> top-p -> renormalise ->
draw, and takes the argmax for rows whose temperature is <= 0 (the reference fixes those up through
the host afterwards).

Two things differ on purpose.  The uniform number of a draw comes from a counter-based generator
keyed by (seed, tokens generated so far), so a seeded request gives the same tokens whatever
else is in the batch; the reference passes the same seed at every step and so draws the same
number each time (src/sampler/configurable_sampler.cpp:282).  And a greedy row with a repetition
penalty gets the penalty, also when all rows are greedy.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
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
        # every per-row option in one upload: four float arrays and three int arrays, as int32 words
        floats = np.array([[p.temperature for p in params],
                           [p.top_p if p.use_top_p() else 1.0 for p in params],
                           [p.repetition_penalty for p in params],
                           [uniform_from_counter(max(p.seed, 0), c) for p, c in zip(params, counters)]], dtype=np.float32)
        ints = np.array([p.top_k if p.use_top_k() else 0 for p in params] + pen_off + (pen_ids or [0]), dtype=np.int32)
        packed = torch.from_numpy(np.concatenate([floats.reshape(-1).view(np.int32), ints])).to(self.device)
        as_float = packed[: 4 * R].view(torch.float32)
        temperature, top_p, penalty, uniform = (as_float[i * R:(i + 1) * R] for i in range(4))
        top_k = packed[4 * R: 5 * R]
        off = packed[5 * R: 6 * R + 1]
        ids = packed[6 * R + 1:]
        work = torch.empty_like(logits)
        out = torch.empty(R, dtype=torch.int32, device=self.device)
        K.sample(logits, work, temperature, top_k, top_p, penalty, ids, off, uniform, out,
                 uses_top_k=any(p.use_top_k() and p.temperature > 0 for p in params),
                 uses_top_p=any(p.use_top_p() and p.temperature > 0 for p in params))
        return out.tolist()

    def draw_tables(self, params: Sequence[SamplingParams], generated: Sequence[Sequence[int]], steps: int) -> "DrawTables":
        """The same draws as :meth:`plan` prepares, as host tables for a runner whose recorded decode steps
        draw by themselves (requests without a repetition penalty)."""
        return DrawTables(params, generated, steps)

    def plan(self, params: Sequence[SamplingParams], generated: Sequence[Sequence[int]], steps: int) -> "SamplingPlan":
        """The draws of ``steps`` successive tokens for the same rows, prepared in one upload: the
        uniform numbers of a seeded request do not depend on the tokens drawn before (they are keyed
        by the seed and the count of generated tokens), so a caller can launch step after step
        without reading a token in between.  The tokens of a row with a repetition penalty are kept
        on the device, where every draw adds the token it chose."""
        return SamplingPlan(self.device, params, generated, steps)


class DrawTables:
    """The options of R rows and the uniform numbers of ``steps`` draws as host arrays, for a runner that has
    the draw recorded into its decode steps: ``rows(i)`` is what step i's kernels read, as int32 words
    [temperature | top_p | uniform of step i | top_k], R each.  For requests without a repetition penalty
    (the tokens a penalty looks at grow with every draw; such requests go through :class:`SamplingPlan`)."""

    def __init__(self, params: Sequence[SamplingParams], generated: Sequence[Sequence[int]], steps: int):
        if any(p.use_repetition_penalty() for p in params):
            raise ValueError("draw tables are for requests without a repetition penalty")
        self.steps = int(steps)
        self.uses_top_k = any(p.use_top_k() and p.temperature > 0 for p in params)
        self.uses_top_p = any(p.use_top_p() and p.temperature > 0 for p in params)
        self._head = np.array([[p.temperature for p in params],
                               [p.top_p if p.use_top_p() else 1.0 for p in params]], dtype=np.float32).reshape(-1).view(np.int32)
        self._uniform = np.array([[uniform_from_counter(max(p.seed, 0), len(g) + i) for p, g in zip(params, generated)]
                                  for i in range(self.steps)], dtype=np.float32).view(np.int32)
        self._top_k = np.array([p.top_k if p.use_top_k() else 0 for p in params], dtype=np.int32)

    @property
    def flags(self):
        return (self.uses_top_k, self.uses_top_p)

    def rows(self, i: int) -> np.ndarray:
        return np.concatenate([self._head, self._uniform[i], self._top_k])


class SamplingPlan:
    """Options of R rows and their uniform numbers for ``steps`` draws, on the device."""

    def __init__(self, device, params: Sequence[SamplingParams], generated: Sequence[Sequence[int]], steps: int):
        R = len(params)
        floats = np.array([[p.temperature for p in params],
                           [p.top_p if p.use_top_p() else 1.0 for p in params],
                           [p.repetition_penalty for p in params]], dtype=np.float32)
        uniform = np.array([[uniform_from_counter(max(p.seed, 0), len(g) + i) for p, g in zip(params, generated)]
                            for i in range(steps)], dtype=np.float32)
        # penalised tokens: what a row has generated, and room for the tokens of the run
        pen_ids, pen_off, pen_count = [], [0], []
        for p, g in zip(params, generated):
            mine = sorted(set(int(t) for t in g)) if p.use_repetition_penalty() else []
            pen_count.append(len(mine))
            pen_ids.extend(mine + [0] * steps)
            pen_off.append(len(pen_ids))
        ints = np.array([p.top_k if p.use_top_k() else 0 for p in params] + pen_off + pen_count + pen_ids, dtype=np.int32)
        packed = torch.from_numpy(np.concatenate([floats.reshape(-1).view(np.int32), uniform.reshape(-1).view(np.int32),
                                                  ints])).to(device)
        as_float = packed[: (3 + steps) * R].view(torch.float32)
        self.temperature, self.top_p, self.penalty = (as_float[i * R:(i + 1) * R] for i in range(3))
        self.uniform = as_float[3 * R:].view(steps, R)
        ints_dev = packed[(3 + steps) * R:]
        self.top_k = ints_dev[:R]
        self.pen_off = ints_dev[R: 2 * R + 1]
        self.pen_count = ints_dev[2 * R + 1: 3 * R + 1]
        self.pen_ids = ints_dev[3 * R + 1:]
        self.uses_top_k = any(p.use_top_k() and p.temperature > 0 for p in params)
        self.uses_top_p = any(p.use_top_p() and p.temperature > 0 for p in params)
        self.steps = steps

    def launch(self, i: int, logits: torch.Tensor, out: torch.Tensor) -> None:
        """Launch draw ``i`` over ``logits`` [R, vocab] into ``out`` (int32 [R], device); nothing waits."""
        K.sample(logits, torch.empty_like(logits), self.temperature, self.top_k, self.top_p, self.penalty,
                 self.pen_ids, self.pen_off, self.uniform[i], out, uses_top_k=self.uses_top_k, uses_top_p=self.uses_top_p,
                 pen_count=self.pen_count)
