"""Per-request sampling options, with the names, meanings and defaults of the reference
(include/nanoinfer/sampler/sampling_params.h:25-79)."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0         # logits are divided by it; <= 0 means greedy argmax; 1 leaves them
    top_k: int = -1                  # keep the k largest logits; <= 0 switches it off
    top_p: float = 1.0               # keep the smallest set of tokens whose mass reaches p; active for 0 < p < 1
    repetition_penalty: float = 1.0  # on tokens already generated: l > 0 ? l / p : l * p; 1 switches it off
    seed: int = -1                   # >= 0: reproducible draws; -1: a seed is drawn when the request is added

    def use_greedy(self) -> bool:
        return self.temperature <= 0.0

    def use_top_k(self) -> bool:
        return self.top_k > 0

    def use_top_p(self) -> bool:
        return 0.0 < self.top_p < 1.0

    def use_repetition_penalty(self) -> bool:
        return self.repetition_penalty != 1.0

    @staticmethod
    def greedy() -> "SamplingParams":
        return SamplingParams(temperature=0.0)

    def validate(self) -> None:
        if self.repetition_penalty <= 0:
            raise ValueError(f"repetition_penalty must be positive, got {self.repetition_penalty}")
        if self.top_p < 0 or self.top_p > 1:
            raise ValueError(f"top_p must lie in [0, 1], got {self.top_p}")
