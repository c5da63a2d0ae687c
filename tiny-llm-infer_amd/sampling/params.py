"""Sampling parameters of a request, with the reference's names, defaults and
checks (engine/include/sampling_params.h:10-34)."""
from __future__ import annotations

from dataclasses import dataclass

GREEDY_BELOW = 1.0e-6      # temperatures at or below this are greedy (engine/src/llm_engine.cpp:81)


@dataclass
class SamplingParams:
    max_tokens: int = 64
    temperature: float = 0.0
    top_p: float = 1.0
    ignore_eos: bool = False
    seed: int = 0              # 0: the request id seeds the draws (engine/src/sequence.cpp:14)

    def validate(self) -> None:
        if self.max_tokens < 0:
            raise ValueError(f"max_tokens is {self.max_tokens}; it counts tokens and cannot be below zero")
        if self.temperature < 0.0:
            raise ValueError(f"temperature is {self.temperature}; 0 means greedy, anything above draws")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p is {self.top_p}; it is the share of the probability mass that is kept, above 0 and at most 1")
        if self.seed < 0:
            raise ValueError(f"seed is {self.seed}; seeds are unsigned (0: the request id seeds the draws)")

    @property
    def greedy(self) -> bool:
        return self.temperature <= GREEDY_BELOW
