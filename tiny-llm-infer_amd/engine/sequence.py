"""A request as the scheduler sees it: all its tokens (prompt and completion),
how many of them are in the cache, and its sampling state
(engine/include/sequence.h:12-54)."""
from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import List

from ..sampling.params import SamplingParams


class Status(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass
class Sequence:
    request_id: int
    token_ids: List[int]
    prompt_size: int
    sampling: SamplingParams
    status: Status = Status.WAITING
    tokens_in_cache: int = 0          # tokens whose keys and values are in the cache
    admitted: bool = False              # holds a state slot and pages
    num_sampled: int = 0                # draws used so far; survives preemption
    preemptions: int = 0

    @property
    def size(self) -> int:
        return len(self.token_ids)

    @property
    def completion_size(self) -> int:
        return len(self.token_ids) - self.prompt_size

    @property
    def completion_tokens(self) -> List[int]:
        return self.token_ids[self.prompt_size:]

    @property
    def rng_seed(self) -> int:
        return self.sampling.seed if self.sampling.seed != 0 else self.request_id
