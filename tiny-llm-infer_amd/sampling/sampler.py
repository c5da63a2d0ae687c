"""Choosing the next token of each request from its float32 logits, on the
device.

Greedy: the largest logit, lowest id on ties.  With a temperature: Gumbel-max,
token = argmax(logit + T * g) with g = -log(-log u), as the reference's device
sampler does (kernels/src/sampling_kernel_cuda.cu:44-57).  top_p < 1 keeps the
most probable tokens until their probabilities sum to top_p
(engine/src/llm_engine.cpp:118-141) and draws among those.

Each sampled step of a request uses one draw seed derived from (request seed,
how many tokens the request has sampled so far), so a request's tokens depend
on its own seed and logits only, never on the batch
(engine/src/llm_engine.cpp:197-202 keeps the same invariant with a per-request
mt19937_64)."""
from __future__ import annotations

from typing import List, Sequence

import torch

from .params import SamplingParams

_MASK = (1 << 64) - 1


def splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def draw_seed(request_seed: int, sample_index: int) -> int:
    """The seed of a request's ``sample_index``-th draw."""
    return splitmix64((request_seed * 0x9E3779B97F4A7C15 + sample_index) & _MASK)


class Sampler:
    def __init__(self, ops, device):
        self.ops = ops
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               request_seeds: Sequence[int], sample_indices: Sequence[int]) -> List[int]:
        """One token id per row of ``logits`` [rows, vocab] (float32, on the device)."""
        return self.launch(logits, params, request_seeds, sample_indices).tolist()

    def launch(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               request_seeds: Sequence[int], sample_indices: Sequence[int]) -> torch.Tensor:
        """The same without waiting: the token ids as an int32 tensor on the device."""
        rows = logits.shape[0]
        assert rows == len(params) == len(request_seeds) == len(sample_indices)
        if all(p.greedy for p in params):
            return self.ops.sample(logits)
        seeds = [draw_seed(s, i) for s, i in zip(request_seeds, sample_indices)]
        with_top_p = any(p.top_p < 1.0 and not p.greedy for p in params)
        # One staging buffer for the step's seeds, temperatures and top_p, in page-locked memory where the
        # device is a GPU: its copy is queued behind the step's kernels and does not wait for them, which a
        # copy from ordinary memory does (and with it the host, which then plans the next step beside an
        # idle device).
        staged = torch.empty(rows * 16, dtype=torch.uint8, pin_memory=self.device.type == "cuda")
        staged[:rows * 8].view(torch.int64).copy_(
            torch.tensor([s - (1 << 64) if s >= (1 << 63) else s for s in seeds], dtype=torch.int64))
        staged[rows * 8:rows * 12].view(torch.float32).copy_(
            torch.tensor([0.0 if p.greedy else p.temperature for p in params], dtype=torch.float32))
        staged[rows * 12:].view(torch.float32).copy_(torch.tensor([p.top_p for p in params], dtype=torch.float32))
        dev = staged.to(self.device, non_blocking=True)
        return self.ops.sample(logits, dev[rows * 8:rows * 12].view(torch.float32), dev[:rows * 8].view(torch.int64),
                               top_p=dev[rows * 12:].view(torch.float32) if with_top_p else None)
