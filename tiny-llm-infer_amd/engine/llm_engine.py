"""The engine: requests in, tokens out (engine/include/llm_engine.h:27-55).

``add_request`` admits a prompt of token ids with its sampling parameters,
``step`` runs one scheduled batch through the step function and samples,
``generate`` runs a list of prompts to the end.  Text is not handled here: the
engine works between a request's tokens and its next token."""
from __future__ import annotations

import threading
from dataclasses import dataclass, field
from typing import List, Optional, Sequence as Seq, Union

import torch

from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .runner import ModelRunner, StepEntry
from .scheduler import BatchPlan, Scheduler, SchedulerConfig
from .sequence import Sequence


@dataclass
class GenerationResult:
    request_id: int
    token_ids: List[int]                 # the completion only
    prompt_token_ids: List[int] = field(default_factory=list)
    preemptions: int = 0


class LLMEngine:
    def __init__(self, runner: ModelRunner, max_model_len: int, max_num_seqs: int,
                 max_num_batched_tokens: int, eos_token_ids: Seq[int] = ()):
        if max_model_len <= 0:
            raise ValueError("Engine capacities and block size must be positive.")
        self.runner = runner
        self.max_model_len = min(max_model_len, runner.max_model_len)
        self.scheduler = Scheduler(SchedulerConfig(max_num_seqs, max_num_batched_tokens), runner.cache)
        self.sampler = Sampler(runner.env.ops, runner.env.device)
        self.eos_token_ids = set(int(t) for t in eos_token_ids)
        self._lock = threading.Lock()        # add_request may come from another thread
        self._next_request_id = 1
        self.total_generated_tokens = 0
        self.num_steps = 0

    # ---- construction ---------------------------------------------------------
    @classmethod
    def from_folder(cls, model_dir: str, dtype="bfloat16", device="cuda:0", max_model_len: int = 2048,
                    page_size: int = 16, num_kv_blocks: int = 0, max_num_seqs: int = 16,
                    max_num_batched_tokens: int = 256, gpu_memory_utilization: float = 0.9,
                    enable_prefix_caching: bool = False, ops=None) -> "LLMEngine":
        from .loading import load_model
        model, cfg = load_model(model_dir, dtype, device, max_model_len, ops)
        return cls.from_model(model, max_model_len=max_model_len, page_size=page_size,
                              num_kv_blocks=num_kv_blocks, max_num_seqs=max_num_seqs,
                              max_num_batched_tokens=max_num_batched_tokens,
                              gpu_memory_utilization=gpu_memory_utilization,
                              enable_prefix_caching=enable_prefix_caching)

    @classmethod
    def from_model(cls, model, max_model_len: int = 2048, page_size: int = 16, num_kv_blocks: int = 0,
                   max_num_seqs: int = 16, max_num_batched_tokens: int = 256,
                   gpu_memory_utilization: float = 0.9, enable_prefix_caching: bool = False) -> "LLMEngine":
        from .sizing import estimate_num_pages
        max_model_len = min(max_model_len, model.spec.max_positions)
        page_size = min(page_size, max_model_len)
        if num_kv_blocks <= 0:
            num_kv_blocks = estimate_num_pages(model, page_size, max_num_batched_tokens,
                                               max_num_seqs, max_model_len, gpu_memory_utilization)
        runner = ModelRunner(model, model.env, page_size=page_size, num_pages=num_kv_blocks,
                             max_requests=max_num_seqs, max_batch_tokens=max_num_batched_tokens,
                             prefix_caching=enable_prefix_caching)
        return cls(runner, max_model_len, max_num_seqs, max_num_batched_tokens,
                   model.spec.eos_token_ids)

    # ---- requests -----------------------------------------------------------------
    def _check_request(self, prompt: Seq[int], sampling: SamplingParams) -> None:
        """engine/src/llm_engine.cpp:41-64."""
        sampling.validate()
        if sampling.max_tokens == 0:
            raise ValueError("max_tokens must be greater than zero.")
        if len(prompt) == 0:
            raise ValueError("A prompt must encode to at least one token.")
        if len(prompt) > self.max_model_len:
            raise ValueError("The prompt exceeds max_model_len.")
        if sampling.max_tokens > self.max_model_len - len(prompt) + 1:
            raise ValueError("The requested completion exceeds max_model_len.")
        vocab = self.runner.model.spec.vocab_size
        for t in prompt:
            if not 0 <= int(t) < vocab:
                raise ValueError(f"Token id {t} is outside the vocabulary of {vocab}.")

    def add_request(self, prompt_tokens: Seq[int], sampling: Optional[SamplingParams] = None) -> int:
        sampling = sampling or SamplingParams()
        self._check_request(prompt_tokens, sampling)
        with self._lock:
            request_id = self._next_request_id
            self._next_request_id += 1
            self.scheduler.add(Sequence(request_id, [int(t) for t in prompt_tokens],
                                        len(prompt_tokens), sampling))
        return request_id

    def is_finished(self) -> bool:
        with self._lock:
            return self.scheduler.is_finished()

    def is_eos(self, token: int) -> bool:
        return token in self.eos_token_ids

    # ---- one step -------------------------------------------------------------------
    def step(self) -> List[GenerationResult]:
        """engine/src/llm_engine.cpp:148-248."""
        with self._lock:
            plan = self.scheduler.schedule()
        if not plan.sequences:
            return []
        entries, sampled_items = [], []
        for i, item in enumerate(plan.sequences):
            seq = item.sequence
            toks = seq.token_ids[item.token_start:item.token_start + item.token_count]
            want = [item.token_count - 1] if item.samples else []
            entries.append(StepEntry(seq.request_id, toks, want))
            if item.samples:
                sampled_items.append(i)
        logits = self.runner.step(entries)
        sampled: List[Optional[int]] = [None] * len(plan.sequences)
        if sampled_items:
            seqs = [plan.sequences[i].sequence for i in sampled_items]
            tokens = self.sampler.sample(logits, [s.sampling for s in seqs],
                                         [s.rng_seed for s in seqs], [s.num_sampled for s in seqs])
            for i, tok in zip(sampled_items, tokens):
                sampled[i] = int(tok)
        with self._lock:
            finished = self.scheduler.postprocess(plan, sampled, self.is_eos)
        self.total_generated_tokens += len(sampled_items)
        self.num_steps += 1
        return [GenerationResult(s.request_id, s.completion_tokens, s.token_ids[:s.prompt_size],
                                 s.preemptions) for s in finished]

    # ---- many prompts to the end --------------------------------------------------------
    def generate(self, prompts: Seq[Seq[int]],
                 sampling: Union[SamplingParams, Seq[SamplingParams], None] = None
                 ) -> List[GenerationResult]:
        """engine/src/llm_engine.cpp:250-317: all prompts are checked before any
        is added; results come back in the order of the prompts."""
        if not prompts:
            return []
        if not self.is_finished():
            raise ValueError("Finish or step existing requests before calling generate.")
        if sampling is None:
            sampling = SamplingParams()
        params = [sampling] * len(prompts) if isinstance(sampling, SamplingParams) else list(sampling)
        if len(params) == 1 and len(prompts) > 1:
            params = params * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("Pass one SamplingParams object or one per prompt.")
        import copy
        for prompt, p in zip(prompts, params):
            self._check_request(prompt, p)
        for prompt, p in zip(prompts, params):
            self.add_request(prompt, copy.copy(p))
        results: List[GenerationResult] = []
        while not self.is_finished():
            results.extend(self.step())
        results.sort(key=lambda r: r.request_id)
        return results
