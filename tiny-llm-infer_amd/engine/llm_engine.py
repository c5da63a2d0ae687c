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
from .scheduler import StepPlan, Scheduler, SchedulerConfig
from .sequence import Sequence, Status


@dataclass
class _Inflight:
    """A step that is on the device: its plan, which items sample, the sampled token
    ids (int32 tensor on the device, not yet read) and each request's row in them."""
    plan: StepPlan
    sampled_items: List[int]
    tokens: Optional[torch.Tensor]
    row_of: dict
    host_copy: Optional[tuple] = None        # (pinned tensor the ids are being copied to, event after the copy)

    def token_list(self) -> List[int]:
        if self.host_copy is None:
            return self.tokens.tolist()
        host, done = self.host_copy
        done.synchronize()
        return host.tolist()


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
            raise ValueError(f"max_model_len is {max_model_len}; a request needs room for at least one token")
        self.runner = runner
        self.max_model_len = min(max_model_len, runner.max_model_len)
        self.scheduler = Scheduler(SchedulerConfig(max_num_seqs, max_num_batched_tokens), runner.cache)
        self.sampler = Sampler(runner.env.ops, runner.env.device)
        self.eos_token_ids = set(int(t) for t in eos_token_ids)
        self._lock = threading.Lock()        # add_request may come from another thread
        self._next_request_id = 1
        self.total_generated_tokens = 0
        self.num_steps = 0
        self.num_steps_ahead = 0
        self.lookahead = True                # put the next step on the device before reading this one
        self._inflight: Optional[_Inflight] = None

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
            raise ValueError("max_tokens is 0: a request has to ask for at least one new token")
        if len(prompt) == 0:
            raise ValueError("the prompt is empty: a request starts from at least one token id")
        if len(prompt) > self.max_model_len:
            raise ValueError(f"the prompt has {len(prompt)} tokens, this engine holds at most {self.max_model_len} a request (max_model_len)")
        if sampling.max_tokens > self.max_model_len - len(prompt) + 1:
            raise ValueError(f"{len(prompt)} prompt tokens and {sampling.max_tokens} new ones do not fit max_model_len = {self.max_model_len}")
        # what the request holds at its longest (its last token is never run) must fit the pools
        # even when it is the only one: else it would be preempted for ever
        cache = self.runner.cache
        longest = len(prompt) + sampling.max_tokens - 1
        need = cache.most_pages_needed(longest, self.scheduler.config.max_num_batched_tokens)
        for g, (n, have) in enumerate(zip(need, cache.pages_per_group())):
            if n > have:
                raise ValueError(f"{len(prompt)} prompt tokens and {sampling.max_tokens} new ones need {n} cache pages "
                                 f"of {cache.page_size} tokens, the cache has {have} (group {g} of its layers)")
        vocab = self.runner.model.spec.vocab_size
        for t in prompt:
            if not 0 <= int(t) < vocab:
                raise ValueError(f"token id {t} in the prompt: the vocabulary has ids 0..{vocab - 1}")

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
            return self.scheduler.is_finished() and self._inflight is None

    def is_eos(self, token: int) -> bool:
        return token in self.eos_token_ids

    def stats(self) -> dict:
        """Counters since construction (the reference counts generated tokens only,
        engine/include/llm_engine.h:46)."""
        cache = self.runner.cache
        with self._lock:
            return {
                "steps": self.num_steps,
                "steps_launched_ahead": self.num_steps_ahead,
                "generated_tokens": self.total_generated_tokens,
                "preemptions": self.scheduler.num_preemptions,
                "waiting": len(self.scheduler.waiting),
                "running": len(self.scheduler.running),
                "pages": cache.num_pages,                  # of the largest group
                "pages_per_group": cache.pages_per_group(),
                "pages_free": cache.free_pages(),          # one count per group of layers
                "pages_taken_total": cache.pages_taken_total,
                "prefix_pages_reused": cache.prefix_hits,
                "recorded_decode_shapes": len(self.runner.graphs),
                "weight_bytes": self.runner.model.weight_bytes(),
                "cache_bytes": self.runner.cache_bytes(),
                # shapes of products of more than 128 rows measured so far, and how many went to this library's kernel
                "product_shapes_measured": len(getattr(self.runner.env.ops, "measured", {})),
                "product_shapes_own_kernel": sum(getattr(self.runner.env.ops, "measured", {}).values()),
            }

    # ---- one step -------------------------------------------------------------------
    def _launch(self, plan: StepPlan, ahead_of: Optional["_Inflight"] = None) -> "_Inflight":
        """Put one planned step on the device: the batch, then the sampling.  Nothing
        is waited for.  With ``ahead_of``, the token of every decoding request is the
        one that step sampled for it and is taken on the device; portions of prompts
        are known on the host as ever."""
        entries, sampled_items = [], []
        fed = {} if ahead_of is None else ahead_of.row_of
        for i, item in enumerate(plan.items):
            seq = item.seq
            want = [item.count - 1] if item.samples else []
            if not item.prompt_portion and seq.request_id in fed:
                entries.append(StepEntry(seq.request_id, [0], want, token_from=fed[seq.request_id]))
            else:
                toks = seq.token_ids[item.first:item.first + item.count]
                if len(toks) != item.count:
                    raise RuntimeError(f"request {seq.request_id}: tokens {item.first} to {item.first + item.count} are planned, it has {seq.size}")
                entries.append(StepEntry(seq.request_id, toks, want))
            if item.samples:
                sampled_items.append(i)
        logits = self.runner.step(entries, feed=ahead_of.tokens if fed else None)
        tokens = None
        row_of = {}
        if sampled_items:
            seqs = [plan.items[i].seq for i in sampled_items]
            # a request whose previous draw is still on the device has one more sample behind it
            tokens = self.sampler.launch(logits, [s.sampling for s in seqs], [s.rng_seed for s in seqs],
                                         [s.num_sampled + (1 if s.request_id in fed else 0) for s in seqs])
            row_of = {s.request_id: j for j, s in enumerate(seqs)}
        return _Inflight(plan, sampled_items, tokens, row_of, self._read_back(tokens))

    def _read_back(self, tokens: Optional[torch.Tensor]):
        """Start copying sampled token ids to the host now, so that reading them later
        waits for this step only and not for whatever is put on the device after it."""
        if tokens is None or tokens.device.type != "cuda":
            return None
        host = torch.empty(tokens.shape, dtype=tokens.dtype, pin_memory=True)
        host.copy_(tokens, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return host, done

    def step(self) -> List[GenerationResult]:
        """One step of the engine (engine/src/llm_engine.cpp:148-248): schedule, run the
        batch, sample, post-process.  When the step after this one is already known
        (see Scheduler.plan_ahead) it is put on the device before this step's tokens
        are read back, its decoding requests fed on the device with the tokens sampled
        here, so the device does not wait for the host between steps."""
        cur = self._inflight
        if cur is None:
            with self._lock:
                plan = self.scheduler.schedule()
            if not plan.items:
                return []
            cur = self._launch(plan)
        nxt = None
        if self.lookahead:
            with self._lock:
                ahead = self.scheduler.plan_ahead(cur.plan)
            if ahead is not None:
                nxt = self._launch(ahead, ahead_of=cur)
                self.num_steps_ahead += 1
        sampled: List[Optional[int]] = [None] * len(cur.plan.items)
        if cur.sampled_items:
            for i, tok in zip(cur.sampled_items, cur.token_list()):         # waits for this step only
                sampled[i] = int(tok)
        live = sum(1 for i in cur.sampled_items if cur.plan.items[i].seq.status != Status.FINISHED)
        with self._lock:
            finished = self.scheduler.postprocess(cur.plan, sampled, self.is_eos)
        self._inflight = nxt
        self.total_generated_tokens += live
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
            raise ValueError("generate() starts from an idle engine: requests added earlier are still being served (step() until is_finished())")
        if sampling is None:
            sampling = SamplingParams()
        params = [sampling] * len(prompts) if isinstance(sampling, SamplingParams) else list(sampling)
        if len(params) == 1 and len(prompts) > 1:
            params = params * len(prompts)
        if len(params) != len(prompts):
            raise ValueError(f"{len(params)} sampling parameter sets for {len(prompts)} prompts: give one for all or one each")
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
