"""The scheduler: which requests run in the next step and with how many tokens.

The policy is the reference's (engine/src/scheduler.cpp:40-121):

1. Decode first.  Every running request, in round-robin order, gets one token
   while ``max_num_seqs`` and the token budget ``max_num_batched_tokens`` allow.
   A running request that needs a page when none is free is preempted: all it
   holds is given back, it goes to the FRONT of the waiting queue and is later
   computed again from its prompt and everything it has generated.
2. Then prompts.  Waiting requests, in order, each get at most one portion per
   step, cut to the budget that is left.  A request is admitted only when the
   pages for all its current tokens are free (and a state slot); otherwise it
   goes to the back of the queue.  (Layers that keep a window of keys have pages
   of their own, which a request takes portion by portion and gives back as the
   window passes; an admitted request whose portion finds none waits a step.)  With prefix caching, leading full pages that
   the cache knows are taken over and not computed again.  A prompt that needs more pages than the pool
   owns is an error.
3. If nothing could be scheduled while work remains, that is an error.

After the step (engine/src/scheduler.cpp:123-159) a request whose portion
reached its last token, or that decoded, takes its sampled token; it finishes
on an end-of-sequence token (unless ``ignore_eos``) or at ``max_tokens``, and
gives back what it holds.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, List, Optional, Sequence as Seq

from ..cache.manager import CacheFull, CacheManager
from .sequence import Sequence, Status


class SchedulerError(RuntimeError):
    pass


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 16
    max_num_batched_tokens: int = 1024


@dataclass
class PlanItem:
    seq: Sequence
    first: int
    count: int
    prompt_portion: bool

    @property
    def samples(self) -> bool:
        """Does this item end at the request's last token (so a token is sampled)?"""
        return (not self.prompt_portion) or self.first + self.count == self.seq.size


@dataclass
class StepPlan:
    items: List[PlanItem] = field(default_factory=list)
    num_tokens: int = 0


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache: CacheManager):
        if config.max_num_seqs <= 0 or config.max_num_batched_tokens <= 0:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
        self.config = config
        self.cache = cache
        self.waiting: Deque[Sequence] = deque()
        self.running: Deque[Sequence] = deque()
        self.num_preemptions = 0

    def add(self, seq: Sequence) -> None:
        if seq.size == 0:
            raise ValueError("a request without tokens cannot be queued")
        self.waiting.append(seq)

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def plan_ahead(self, plan: StepPlan) -> Optional[StepPlan]:
        """The plan of the step after ``plan``, made while ``plan`` is still running on
        the device, or None if it cannot be known yet.  It is what ``schedule`` would
        give once ``plan`` has been post-processed, as far as that can be told now:

        - every running request is in ``plan`` and is sampled there, so its next token
          (which the host does not know yet) can be fed on the device; it decodes one
          token, unless the running step's token is its last by ``max_tokens``.  One that
          will stop on an end-of-sequence token cannot be known and is skipped when its
          result comes in;
        - waiting requests that hold their pages already go on with their prompts, in the
          same order and under the same budget, starting after the portion that ``plan``
          runs.  A request that is not admitted yet ends the look ahead: admission takes
          pages and a slot, and which are free is known after ``plan``;
        - the pages for all of it are free.  The requests compete for the same pools, so
          the whole step is counted before anything is taken; if it does not fit, nothing
          is taken and the ordinary path decides who waits and who is preempted."""
        if not plan.items:
            return None
        in_plan = {}
        for item in plan.items:
            if item.seq.status == Status.FINISHED:
                return None
            in_plan[id(item.seq)] = item
        cfg = self.config
        budget = cfg.max_num_batched_tokens
        ahead = StepPlan()
        need = [0] * len(self.cache.groups)
        tokens = 0
        for seq in self.running:
            item = in_plan.get(id(seq))
            if item is None or not item.samples:
                return None
            if seq.completion_size + 1 >= seq.sampling.max_tokens:
                continue                      # the running step's token is its last
            if len(ahead.items) >= cfg.max_num_seqs or tokens >= budget:
                return None                   # someone has to wait a turn: the ordinary path rotates them
            # seq.size does not count the running step's token yet: that token goes to position seq.size
            for g, n in enumerate(self.cache.pages_needed(seq.request_id, seq.size + 1)):
                need[g] += n
            ahead.items.append(PlanItem(seq, seq.size, 1, False))
            tokens += 1
        visited = 0
        for seq in self.waiting:
            if len(ahead.items) >= cfg.max_num_seqs or tokens >= budget:
                break
            if not seq.admitted:
                return None
            item = in_plan.get(id(seq))
            first = seq.tokens_in_cache + (item.count if item is not None else 0)
            count = min(seq.size - first, budget - tokens)
            if count <= 0:
                return None
            for g, n in enumerate(self.cache.pages_needed(seq.request_id, first + count)):
                need[g] += n
            ahead.items.append(PlanItem(seq, first, count, True))
            tokens += count
            visited += 1
        if not ahead.items:
            return None
        if any(n > g.pool.free_count for n, g in zip(need, self.cache.groups)):
            return None
        for item in ahead.items:
            self.cache.reserve(item.seq.request_id, item.first + item.count)
        # the queues move as ``schedule`` moves them: each request that got a portion goes to the
        # back of the waiting ones, or to the running ones when the portion reaches its last token
        for item in ahead.items[len(ahead.items) - visited:]:
            seq = self.waiting.popleft()
            assert seq is item.seq
            if item.first + item.count == seq.size:
                seq.status = Status.RUNNING
                self.running.append(seq)
            else:
                self.waiting.append(seq)
        ahead.num_tokens = tokens
        return ahead

    # ---- pages ------------------------------------------------------------
    def _preempt(self, seq: Sequence) -> None:
        if seq.admitted:
            self.cache.release(seq.request_id)
            seq.admitted = False
        seq.status = Status.WAITING
        seq.tokens_in_cache = 0
        seq.preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(seq)

    def _pages_for_whole_pool(self, size: int) -> bool:
        need = self.cache.most_pages_needed(size, self.config.max_num_batched_tokens)
        return all(n <= have for n, have in zip(need, self.cache.pages_per_group()))

    def _admit(self, seq: Sequence) -> bool:
        if self.cache.free_slots() == 0:
            return False
        self.cache.admit(seq.request_id)
        # with prefix caching the leading full pages that are known are taken over
        cached = self.cache.adopt_prefix(seq.request_id, seq.token_ids) if self.cache.prefix_caching else 0
        if not self.cache.can_hold_ahead(seq.request_id, seq.size):
            self.cache.release(seq.request_id)
            return False
        self.cache.hold_ahead(seq.request_id, seq.size)
        seq.admitted = True
        seq.tokens_in_cache = cached
        return True

    # ---- one step's plan -----------------------------------------------------
    def schedule(self) -> StepPlan:
        plan = StepPlan()
        budget = self.config.max_num_batched_tokens
        tokens = 0
        for _ in range(len(self.running)):
            if len(plan.items) >= self.config.max_num_seqs or tokens >= budget:
                break
            seq = self.running.popleft()
            if not self.cache.can_reserve(seq.request_id, seq.size):
                self._preempt(seq)
                continue
            self.cache.reserve(seq.request_id, seq.size)
            plan.items.append(PlanItem(seq, seq.size - 1, 1, False))
            self.running.append(seq)
            tokens += 1

        for _ in range(len(self.waiting)):
            if len(plan.items) >= self.config.max_num_seqs or tokens >= budget:
                break
            seq = self.waiting.popleft()
            if not seq.admitted and not self._admit(seq):
                if not self._pages_for_whole_pool(seq.size):
                    raise SchedulerError(f"request {seq.request_id} holds {seq.size} tokens, more than all {self.cache.num_pages} pages of {self.cache.page_size} can take")
                self.waiting.append(seq)
                continue
            remaining = seq.size - seq.tokens_in_cache
            if remaining <= 0:
                raise SchedulerError(f"request {seq.request_id} waits although all its {seq.size} tokens are in the cache")
            count = min(remaining, budget - tokens)
            if not self.cache.can_reserve(seq.request_id, seq.tokens_in_cache + count):
                # a window group has no pages for this portion yet: the request waits for others to give
                # theirs back, unless no pool could ever hold it
                if not self._pages_for_whole_pool(seq.size):
                    raise SchedulerError(f"request {seq.request_id} holds {seq.size} tokens, more than all {self.cache.num_pages} pages of {self.cache.page_size} can take")
                self.waiting.append(seq)
                continue
            self.cache.reserve(seq.request_id, seq.tokens_in_cache + count)
            plan.items.append(PlanItem(seq, seq.tokens_in_cache, count, True))
            tokens += count
            if seq.tokens_in_cache + count == seq.size:
                seq.status = Status.RUNNING
                self.running.append(seq)
            else:
                self.waiting.append(seq)
        plan.num_tokens = tokens
        if not plan.items and not self.is_finished():
            raise SchedulerError("nothing can run: requests remain, but neither a decode token nor a prompt portion found pages")
        return plan

    # ---- after the step --------------------------------------------------------
    def postprocess(self, plan: StepPlan, sampled: Seq[Optional[int]],
                    is_eos: Callable[[int], bool]) -> List[Sequence]:
        """``sampled[i]`` is the token of plan item i, None where nothing was
        sampled.  Returns the requests that finished."""
        if len(sampled) != len(plan.items):
            raise SchedulerError(f"{len(sampled)} sampled tokens came back for a plan of {len(plan.items)} items")
        finished = []
        for item, token in zip(plan.items, sampled):
            seq = item.seq
            if seq.status == Status.FINISHED:
                continue            # it ended in the step before, while this one was already running
            seq.tokens_in_cache += item.count
            self.cache.register_pages(seq.request_id, seq.token_ids)     # full pages enter the prefix cache
            if item.prompt_portion and seq.tokens_in_cache < seq.size:
                continue
            if token is None or token < 0:
                raise SchedulerError(f"request {seq.request_id} reached its last token in this step but no token was sampled for it")
            seq.token_ids.append(int(token))
            seq.num_sampled += 1
            stopped = (not seq.sampling.ignore_eos) and is_eos(int(token))
            if stopped or seq.completion_size >= seq.sampling.max_tokens:
                seq.status = Status.FINISHED
                self.cache.release(seq.request_id)
                seq.admitted = False
                try:
                    self.running.remove(seq)
                except ValueError:
                    pass
                finished.append(seq)
        return finished
