"""The step function.

``ModelRunner.step(entries)`` takes a batch of (request, its next tokens,
places whose logits are wanted): portions of prompts beside single decoded
tokens, cut anywhere.  It runs only those tokens, as one batch, against the
cache that earlier steps left, and returns float32 logits at the wanted places.
The reference's counterpart is Qwen3Model::forward_paged_batch
(model/src/qwen3_paged_batch.cpp:44-366) with the batch assembly of
LLMEngine::step (engine/src/llm_engine.cpp:164-183); there every row carries a
copy of its request's block table, here tables are per request and rows carry
the index of their request.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheFull, CacheManager
from ..parts.base import BuildEnv, GroupView, LayerCache, StepView, run_norm
from .model import Model


@dataclass
class StepEntry:
    key: Hashable                 # the request
    tokens: Sequence[int]         # its next tokens
    want: Sequence[int] = ()      # places among ``tokens`` whose logits are wanted
    token_from: Optional[int] = None   # a single token that is not known on the host yet: its value is
                                       # element ``token_from`` of the tensor given to step(feed=...)


class StepError(ValueError):
    pass


def _pow2_at_least(n: int, floor: int = 4) -> int:
    w = floor
    while w < n:
        w *= 2
    return w


def _pad4(n: int) -> int:
    return (n + 3) & ~3


def _decode_bucket(n: int) -> int:
    """Recorded decode steps come in these numbers of rows: powers of two up to 64 (up to
    16 rows, and from 17 to 64, the matrix products cost the same), then multiples of 32 (the
    products cost the same from 65 to 128 rows; attention and norms do not)."""
    return _pow2_at_least(n, 1) if n <= 64 else (n + 31) // 32 * 32


class StepInputs:
    """One host staging buffer and one device buffer that hold every integer
    input of a step; a step costs one host-to-device copy.  The layout depends
    only on (rows, sequences, wanted, table width)."""

    def __init__(self, device, max_rows: int, max_seqs: int, num_groups: int, max_width: int):
        self.device = torch.device(device)
        cap = (4 * _pad4(max_rows) + _pad4(max_rows) + _pad4(max_seqs + 1) + 3 * _pad4(max_seqs)
               + num_groups * max_seqs * max_width + 64)
        pin = self.device.type == "cuda"
        self.host = [torch.zeros(cap, dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self.host_np = [h.numpy() for h in self.host]
        self.events = [None, None]
        self.dev = torch.zeros(cap, dtype=torch.int32, device=self.device)
        self.turn = 0
        self.num_groups = num_groups

    def layout(self, rows: int, seqs: int, wanted: int, width: int) -> Dict[str, slice]:
        off = 0
        out = {}
        for name, n in (("token_ids", rows), ("token_from", rows), ("positions", rows), ("seq_of_row", rows),
                        ("row_start", seqs + 1), ("seq_start", seqs), ("seq_len", seqs),
                        ("slots", seqs), ("sample_rows", wanted)):
            out[name] = slice(off, off + n)
            off += _pad4(max(n, 1))
        for g in range(self.num_groups):
            out[f"tables{g}"] = slice(off, off + seqs * width)
            off += _pad4(seqs * width)
        out["_end"] = slice(0, off)
        return out

    def begin(self):
        self.turn ^= 1
        ev = self.events[self.turn]
        if ev is not None:
            ev.synchronize()
        return self.host_np[self.turn]

    def upload(self, n: int) -> None:
        if self.device.type == "cuda":
            self.dev[:n].copy_(self.host[self.turn][:n], non_blocking=True)
            ev = self.events[self.turn] or torch.cuda.Event()
            ev.record()
            self.events[self.turn] = ev
        else:
            self.dev[:n].copy_(self.host[self.turn][:n])


class ModelRunner:
    def __init__(self, model: Model, env: BuildEnv, page_size: int, num_pages: int,
                 max_requests: int, max_batch_tokens: int, prefix_caching: bool = False):
        self.model = model
        self.env = env
        self.page_size = page_size
        self.max_batch_tokens = max_batch_tokens
        self.max_requests = max_requests
        self.max_model_len = min(env.max_model_len, model.spec.max_positions)
        env.ops.check_page_size(page_size)
        if prefix_caching and any(n is not None for n in model.state_needs()):
            raise ValueError("prefix caching cannot take over per-request state of a mixer")
        self.cache = CacheManager(model.cache_needs(), page_size, num_pages, max_requests, prefix_caching,
                                  max_step_tokens=max_batch_tokens)
        # The pages' contents: for every group the records its mixers declared, one tensor each,
        # [layers in group, pages, *the record's page shape], zeroed.  A group that keeps all keys has
        # ``num_pages`` pages, a window group no more than its requests can hold together.  (One page
        # and one state slot more than the manager hands out: what the padding rows of a recorded
        # decode step write to.)
        self.group_tensors: List[Dict[str, torch.Tensor]] = []
        for g in self.cache.groups:
            self.group_tensors.append({
                rec.name: torch.zeros((len(g.cache_layers), g.pool.num_pages + 1) + rec.page_shape(page_size),
                                      dtype=rec.dtype or env.dtype, device=env.device)
                for rec in g.need.records})
        self.pad_pages, self.pad_slot = [g.pool.num_pages for g in self.cache.groups], max_requests
        self.states: List[Optional[torch.Tensor]] = []
        for need in model.state_needs():
            self.states.append(None if need is None else torch.zeros(
                (max_requests + 1,) + tuple(need.shape), dtype=need.dtype, device=env.device))
        max_width = _pow2_at_least((self.max_model_len + page_size - 1) // page_size)
        self.inputs = StepInputs(env.device, max(max_batch_tokens, _decode_bucket(max_requests)),
                                 _decode_bucket(max_requests), len(self.cache.groups), max_width)
        self.steps_run = 0
        # Decode steps (one token for every request, every logit wanted) launch the same
        # kernels with the same arguments whenever (requests, table width, reach, skew) agree:
        # their launch sequence is recorded once as a HIP graph and replayed.
        parts = [model.embedding, model.final_norm, model.head] + list(model.blocks)
        self.use_graphs = (env.device.type == "cuda" and env.dtype == torch.bfloat16
                           and all(p.replayable for p in parts))
        self.graphs = {}
        self.graph_pool = None
        self.graph_replays = 0
        # for the replay tool's index: with ``keep_tables`` set, the block tables that the last step
        # ran with (request -> per group a list of pages), taken after its pages were reserved and
        # before a window gave any back
        self.keep_tables = False
        self.tables_run: Dict[Hashable, List[List[int]]] = {}

    # ---- requests ---------------------------------------------------------
    def admit(self, key: Hashable):
        return self.cache.admit(key)

    def release(self, key: Hashable) -> None:
        self.cache.release(key)

    def cache_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for tensors in self.group_tensors for t in tensors.values())

    # ---- the step -----------------------------------------------------------
    def _check(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        if len(entries) > self.max_requests:
            raise StepError(f"{len(entries)} requests in one step, at most {self.max_requests}")
        seen = set()
        rows = 0
        vocab = self.model.spec.vocab_size
        for e in entries:
            if e.key in seen:
                raise StepError(f"request {e.key!r} appears twice in one step")
            seen.add(e.key)
            if e.key not in self.cache:
                raise StepError(f"request {e.key!r} has not been admitted")
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.key!r} brings no tokens")
            rows += n
            total = self.cache.get(e.key).num_tokens + n
            if total > self.max_model_len:
                raise StepError(f"request {e.key!r} would reach {total} tokens, "
                                f"the limit is {self.max_model_len}")
            lo, hi = (min(e.tokens), max(e.tokens))
            if lo < 0 or hi >= vocab:
                raise StepError(f"token id {lo if lo < 0 else hi} of request {e.key!r} is outside the "
                                f"vocabulary of {vocab}")
            if e.token_from is not None and n != 1:
                raise StepError(f"request {e.key!r}: only a single token can come from the device")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"wanted place {w} of request {e.key!r} is outside its "
                                    f"{n} tokens")
        if rows > self.max_batch_tokens:
            raise StepError(f"{rows} tokens in one step, at most {self.max_batch_tokens}")

    def _pack(self, entries: Sequence[StepEntry], feed: Optional[torch.Tensor] = None, pad_to: int = 0) -> StepView:
        """``pad_to``: a decode step is filled up to this many rows with rows of no
        request (token 0 at position 0 of a one-token sequence that lives in the spare
        page and the spare state slot), so that steps of a few different sizes cover
        every number of requests."""
        page = self.page_size
        rcs = [self.cache.get(e.key) for e in entries]
        starts = [rc.num_tokens for rc in rcs]
        counts = [len(e.tokens) for e in entries]
        totals = [s + c for s, c in zip(starts, counts)]
        rows, seqs = sum(counts), len(entries)
        wanted = sum(len(e.want) for e in entries)
        width = _pow2_at_least(max(max((len(tab) for tab in rc.tables), default=1) for rc in rcs))
        pads = max(0, pad_to - seqs)
        lay = self.inputs.layout(rows + pads, seqs + pads, wanted + pads, width)
        buf = self.inputs.begin()
        # every field is put together as one list and written with one assignment
        tok, pos, sor, sample, row_start, src = [], [], [], [], [0], []
        r = 0
        for i, e in enumerate(entries):
            n = counts[i]
            tok.extend(e.tokens)
            src.extend([-1] * n if e.token_from is None else [int(e.token_from)])
            pos.extend(range(starts[i], starts[i] + n))
            sor.extend([i] * n)
            sample.extend(r + int(w) for w in e.want)
            r += n
            row_start.append(r)
        slots = [rc.slot for rc in rcs]
        if pads:
            tok.extend([0] * pads)
            src.extend([-1] * pads)
            pos.extend([0] * pads)
            sor.extend(range(seqs, seqs + pads))
            sample.extend(range(rows, rows + pads))
            row_start.extend(range(rows + 1, rows + pads + 1))
            starts = starts + [0] * pads
            totals = totals + [1] * pads
            counts = counts + [1] * pads
            slots = slots + [self.pad_slot] * pads
        buf[lay["token_ids"]] = tok
        buf[lay["token_from"]] = src
        buf[lay["positions"]] = pos
        buf[lay["seq_of_row"]] = sor
        buf[lay["row_start"]] = row_start
        buf[lay["seq_start"]] = starts
        buf[lay["seq_len"]] = totals
        buf[lay["slots"]] = slots
        if wanted + pads:
            buf[lay["sample_rows"]] = sample
        for g in range(len(self.cache.groups)):
            # (a request's table is one piece of memory: a copy each, whatever their length)
            rows_of = buf[lay[f"tables{g}"]].reshape(seqs + pads, width)
            rows_of.fill(-1)
            for i, rc in enumerate(rcs):
                tab = rc.tables[g]
                if len(tab):
                    rows_of[i, :len(tab)] = np.frombuffer(tab, dtype=np.int32)
            if pads:
                rows_of[seqs:, 0] = self.pad_pages[g]
        self.inputs.upload(lay["_end"].stop)
        dev = self.inputs.dev
        rows, seqs = rows + pads, seqs + pads
        if feed is not None:
            self.env.ops.feed_tokens(dev[lay["token_ids"]], dev[lay["token_from"]], feed, rows)
        groups = []
        for g, gl in enumerate(self.cache.groups):
            groups.append(GroupView(tensors=self.group_tensors[g], tables=dev[lay[f"tables{g}"]].view(seqs, width),
                                    table_width=width, page_size=page, window=gl.need.window))
        return StepView(
            num_rows=rows, num_seqs=seqs,
            token_ids=dev[lay["token_ids"]], positions=dev[lay["positions"]],
            seq_of_row=dev[lay["seq_of_row"]], row_start=dev[lay["row_start"]],
            seq_start=dev[lay["seq_start"]], seq_len=dev[lay["seq_len"]],
            slots=dev[lay["slots"]], sample_rows=dev[lay["sample_rows"]],
            h_row_start=row_start, h_seq_start=starts, h_seq_len=totals,
            h_slots=slots, max_rows_per_seq=max(counts),
            max_seq_len=max(totals), reach=max(128, 1 << (max(totals) - 1).bit_length()),
            skew=min(16, 1 << ((max(totals) * len(totals)) // max(sum(totals), 1)).bit_length() - 1),
            groups=groups)

    def forward(self, step: StepView, num_wanted: int) -> Optional[torch.Tensor]:
        """Run the model over a packed step; float32 logits [wanted, vocab] or None."""
        hold = getattr(self.env.ops, "hold_stream", None)
        if hold is None:
            return self._forward(step, num_wanted)
        with hold():
            return self._forward(step, num_wanted)

    def _forward(self, step: StepView, num_wanted: int) -> Optional[torch.Tensor]:
        model = self.model
        resid = model.embedding.forward(step.token_ids, step.num_rows)
        pending = None
        for i, call in enumerate(model.schedule):
            if call.cache >= 0 and call.cache in self.cache.group_of_layer:
                gi = self.cache.group_of_layer[call.cache]
                step.cache = LayerCache(step.groups[gi],
                                        self.cache.groups[gi].local_layer(call.cache),
                                        call.writes_cache)
            else:
                step.cache = None
            step.state = self.states[i]
            pending = model.blocks[call.block].forward(resid, pending, step)
        step.cache = None
        step.state = None
        if num_wanted == 0:
            return None
        x = run_norm(model.final_norm, resid, pending, rows=step.sample_rows, num_rows=num_wanted)
        return model.head.forward(x)

    def _replay(self, view: StepView, wanted: int) -> torch.Tensor:
        """A decode step through its recorded launch sequence.  The step's inputs
        already lie in the device buffer whose layout depends on the key alone."""
        key = (view.num_seqs, view.groups[0].table_width if view.groups else 0, view.reach, view.skew)
        entry = self.graphs.get(key)
        if entry is None:
            self.forward(view, wanted)                 # once eagerly: anything lazy happens now
            torch.cuda.synchronize(self.env.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, pool=self.graph_pool):
                out = self.forward(view, wanted)
            if self.graph_pool is None:
                self.graph_pool = graph.pool()
            entry = (graph, out)
            self.graphs[key] = entry
        entry[0].replay()
        self.graph_replays += 1
        return entry[1]

    def step(self, entries: Sequence[StepEntry], feed: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run one batch.  Pages are reserved for every entry first; if the pool
        cannot hold the batch, CacheFull is raised and no token has been run.
        ``feed``: int32 tensor on the device that entries with ``token_from`` take
        their token from (the tokens the previous step sampled).

        The logits that come back belong to the runner: for a recorded decode step they are
        a view of the recording's output buffer, which the next step of the same shape
        writes again.  Use them (sample from them, copy them) before the next call of
        ``step``; ``clone()`` what has to outlive it."""
        self._check(entries)
        # all or nothing over the whole batch: groups are independent, requests compete
        need = [0] * len(self.cache.groups)
        for e in entries:
            total = self.cache.get(e.key).num_tokens + len(e.tokens)
            for g, n in enumerate(self.cache.pages_needed(e.key, total)):
                need[g] += n
        for g, n in enumerate(need):
            if n > self.cache.groups[g].pool.free_count:
                raise CacheFull(f"the step needs {n} pages of group {g}, "
                                f"{self.cache.groups[g].pool.free_count} are free")
        for e in entries:
            self.cache.reserve(e.key, self.cache.get(e.key).num_tokens + len(e.tokens))
        if feed is None and any(e.token_from is not None for e in entries):
            raise StepError("an entry takes its token from the device but no tensor was given")
        if self.keep_tables:
            self.tables_run = {e.key: [list(t) for t in self.cache.get(e.key).tables] for e in entries}
        wanted = sum(len(e.want) for e in entries)
        if self.use_graphs and wanted == len(entries) and all(len(e.tokens) == 1 for e in entries):
            view = self._pack(entries, feed, pad_to=_decode_bucket(len(entries)))
            logits = self._replay(view, view.num_rows)[:wanted]
        else:
            view = self._pack(entries, feed)
            logits = self.forward(view, wanted)
        for e in entries:
            self.cache.advance(e.key, self.cache.get(e.key).num_tokens + len(e.tokens))
        self.steps_run += 1
        return logits
