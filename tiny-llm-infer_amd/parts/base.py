"""Interfaces of the parts a model is put together from, and their registries.

Kinds of parts: position encoding, norm, mixer, feed-forward, block
(arrangement), embedding, head.  A part is built from a ``PartSpec`` alone: its
sizes and constants are ``spec.params``, the checkpoint names of its weights
are ``spec.names``, nested parts are ``spec.parts``.  Life cycle:

    part = build_part(kind_of_part, spec)        # no device needed
    part.tensors()                               # -> [TensorDecl] it wants loaded
    part.load(weights, env)                      # weights: name -> tensor on env.device
    part.forward(...)                            # see each interface

No part knows which architecture it is in.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, NamedTuple, Optional

import torch

from ..cache.manager import CacheNeed, StateNeed
from ..config.base import PartSpec
from ..weights.loader import TensorDecl


@dataclass
class BuildEnv:
    """Where and how parts run."""
    dtype: torch.dtype            # torch.bfloat16 or torch.float32: storage of activations and matrices
    device: torch.device
    ops: Any                      # the kernel library (kernels.ops.HipOps)
    max_model_len: int            # highest number of positions a request may reach
    shared: Dict[Any, Any] = field(default_factory=dict)   # what parts of one model build once and share
                                  # (a rotation table that every layer would otherwise build for itself)


@dataclass
class GroupView:
    """One cache group as a step sees it."""
    tensors: Dict[str, torch.Tensor]   # record name -> [layers in group, pages, *page shape of the record]
    tables: torch.Tensor          # int32 [sequences in step, table width], -1 where no page
    table_width: int
    page_size: int
    window: Optional[int]


@dataclass
class LayerCache:
    """The cache of the one layer call that is running."""
    group: GroupView
    layer: int                    # index inside the group's tensors
    writes: bool                  # False: keys/values were written by another call of this step

    def record(self, name: str) -> torch.Tensor:
        """This layer's tensor of the record ``name``: [pages, *page shape]."""
        return self.group.tensors[name][self.layer]


@dataclass
class StepView:
    """The flattened batch of one step.  Rows of one sequence are contiguous
    and in ascending position.  Device tensors are int32."""
    num_rows: int
    num_seqs: int
    token_ids: torch.Tensor       # [rows]
    positions: torch.Tensor       # [rows]
    seq_of_row: torch.Tensor      # [rows]  index into this step's sequences
    row_start: torch.Tensor       # [seqs + 1]  first row of each sequence
    seq_start: torch.Tensor       # [seqs]  position of the sequence's first row
    seq_len: torch.Tensor         # [seqs]  tokens of the sequence after this step
    slots: torch.Tensor           # [seqs]  the sequence's state slot
    sample_rows: torch.Tensor     # [wanted]
    # the same on the host, for parts that plan launches
    h_row_start: List[int] = field(default_factory=list)
    h_seq_start: List[int] = field(default_factory=list)
    h_seq_len: List[int] = field(default_factory=list)
    h_slots: List[int] = field(default_factory=list)
    max_rows_per_seq: int = 1
    max_seq_len: int = 1
    reach: int = 1                # max_seq_len rounded up to a power of two: launches are shaped by
                                  # this, so that steps of like shape launch alike (and can be replayed)
    skew: int = 1                 # the longest sequence has at least this many times the tokens of the average
                                  # one (a power of two, at most 16): launches may split the long ones' work by it
    groups: List[GroupView] = field(default_factory=list)
    # filled by the runner for the layer call that is running
    cache: Optional[LayerCache] = None
    state: Optional[torch.Tensor] = None      # [slots, *StateNeed.shape] of the running mixer


class Part:
    # True if forward() looks at nothing on the host but the step's shape (rows,
    # sequences, table width, reach, skew): then a recorded launch sequence can be replayed
    replayable = False

    def __init__(self, spec: PartSpec):
        self.spec = spec

    def tensors(self) -> List[TensorDecl]:
        return []

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        self.env = env

    def workspace_elems(self, rows: int) -> int:
        """How many elements of activations ``forward`` holds at its widest for a step of
        ``rows`` rows, beyond its input and its result (the q/k/v rows of an attention, the gate
        and up rows of a gated feed-forward).  The engine sums this over a block's parts
        when it sets memory aside for a step before it sizes the cache."""
        return 0


class RotaryTables(NamedTuple):
    """What a rotary encoding hands to the mixer that applies it.  Pair i of a head, i <
    rotary_dim/2, is turned by the angle whose cosine and sine are ``cos[position, i]`` and
    ``sin[position, i]``; ``pairing`` says which two elements pair i is: "half" = (i, i +
    rotary_dim/2), "interleaved" = (2i, 2i + 1).  Elements from ``rotary_dim`` on are left alone."""
    cos: torch.Tensor             # float32 [positions, rotary_dim / 2]
    sin: torch.Tensor
    rotary_dim: int
    pairing: str = "half"


ROTARY_PAIRINGS = ("half", "interleaved")


class PositionEncoding(Part):
    """Rotary encodings expose ``rotary()``: a ``RotaryTables`` (None for an encoding that
    is not rotary and acts elsewhere)."""

    def rotary(self) -> Optional[RotaryTables]:
        return None


class Norm(Part):
    # A norm that sets this also takes ``lazy=True`` in ``forward``: its rows go to matrix
    # products only (the part after it has ``takes_normed_rows``), and it may answer with
    # whatever ``ops.linear`` / ``ops.linear_swiglu`` accept in place of a tensor (rows whose
    # scalar factor the product applies).  A norm without it is never asked.
    supports_lazy = False
    # A norm that sets this takes as ``delta`` whatever ``ops.linear(..., deferred=True)``
    # returned (a product not run yet, or partial sums).  For a norm without it the caller
    # makes a tensor of the delta first.
    takes_unfinished_products = False

    def as_rms(self):
        """(weight float32 [size], eps) if this norm is y = weight * x / sqrt(mean(x^2) + eps) and
        nothing else, so that a kernel which has that formula built in (the attention kernels, for
        the norms of q and k per head) can apply it; None for every other kind of norm."""
        return None

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor],
                rows: Optional[torch.Tensor] = None, num_rows: Optional[int] = None) -> torch.Tensor:
        """``resid`` (float32 [T, n]) += ``delta`` (run dtype [T, n]) if given; return the
        normalised rows in the run dtype.  With ``rows`` (int32 on the device, the first
        ``num_rows`` of them) only those rows are computed and returned, and ``resid`` is left
        unchanged."""
        raise NotImplementedError


def run_norm(norm: "Norm", resid: torch.Tensor, delta, consumer=None, rows=None, num_rows=None):
    """Call a norm as blocks and the step function do: ``delta`` is what the part before still
    owes the residual (None, a tensor, or an unfinished product), ``consumer`` the part that
    reads the normalised rows (None: they are needed as a tensor)."""
    if delta is not None and not isinstance(delta, torch.Tensor) and not norm.takes_unfinished_products:
        delta = norm.env.ops.resolve(delta)
    extra = {}
    if rows is not None:
        extra.update(rows=rows, num_rows=num_rows)
    if consumer is not None and norm.supports_lazy and getattr(consumer, "takes_normed_rows", False):
        extra["lazy"] = True
    return norm.forward(resid, delta, **extra)


class Mixer(Part):
    # True if ``forward`` hands x to ``ops.linear`` / ``ops.linear_swiglu`` only: the norm
    # before it may then leave its scalar factor to that product (``lazy`` norms)
    takes_normed_rows = False

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, x: torch.Tensor, step: StepView) -> torch.Tensor:
        """x: normalised rows [T, hidden] in the run dtype; returns what is
        added to the residual, same shape: a tensor, or whatever
        ``ops.linear(..., deferred=True)`` returned (a norm's ``forward`` takes
        either as its delta; ``ops.resolve`` makes a tensor of it)."""
        raise NotImplementedError


class FeedForward(Part):
    takes_normed_rows = False        # as for a mixer

    def forward(self, x: torch.Tensor, step: StepView) -> torch.Tensor:
        """As ``Mixer.forward``."""
        raise NotImplementedError


class Block(Part):
    """An arrangement of norms, a mixer and a feed-forward around the residual.
    ``forward(resid, pending, step)``: ``pending`` is what the previous block
    still owes the residual (None for the first); returns the new pending."""
    mixer: Mixer
    ffn: FeedForward

    def forward(self, resid: torch.Tensor, pending: Optional[torch.Tensor],
                step: StepView) -> torch.Tensor:
        raise NotImplementedError


_REGISTRIES: Dict[str, Dict[str, Callable[[PartSpec], Part]]] = {
    "position": {}, "norm": {}, "mixer": {}, "ffn": {}, "block": {}, "embedding": {}, "head": {},
}


def register_part(family: str, kind: str, factory: Callable[..., Part], replace: bool = False) -> None:
    """Make ``factory(spec)`` (``factory(spec, mixer, ffn, norms)`` for blocks)
    the implementation of ``kind`` in ``family`` (position, norm, mixer, ffn,
    block, embedding, head)."""
    reg = _REGISTRIES[family]
    if kind in reg and not replace:
        raise ValueError(f"{family} part '{kind}' is already registered")
    reg[kind] = factory


def build_part(family: str, spec: PartSpec, *args) -> Part:
    reg = _REGISTRIES[family]
    if spec.kind not in reg:
        raise KeyError(f"no {family} part of kind '{spec.kind}' is registered; known: "
                       f"{', '.join(sorted(reg)) or 'none'}")
    return reg[spec.kind](spec, *args)
