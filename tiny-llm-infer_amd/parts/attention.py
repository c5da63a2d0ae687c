"""Attention over the paged cache with grouped heads.

Order (model/src/qwen3_paged_batch.cpp:147-271): q, k, v projections (no
bias) -> optional per-head norm of q and of k -> optional rotation of q and k (pairs (i, i + d/2) as the reference turns them,
kernels/src/rope_kernel_cpu.cpp:156-179, or neighbours for an encoding that says so)
-> k and v into the cache at (table[pos // page], pos % page) -> for the row at
position p and head h, kv head h // (heads / kv_heads), scores (q.k) * scale
over the keys 0..p (kernels/src/paged_attention_cpu.cpp:16-69), or over
p-window+1..p for a windowed layer, softmax, weighted sum of values -> output
projection.  v is neither normed nor rotated.  Every row reads its keys from
the cache, the step's own rows included, so a portion of a prompt and a single
decoded token are the same case.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import CacheNeed
from ..weights.loader import TensorDecl
from .base import ROTARY_PAIRINGS, BuildEnv, Mixer, RotaryTables, StepView, build_part, register_part
from .linear import as_matrix, fuse_rows


class PagedAttention(Mixer):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.scale = float(p["scale"])
        self.window = None if p.get("window") is None else int(p["window"])
        if self.heads % self.kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if self.window is not None and self.window <= 0:
            raise ValueError("window must be positive")
        self.q_dim = self.heads * self.head_dim
        self.kv_dim = self.kv_heads * self.head_dim
        self.position = build_part("position", spec.parts["position"]) if "position" in spec.parts else None
        self.q_norm = build_part("norm", spec.parts["q_norm"]) if "q_norm" in spec.parts else None
        self.k_norm = build_part("norm", spec.parts["k_norm"]) if "k_norm" in spec.parts else None

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        out = [TensorDecl(n["q"], (self.q_dim, self.hidden)),
               TensorDecl(n["k"], (self.kv_dim, self.hidden)),
               TensorDecl(n["v"], (self.kv_dim, self.hidden)),
               TensorDecl(n["o"], (self.hidden, self.q_dim))]
        for part in (self.q_norm, self.k_norm, self.position):
            if part is not None:
                out += part.tensors()
        return out

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        for part in (self.q_norm, self.k_norm, self.position):
            if part is not None:
                part.load(weights, env)
        env.ops.check_attention_sizes(self.heads, self.kv_heads, self.head_dim)
        # The kernels turn the pairs (i, i + rotary_dim/2) of a head.  An encoding that pairs
        # neighbours (2i, 2i + 1) is served by the same kernels: a head's scores q.k do not change
        # when q and k are permuted alike, so the rows of the q and k projections (and the weights
        # of their norms) are put in the order 0, 2, 4, .., 1, 3, 5, .. once, here.
        self.rotary, order = None, None
        tables = self.position.rotary() if self.position is not None else None
        if tables is not None:
            tables = RotaryTables(*tables)
            if tables.pairing not in ROTARY_PAIRINGS:
                raise ValueError(f"rotary pairing '{tables.pairing}' is not known; known: {', '.join(ROTARY_PAIRINGS)}")
            rd = int(tables.rotary_dim)
            if rd <= 0 or rd % 2 or rd > self.head_dim:
                raise ValueError(f"rotary_dim {rd} must be even and at most head_dim {self.head_dim}")
            if tables.pairing == "interleaved":
                order = torch.cat([torch.arange(0, rd, 2), torch.arange(1, rd, 2), torch.arange(rd, self.head_dim)])
            self.rotary = (tables.cos, tables.sin, rd)
        # The norms of q and k per head are applied inside the kernels, which have the RMS norm
        # built in: any other kind of norm there is refused, not taken for one.
        self.head_norms = []
        for role, norm in (("q", self.q_norm), ("k", self.k_norm)):
            rms = None
            if norm is not None:
                rms = norm.as_rms()
                if rms is None:
                    raise ValueError(f"the {role} norm of an attention layer is '{norm.spec.kind}': the attention "
                                     f"kernels apply it per head themselves and have the RMS norm only")
                weight, eps = rms
                if tuple(weight.shape) != (self.head_dim,):
                    raise ValueError(f"the {role} norm has {tuple(weight.shape)} weights, a head has {self.head_dim} elements")
                rms = (weight[order.to(weight.device)].contiguous() if order is not None else weight, float(eps))
            self.head_norms.append(rms)

        def heads_in_order(w: torch.Tensor, heads: int) -> torch.Tensor:
            if order is None:
                return w
            return w.view(heads, self.head_dim, self.hidden)[:, order.to(w.device)].reshape(heads * self.head_dim, self.hidden)
        self.w_qkv = fuse_rows([heads_in_order(weights[n["q"]], self.heads),
                                heads_in_order(weights[n["k"]], self.kv_heads), weights[n["v"]]], env)
        self.w_o = as_matrix(weights[n["o"]], env)

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed.keys_and_values(self.kv_heads, self.head_dim, self.window)

    def workspace_elems(self, rows: int) -> int:
        # q, k, v rows (as float32 partial sums at worst), the rotated q, the attention's output
        return rows * (3 * (self.q_dim + 2 * self.kv_dim) + 2 * self.q_dim)

    @property
    def takes_normed_rows(self) -> bool:       # x goes to the q/k/v product only
        return getattr(self.w_qkv, "tiled", None) is not None

    def forward(self, x: torch.Tensor, step: StepView) -> torch.Tensor:
        ops = self.env.ops
        qkv = ops.linear(x, self.w_qkv, sums_only=True)      # partial sums, if k was split, are the attention's to add
        o = ops.qkv_attention(qkv, step, step.cache, self.heads, self.kv_heads, self.head_dim,
                              self.head_norms[0], self.head_norms[1], self.rotary, self.scale, self.window)
        return ops.linear(o, self.w_o, deferred=True)       # goes to the next norm as the residual delta


register_part("mixer", "paged_attention", PagedAttention)
