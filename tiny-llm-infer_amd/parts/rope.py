"""Rotary position encoding, half-split ("neox") pairing.

Frequencies f_i = theta^(-2i/d) for i < d/2, computed in float32 with the
exponent -2.0f*i/d in float32; angle = float32(position) * f_i in float32
(kernels/src/rope_kernel_cpu.cpp:127-141).  The pair (x_i, x_{i+d/2}) becomes
(x_i cos - x_{i+d/2} sin, x_i sin + x_{i+d/2} cos)
(kernels/src/rope_kernel_cpu.cpp:156-179).  ``rotary_dim`` = d may be smaller
than the head size; the rest of the head is left as it is.  The table holds
sin and cos of the float32 angle, evaluated in float64 and rounded once.
"""
from __future__ import annotations

import numpy as np
import torch

from .base import BuildEnv, PositionEncoding, RotaryTables, register_part


class NeoxRope(PositionEncoding):
    def __init__(self, spec):
        super().__init__(spec)
        p = spec.params
        self.head_dim = int(p["head_dim"])
        self.rotary_dim = int(p.get("rotary_dim", self.head_dim))
        self.theta = float(p["theta"])
        self.max_positions = int(p["max_positions"])
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim or self.rotary_dim <= 0:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {self.head_dim}")
        self.cos = None
        self.sin = None

    def load(self, weights, env: BuildEnv) -> None:
        super().load(weights, env)
        n = min(self.max_positions, env.max_model_len)
        self.num_positions = n
        key = ("rope_neox", self.theta, self.rotary_dim, n, str(env.device))
        if key in env.shared:                 # layers with the same angles share one table
            self.cos, self.sin = env.shared[key]
            return
        half = self.rotary_dim // 2
        i = np.arange(half, dtype=np.float32)
        exponent = (np.float32(-2.0) * i) / np.float32(self.rotary_dim)
        freq = np.power(np.float32(self.theta), exponent, dtype=np.float32)
        pos = np.arange(n, dtype=np.float32)
        angle = (pos[:, None] * freq[None, :]).astype(np.float32)
        a64 = angle.astype(np.float64)
        self.cos = torch.from_numpy(np.cos(a64).astype(np.float32)).to(env.device).contiguous()
        self.sin = torch.from_numpy(np.sin(a64).astype(np.float32)).to(env.device).contiguous()
        env.shared[key] = (self.cos, self.sin)

    def rotary(self) -> RotaryTables:
        return RotaryTables(self.cos, self.sin, self.rotary_dim, "half")


register_part("position", "rope_neox", NeoxRope)
