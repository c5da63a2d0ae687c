"""Dense gated feed-forward: down( silu(gate(x)) * up(x) ) with
silu(g) = g / (1 + exp(-g)) (model/src/qwen3_paged_batch.cpp:281-295,
kernels/src/swiglu_kernel_cpu.cpp:20-24).  gate and up are stacked into one
matrix so that one product reads x once."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..weights.loader import TensorDecl
from .base import BuildEnv, FeedForward, StepView, register_part
from .linear import GatedMatrix, as_matrix


class SwiGLU(FeedForward):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])

    def tensors(self) -> List[TensorDecl]:
        n = self.spec.names
        return [TensorDecl(n["gate"], (self.inter, self.hidden)),
                TensorDecl(n["up"], (self.inter, self.hidden)),
                TensorDecl(n["down"], (self.hidden, self.inter))]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        n = self.spec.names
        self.w_gate_up = GatedMatrix(weights[n["gate"]], weights[n["up"]], env)
        self.w_down = as_matrix(weights[n["down"]], env)

    def workspace_elems(self, rows: int) -> int:
        return rows * 3 * self.inter            # gate and up rows side by side, then the activation

    @property
    def takes_normed_rows(self) -> bool:       # x goes to the gate/up product only
        return getattr(self.w_gate_up, "gated", None) is not None

    def forward(self, x: torch.Tensor, step: StepView) -> torch.Tensor:
        ops = self.env.ops
        return ops.linear(ops.linear_swiglu(x, self.w_gate_up), self.w_down, deferred=True)   # a delta for the next norm


register_part("ffn", "swiglu", SwiGLU)
