"""Pre-norm residual block: n = norm(h); r = h + mixer(n); m = norm(r);
h' = r + ffn(m) (model/src/qwen3_paged_batch.cpp:146-148, 273-279, 297-301).
The second sum is left to whoever normalises next (the following block or the
final norm), which adds it in float32 in the same pass as its norm.  Without a
feed-forward the block is n = norm(h); h' = h + mixer(n), that one sum left
to the next norm likewise."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorDecl
from .base import Block, BuildEnv, StepView, register_part, run_norm


class PreNormBlock(Block):
    def __init__(self, spec, mixer, ffn, norms):
        super().__init__(spec)
        self.mixer = mixer
        self.ffn = ffn
        self.norm_mixer = norms["mixer"]
        self.norm_ffn = norms["ffn"] if ffn is not None else None
        self.replayable = all(p.replayable for p in self._parts())

    def _parts(self):
        return [p for p in (self.norm_mixer, self.mixer, self.norm_ffn, self.ffn) if p is not None]

    def tensors(self) -> List[TensorDecl]:
        return [d for p in self._parts() for d in p.tensors()]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        for part in self._parts():
            part.load(weights, env)

    def forward(self, resid: torch.Tensor, pending: Optional[torch.Tensor],
                step: StepView) -> torch.Tensor:
        # (a part that gives its input to matrix products only lets the norm before it be
        # taken into those products, if the norm can do that)
        n = run_norm(self.norm_mixer, resid, pending, consumer=self.mixer)
        a = self.mixer.forward(n, step)
        if self.ffn is None:
            return a
        m = run_norm(self.norm_ffn, resid, a, consumer=self.ffn)
        return self.ffn.forward(m, step)


register_part("block", "prenorm", PreNormBlock)
