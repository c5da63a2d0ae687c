"""Token embedding (x_t = E[token_t], no scaling; layers/src/embedding.cpp:37-44)
and the head that turns final hidden rows into float32 logits
(model/src/qwen3_paged_batch.cpp:343-346).  The reference always uses the
embedding matrix as the head (model/src/qwen3_layers.cpp:246-265) and rounds
logits to half precision; here a head has its own matrix unless the model ties
it, and logits leave the product in float32."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..weights.loader import TensorDecl
from .base import BuildEnv, Part, register_part
from .linear import as_matrix


class TokenEmbedding(Part):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        self.vocab = int(spec.params["vocab_size"])
        self.hidden = int(spec.params["hidden_size"])
        self.name = spec.names["weight"]

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.vocab, self.hidden))]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        self.table = weights[self.name].to(env.dtype).contiguous()      # rows are gathered: row-major only

    def forward(self, token_ids: torch.Tensor, num_rows: int) -> torch.Tensor:
        """Rows of the table as a float32 residual stream [rows, hidden]."""
        return self.env.ops.embed(self.table, token_ids, num_rows)


class LinearHead(Part):
    replayable = True

    def __init__(self, spec):
        super().__init__(spec)
        self.vocab = int(spec.params["vocab_size"])
        self.hidden = int(spec.params["hidden_size"])
        self.name = spec.names["weight"]

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.name, (self.vocab, self.hidden))]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv, share_with=None) -> None:
        super().load(weights, env)
        if share_with is not None and share_with.name == self.name:
            self.weight = as_matrix(share_with.table, env)     # tied: the row-major copy is shared
        else:
            self.weight = as_matrix(weights[self.name], env)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.env.ops.linear(x, self.weight, out_dtype=torch.float32)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
