"""RMSNorm: y_j = w_j * x_j / sqrt(mean(x^2) + eps), all in float32
(kernels/src/rmsnorm_kernel_cpu.cpp:27-43).  The weight is a plain multiplier.
The residual stream is float32; the norm adds what the previous part owes the
residual before it normalises, so the residual sum is never rounded."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..weights.loader import TensorDecl
from .base import BuildEnv, Norm, register_part


class RMSNorm(Norm):
    replayable = True
    supports_lazy = True
    takes_unfinished_products = True

    def __init__(self, spec):
        super().__init__(spec)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight_name = spec.names["weight"]
        self.weight: Optional[torch.Tensor] = None

    def tensors(self) -> List[TensorDecl]:
        return [TensorDecl(self.weight_name, (self.size,), "ones_normal")]

    def load(self, weights: Dict[str, torch.Tensor], env: BuildEnv) -> None:
        super().load(weights, env)
        # vectors are held in float32: exact for 16-bit storage, unchanged for 32-bit
        self.weight = weights[self.weight_name].to(torch.float32).contiguous()

    def as_rms(self):
        return self.weight, self.eps

    def forward(self, resid, delta, rows=None, num_rows=None, lazy=False):
        """``lazy``: the rows go to matrix products only, which may then apply the rows'
        scalar factor themselves (the kernel library decides; see its ``add_rmsnorm``)."""
        return self.env.ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.env.dtype,
                                        rows=rows, num_rows=num_rows, **({"lazy": True} if lazy else {}))


register_part("norm", "rmsnorm", RMSNorm)
