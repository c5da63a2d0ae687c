"""Matrices applied as y = x W^T with W stored [out, in] row-major
(kernels/src/matmul_kernel_cpu.cpp:27-35).  Accumulation is float32."""
from __future__ import annotations

from typing import Sequence

import torch

from .base import BuildEnv


def as_matrix(t: torch.Tensor, env: BuildEnv) -> torch.Tensor:
    """A loaded matrix in the dtype the run multiplies in."""
    return t.to(env.dtype).contiguous()


def fuse_rows(mats: Sequence[torch.Tensor], env: BuildEnv) -> torch.Tensor:
    """Stack matrices that read the same input ([out_i, in] each) into one
    [sum out_i, in], so that one product gives all their outputs."""
    return torch.cat([as_matrix(m, env) for m in mats], dim=0).contiguous()
