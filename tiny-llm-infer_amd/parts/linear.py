"""Matrices applied as y = x W^T with W stored [out, in] row-major
(kernels/src/matmul_kernel_cpu.cpp:27-35).  Accumulation is float32."""
from __future__ import annotations

from typing import Sequence

import torch

from .base import BuildEnv


class Matrix:
    """A weight matrix as the products use it: ``w`` [out, in] row-major in the
    run's dtype (many rows: prefill) and, for a bfloat16 run, ``tiled``, the same
    values in the layout the weight-streaming kernel for few rows reads in a row
    (decode).  Holding both costs the matrix's bytes twice; a decode step reads
    only ``tiled``, a prefill step only ``w``."""

    def __init__(self, w: torch.Tensor, env: BuildEnv, decode_layout: bool = True):
        self.w = w.to(env.dtype).contiguous()
        tile = getattr(env.ops, "tile_matrix", None)
        self.tiled = tile(self.w) if (decode_layout and tile is not None) else None

    @property
    def shape(self):
        return self.w.shape


def as_matrix(t: torch.Tensor, env: BuildEnv) -> Matrix:
    """A loaded matrix ready for products."""
    return Matrix(t, env)


def fuse_rows(mats: Sequence[torch.Tensor], env: BuildEnv) -> Matrix:
    """Stack matrices that read the same input ([out_i, in] each) into one
    [sum out_i, in], so that one product gives all their outputs."""
    return Matrix(torch.cat([m.to(env.dtype) for m in mats], dim=0), env)
