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


class GatedMatrix(Matrix):
    """A gate matrix and an up matrix that read the same input, for
    silu(x gate^T) * (x up^T).  ``w`` stacks them ([gate; up], one product for many
    rows, the activation in a pass of its own); ``gated`` is the decode layout with
    the 16-row blocks of gate and up alternating, so that the weight-streaming
    kernel holds both sums of an output and writes the activation itself."""

    def __init__(self, gate: torch.Tensor, up: torch.Tensor, env: BuildEnv):
        super().__init__(torch.cat([gate.to(env.dtype), up.to(env.dtype)], dim=0), env, decode_layout=False)
        self.inter = gate.shape[0]
        self.gated = None
        tile = getattr(env.ops, "tile_matrix", None)
        if tile is not None and self.inter % 16 == 0 and env.dtype == torch.bfloat16:
            k = gate.shape[1]
            pairs = torch.stack([self.w[:self.inter].view(-1, 16, k), self.w[self.inter:].view(-1, 16, k)], dim=1)
            self.gated = tile(pairs.reshape(2 * self.inter, k))
            if self.gated is None:          # the kernel cannot take this width: plain decode layout
                self.tiled = tile(self.w)
        elif tile is not None:
            self.tiled = tile(self.w)


def as_matrix(t: torch.Tensor, env: BuildEnv) -> Matrix:
    """A loaded matrix ready for products."""
    return Matrix(t, env)


def fuse_rows(mats: Sequence[torch.Tensor], env: BuildEnv) -> Matrix:
    """Stack matrices that read the same input ([out_i, in] each) into one
    [sum out_i, in], so that one product gives all their outputs."""
    return Matrix(torch.cat([m.to(env.dtype) for m in mats], dim=0), env)
