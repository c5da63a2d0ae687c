"""Matrices applied as y = x W^T with W stored [out, in] row-major
(kernels/src/matmul_kernel_cpu.cpp:27-35).  Accumulation is float32."""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from .base import BuildEnv


class Matrix:
    """A weight matrix as the products use it.  In a bfloat16 run it is held once, in the
    "decode layout" (``tiled``) that this library's product kernels for any number of rows
    stream in a row; the row-major form ``w`` [out, in] is held beside it only where the
    kernel library says it multiplies with it (products of many rows given to the BLAS
    library) or where there is no decode layout (a float32 run, a width the layout does not
    take).  Asked for all the same (the plain kernels, a product too large for the offsets of
    the kernel for many rows), ``w`` is put together from the decode layout once and kept from
    then on (``rebuilt`` counts how often that happened in the process): a default run never
    asks for it, and one that does pays the second copy once, not at every product."""

    rebuilt = 0

    def __init__(self, w: torch.Tensor, env: BuildEnv, decode_layout: bool = True):
        w = w.to(env.dtype).contiguous()
        self.shape = tuple(w.shape)
        self.dtype = w.dtype
        self.ops = env.ops
        tile = getattr(env.ops, "tile_matrix", None)
        self.tiled = tile(w) if (decode_layout and tile is not None) else None
        self._w: Optional[torch.Tensor] = w if (self.tiled is None or self._keeps_row_major()) else None

    def _keeps_row_major(self) -> bool:
        return bool(getattr(self.ops, "keep_row_major", True))

    @property
    def w(self) -> torch.Tensor:
        if self._w is None:
            self._w = self._rebuild()
            Matrix.rebuilt += 1
        return self._w

    def _rebuild(self) -> torch.Tensor:
        return self.ops.untile_matrix(self.tiled, self.shape)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self._w, self.tiled) if t is not None)


class GatedMatrix(Matrix):
    """A gate matrix and an up matrix that read the same input, for
    silu(x gate^T) * (x up^T).  ``gated`` is the decode layout with the 16-row blocks of
    gate and up alternating, so that a product kernel holds both sums of an output and
    writes the activation itself.  ``w`` stacks them row-major ([gate; up]: one product,
    the activation in a pass of its own), held or put together as for a ``Matrix``."""

    def __init__(self, gate: torch.Tensor, up: torch.Tensor, env: BuildEnv):
        self.inter = gate.shape[0]
        self.gated = None
        stacked = torch.cat([gate.to(env.dtype), up.to(env.dtype)], dim=0)
        tile = getattr(env.ops, "tile_matrix", None)
        interleave = tile is not None and self.inter % 16 == 0 and env.dtype == torch.bfloat16
        if interleave:
            k = gate.shape[1]
            pairs = torch.stack([stacked[:self.inter].view(-1, 16, k), stacked[self.inter:].view(-1, 16, k)], dim=1)
            self.gated = tile(pairs.reshape(2 * self.inter, k))
            del pairs
        # (the kernel cannot take this width, or the blocks do not pair up: the plain decode layout)
        super().__init__(stacked, env, decode_layout=self.gated is None)
        if self.gated is not None and not self._keeps_row_major():
            self._w = None

    def _rebuild(self) -> torch.Tensor:
        if self.gated is None:
            return super()._rebuild()
        rows, k = self.shape
        pairs = self.ops.untile_matrix(self.gated, (rows, k)).view(-1, 2, 16, k)      # [block, gate/up, 16, k]
        return torch.cat([pairs[:, 0].reshape(self.inter, k), pairs[:, 1].reshape(self.inter, k)], dim=0)

    def nbytes(self) -> int:
        return super().nbytes() + (self.gated.numel() * self.gated.element_size() if self.gated is not None else 0)


def as_matrix(t: torch.Tensor, env: BuildEnv) -> Matrix:
    """A loaded matrix ready for products."""
    return Matrix(t, env)


def fuse_rows(mats: Sequence[torch.Tensor], env: BuildEnv) -> Matrix:
    """Stack matrices that read the same input ([out_i, in] each) into one
    [sum out_i, in], so that one product gives all their outputs."""
    return Matrix(torch.cat([m.to(env.dtype) for m in mats], dim=0), env)
