"""Seeded random weights that are the same wherever they are drawn.

Element e of the ``index``-th tensor of a model with seed s is a function of (s, index,
e) alone: a 32-bit hash picks a point on the normal distribution's quantile function
(a table of 65,537 float32 values, straight lines between them), scaled to N(mean,
std^2) in float32 operations that are each rounded on their own.  The kernel library
computes it, on the device for a tensor that lives there and on the host otherwise, with
the same bits; ``--random-weights --seed N`` on the device and a model folder written
with seed N therefore hold the same model.  (The reference has no random-weights mode.)
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

_TABLE = None
_TABLE_ON: Dict[str, torch.Tensor] = {}

TABLE_INTERVALS = 65536
TAIL = 2.0 ** -18            # the probability at which the two ends of the table stand in for 0 and 1


def quantile_table() -> torch.Tensor:
    """float32 [65537]: the standard normal quantile at i / 65536, computed in float64 and
    rounded once; entries 0 and 65536 at a probability of 2^-18 from the ends."""
    global _TABLE
    if _TABLE is None:
        p = torch.arange(TABLE_INTERVALS + 1, dtype=torch.float64) / TABLE_INTERVALS
        p[0], p[-1] = TAIL, 1.0 - TAIL
        _TABLE = torch.special.ndtri(p).to(torch.float32).contiguous()
    return _TABLE


def _table_on(device: torch.device) -> torch.Tensor:
    key = str(device)
    if key not in _TABLE_ON:
        _TABLE_ON[key] = quantile_table().to(device)
    return _TABLE_ON[key]


def draw_normal(shape: Tuple[int, ...], seed: int, index: int, std: float, mean: float = 0.0,
                device="cpu") -> torch.Tensor:
    """float32 tensor of ``shape`` on ``device``; element e (row-major) depends on (seed, index, e)."""
    from ..kernels.ops import KernelError, load_library
    lib = load_library()
    device = torch.device(device)
    out = torch.empty(tuple(shape), dtype=torch.float32, device=device)
    n = out.numel()
    seed &= (1 << 64) - 1
    on_device = device.type == "cuda"
    table = _table_on(device) if on_device else quantile_table()
    stream = torch.cuda.current_stream(device).cuda_stream if on_device else None
    if on_device:
        with torch.cuda.device(device):
            code = lib.tli_random_normal(out.data_ptr(), n, seed & 0xFFFFFFFF, seed >> 32, int(index) & 0xFFFFFFFF,
                                         table.data_ptr(), float(std), float(mean), 1, stream)
    else:
        code = lib.tli_random_normal(out.data_ptr(), n, seed & 0xFFFFFFFF, seed >> 32, int(index) & 0xFFFFFFFF,
                                     table.data_ptr(), float(std), float(mean), 0, None)
    if code != 0:
        raise KernelError(lib.tli_last_error().decode())
    return out
