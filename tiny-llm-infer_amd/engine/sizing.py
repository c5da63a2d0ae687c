"""How many cache pages fit: the memory the device has left after the weights,
less a reserve for the step's activations and what the window groups take (a
fixed number of pages each, see ``cache.manager.window_group_pages``), divided
by the bytes of one page of the layers that keep all keys.  The policy follows
the reference's estimator (model/src/qwen3.cpp:96-151): budget = utilisation *
total - used; reserve = max(256 MiB, total / 20, workspace)."""
from __future__ import annotations

import torch


def _elem_size(dtype, run_dtype) -> int:
    return torch.empty((), dtype=dtype or run_dtype).element_size()


def page_bytes(model, page_size: int, windowed=None) -> int:
    """Bytes of one page id across the cache layers (``windowed``: None all of them, False
    those that keep all keys, True those with a window): every record that the mixers declared."""
    total = 0
    for need in model.cache_needs():
        if need is not None and (windowed is None or (need.window is not None) == windowed):
            total += need_page_bytes(need, page_size, model.env.dtype)
    return total


def need_page_bytes(need, page_size: int, run_dtype) -> int:
    """Bytes of one page of one cache layer with this need."""
    return sum(rec.elems_per_token() * page_size * _elem_size(rec.dtype, run_dtype) for rec in need.records)


def window_bytes(model, page_size: int, max_batch_tokens: int, max_num_seqs: int) -> int:
    """What the window groups take: their fixed number of pages, for every layer of the group."""
    from ..cache.manager import window_group_pages
    total = 0
    for need in model.cache_needs():
        if need is not None and need.window is not None:
            pages = window_group_pages(need.window, page_size, max_num_seqs, max_batch_tokens)
            total += pages * need_page_bytes(need, page_size, model.env.dtype)
    return total


def workspace_bytes(model, max_batch_tokens: int) -> int:
    """A bound on the activations of one step: the residual stream, its normed rows and two
    deltas, and what the parts of the hungriest block say they hold (``workspace_elems``),
    every element counted as four bytes, twice over for what the allocator keeps around."""
    rows = max_batch_tokens
    parts = max((b.mixer.workspace_elems(rows) + (b.ffn.workspace_elems(rows) if b.ffn is not None else 0)
                 for b in model.blocks), default=0)
    return 2 * 4 * (4 * rows * model.spec.hidden_size + parts)


def estimate_num_pages(model, page_size: int, max_batch_tokens: int, max_num_seqs: int,
                       max_model_len: int, utilization: float = 0.9) -> int:
    if not 0.0 < utilization <= 0.95:
        raise ValueError("gpu_memory_utilization must be in (0, 0.95]")
    per_page = page_bytes(model, page_size, windowed=False)
    most_useful = max_num_seqs * ((max_model_len + page_size - 1) // page_size)
    if page_bytes(model, page_size) == 0:
        return 1
    device = model.env.device
    if device.type != "cuda" or per_page == 0:
        return most_useful              # (only window groups: each takes what it can use of this, no more)
    free, total = torch.cuda.mem_get_info(device)
    used = total - free
    budget = utilization * total - used
    reserve = max(256 << 20, total // 20, workspace_bytes(model, max_batch_tokens))
    pages = int((budget - reserve - window_bytes(model, page_size, max_batch_tokens, max_num_seqs)) // per_page)
    if pages <= 0:
        raise RuntimeError("no device memory is left for the cache")
    return min(pages, most_useful)
