"""How many cache pages fit: the memory the device has left after the weights,
less a reserve for the step's activations, divided by the bytes of one page in
every group.  The policy follows the reference's estimator
(model/src/qwen3.cpp:96-151): budget = utilisation * total - used; reserve =
max(256 MiB, total / 20, workspace)."""
from __future__ import annotations

import torch


def page_bytes(model, page_size: int) -> int:
    """Bytes of one page id across all groups (each group owns as many pages)."""
    elem = 2 if model.env.dtype == torch.bfloat16 else 4
    total = 0
    for need in model.cache_needs():
        if need is not None:
            total += 2 * need.num_kv_heads * need.head_dim * page_size * elem
    return total


def workspace_bytes(model, max_batch_tokens: int) -> int:
    """A bound on the activations of one step."""
    widest = model.spec.hidden_size
    for b in model.blocks:
        for attr in ("inter", "q_dim"):
            for part in (b.mixer, b.ffn):
                widest = max(widest, 2 * int(getattr(part, attr, 0)))
    return max_batch_tokens * (6 * widest + 4 * model.spec.hidden_size) * 4


def estimate_num_pages(model, page_size: int, max_batch_tokens: int, max_num_seqs: int,
                       max_model_len: int, utilization: float = 0.9) -> int:
    if not 0.0 < utilization <= 0.95:
        raise ValueError("gpu_memory_utilization must be in (0, 0.95]")
    per_page = page_bytes(model, page_size)
    most_useful = max_num_seqs * ((max_model_len + page_size - 1) // page_size)
    if per_page == 0:
        return 1
    device = model.env.device
    if device.type != "cuda":
        return most_useful
    free, total = torch.cuda.mem_get_info(device)
    used = total - free
    budget = utilization * total - used
    reserve = max(256 << 20, total // 20, workspace_bytes(model, max_batch_tokens))
    pages = int((budget - reserve) // per_page)
    if pages <= 0:
        raise RuntimeError("no device memory is left for the cache")
    return min(pages, most_useful)
