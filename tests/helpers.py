"""Shared by the tests: the tiny configurations, traces cut in different ways,
and the comparison with the plain implementation."""
from __future__ import annotations

import random
from typing import Dict, List

import numpy as np
import torch

ARCH = "Qwen3ForCausalLM"

# Tiny configurations that differ in every size and option.
TINY = {
    # 2 layers, head_dim = hidden/heads, tied head, all keys everywhere
    "A": dict(hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, head_dim=16, vocab_size=256, max_position_embeddings=512,
              rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              use_sliding_window=False, seed=11, page_size=8),
    # 3 layers, head_dim != hidden/heads, untied head, layers 1 and 2 windowed
    "B": dict(hidden_size=96, intermediate_size=160, num_hidden_layers=3, num_attention_heads=6,
              num_key_value_heads=3, head_dim=32, vocab_size=384, max_position_embeddings=640,
              rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
              use_sliding_window=True, sliding_window=40, max_window_layers=1, seed=23, page_size=16),
    # sizes that are no power of two, one kv head, head_dim 48, odd vocabulary,
    # windows named layer by layer
    "C": dict(hidden_size=80, intermediate_size=112, num_hidden_layers=4, num_attention_heads=5,
              num_key_value_heads=1, head_dim=48, vocab_size=301, max_position_embeddings=400,
              rope_theta=50000.0, rms_norm_eps=3e-6, tie_word_embeddings=False,
              use_sliding_window=True, sliding_window=19,
              layer_types=["sliding_attention", "full_attention", "sliding_attention", "full_attention"],
              seed=37, page_size=32),
    # heads of 64: the attention kernels that take q (and for decode steps k and v) from the
    # raw projections themselves; one windowed layer, one not
    "D": dict(hidden_size=128, intermediate_size=192, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, head_dim=64, vocab_size=320, max_position_embeddings=512,
              rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
              use_sliding_window=True, sliding_window=24,
              layer_types=["sliding_attention", "full_attention"], seed=41, page_size=8),
}


def config_json(name: str) -> dict:
    c = {k: v for k, v in TINY[name].items() if k not in ("seed", "page_size")}
    c["architectures"] = [ARCH]
    c["model_type"] = "qwen3"
    return c


def make_model_folder(folder: str, name: str) -> str:
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.loading import write_random_model
    cfg = Qwen3Config.from_dict(config_json(name))
    return write_random_model(folder, ARCH, cfg, TINY[name]["seed"])


def random_prompt(vocab: int, n: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


# ------------------------------------------------------------------ traces ---
def trace_whole(reqs: Dict[str, List[int]]) -> List[dict]:
    """Each request alone and whole."""
    steps = []
    for i, (rid, toks) in enumerate(reqs.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks,
                                              "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def trace_prefill_then_decode(reqs: Dict[str, List[int]], tail: int = 32) -> List[dict]:
    """Most of a request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in reqs.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [
            {"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for j in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": [toks[j]], "want": [0]}],
                "end": [rid] if j == len(toks) - 1 else []})
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def trace_portions(reqs: Dict[str, List[int]], seed: int = 0) -> List[dict]:
    """Portions of changing size, down to two tokens."""
    rng = random.Random(seed)
    sizes = [2, 7, 3, 16, 5, 2, 31, 9, 1, 17, 64, 2, 33]
    steps = []
    for rid, toks in reqs.items():
        at = 0
        k = rng.randrange(len(sizes))
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                "end": [rid] if at + n == len(toks) else []})
            at += n
    return steps


def trace_mixed(reqs: Dict[str, List[int]], max_tokens: int, seed: int = 0, max_live: int = 4,
                round_to: int = 64) -> List[dict]:
    """Up to ``max_live`` live requests: portions of some beside single tokens
    of others, some left out of a step, admitted only while the live requests'
    token counts, each rounded up to ``round_to``, fit in ``max_tokens`` (so
    pages are given back and used again)."""
    rng = random.Random(seed)
    waiting = list(reqs.items())
    live: Dict[str, int] = {}          # id -> tokens fed so far
    steps = []

    def rounded(n):
        return (n + round_to - 1) // round_to * round_to

    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting[0]
            held = sum(rounded(len(reqs[r])) for r in live)
            if held + rounded(len(toks)) > max_tokens:
                break
            waiting.pop(0)
            live[rid] = 0
        assert live, "max_tokens is too small for the next request"
        entries, ended = [], []
        ids = list(live)
        rng.shuffle(ids)
        for rid in ids:
            if len(ids) > 1 and rng.random() < 0.25:
                continue                                   # left out of this step
            toks, at = reqs[rid], live[rid]
            left = len(toks) - at
            if at > len(toks) // 2 or rng.random() < 0.3:
                n = 1                                      # a decoded token
            else:
                n = min(left, rng.choice([2, 3, 5, 8, 13, 21, 34]))
            entries.append({"id": rid, "tokens": toks[at:at + n], "want": list(range(n))})
            live[rid] = at + n
            if at + n == len(toks):
                ended.append(rid)
        if not entries:
            continue
        for rid in ended:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


# ------------------------------------------------------------ comparison -----
def collect(steps: List[dict], outputs: Dict[int, np.ndarray]) -> Dict[str, np.ndarray]:
    """Reassemble per-request logits [tokens, vocab] from the outputs of a
    replay (step number -> [wanted, vocab])."""
    rows: Dict[str, Dict[int, np.ndarray]] = {}
    fed: Dict[str, int] = {}
    for st in steps:
        out = outputs.get(st["step"])
        r = 0
        for e in st["entries"]:
            at = fed.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[at + w] = out[r]
                r += 1
            fed[e["id"]] = at + len(e["tokens"])
        assert out is None or r == out.shape[0]
    return {rid: np.stack([d[i] for i in sorted(d)]) for rid, d in rows.items()}


def plain_logits(folder: str, reqs: Dict[str, List[int]]) -> Dict[str, np.ndarray]:
    import plain_qwen3
    cfg, w = plain_qwen3.read_model(folder)
    return {rid: plain_qwen3.forward(cfg, w, toks).numpy() for rid, toks in reqs.items()}


def max_error(got: np.ndarray, want: np.ndarray):
    """(largest absolute difference, its row, scale of the wanted logits)."""
    diff = np.abs(got.astype(np.float64) - want)
    row = int(diff.max(axis=1).argmax())
    return float(diff.max()), row, float(np.abs(want).max())
