"""What the C ABI of the engine (``capi/tli_engine.h``) calls: an engine built from a plain
dictionary, requests added from plain lists, results handed back as plain lists.  The engine
is ``LLMEngine``; nothing here computes."""
from __future__ import annotations

import json
from typing import Dict, List, Tuple

from ..sampling.params import SamplingParams
from .llm_engine import LLMEngine


def create(config: Dict) -> LLMEngine:
    limits = dict(max_model_len=int(config.get("max_model_len") or 2048),
                  page_size=int(config.get("page_size") or 16),
                  num_kv_blocks=int(config.get("num_kv_blocks") or 0),
                  max_num_seqs=int(config.get("max_num_seqs") or 16),
                  max_num_batched_tokens=int(config.get("max_num_batched_tokens") or 256),
                  gpu_memory_utilization=float(config.get("gpu_memory_utilization") or 0.9),
                  enable_prefix_caching=bool(config.get("enable_prefix_caching")))
    dtype = config.get("dtype") or "bfloat16"
    if config.get("model_dir"):
        return LLMEngine.from_folder(config["model_dir"], dtype=dtype, device="cuda:0", **limits)
    # seeded random weights from a config.json
    from ..registry import architecture_of
    from .loading import random_model
    path = config["config_json"]
    with open(path) as fh:
        data = json.load(fh)
    arch = architecture_of(data, path)
    model = random_model(arch.name, arch.read_config(data, path), int(config.get("weights_seed") or 0), dtype,
                         "cuda:0", limits["max_model_len"])
    return LLMEngine.from_model(model, **limits)


def add_request(engine: LLMEngine, tokens: List[int], sampling: Dict) -> int:
    return engine.add_request(tokens, SamplingParams(
        max_tokens=int(sampling["max_tokens"]), temperature=float(sampling["temperature"]),
        top_p=float(sampling["top_p"]), ignore_eos=bool(sampling["ignore_eos"]), seed=int(sampling["seed"])))


def step(engine: LLMEngine) -> List[Tuple[int, List[int]]]:
    return [(int(r.request_id), [int(t) for t in r.token_ids]) for r in engine.step()]


def is_finished(engine: LLMEngine) -> int:
    return int(engine.is_finished())


def total_generated_tokens(engine: LLMEngine) -> int:
    return int(engine.total_generated_tokens)
