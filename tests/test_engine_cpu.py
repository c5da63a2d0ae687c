"""The engine's own logic (packing, block tables, cache manager, run order)
checked on the CPU: the kernel library is replaced by the plain-torch stand-in
of tests/cpu_ops.py, everything else is the product's code.  All ways of
cutting the work must give the plain implementation's logits."""
import numpy as np
import pytest
import torch

from cpu_ops import CpuOps
from helpers import (TINY, collect, max_error, plain_logits, random_prompt, trace_mixed,
                     trace_portions, trace_prefill_then_decode, trace_whole)
from tiny_llm_infer_amd.engine.loading import load_model
from tiny_llm_infer_amd.engine.replay import Replayer
from tiny_llm_infer_amd.engine.runner import ModelRunner


def _runner(folder, name, max_tokens):
    model, cfg = load_model(folder, "float32", "cpu", ops=CpuOps())
    page = TINY[name]["page_size"]
    return ModelRunner(model, model.env, page_size=page, num_pages=max_tokens // page,
                       max_requests=4, max_batch_tokens=512)


def _requests(name, lengths, seed):
    vocab = TINY[name]["vocab_size"]
    return {f"r{i}": random_prompt(vocab, n, seed + i) for i, n in enumerate(lengths)}


def _replay(runner, steps):
    rp = Replayer(runner)
    return {st["step"]: rp.run_step(st) for st in steps}


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_all_cuts_match_plain(model_folders, name):
    folder = model_folders[name]
    reqs = _requests(name, [70, 45, 97, 33, 58], seed=5)
    want = plain_logits(folder, reqs)
    max_tokens = 256
    cuts = {
        "whole": trace_whole(reqs),
        "decode": trace_prefill_then_decode(reqs),
        "portions": trace_portions(reqs, seed=3),
        "mixed": trace_mixed(reqs, max_tokens=max_tokens, seed=9),
    }
    for cut, steps in cuts.items():
        runner = _runner(folder, name, max_tokens)
        got = collect(steps, _replay(runner, steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], want[rid])
            assert err <= 2e-5 * max(1.0, scale), f"{name}/{cut}/{rid}: error {err} at token {row}"
        runner.cache.check()
        assert not runner.cache.live()
        assert runner.cache.free_pages() == runner.cache.pages_per_group()
        if cut == "mixed":
            assert runner.cache.pages_taken_total > runner.cache.num_pages * len(runner.cache.groups) // 2
