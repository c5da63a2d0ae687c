"""Replay on the GPU against the plain implementation, in float32 and in
bfloat16: each request alone and whole; most of it in one step and the last 32
tokens one by one; in portions of changing size, down to two tokens; and
mixed, up to four live requests with so few pages that they are used again."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import (TINY, collect, max_error, plain_logits, random_prompt, trace_mixed,
                     trace_portions, trace_prefill_then_decode, trace_whole)

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# largest |difference| allowed, relative to the largest |logit| of the request
TOL = {"float32": 2e-5, "bfloat16": 2.5e-2}
# The tiny configurations in bfloat16: their rounding error against the plain implementation is 2.5e-3
# (A) to 7.5e-3 (C) of the largest logit in every cut, and the bound for them is set just above it.
TOL_TINY = {"float32": 2e-5, "bfloat16": 1.2e-2}


def _runner(folder, name, dtype, max_tokens, page=None):
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    model, cfg = load_model(folder, dtype, "cuda:0")
    page = page or TINY[name]["page_size"]
    return ModelRunner(model, model.env, page_size=page, num_pages=max_tokens // page,
                       max_requests=4, max_batch_tokens=1024)


def _requests(name, lengths, seed):
    vocab = TINY[name]["vocab_size"]
    return {f"r{i}": random_prompt(vocab, n, seed + i) for i, n in enumerate(lengths)}


def _replay(runner, steps):
    from tiny_llm_infer_amd.engine.replay import Replayer
    rp = Replayer(runner)
    return {st["step"]: rp.run_step(st) for st in steps}


def _check(got, want, dtype, label, tol=TOL):
    worst = 0.0
    for rid in want:
        err, row, scale = max_error(got[rid], want[rid])
        worst = max(worst, err / scale)
        assert err <= tol[dtype] * scale, (f"{label}/{rid}: error {err:.3e} at token {row} "
                                           f"(logit scale {scale:.3e})")
    return worst


@pytest.fixture(scope="module")
def oracle(model_folders):
    out = {}
    for name in TINY:
        reqs = _requests(name, [70, 45, 97, 33, 58, 121], seed=5)
        out[name] = (reqs, plain_logits(model_folders[name], reqs))
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("cut", ["whole", "decode", "portions", "mixed"])
def test_cuts_match_plain(model_folders, oracle, name, dtype, cut):
    reqs, want = oracle[name]
    max_tokens = 320
    steps = {"whole": lambda: trace_whole(reqs),
             "decode": lambda: trace_prefill_then_decode(reqs),
             "portions": lambda: trace_portions(reqs, seed=3),
             "mixed": lambda: trace_mixed(reqs, max_tokens=max_tokens, seed=9)}[cut]()
    runner = _runner(model_folders[name], name, dtype, max_tokens)
    got = collect(steps, _replay(runner, steps))
    worst = _check(got, want, dtype, f"{name}/{dtype}/{cut}", TOL_TINY)
    print(f"{name} {dtype} {cut}: worst relative error {worst:.2e}")
    runner.cache.check()
    assert runner.cache.free_pages() == runner.cache.pages_per_group()
    if cut == "mixed":
        assert runner.cache.pages_taken_total > runner.cache.num_pages


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random_match_plain(tmp_path, seed):
    """Sizes beyond the four tiny configurations: a configuration drawn from the seed (head sizes from 16
    to 256 in steps of 16, one to four kv heads with groups of one to eight, a width that is a multiple
    of 8, a vocabulary of any size, one to four layers, windows on some of them) with random weights,
    replayed whole, in portions and mixed on few pages, in float32 and bfloat16, against the plain
    implementation; the float32 cuts agree bit for bit."""
    import random
    from helpers import ARCH
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    rng = random.Random(4000 + seed)
    kv, group, layers = rng.randrange(1, 5), rng.choice([1, 2, 3, 4, 5, 7, 8]), rng.randrange(1, 5)
    cfg = dict(hidden_size=8 * rng.randrange(4, 40), intermediate_size=16 * rng.randrange(2, 30),
               num_hidden_layers=layers, num_attention_heads=kv * group, num_key_value_heads=kv,
               head_dim=16 * rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16]), vocab_size=rng.randrange(40, 3000),
               max_position_embeddings=512, rope_theta=rng.choice([1e4, 5e4, 1e6]),
               rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]), tie_word_embeddings=rng.random() < 0.5,
               use_sliding_window=rng.random() < 0.4, architectures=[ARCH], model_type="qwen3")
    if cfg["use_sliding_window"]:
        cfg["sliding_window"] = rng.randrange(5, 70)
        cfg["layer_types"] = [rng.choice(["sliding_attention", "full_attention"]) for _ in range(layers)]
    folder = write_random_model(str(tmp_path / "m"), ARCH, Qwen3Config.from_dict(cfg), 100 + seed)
    lengths = [rng.randrange(2, 150) for _ in range(rng.randrange(2, 6))]
    reqs = {f"r{i}": random_prompt(cfg["vocab_size"], n, rng.randrange(10 ** 6)) for i, n in enumerate(lengths)}
    want = plain_logits(folder, reqs)
    page = rng.choice([8, 16, 32, 64])
    max_tokens = 64 * ((max(lengths) + 63) // 64) * rng.choice([1, 2, 3])
    cuts = {"mixed": trace_mixed(reqs, max_tokens=max(max_tokens, 192), seed=seed, max_live=rng.randrange(1, 5)),
            "whole": trace_whole(reqs), "portions": trace_portions(reqs, seed=seed)}
    for dtype in ("float32", "bfloat16"):
        model, _ = load_model(folder, dtype, "cuda:0")
        first = None
        for cut, steps in cuts.items():
            runner = ModelRunner(model, model.env, page_size=page, num_pages=max(max_tokens, 192) // page + (0 if cut == "mixed" else 8),
                                 max_requests=4, max_batch_tokens=1024)
            got = collect(steps, _replay(runner, steps))
            _check(got, want, dtype, f"{cfg}/{dtype}/{cut}", TOL_TINY)
            if dtype == "float32":
                first = first or got
                assert all(np.array_equal(first[rid], got[rid]) for rid in reqs), cut
            runner.cache.check()
            assert runner.cache.free_pages() == runner.cache.pages_per_group()


@pytest.mark.parametrize("name", ["A", "B"])
def test_float32_cuts_agree_bit_for_bit(model_folders, oracle, name):
    """In float32 every kernel adds in an order that depends on the row alone,
    so all ways of cutting give identical logits."""
    reqs, _ = oracle[name]
    outs = []
    for steps in (trace_whole(reqs), trace_prefill_then_decode(reqs), trace_portions(reqs, 1),
                  trace_mixed(reqs, 320, seed=4)):
        runner = _runner(model_folders[name], name, "float32", 320)
        outs.append(collect(steps, _replay(runner, steps)))
    for other in outs[1:]:
        for rid in reqs:
            assert np.array_equal(outs[0][rid], other[rid]), rid


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_bfloat16_through_the_plain_kernels_does_not_depend_on_the_cut(model_folders, oracle, name):
    """bfloat16 storage with the plain kernels (float32 arithmetic in a fixed order, rounded where
    the tuned path rounds to store): the logits of every cut are bit for bit those of the whole
    requests, so whatever the cache or the batch did wrong in bfloat16 (a stale slot, a key of a
    page that is used again) would show however small.  The tuned kernels stay within rounding
    of them in every cut."""
    reqs, _ = oracle[name]
    cuts = {"whole": trace_whole(reqs), "decode": trace_prefill_then_decode(reqs),
            "portions": trace_portions(reqs, seed=3), "mixed": trace_mixed(reqs, max_tokens=320, seed=9)}
    first = None
    for cut, steps in cuts.items():
        runner = _runner(model_folders[name], name, "bfloat16", 320)
        runner.env.ops.use_plain_kernels()
        plain = collect(steps, _replay(runner, steps))
        if first is None:
            first = plain
        for rid in reqs:
            assert np.array_equal(first[rid], plain[rid]), (cut, rid)
        tuned = collect(steps, _replay(_runner(model_folders[name], name, "bfloat16", 320), steps))
        for rid in reqs:
            err, row, scale = max_error(tuned[rid], plain[rid].astype(np.float64))
            assert err <= 1e-2 * scale, f"{name}/{cut}/{rid}: tuned and plain kernels differ by {err / scale:.2e} at token {row}"


def test_long_decoding_and_first_tokens(model_folders):
    """One request decoded token by token from its very first token, far past
    several pages and past the window of configuration B."""
    name = "B"
    reqs = _requests(name, [300], seed=77)
    want = plain_logits(model_folders[name], reqs)
    toks = reqs["r0"]
    steps = [{"step": i, "entries": [{"id": "r0", "tokens": [t], "want": [0]}],
              "end": ["r0"] if i == len(toks) - 1 else []} for i, t in enumerate(toks)]
    for dtype in ("float32", "bfloat16"):
        runner = _runner(model_folders[name], name, dtype, 320)
        got = collect(steps, _replay(runner, steps))
        _check(got, want, dtype, f"long decode {dtype}")
        # the first tokens on their own
        err, _, scale = max_error(got["r0"][:3], want["r0"][:3])
        assert err <= TOL[dtype] * scale


def test_trace_run_program(model_folders, tmp_path):
    """bin/trace_run as a user runs it: JSON lines in, 'done <step>' lines and
    <step>.f32 files out."""
    name = "A"
    reqs = _requests(name, [40, 70], seed=31)
    want = plain_logits(model_folders[name], reqs)
    steps = trace_mixed(reqs, max_tokens=192, seed=2)
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / dtype
        proc = subprocess.run(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folders[name],
             "--dtype", dtype, "--out", str(out_dir), "--max-tokens", "192"],
            input="".join(json.dumps(s) + "\n" for s in steps), text=True,
            stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert proc.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
        vocab = TINY[name]["vocab_size"]
        outputs = {}
        for s in steps:
            path = out_dir / f"{s['step']}.f32"
            if sum(len(e["want"]) for e in s["entries"]):
                outputs[s["step"]] = np.fromfile(path, dtype="<f4").reshape(-1, vocab)
        got = collect(steps, outputs)
        _check(got, want, dtype, f"trace_run {dtype}")
    # `model_main --replay` is the same program; with --kernels plain bfloat16 goes through the plain kernels
    out_dir = tmp_path / "plain"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "model_main"), "--replay", "--model", model_folders[name],
         "--dtype", "bfloat16", "--out", str(out_dir), "--max-tokens", "192", "--kernels", "plain"],
        input="".join(json.dumps(s) + "\n" for s in steps), text=True,
        stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    outputs = {s["step"]: np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(-1, vocab)
               for s in steps if sum(len(e["want"]) for e in s["entries"])}
    _check(collect(steps, outputs), want, "bfloat16", "model_main --replay --kernels plain")


def test_random_weights_without_a_folder(model_folders, tmp_path):
    """One random model everywhere: the tensors drawn on the device are, bit for bit, those of
    the folder written with the same seed; and ``--config FILE --random-weights --seed S``
    replays a trace against the plain implementation run on weights that the test draws for
    itself in numpy, with no model folder anywhere."""
    import plain_qwen3
    import plain_random
    from helpers import config_json
    from tiny_llm_infer_amd import lookup_architecture
    from tiny_llm_infer_amd.engine.model import Model
    from tiny_llm_infer_amd.weights import Checkpoint, random_tensors
    name, seed = "C", 12345
    arch = lookup_architecture("Qwen3ForCausalLM")
    conf = config_json(name)
    decls = Model(arch.make_spec(arch.read_config(conf, "x"))).tensors()
    ck = Checkpoint(model_folders[name])
    for n, t in random_tensors(decls, TINY[name]["seed"], torch.bfloat16, "cuda:0"):
        assert t.device.type == "cuda" and torch.equal(t.cpu(), ck.read(n)), n
    ck.close()
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(conf))
    w = {k: torch.from_numpy(v) for k, v in
         plain_random.model_weights([(d.name, d.shape, d.init) for d in decls], seed).items()}
    reqs = _requests(name, [50, 23, 77], seed=8)
    want = {rid: plain_qwen3.forward(conf, w, toks).numpy() for rid, toks in reqs.items()}
    steps = trace_mixed(reqs, max_tokens=192, seed=5)
    vocab = TINY[name]["vocab_size"]
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / dtype
        proc = subprocess.run(
            [sys.executable, os.path.join(ROOT, "bin", "model_main"), "--replay", "--config", str(cfg_path),
             "--random-weights", "--seed", str(seed), "--dtype", dtype, "--out", str(out_dir), "--max-tokens", "192",
             "--page-size", "32"],
            input="".join(json.dumps(s) + "\n" for s in steps), text=True,
            stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        outputs = {s["step"]: np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(-1, vocab)
                   for s in steps if sum(len(e["want"]) for e in s["entries"])}
        _check(collect(steps, outputs), want, dtype, f"random weights without a folder, {dtype}", TOL_TINY)


@pytest.mark.parametrize("sizes", [
    dict(hidden_size=4096, intermediate_size=12288, num_attention_heads=32, num_key_value_heads=8),   # Qwen3-8B
    # the width and the head grouping of Qwen3-14B (5 query heads a kv head) and of Qwen3-32B (8),
    # fewer heads and a narrower feed-forward to keep the plain implementation's time down
    dict(hidden_size=5120, intermediate_size=1536, num_attention_heads=10, num_key_value_heads=2),
    dict(hidden_size=5120, intermediate_size=2560, num_attention_heads=16, num_key_value_heads=2),
    # and their true layers: 40 and 64 query heads over 8 kv heads (q as wide as, and wider than, the
    # hidden size), intermediate 17408 and 25600; two shorter requests
    dict(hidden_size=5120, intermediate_size=17408, num_attention_heads=40, num_key_value_heads=8),
    dict(hidden_size=5120, intermediate_size=25600, num_attention_heads=64, num_key_value_heads=8),
], ids=["8B", "14B-like", "32B-like", "14B", "32B"])
def test_real_layer_sizes(tmp_path, sizes):
    """Qwen3-8B layer sizes (hidden 4096, 32 query / 8 kv heads of 128, intermediate
    12288) with random weights, one layer and a small vocabulary to keep the plain
    implementation's time down: all cuts in float32 and in bfloat16, through the
    kernels' full-size code paths (decode layout, MFMA attention, recorded decode
    steps).  Also the width and head grouping of the larger models."""
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    cfg = Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=1, head_dim=128, vocab_size=2048,
        max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, **sizes))
    folder = write_random_model(str(tmp_path / "big"), "Qwen3ForCausalLM", cfg, seed=5)
    lengths = [150, 97, 40] if sizes["intermediate_size"] <= 12288 else [150, 45]
    reqs = {f"r{i}": random_prompt(2048, n, 300 + i) for i, n in enumerate(lengths)}
    want = plain_logits(folder, reqs)
    for dtype in ("float32", "bfloat16"):
        model, _ = load_model(folder, dtype, "cuda:0")
        for cut, steps in (("whole", trace_whole(reqs)), ("decode", trace_prefill_then_decode(reqs)),
                           ("portions", trace_portions(reqs, seed=2)),
                           ("mixed", trace_mixed(reqs, max_tokens=384, seed=6))):
            runner = ModelRunner(model, model.env, page_size=16, num_pages=24, max_requests=4,
                                 max_batch_tokens=512)
            got = collect(steps, _replay(runner, steps))
            worst = _check(got, want, dtype, f"{sizes['hidden_size']} wide/{dtype}/{cut}")
            print(f"{sizes['hidden_size']} wide, {sizes['num_attention_heads']} heads, {dtype} {cut}: worst relative error {worst:.2e}")
            runner.cache.check()
    # bfloat16 once more with the products of more than 128 rows (the whole prompt of 150 tokens, and
    # the 118 + 32 of "decode" is below) through the BLAS library instead of this library's own kernel
    # (the row-major matrices it reads are put together from the decode layout at every call)
    model.env.ops.many_rows = "library"
    steps = trace_whole(reqs)
    runner = ModelRunner(model, model.env, page_size=16, num_pages=24, max_requests=4, max_batch_tokens=512)
    worst = _check(collect(steps, _replay(runner, steps)), want, "bfloat16", f"{sizes['hidden_size']} wide/library products")
    print(f"{sizes['hidden_size']} wide, library products of many rows: worst relative error {worst:.2e}")


def test_three_layers_at_the_width_of_qwen3_8b(tmp_path):
    """Three layers of the Qwen3-8B sizes against the plain implementation, requests mixed so
    that pages are used again: which layer of the cache a page's keys belong to, at the true
    strides of the pool (8 kv heads of 128, pages of 16), in float32 and in bfloat16."""
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    cfg = Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3, head_dim=128, vocab_size=1024,
        max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False,
        hidden_size=4096, intermediate_size=12288, num_attention_heads=32, num_key_value_heads=8))
    folder = write_random_model(str(tmp_path / "three"), "Qwen3ForCausalLM", cfg, seed=8)
    reqs = {f"r{i}": random_prompt(1024, n, 500 + i) for i, n in enumerate([120, 61, 40, 97])}
    want = plain_logits(folder, reqs)
    steps = trace_mixed(reqs, max_tokens=256, seed=4)
    for dtype in ("float32", "bfloat16"):
        model, _ = load_model(folder, dtype, "cuda:0")
        runner = ModelRunner(model, model.env, page_size=16, num_pages=16, max_requests=4, max_batch_tokens=512)
        got = collect(steps, _replay(runner, steps))
        worst = _check(got, want, dtype, f"three layers/{dtype}")
        print(f"three layers at 4096 wide, {dtype}, mixed: worst relative error {worst:.2e}")
        runner.cache.check()
        assert runner.cache.pages_taken_total > runner.cache.num_pages


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_selective_attention_through_every_cut(model_folders, tmp_path, name):
    """With random weights every key weighs about the same, and a key that is
    left out or counted twice changes little.  Here the head norms of q and k are
    doubled, so scores are four times as far apart and few keys carry a row: in
    float32 every cut still matches the plain implementation and they agree with
    each other bit for bit; in bfloat16 (where such scores amplify the rounding
    of q and k) the tuned kernels stay as close to it as the plain kernels do."""
    import shutil
    from tiny_llm_infer_amd.weights.safetensors_io import SafetensorsFile, write_safetensors
    folder = str(tmp_path / name)
    shutil.copytree(model_folders[name], folder)
    path = os.path.join(folder, "model.safetensors")
    src = SafetensorsFile(path)
    tensors = []
    for n in src.names():
        t = src.read(n).clone()
        if n.endswith("q_norm.weight") or n.endswith("k_norm.weight"):
            t = (t.float() * 2).to(t.dtype)
        tensors.append((n, t))
    src.close()
    write_safetensors(path, tensors)
    reqs = _requests(name, [70, 45, 97, 33, 121], seed=15)
    want = plain_logits(folder, reqs)
    cuts = {"decode": trace_prefill_then_decode(reqs), "portions": trace_portions(reqs, seed=5),
            "mixed": trace_mixed(reqs, max_tokens=320, seed=12)}
    first = None
    for cut, steps in cuts.items():
        got = collect(steps, _replay(_runner(folder, name, "float32", 320), steps))
        _check(got, want, "float32", f"selective {name}/float32/{cut}")
        if first is None:
            first = got
        for rid in reqs:
            assert np.array_equal(first[rid], got[rid]), (cut, rid)

    def worst(got):
        return max(max_error(got[rid], want[rid])[0] / max_error(got[rid], want[rid])[2] for rid in want)
    for cut, steps in cuts.items():
        tuned = worst(collect(steps, _replay(_runner(folder, name, "bfloat16", 320), steps)))
        runner = _runner(folder, name, "bfloat16", 320)
        runner.env.ops.use_plain_kernels()
        plain = worst(collect(steps, _replay(runner, steps)))
        print(f"selective {name} bfloat16 {cut}: tuned {tuned:.2e}, plain kernels {plain:.2e}")
        assert tuned <= 1.5 * plain + 0.1 * TOL["bfloat16"], (cut, tuned, plain)


@pytest.mark.parametrize("batch", [40, 140])
def test_many_rows_decoded_together_at_real_width(tmp_path, batch):
    """40 and 140 requests at the width of Qwen3-8B (one layer): prompts in two steps of many
    rows, then every request's last tokens one by one, all requests in one step: the products
    for 17..128 rows with their partial sums, those for more rows, the recorded decode steps."""
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner, StepEntry
    cfg = Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=1, head_dim=128, vocab_size=1024,
        max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, hidden_size=4096,
        intermediate_size=12288, num_attention_heads=32, num_key_value_heads=8))
    folder = write_random_model(str(tmp_path / "wide"), "Qwen3ForCausalLM", cfg, seed=3)
    rng = np.random.default_rng(batch)
    reqs = {f"r{i}": random_prompt(1024, int(n), 50 * batch + i) for i, n in enumerate(rng.integers(12, 50, batch))}
    want = plain_logits(folder, reqs)
    model, _ = load_model(folder, "bfloat16", "cuda:0")
    runner = ModelRunner(model, model.env, page_size=16, num_pages=batch * 4, max_requests=batch, max_batch_tokens=8192)
    ids, keep = list(reqs), 4
    for rid in ids:
        runner.admit(rid)
    for part in (ids[:batch // 2], ids[batch // 2:]):
        runner.step([StepEntry(r, reqs[r][:-keep], []) for r in part])
    worst = 0.0
    for t in range(keep):
        out = runner.step([StepEntry(r, [reqs[r][len(reqs[r]) - keep + t]], [0]) for r in ids]).float().cpu().numpy()
        for i, r in enumerate(ids):
            w = want[r][len(reqs[r]) - keep + t]
            worst = max(worst, float(np.abs(out[i] - w).max() / np.abs(w).max()))
    print(f"{batch} rows decoded together: worst relative error {worst:.2e}")
    assert worst <= TOL["bfloat16"]
    assert runner.graph_replays == keep
    for rid in ids:
        runner.release(rid)
    runner.cache.check()


def test_trace_run_twice_gives_the_same_bytes_and_an_index(model_folders, tmp_path):
    """Two runs of bin/trace_run on the same bfloat16 trace (prompt portions of more than 128
    rows among them, whose products could go to one of two kernels) write byte-identical
    logits; index.jsonl names the request and position of every row and the block tables
    of every step, in which no page belongs to two live requests."""
    name = "D"
    reqs = _requests(name, [200, 150, 70], seed=61)
    steps = trace_mixed(reqs, max_tokens=512, seed=3)
    first = {"step": 0, "entries": [{"id": "whole", "tokens": reqs["r0"], "want": [0, 199]}], "end": ["whole"]}
    steps = [first] + [dict(s, step=s["step"] + 1) for s in steps]
    runs = []
    for run in range(2):
        out_dir = tmp_path / f"run{run}"
        proc = subprocess.run(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folders[name],
             "--dtype", "bfloat16", "--out", str(out_dir), "--max-tokens", "512"],
            input="".join(json.dumps(s) + "\n" for s in steps), text=True,
            stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert "kernels: own-products" in proc.stderr
        runs.append({f: (out_dir / f).read_bytes() for f in sorted(os.listdir(out_dir))})
    assert runs[0].keys() == runs[1].keys() and len(runs[0]) > 10
    for f in runs[0]:
        assert runs[0][f] == runs[1][f], f
    index = [json.loads(line) for line in runs[0]["index.jsonl"].decode().splitlines()]
    assert [i["step"] for i in index] == [s["step"] for s in steps]
    vocab = TINY[name]["vocab_size"]
    fed = {}
    for s, i in zip(steps, index):
        rows = []
        for e in s["entries"]:
            rows += [{"id": e["id"], "position": fed.get(e["id"], 0) + w} for w in e["want"]]
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        assert i["rows"] == rows
        if rows:
            assert len(runs[0][i["file"]]) == 4 * vocab * len(rows)
        assert sorted(i["block_tables"]) == sorted(e["id"] for e in s["entries"])
        for group in range(2):                                 # D: a windowed layer and a full one
            held = [p for t in i["block_tables"].values() for p in t[group] if p >= 0]
            assert len(held) == len(set(held)) and all(0 <= p < 512 // 16 for p in held)
