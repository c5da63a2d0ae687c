"""Generation through the entry points on the GPU: the Python engine and the
command line, greedy against the plain implementation, the small serving workloads
of the two tiny configurations, and top-p sampling against a plain version."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_qwen3
from cpu_ops import CpuOps
from helpers import TINY, random_prompt

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _engine(folder, name, dtype, **kw):
    from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
    args = dict(dtype=dtype, device="cuda:0", max_model_len=128, page_size=TINY[name]["page_size"],
                num_kv_blocks=64, max_num_seqs=4, max_num_batched_tokens=24)
    args.update(kw)
    return LLMEngine.from_folder(folder, **args)


def test_greedy_generation_float32_equals_plain(model_folders):
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders["A"]
    cfg, w = plain_qwen3.read_model(folder)
    prompts = [random_prompt(256, n, 40 + n) for n in (5, 17, 33)]
    want = [plain_qwen3.greedy(cfg, w, p, 16) for p in prompts]
    eng = _engine(folder, "A", "float32")
    got = eng.generate(prompts, SamplingParams(max_tokens=16, ignore_eos=True))
    assert [r.token_ids for r in got] == want
    small = _engine(folder, "A", "float32", num_kv_blocks=9)       # preemption and recompute
    got = small.generate(prompts, SamplingParams(max_tokens=16, ignore_eos=True))
    assert [r.token_ids for r in got] == want and small.scheduler.num_preemptions > 0
    small.runner.cache.check()


@pytest.mark.parametrize("ahead", [False, True])
@pytest.mark.parametrize("name,pages", [("B", 5), ("B", 8), ("D", 7), ("D", 12)])
def test_preemption_with_two_groups_of_cache_layers(model_folders, name, pages, ahead):
    """Configurations with a windowed group and one that keeps all keys, in a pool so small
    that requests are preempted and computed again, with and without steps launched ahead:
    float32 tokens are the plain greedy ones, no page is lost, every pool is whole at the end."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders[name]
    cfg, w = plain_qwen3.read_model(folder)
    vocab = TINY[name]["vocab_size"]
    prompts = [random_prompt(vocab, n, 30 + n) for n in (5, 17, 33, 9)]
    want = [plain_qwen3.greedy(cfg, w, p, 16) for p in prompts]
    eng = _engine(folder, name, "float32", num_kv_blocks=pages)
    eng.lookahead = ahead
    got = eng.generate(prompts, SamplingParams(max_tokens=16, ignore_eos=True))
    assert [r.token_ids for r in got] == want
    assert eng.scheduler.num_preemptions > 0 and sum(r.preemptions for r in got) == eng.scheduler.num_preemptions
    eng.runner.cache.check()
    assert len(eng.runner.cache.groups) == 2 and eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()
    # bfloat16 through the same schedule: every token within rounding of the plain best for its own prefix
    eng = _engine(folder, name, "bfloat16", num_kv_blocks=pages)
    eng.lookahead = ahead
    got = eng.generate(prompts, SamplingParams(max_tokens=16, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0
    for p, r in zip(prompts, got):
        logits = plain_qwen3.forward(cfg, w, p + r.token_ids[:-1])[len(p) - 1:]
        for t, row in zip(r.token_ids, logits):
            assert float(row.max() - row[t]) <= 5e-2 * float(row.abs().max())
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()


def test_a_window_group_has_the_smaller_pool_on_the_device(model_folders):
    """Configuration B: layer 0 keeps all keys, layers 1 and 2 a window of 40.  With room for
    4 requests of 640 tokens the windowed layers get 4 * (3 + 2) + 2 pages (the window's blocks
    and two for its edges a request, a step's 24 tokens on top), not 160, and their tensors are
    that small; generation is what it is with equal pools."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    eng = _engine(model_folders["B"], "B", "float32", num_kv_blocks=160, max_model_len=640)
    cache = eng.runner.cache
    assert cache.pages_per_group() == [160, 22]
    assert [t["k"].shape[:2] for t in eng.runner.group_tensors] == [(1, 161), (2, 23)]
    assert eng.stats()["pages_per_group"] == [160, 22]
    prompts = [random_prompt(384, n, 11 * n) for n in (150, 3, 77, 240)]
    got = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    cfg, w = plain_qwen3.read_model(model_folders["B"])
    assert [r.token_ids for r in got] == [plain_qwen3.greedy(cfg, w, p, 12) for p in prompts]
    assert eng.scheduler.num_preemptions == 0
    cache.check()
    assert cache.free_pages() == [160, 22]


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_bfloat16_follows_plain(model_folders, name):
    """In bfloat16 a near-tie may fall the other way, so each generated token
    is checked against the plain logits for the engine's own prefix: it must be
    the plain arg-max or within the rounding margin of it."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders[name]
    cfg, w = plain_qwen3.read_model(folder)
    vocab = TINY[name]["vocab_size"]
    prompts = [random_prompt(vocab, n, 90 + n) for n in (3, 21, 40)]
    eng = _engine(folder, name, "bfloat16")
    got = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    same = 0
    for p, r in zip(prompts, got):
        logits = plain_qwen3.forward(cfg, w, p + r.token_ids[:-1])[len(p) - 1:]
        for t, row in zip(r.token_ids, logits):
            # (bfloat16 logits of these configurations are within 1.2e-2 of the largest logit of the plain
            # ones, so a token the engine prefers is at most twice that below the plain best)
            margin = 1.2e-2 * float(row.abs().max())
            assert float(row.max() - row[t]) <= 2 * margin
            same += int(t == int(row.argmax()))
    assert same >= 32          # of 36


def test_temperature_workload_of_configuration_b(model_folders):
    """Five requests with prompts of 1..40 tokens, 12 tokens each at temperature
    0.7 with fixed seeds, page 16, budget 32: the tokens are those a plain
    sampler draws from the engine's own float32 logits, and do not depend on
    the batch."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders["B"]
    prompts = [random_prompt(384, n, 70 + n) for n in (1, 9, 40, 23, 14)]
    params = [SamplingParams(max_tokens=12, temperature=0.7, ignore_eos=True, seed=100 + i)
              for i in range(5)]
    eng = _engine(folder, "B", "float32", max_num_batched_tokens=32)
    together = eng.generate(prompts, params)
    alone = [_engine(folder, "B", "float32", max_num_batched_tokens=32).generate([p], [s])[0]
             for p, s in zip(prompts, params)]
    assert [r.token_ids for r in together] == [r.token_ids for r in alone]
    # the same engine logic on the CPU stand-in draws the same tokens
    from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
    cpu = LLMEngine.from_folder(folder, dtype="float32", device="cpu", max_model_len=128, page_size=16,
                                num_kv_blocks=64, max_num_seqs=4, max_num_batched_tokens=32, ops=CpuOps())
    ref = cpu.generate(prompts, params)
    agree = sum(a == b for r, c in zip(together, ref) for a, b in zip(r.token_ids, c.token_ids))
    assert agree >= 55         # of 60; a draw on a near-tie may differ between float32 libraries


def test_top_p_kernel_against_plain():
    from tiny_llm_infer_amd.kernels.ops import HipOps
    ops = HipOps("cuda:0")
    rows, vocab = 6, 500
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(rows, vocab, generator=g) * 3
    temps = torch.tensor([0.7, 1.0, 0.0, 0.5, 2.0, 1.0])
    top_p = torch.tensor([0.9, 0.5, 0.3, 1.0, 0.05, 1e-6])
    seeds = torch.arange(1, rows + 1, dtype=torch.int64) * 104729
    got = ops.sample(logits.cuda(), temps.cuda(), seeds.cuda(), top_p=top_p.cuda()).cpu().tolist()
    want = CpuOps().sample(logits, temps, seeds, top_p).tolist()
    assert got == want
    assert got[5] == int(logits[5].argmax())        # a vanishing top_p keeps the best token only


def test_top_p_over_a_large_vocabulary_against_the_rule():
    """The top-p selection (a histogram of the weights over the logits' range, refined twice) over
    vocabularies of 40,007 and 151,936 tokens, peaked and flat rows, temperatures from 0.3 to 2 and top_p
    from 1e-4 to 0.999: for 24 seeds a row the drawn token is the best of the kept ones under the rule
    written out in float64 (sort, running sum, threshold), with the same Gumbel noise."""
    import numpy as np
    from tiny_llm_infer_amd.kernels.ops import HipOps
    ops = HipOps("cuda:0")

    def uniforms(seed, n):
        def mix(h):
            h = h.copy()
            h ^= h >> np.uint32(16); h *= np.uint32(0x85EBCA6B); h ^= h >> np.uint32(13)
            h *= np.uint32(0xC2B2AE35); h ^= h >> np.uint32(16)
            return h
        lo, hi = np.uint32(seed & 0xFFFFFFFF), np.uint32(seed >> 32)
        with np.errstate(over="ignore"):
            h = mix(np.arange(n, dtype=np.uint32) ^ np.uint32(0x9E3779B9))
            h = mix(h ^ lo)
            h = mix(h + hi * np.uint32(0x85EBCA6B) + np.uint32(0x27D4EB2F))
        return ((h >> np.uint32(9)).astype(np.float64) + 0.5) / 8388608.0

    g = torch.Generator().manual_seed(5)
    for vocab in (40007, 151936):
        cases = []              # (logits, temperature, top_p)
        for std, temp, tp in ((3.0, 0.7, 0.9), (3.0, 1.0, 0.5), (1.0, 2.0, 0.999), (8.0, 0.3, 0.95), (0.01, 1.0, 0.3),
                              (3.0, 0.6, 1e-4), (5.0, 1.0, 0.05), (2.0, 1.5, 0.7)):
            cases.append((torch.randn(vocab, generator=g) * std, temp, tp))
        ties = torch.randn(vocab, generator=g).mul(4).round().div(4)               # many equal logits
        cases.append((ties, 1.0, 0.6))
        logits = torch.stack([c[0] for c in cases])
        rows = len(cases)
        temps = torch.tensor([c[1] for c in cases], dtype=torch.float32)
        top_p = torch.tensor([c[2] for c in cases], dtype=torch.float32)
        kept = []
        for row, temp, tp in cases:
            x = row.double().numpy()
            w = np.exp((x - x.max()) / temp)
            order = np.argsort(-x, kind="stable")
            before = np.concatenate([[0.0], np.cumsum(w[order])[:-1]])             # weights of the tokens before each one
            n = int((before < np.float64(np.float32(tp)) * w.sum()).sum())
            edge = x[order[n - 1]]
            kept.append((x >= edge, n))                                             # tokens equal to the last one kept share its fate
        dev = logits.cuda()
        for s in range(24):
            seeds = torch.arange(rows, dtype=torch.int64) * 7919 + 1000003 * s + 17
            got = ops.sample(dev, temps.cuda(), seeds.cuda(), top_p=top_p.cuda()).cpu().tolist()
            for r, (row, temp, tp) in enumerate(cases):
                x = row.double().numpy()
                score = np.where(kept[r][0], x + temp * -np.log(-np.log(uniforms(int(seeds[r]), vocab))), -np.inf)
                best = int(np.argmax(score))
                assert kept[r][0][got[r]], f"vocabulary {vocab}, row {r}, seed {s}: token {got[r]} is not among the {kept[r][1]} kept"
                assert got[r] == best or score[best] - score[got[r]] < 1e-5, (vocab, r, s, got[r], best)


def test_command_line_infer(model_folders):
    folder = model_folders["A"]
    cfg, w = plain_qwen3.read_model(folder)
    prompts = [random_prompt(256, 7, 1), random_prompt(256, 19, 2)]
    want = [plain_qwen3.greedy(cfg, w, p, 5) for p in prompts]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "model_main"), "--infer", "--model", folder,
           "--dtype", "float32", "--max-new-tokens", "5", "--max-seq-len", "64", "--num-kv-blocks", "16",
           "--page-size", "8", "--ignore-eos"]
    for p in prompts:
        cmd += ["--prompt-ids", ",".join(map(str, p))]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [list(map(int, l.split())) for l in proc.stdout.strip().split("\n")]
    assert lines == want
    # usage errors exit with 2
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "model_main"), "--infer", "--model", folder],
                         stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
    assert bad.returncode == 2


def test_command_line_bench(model_folders):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "model_main"), "--bench", "--model", model_folders["B"],
           "--num-seqs", "3", "--min-input-len", "4", "--max-input-len", "9", "--min-output-len", "3",
           "--max-output-len", "5", "--warmup", "1", "--repeats", "2", "--max-seq-len", "64"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = proc.stdout.strip().split("\n")
    assert out[0].startswith("run=0 output_tokens=") and "output_tokens_per_second=" in out[-1]
    fields = lambda line: dict(f.split("=") for f in line.split() if "=" in f)
    runs = [fields(line) for line in out if line.startswith("run=")]
    total = fields(next(line for line in out if line.startswith("aggregate_runs=")))
    # every request ends at a length between the two bounds, the runs add up, nothing stays held
    assert len(runs) == 2 and all(9 <= int(r["output_tokens"]) <= 15 for r in runs)
    assert int(total["aggregate_runs"]) == 2 and int(total["output_tokens"]) == sum(int(r["output_tokens"]) for r in runs)
    assert abs(float(total["elapsed_seconds"]) - sum(float(r["elapsed_seconds"]) for r in runs)) < 1e-3
    stats = fields(next(line for line in proc.stderr.split("\n") if line.startswith("engine_steps=")))
    free, pages = stats["pages_free"].split("/")
    assert free == pages and int(stats["engine_steps"]) > 0


def test_command_line_plain_kernels_and_prefill_only(model_folders):
    """--kernels plain runs bfloat16 through the plain kernels: the first tokens are those
    of the tuned kernels; --bench --prefill-only counts prompt tokens."""
    folder = model_folders["D"]
    prompt = ",".join(map(str, random_prompt(320, 21, 4)))
    outs = []
    for kernels in ("tuned", "plain"):
        cmd = [sys.executable, os.path.join(ROOT, "bin", "model_main"), "--infer", "--model", folder,
               "--dtype", "bfloat16", "--max-new-tokens", "4", "--max-seq-len", "64", "--num-kv-blocks", "16",
               "--page-size", "8", "--ignore-eos", "--kernels", kernels, "--prompt-ids", prompt]
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        outs.append(list(map(int, proc.stdout.split())))
    assert len(outs[0]) == 4 and outs[0][0] == outs[1][0]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "model_main"), "--bench", "--model", folder, "--prefill-only",
           "--num-seqs", "3", "--min-input-len", "20", "--max-input-len", "40", "--warmup", "0", "--repeats", "1",
           "--max-seq-len", "64"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.startswith("run=0 prompt_tokens=") and "median_prompt_tokens_per_second=" in proc.stdout


def test_the_library_is_needed():
    from tiny_llm_infer_amd.kernels.ops import HipOps, KernelError
    with pytest.raises(KernelError):
        HipOps("cpu")


def test_recorded_decode_steps_equal_eager_ones(model_folders):
    """Decode steps are replayed from a recorded HIP graph.  Every replay is
    compared with the same step run eagerly on a second runner, with eager work
    (prefill of new requests, steps of other shapes) and synchronisation between
    the replays, and while requests come and go so that pages and slots change."""
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner, StepEntry
    name = "B"
    model, _ = load_model(model_folders[name], "bfloat16", "cuda:0")
    make = lambda: ModelRunner(model, model.env, page_size=16, num_pages=40, max_requests=4,
                               max_batch_tokens=256)
    fast, slow = make(), make()
    assert fast.use_graphs
    slow.use_graphs = False
    rng = np.random.default_rng(1)
    live = {}
    compared = 0
    for it in range(60):
        if len(live) < 3 and rng.random() < 0.4:
            key = f"r{it}"
            prompt = rng.integers(0, 384, int(rng.integers(2, 50))).tolist()
            for r in (fast, slow):
                r.admit(key)
                r.step([StepEntry(key, prompt, [])])          # eager work between replays
            live[key] = len(prompt)
        if not live:
            continue
        entries = [StepEntry(k, [int(rng.integers(0, 384))], [0]) for k in live]
        a = fast.step(entries).clone()
        torch.cuda.synchronize()
        b = slow.step(entries)
        assert torch.equal(a, b), f"replay {it} differs from the eager step"
        compared += 1
        for k in list(live):
            live[k] += 1
            if live[k] > 70 or rng.random() < 0.05:
                fast.release(k)
                slow.release(k)
                del live[k]
    assert compared > 30 and fast.graph_replays == compared and len(fast.graphs) >= 3


@pytest.mark.parametrize("first,most,rows,products", [(80, 90, 96, "own"), (140, 150, 160, "own"),
                                                       (140, 150, 160, "library")])
def test_recorded_steps_of_many_rows_equal_eager_ones(tmp_path, first, most, rows, products):
    """Many rows in a decode step, at the layer sizes of Qwen3-8B: up to 128 rows the
    matrix products are the kernel with eight row tiles, beyond they are the kernel for
    any number of rows, or the library's where that was asked for before the weights were
    loaded (it picks its kernels by shape, and its calls are recorded too).  80 to 90 live
    requests in steps of 96 rows, and 140 to 150 in steps of 160; every replay is compared
    with the same step run eagerly on a second runner, with eager prefill work and
    synchronisation between the replays."""
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner, StepEntry
    cfg = Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, head_dim=128, vocab_size=4096,
        hidden_size=4096, intermediate_size=12288, num_attention_heads=32, num_key_value_heads=8,
        max_position_embeddings=4096, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False))
    folder = write_random_model(str(tmp_path / "wide"), "Qwen3ForCausalLM", cfg, seed=9)
    from tiny_llm_infer_amd.kernels.ops import HipOps
    ops = HipOps("cuda:0")
    ops.many_rows = products
    model, _ = load_model(folder, "bfloat16", "cuda:0", ops=ops)
    held = model.blocks[0].ffn.w_down
    assert (held._w is not None) == (products == "library") and held.tiled is not None     # one form, or both
    make = lambda: ModelRunner(model, model.env, page_size=16, num_pages=700, max_requests=rows,
                               max_batch_tokens=4096)
    fast, slow = make(), make()
    slow.use_graphs = False
    rng = np.random.default_rng(4)
    live = []
    for it in range(14):
        fresh = [f"r{it}_{j}" for j in range(first if it == 0 else int(rng.integers(0, 4)))]
        fresh = fresh[:most - len(live)]
        if fresh:
            prompts = [rng.integers(0, 4096, int(rng.integers(2, 20))).tolist() for _ in fresh]
            for r in (fast, slow):
                for key in fresh:
                    r.admit(key)
                r.step([StepEntry(k, p, []) for k, p in zip(fresh, prompts)])     # eager work between replays
            live += fresh
        entries = [StepEntry(k, [int(rng.integers(0, 4096))], [0]) for k in live]
        a = fast.step(entries).clone()
        torch.cuda.synchronize()
        b = slow.step(entries)
        assert torch.isfinite(a).all()
        assert torch.equal(a, b), f"replay {it} of {len(entries)} rows differs from the eager step"
        for k in live[:int(rng.integers(0, 3))]:
            fast.release(k)
            slow.release(k)
            live.remove(k)
    assert fast.graph_replays == 14 and {k[0] for k in fast.graphs} == {rows}


def test_decode_steps_are_padded_to_few_sizes(model_folders):
    """Seven requests that finish one after the other: the recorded decode steps come in
    the sizes 8, 4, 2 and 1 only (steps of other sizes are filled with rows of no
    request), and the tokens are those of an engine that records nothing."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders["D"]
    prompts = [random_prompt(320, 6 + 3 * i, 70 + i) for i in range(7)]
    params = [SamplingParams(max_tokens=4 + 5 * i, ignore_eos=True) for i in range(7)]
    args = dict(max_num_seqs=8, max_num_batched_tokens=128, max_model_len=128)
    eng = _engine(folder, "D", "bfloat16", **args)
    got = eng.generate(prompts, params)
    assert eng.runner.graph_replays > 20
    assert {k[0] for k in eng.runner.graphs} == {8, 4, 2, 1}
    plain = _engine(folder, "D", "bfloat16", **args)
    plain.runner.use_graphs = False
    want = plain.generate(prompts, params)
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()


def test_a_default_run_never_asks_for_the_row_major_form_of_a_matrix(tmp_path):
    """bfloat16 matrices are held once, in the decode layout.  Prefill of more than 128 rows,
    portions, recorded decode steps: nothing puts the row-major form together again.  The plain
    kernels do ask for it, and then it is made once for every matrix and kept."""
    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
    from tiny_llm_infer_amd.engine.loading import write_random_model
    from tiny_llm_infer_amd.parts.linear import Matrix
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    cfg = Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, head_dim=64, vocab_size=512,
        hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
        max_position_embeddings=1024, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False))
    folder = write_random_model(str(tmp_path / "m"), "Qwen3ForCausalLM", cfg, seed=2)
    eng = LLMEngine.from_folder(folder, dtype="bfloat16", device="cuda:0", max_model_len=512, page_size=16,
                                num_kv_blocks=128, max_num_seqs=4, max_num_batched_tokens=256)
    before = Matrix.rebuilt
    prompts = [random_prompt(512, n, n) for n in (300, 40, 7, 150)]
    first = eng.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    assert Matrix.rebuilt == before and eng.runner.graph_replays > 0
    eng.runner.env.ops.use_plain_kernels()
    eng.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    made = Matrix.rebuilt - before
    assert made == 2 * 4 + 1                      # q/k/v, o, gate/up, down of two layers, and the head
    eng.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    assert Matrix.rebuilt - before == made        # kept, not made again
    assert all(len(r.token_ids) == 6 for r in first)


def test_prefix_caching_on_the_gpu(model_folders):
    """Requests that share a prompt prefix take its pages over instead of computing
    them; the tokens are those of an engine without the cache."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders["A"]
    shared = random_prompt(256, 40, 9)
    prompts = [shared + random_prompt(256, n, 20 + n) for n in (3, 9, 1)] + [shared[:33]]
    params = SamplingParams(max_tokens=6, ignore_eos=True)
    for dtype in ("float32", "bfloat16"):
        plain = _engine(folder, "A", dtype).generate(prompts, params)
        eng = _engine(folder, "A", dtype, enable_prefix_caching=True, max_num_seqs=1)
        got = eng.generate(prompts, params)
        if dtype == "float32":
            assert [r.token_ids for r in got] == [r.token_ids for r in plain]
        assert eng.runner.cache.prefix_hits == 14
        eng.runner.cache.check()


@pytest.mark.parametrize("name", ["B", "D"])
def test_a_request_that_ends_while_its_next_step_is_on_the_device(model_folders, name):
    """An end-of-sequence token stops one request of a batch in the middle of a run while the
    step after it is already on the device (fed on the device, replayed from its recording in
    bfloat16) and writes into pages that are given back meanwhile: the tokens are those of the
    engine that launches nothing ahead, the request stops where the plain greedy run meets the
    token, and no page is lost."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders[name]
    cfg, w = plain_qwen3.read_model(folder)
    vocab = TINY[name]["vocab_size"]
    prompts = [random_prompt(vocab, n, 60 + n) for n in (6, 19, 11, 27)]
    for dtype in ("float32", "bfloat16"):
        free = _engine(folder, name, dtype, max_num_batched_tokens=64)
        free.lookahead = False
        runs = [r.token_ids for r in free.generate(prompts, SamplingParams(max_tokens=14, ignore_eos=True))]
        # a token that request 1 meets in the middle of its run, and the others late or never if there is one
        others = [t for i, run in enumerate(runs) if i != 1 for t in run[:10]]
        eos = next((t for t in runs[1][3:7] if t not in others), runs[1][5])
        outs = []
        for ahead in (False, True):
            eng = _engine(folder, name, dtype, max_num_batched_tokens=64)
            eng.lookahead = ahead
            eng.eos_token_ids = {eos}
            outs.append([r.token_ids for r in eng.generate(prompts, SamplingParams(max_tokens=14))])
            assert (eng.num_steps_ahead > 0) == ahead
            if ahead and dtype == "bfloat16":
                assert eng.runner.graph_replays > 0
            eng.runner.cache.check()
            assert eng.is_finished() and eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()
            # and the engine serves again afterwards from the pages that were given back
            again = [r.token_ids for r in eng.generate(prompts[:2], SamplingParams(max_tokens=14))]
            assert again == outs[-1][:2]
        assert outs[0] == outs[1]
        for run, got in zip(runs, outs[1]):               # each request is its free run cut after the token
            cut = run.index(eos) + 1 if eos in run else len(run)
            assert got == run[:cut]
        assert len(outs[1][1]) <= 7
        if dtype == "float32":
            assert runs == [plain_qwen3.greedy(cfg, w, p, 14) for p in prompts]


@pytest.mark.parametrize("name", ["B", "D"])
def test_steps_with_prompt_portions_are_launched_ahead_too(model_folders, name):
    """A budget of 7 tokens and three live requests among five: while prompts go through in
    portions beside decoding requests, and while requests wait for a place, the next step is on
    the device before this one's tokens are read, its decoding rows fed on the device.  Greedy
    float32 tokens are the plain ones; drawn tokens (seeded) and an end-of-sequence stop are
    those of the engine that launches nothing ahead."""
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = model_folders[name]
    cfg, w = plain_qwen3.read_model(folder)
    vocab = TINY[name]["vocab_size"]
    prompts = [random_prompt(vocab, n, 80 + n) for n in (23, 4, 31, 12, 18)]
    want = [plain_qwen3.greedy(cfg, w, p, 10) for p in prompts]
    params = [SamplingParams(max_tokens=10, temperature=t, seed=3 + i, ignore_eos=(i != 2))
              for i, t in enumerate([0.0, 0.7, 0.0, 0.0, 0.9])]
    outs = []
    for ahead in (False, True):
        eng = _engine(folder, name, "float32", max_num_batched_tokens=7, max_num_seqs=3)
        eng.lookahead = ahead
        eng.eos_token_ids = {want[2][5]}                  # request 2 stops in the middle of its run
        for p, sp in zip(prompts, params):
            eng.add_request(p, sp)
        mixed_ahead, results = 0, []
        while not eng.is_finished():
            results.extend(eng.step())
            nxt = eng._inflight
            if nxt is not None and any(i.prompt_portion for i in nxt.plan.items) \
                    and any(not i.prompt_portion for i in nxt.plan.items):
                mixed_ahead += 1
        assert (mixed_ahead > 3) == ahead
        results.sort(key=lambda r: r.request_id)
        outs.append([r.token_ids for r in results])
        eng.runner.cache.check()
        assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()
    assert outs[0] == outs[1]
    for i in (0, 3):
        assert outs[1][i] == want[i]
    assert outs[1][2] == want[2][:want[2].index(want[2][5]) + 1]
    assert outs[1][1] != want[1] and outs[1][4] != want[4]          # the draws are draws
