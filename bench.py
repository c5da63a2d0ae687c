"""Serving benchmark on one MI355X: decode tokens a second of a Qwen3-8B-shaped
model with random bfloat16 weights (the layer sizes of Qwen3-8B), plus the prefill
of one 2,048-token prompt and decode at batch 1 and 64.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of the engine (schedule, run the batch, sample,
post-process).  One JSON line is printed.  Beside the headline, ``points`` holds (all
with 128-token prompts unless the name says otherwise, tokens a second and the fraction of
the HBM peak that the bytes a step has to read make of its time):
  decode_b1, decode_b64, decode_b256         a few steps at batch 1, 64 and 256
  decode_b{1,8,64}_128out                    all 128 output tokens of 128-token prompts
  decode_b{8,64}_ctx4096                     contexts that end at 4,096 tokens
  qwen3_14b_*, qwen3_32b_*                   decode at batch 8 and the prefill of 2,048 tokens at
                                             the layer sizes of the larger models (configs/), and
                                             one serving workload each through the scheduler: 32
                                             requests with prompts of 64 to 2,048 tokens in portions
                                             beside decoding (14B), 64 requests that join while the
                                             others are served (32B)
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12            # bytes/s, MI355X HBM3E
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_size=4096,
                intermediate_size=12288, num_hidden_layers=36, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, vocab_size=151936, max_position_embeddings=40960,
                rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False)


def weight_bytes(cfg, layers, elem=2):
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    Q = cfg["num_attention_heads"] * cfg["head_dim"]
    KV = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = (Q + 2 * KV) * H + H * Q + 3 * I * H
    return (layers * per_layer + V * H) * elem       # what a decode step reads (embedding rows aside)


def kv_bytes_per_token(cfg, layers, elem=2):
    return 2 * layers * cfg["num_key_value_heads"] * cfg["head_dim"] * elem


def step_flops(cfg, layers, rows, ctx_sum, wanted):
    """2*rows*params for the matrices, 4*heads*head_dim per (row, key) for attention."""
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    Q = cfg["num_attention_heads"] * cfg["head_dim"]
    KV = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = (Q + 2 * KV) * H + H * Q + 3 * I * H
    return 2.0 * rows * layers * per_layer + 4.0 * Q * ctx_sum * layers + 2.0 * wanted * V * H


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0: all)")
    ap.add_argument("--prompt-len", type=int, default=128)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip every point beside the headline")
    ap.add_argument("--no-other-shapes", action="store_true", help="skip the points at the layer sizes of the larger models")
    ap.add_argument("--no-big-batch", action="store_true", help="skip the point at batch 256")
    ap.add_argument("--no-workloads", action="store_true", help="skip the two serving workloads at those sizes")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill measurement (for profiles)")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode measurement (for profiles)")
    ap.add_argument("--own-products", action="store_true",
                    help="every product of more than 128 rows by this library's kernel (the default)")
    ap.add_argument("--library-products", action="store_true", help="... by the BLAS library (every matrix is then held twice)")
    ap.add_argument("--measured-products", action="store_true", help="... by whichever was timed faster for the shape")
    ap.add_argument("--rows-cfg", type=int, default=0, help="with --own-products: force a launch shape (measurements)")
    ap.add_argument("--no-check", action="store_true", help="skip the untimed comparison of logits with the 32-bit path")
    ap.add_argument("--shape", default=None,
                    help="a config.json whose layer sizes replace the default ones (configs/ holds the larger shapes of the family)")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py runs on one GPU only; --gpus {args.gpus} is not supported (single-GPU engine)")
        return 2

    import gc
    import random

    import torch

    from tiny_llm_infer_amd.config import Qwen3Config
    from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
    from tiny_llm_infer_amd.engine.loading import random_model
    from tiny_llm_infer_amd.sampling.params import SamplingParams

    cfg_json = dict(QWEN3_8B)
    shape_name = "Qwen3-8B shape"
    if args.shape:
        with open(args.shape) as fh:
            cfg_json = json.load(fh)
        shape_name = os.path.splitext(os.path.basename(args.shape))[0].replace("_", " ")
    full_layers = cfg_json["num_hidden_layers"]
    layers = args.layers or full_layers
    cfg_json["num_hidden_layers"] = layers
    cfg = Qwen3Config.from_dict(cfg_json)
    elem = 2 if args.dtype == "bfloat16" else 4
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    from tiny_llm_infer_amd.kernels.ops import HipOps
    page = 16
    budget = max(args.prefill_tokens, 2048)
    rng = random.Random(args.seed)

    def make_engine(conf, max_batch, longest, outputs, context=None):
        """A model of ``conf`` with random weights (for up to ``context`` positions) and an engine
        whose cache holds ``max_batch`` requests of ``longest`` prompt tokens and ``outputs`` new
        ones beside one prompt of --prefill-tokens."""
        context = context or args.context
        t0 = time.time()
        ops = HipOps("cuda:0")
        # which kernel multiplies more than 128 rows is settled before the weights are loaded: a matrix
        # keeps its row-major form only where the library (or the plain kernels of the untimed check) reads it
        ops.many_rows = "library" if args.library_products else ("measure" if args.measured_products else "own")
        ops.rows_cfg = args.rows_cfg
        before = torch.cuda.memory_allocated()
        m = random_model("Qwen3ForCausalLM", Qwen3Config.from_dict(conf), args.seed, args.dtype, "cuda:0",
                         context, ops=ops)
        gb = (torch.cuda.memory_allocated() - before) / 1e9
        torch.cuda.synchronize()
        print(f"[bench] model with {conf['num_hidden_layers']} layers of {conf['hidden_size']} on the device in "
              f"{time.time() - t0:.1f} s", file=sys.stderr, flush=True)
        pages = max_batch * ((longest + outputs + 64 + page - 1) // page) + (args.prefill_tokens + page - 1) // page + 8
        e = LLMEngine.from_model(m, max_model_len=context, page_size=page, num_kv_blocks=pages,
                                 max_num_seqs=max_batch, max_num_batched_tokens=budget)
        return m, e, gb

    def prefill_steps(batch, prompt_len):
        """Steps in which the prompts are taken in; those taken in first decode meanwhile."""
        return (batch * prompt_len + budget - 1) // budget + 1

    def decode_run(engine, conf, batch, steps, warmup, prompt_len):
        """Prefill ``batch`` prompts, then time ``steps`` decode steps after ``warmup`` untimed ones.
        Returns (seconds, tokens of context a step reads on average, fraction of the HBM peak)."""
        vocab = conf["vocab_size"]
        # (the margin keeps every request alive through the timed steps)
        params = SamplingParams(max_tokens=steps + warmup + prefill_steps(batch, prompt_len) + 16, temperature=0.0,
                                ignore_eos=True)
        for _ in range(batch):
            engine.add_request([rng.randrange(vocab) for _ in range(prompt_len)], params)
        while engine.scheduler.waiting:
            engine.step()
        for _ in range(warmup):
            engine.step()
        assert len(engine.scheduler.running) == batch
        ctx0 = sum(s.size for s in engine.scheduler.running)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx1 = sum(s.size for s in engine.scheduler.running)
        assert len(engine.scheduler.running) == batch, "a request ended inside the timed steps"
        while not engine.is_finished():
            engine.step()
        ctx = (ctx0 + ctx1) / 2.0
        n_layers = conf["num_hidden_layers"]
        nbytes = weight_bytes(conf, n_layers, elem) + ctx * kv_bytes_per_token(conf, n_layers, elem)
        return dt, ctx, nbytes / (dt / steps) / HBM_PEAK

    def prefill_run(engine, conf, tokens):
        """One prompt of ``tokens`` tokens in one step: (median of five, best) in seconds, after one
        untimed run, and the fraction of the matrix cores' peak that the median makes."""
        vocab = conf["vocab_size"]

        def once():
            engine.add_request([rng.randrange(vocab) for _ in range(tokens)], SamplingParams(max_tokens=1, ignore_eos=True))
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            assert engine.is_finished()
            return dt
        once()
        runs = sorted(once() for _ in range(5))
        flops = step_flops(conf, conf["num_hidden_layers"], tokens, tokens * (tokens + 1) / 2.0, 1)
        return runs[2], runs[0], flops / runs[2] / MFMA_PEAK[dkey]

    points = {}
    most = args.batch if args.no_points else max(64, args.batch)
    model, engine, weight_gb = make_engine(cfg_json, most, args.prompt_len if args.no_points else args.context - 192,
                                           max(args.steps + args.warmup, 128) + 64)
    vocab = cfg.vocab_size

    if args.no_decode:
        dt, ctx_tokens, frac = float("nan"), 0.0, float("nan")
    else:
        dt, ctx_tokens, frac = decode_run(engine, cfg_json, args.batch, args.steps, args.warmup, args.prompt_len)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    achieved = frac * HBM_PEAK

    # prefill of one prompt in one step
    T = args.prefill_tokens
    if args.no_prefill:
        pre = pre_best = pre_frac = float("nan")
    else:
        pre, pre_best, pre_frac = prefill_run(engine, cfg_json, T)

    if not args.no_points:
        n = min(args.steps, 32)
        for b in (1, 64):
            d, _, f = decode_run(engine, cfg_json, b, n, 4, args.prompt_len)
            points[f"decode_b{b}"] = round(b * n / d, 2)
            points[f"decode_b{b}_hbm_frac"] = round(f, 4)
        # a decode step of hundreds of requests, on an engine of its own over the same model (the cache
        # of the first one is sized for 64 requests of the full context)
        if not args.no_big_batch:
            big = LLMEngine.from_model(model, max_model_len=args.context, page_size=page, max_num_seqs=256,
                                       num_kv_blocks=256 * ((args.prompt_len + n + 64 + page - 1) // page) + 136,
                                       max_num_batched_tokens=budget)
            d, _, f = decode_run(big, cfg_json, 256, n, 4, args.prompt_len)
            points["decode_b256"] = round(256 * n / d, 2)
            points["decode_b256_hbm_frac"] = round(f, 4)
            del big
        # every one of the 128 output tokens of 128-token prompts (the first token comes with the
        # prompt's last step); once untimed before, because the steps past 256 tokens are recorded anew
        for b in (1, 8, 64):
            decode_run(engine, cfg_json, b, 127, 0, 128)
            d, _, f = decode_run(engine, cfg_json, b, 127, 0, 128)
            points[f"decode_b{b}_128out"] = round(b * 127 / d, 2)
            points[f"decode_b{b}_128out_hbm_frac"] = round(f, 4)
        # contexts that end at the limit (4,096 tokens unless --context says otherwise): prompts as
        # long as leaves every request room for the steps it takes while the others' prompts come in
        for b in (8, 64):
            long_prompt = args.context - (n + 4 + prefill_steps(b, args.context) + 16)
            d, ctx, f = decode_run(engine, cfg_json, b, n, 4, long_prompt)
            points[f"decode_b{b}_ctx{args.context}"] = round(b * n / d, 2)
            points[f"decode_b{b}_ctx{args.context}_hbm_frac"] = round(f, 4)
            points[f"decode_b{b}_ctx{args.context}_mean_context"] = round(ctx / b, 1)

    def logit_check():
        """Outside every timed region: the logits of the last prompt token and of a few decoded
        tokens on the whole model (all layers, the whole vocabulary), through the tuned kernels
        (recorded decode steps included), through the plain kernels in bfloat16, and through the
        true 32-bit path on the same weights; the largest difference to the 32-bit logits
        relative to the largest logit, for the tuned and for the plain kernels."""
        from tiny_llm_infer_amd.engine.runner import ModelRunner, StepEntry
        runner, ops = engine.runner, model.env.ops
        prompt = [rng.randrange(vocab) for _ in range(48)]
        tail = [rng.randrange(vocab) for _ in range(3)]

        def run(r):
            r.admit("check")
            rows = [r.step([StepEntry("check", prompt, [len(prompt) - 1])]).clone()]
            for t in tail:
                rows.append(r.step([StepEntry("check", [t], [0])]).clone())
            r.release("check")
            return torch.cat(rows).double()
        tuned = run(runner)
        flags = ("force_plain", "plain_products", "separate_norms", "unfused_decode")
        saved, graphs = [getattr(ops, f) for f in flags], runner.use_graphs
        ops.use_plain_kernels()
        runner.use_graphs = False
        try:
            plain = run(runner)
        finally:
            for f, v in zip(flags, saved):
                setattr(ops, f, v)
            runner.use_graphs = graphs
        exact_model = random_model("Qwen3ForCausalLM", cfg, args.seed, "float32", "cuda:0", args.context)
        exact = run(ModelRunner(exact_model, exact_model.env, page_size=page, num_pages=8, max_requests=1,
                                max_batch_tokens=64))
        del exact_model

        def rel(x):
            return round(float(((x - exact).abs().amax(dim=1) / exact.abs().amax(dim=1)).max()), 5)
        same = int((tuned.argmax(dim=1) == exact.argmax(dim=1)).sum())
        return {"rel_err_tuned_vs_fp32": rel(tuned), "rel_err_plain_kernels_vs_fp32": rel(plain),
                "argmax_same_as_fp32": same, "rows": int(tuned.shape[0])}
    check = logit_check() if (args.dtype == "bfloat16" and not args.no_check) else {}

    def serving_workload(tag, m):
        """The two serving workloads that go with the larger shapes, through the scheduler (output
        tokens a second over the whole run, prompts included in the time).  14B: 32 requests at
        once, prompts of 64 to 2,048 tokens taken in in portions under a budget of 2,048 tokens
        a step beside the decoding of the others, 256 new tokens each, up to 8,192 positions.
        32B: 64 requests of 512 prompt tokens and 512 new ones that join eight steps apart while
        the earlier ones are served, up to 16,384 positions, the cache sized from the memory that
        the weights leave.  Every request has to come back with its full length and the cache
        whole."""
        from tiny_llm_infer_amd.cli import _generate_arriving, make_benchmark_requests
        if tag == "14b":
            name, reqs = "mixed_32_requests", make_benchmark_requests(32, 64, 2048, 256, 256, 10000, m.spec.vocab_size, 7)
            e = LLMEngine.from_model(m, max_model_len=8192, page_size=page, max_num_seqs=32, max_num_batched_tokens=2048,
                                     num_kv_blocks=32 * ((2048 + 256 + page - 1) // page) + 8)
            run = lambda: e.generate([q for q, _ in reqs], [sp for _, sp in reqs])
        else:
            name, reqs = "continuous_64_requests", make_benchmark_requests(64, 512, 512, 512, 512, 10000, m.spec.vocab_size, 9)
            e = LLMEngine.from_model(m, max_model_len=16384, page_size=page, max_num_seqs=64, max_num_batched_tokens=2048,
                                     num_kv_blocks=0, gpu_memory_utilization=0.9)
            run = lambda: _generate_arriving(e, reqs, 8)
        torch.cuda.synchronize()
        t = time.perf_counter()
        results = run()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        assert [len(r.token_ids) for r in results] == [sp.max_tokens for _, sp in reqs], "a request came back short"
        e.runner.cache.check()
        assert e.runner.cache.free_pages() == e.runner.cache.pages_per_group() and e.is_finished()
        st = e.stats()
        out = sum(len(r.token_ids) for r in results)
        return {f"qwen3_{tag}_{name}_tok_s": round(out / dt, 1), f"qwen3_{tag}_{name}_steps": st["steps"],
                f"qwen3_{tag}_{name}_preemptions": st["preemptions"], f"qwen3_{tag}_{name}_cache_pages": st["pages"]}

    # the layer sizes of the larger models of the family: decode at batch 8 and the prefill of 2,048 tokens
    if not args.no_points and not args.no_other_shapes and not args.shape and not args.layers:
        del model, engine
        for tag in ("14b", "32b"):
            gc.collect()
            torch.cuda.empty_cache()
            with open(os.path.join(ROOT, "configs", f"qwen3_{tag}_shape.json")) as fh:
                conf = json.load(fh)
            m2, e2, _ = make_engine(conf, 8, args.prompt_len, 128, context=16384)
            n = min(args.steps, 32)
            d, _, f = decode_run(e2, conf, 8, n, 4, args.prompt_len)
            points[f"qwen3_{tag}_decode_b8"] = round(8 * n / d, 2)
            points[f"qwen3_{tag}_decode_b8_hbm_frac"] = round(f, 4)
            p_med, _, p_frac = prefill_run(e2, conf, T)
            points[f"qwen3_{tag}_prefill_{T}"] = round(T / p_med, 1)
            points[f"qwen3_{tag}_prefill_{T}_mfma_frac"] = round(p_frac, 4)
            del e2
            if not args.no_workloads:
                gc.collect()
                torch.cuda.empty_cache()
                points.update(serving_workload(tag, m2))
            del m2

    out = {
        "metric": f"decode tok/s @ batch {args.batch} ({shape_name}, {dkey}, random weights)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dkey, "data": "synthetic",
        "config": {"model": f"{shape_name}, random weights", "global_batch": args.batch,
                   "seq_len": args.context, "parallelism": "single GPU", "layers": layers,
                   "layers_of_config": full_layers, "hidden_size": cfg.hidden_size,
                   "intermediate_size": cfg.intermediate_size, "heads": cfg.num_attention_heads,
                   "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "vocab_size": cfg.vocab_size, "prompt_len": args.prompt_len,
                   "page_size": page, "prefill_tokens": T, "weights_gb_on_device": round(weight_gb, 2)},
        "prefill": {"value": round(T / pre, 1), "tokens": T, "ms": round(pre * 1e3, 3),
                    "frac": round(pre_frac, 4), "of": "median of 5",
                    "best_ms": round(pre_best * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 4)},
        "points": points,
        # bfloat16 logits of this very model against its true 32-bit path (untimed)
        "logit_check": check,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
