"""The command line, in the manner of the reference's ``model_main``
(model/model_main.cpp:465-604): ``--infer`` generates for the given prompts,
``--bench`` measures output tokens a second over synthetic requests.  Option
names and meanings are the reference's where it has them.  This engine has no
tokenizer: prompts are lists of token ids (``--prompt-ids 1,2,3``) and
completions are printed as token ids.

Exit codes as in the reference: 0 ok, 1 a failure while running, 2 usage.
"""
from __future__ import annotations

import argparse
import json
import random
import statistics
import sys
import time
from typing import List


def _common(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--model", help="model folder (config.json + safetensors) or a .safetensors file in it")
    ap.add_argument("--tokenizer", help="accepted for compatibility and ignored: the engine works on token ids")
    ap.add_argument("--device", default="cuda", help="cuda (the MI355X); there is no cpu path")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--max-seq-len", type=int, default=None)
    ap.add_argument("--num-kv-blocks", type=int, default=0, help="0: sized from free device memory")
    ap.add_argument("--gpu-memory-utilization", type=float, default=None)
    ap.add_argument("--quantization", default="none", help="only 'none' is supported")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-num-batched-tokens", type=int, default=None)
    ap.add_argument("--max-num-seqs", type=int, default=None)
    ap.add_argument("--enable-prefix-caching", action="store_true",
                    help="take over cached full pages of a known prompt prefix instead of computing them")
    ap.add_argument("--random-weights", action="store_true",
                    help="with --config: draw seeded random weights instead of reading a checkpoint")
    ap.add_argument("--config", help="a config.json, for --random-weights")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--kernels", default="tuned", choices=["tuned", "plain", "own-products", "library-products", "measured"],
                    help="tuned (= own-products): every matrix product by this library's kernels, each matrix held "
                         "once; library-products: products of more than 128 rows by the BLAS library (each matrix is "
                         "then held twice); measured: by whichever was timed faster for the shape when it first came "
                         "up; plain: the simple twins of the tuned kernels (bfloat16 too)")


def _device(name: str) -> str:
    if name in ("cuda", "hip", "gpu"):
        return "cuda:0"
    if name.startswith("cuda:"):
        return name
    raise SystemExit2(f"--device {name}: this engine runs on the GPU only (use cuda)")


class SystemExit2(Exception):
    pass


def _load(args, max_seq_len: int):
    from .engine.loading import load_model, random_model
    from .registry import architecture_of
    if args.quantization != "none":
        raise SystemExit2("--quantization: only 'none' is supported")
    device = _device(args.device)
    if args.random_weights:
        if not args.config:
            raise SystemExit2("--random-weights needs --config FILE")
        with open(args.config) as fh:
            data = json.load(fh)
        arch = architecture_of(data, args.config)
        cfg = arch.read_config(data, args.config)
        return random_model(arch.name, cfg, args.seed, args.dtype, device, max_seq_len, ops=_ops(device, args.kernels))
    if not args.model:
        raise SystemExit2("--model is required (or --config with --random-weights)")
    model, _ = load_model(args.model, args.dtype, device, max_seq_len, ops=_ops(device, args.kernels))
    return model


def run_inference(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="model_main --infer")
    _common(ap)
    ap.add_argument("--prompt", action="append", default=[], help="text prompts need a tokenizer: not supported")
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; repeatable")
    ap.add_argument("--max-new-tokens", type=int, default=64)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--sampling-seed", type=int, default=0)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--eos-id", type=int, action="append", default=None)
    args = ap.parse_args(argv)
    if args.prompt:
        raise SystemExit2("--prompt: this engine has no tokenizer; pass token ids with --prompt-ids")
    if not args.prompt_ids:
        raise SystemExit2("at least one --prompt-ids is required")
    try:
        prompts = [[int(t) for t in p.replace(" ", "").split(",") if t != ""] for p in args.prompt_ids]
    except ValueError:
        raise SystemExit2("--prompt-ids takes comma-separated integers") from None
    if any(not p for p in prompts):
        raise SystemExit2("every --prompt-ids needs at least one token id")
    if args.max_new_tokens < 0:
        raise SystemExit2("--max-new-tokens cannot be negative")
    max_seq_len = args.max_seq_len or 2048
    util = args.gpu_memory_utilization if args.gpu_memory_utilization is not None else 0.9
    if not 0.0 < util <= 0.95:
        raise SystemExit2("--gpu-memory-utilization must be in (0, 0.95]")
    from .engine.llm_engine import LLMEngine
    from .sampling.params import SamplingParams
    model = _load(args, max_seq_len)
    if args.max_new_tokens == 0:
        for _ in prompts:
            print()
        return 0
    # engine limits as the reference chooses them (model/model_main.cpp:403-408)
    engine = LLMEngine.from_model(
        model, max_model_len=max_seq_len, page_size=min(args.page_size, max_seq_len),
        num_kv_blocks=args.num_kv_blocks,
        max_num_seqs=args.max_num_seqs or min(16, len(prompts)),
        max_num_batched_tokens=args.max_num_batched_tokens or min(max_seq_len, 256),
        gpu_memory_utilization=util, enable_prefix_caching=args.enable_prefix_caching)
    if args.eos_id is not None:
        engine.eos_token_ids = set(args.eos_id)
    print(f"cache: {engine.runner.cache.num_pages} pages of {engine.runner.page_size} tokens, "
          f"{engine.runner.cache_bytes() >> 20} MiB", file=sys.stderr)
    sampling = SamplingParams(max_tokens=args.max_new_tokens, temperature=args.temperature,
                              top_p=args.top_p, ignore_eos=args.ignore_eos, seed=args.sampling_seed)
    results = engine.generate(prompts, sampling)
    if len(results) != len(prompts):
        print(f"{len(results)} results came back for {len(prompts)} prompts", file=sys.stderr)
        return 1
    for r in results:
        print(" ".join(str(t) for t in r.token_ids))
    return 0


def make_benchmark_requests(num_seqs, min_in, max_in, min_out, max_out, max_token_id, vocab, seed):
    """Seeded synthetic requests (model/model_main.cpp:150-175): uniform prompt
    lengths, uniform token ids in [0, min(max_token_id, vocab-1)], temperature
    0.6, EOS ignored, a seed per request."""
    from .sampling.params import SamplingParams
    rng = random.Random(seed)
    top = min(max_token_id, vocab - 1)
    reqs = []
    for i in range(num_seqs):
        n_in = rng.randint(min_in, max_in)
        n_out = rng.randint(min_out, max_out)
        prompt = [rng.randint(0, top) for _ in range(n_in)]
        reqs.append((prompt, SamplingParams(max_tokens=n_out, temperature=0.6, ignore_eos=True,
                                            seed=seed * 1000003 + i + 1)))
    return reqs


def _generate_arriving(engine, requests, interval: int):
    """Continuous batching: request i joins ``interval`` engine steps after request i-1
    (at once if the engine has run dry), while the earlier ones are being served."""
    import copy
    results, admitted, steps = [], 0, 0
    while admitted < len(requests) or not engine.is_finished():
        while admitted < len(requests) and (steps >= interval * admitted or engine.is_finished()):
            prompt, sampling = requests[admitted]
            engine.add_request(prompt, copy.copy(sampling))
            admitted += 1
        results.extend(engine.step())
        steps += 1
    results.sort(key=lambda r: r.request_id)
    return results


def run_benchmark(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="model_main --bench")
    _common(ap)
    ap.add_argument("--num-seqs", type=int, default=8)
    ap.add_argument("--min-input-len", type=int, default=64)
    ap.add_argument("--max-input-len", type=int, default=128)
    ap.add_argument("--min-output-len", type=int, default=32)
    ap.add_argument("--max-output-len", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--repeats", type=int, default=3)
    ap.add_argument("--max-token-id", type=int, default=10000)
    ap.add_argument("--manifest-prefix", default=None)
    ap.add_argument("--prefill-only", action="store_true",
                    help="one new token a request: measures prompt tokens a second")
    ap.add_argument("--arrival-interval", type=int, default=0,
                    help="engine steps between one request's arrival and the next (0: all are there at the start)")
    ap.add_argument("--kv-from-free-memory", action="store_true",
                    help="with --num-kv-blocks 0: as many pages as --gpu-memory-utilization leaves room for")
    args = ap.parse_args(argv)
    if args.prefill_only:
        args.min_output_len = args.max_output_len = 1
    max_seq_len = args.max_seq_len or 256
    if args.max_input_len + args.max_output_len > max_seq_len + 1:
        raise SystemExit2("max-input-len + max-output-len must be at most max-seq-len + 1")
    if args.min_input_len < 1 or args.min_input_len > args.max_input_len or \
            args.min_output_len < 1 or args.min_output_len > args.max_output_len:
        raise SystemExit2("input and output length ranges must be positive and ordered")
    util = args.gpu_memory_utilization if args.gpu_memory_utilization is not None else 0.7
    from .engine.llm_engine import LLMEngine
    model = _load(args, max_seq_len)
    page = min(args.page_size, max_seq_len)
    blocks = args.num_kv_blocks
    if blocks <= 0 and not args.kv_from_free_memory:
        # as the reference: enough for every request's longest possible sequence
        blocks = ((args.max_input_len + args.max_output_len + page - 1) // page) * args.num_seqs
    engine = LLMEngine.from_model(
        model, max_model_len=max_seq_len, page_size=page, num_kv_blocks=blocks,
        max_num_seqs=args.max_num_seqs or args.num_seqs,
        max_num_batched_tokens=args.max_num_batched_tokens or min(max_seq_len, 256),
        gpu_memory_utilization=util, enable_prefix_caching=args.enable_prefix_caching)
    vocab = model.spec.vocab_size
    import torch
    rates, total_tokens, total_time = [], 0, 0.0
    for run in range(args.warmup + args.repeats):
        warm = run < args.warmup
        seed = args.seed + (run + 1 if warm else 1000 + run - args.warmup)
        reqs = make_benchmark_requests(args.num_seqs, args.min_input_len, args.max_input_len,
                                       args.min_output_len, args.max_output_len,
                                       args.max_token_id, vocab, seed)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if args.arrival_interval > 0:
            results = _generate_arriving(engine, reqs, args.arrival_interval)
        else:
            results = engine.generate([p for p, _ in reqs], [s for _, s in reqs])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        out_tokens = sum(len(r.token_ids) for r in results)
        if args.prefill_only:
            out_tokens = sum(len(p) for p, _ in reqs)          # the tokens that were run
        if args.manifest_prefix and not warm:
            with open(f"{args.manifest_prefix}.run{run - args.warmup}.json", "w") as fh:
                json.dump({"seed": seed, "requests": [
                    {"prompt_token_ids": p, "max_tokens": s.max_tokens, "temperature": s.temperature,
                     "seed": s.seed, "output_token_ids": r.token_ids}
                    for (p, s), r in zip(reqs, results)]}, fh)
        if warm:
            continue
        rates.append(out_tokens / dt)
        total_tokens += out_tokens
        total_time += dt
        what = "prompt" if args.prefill_only else "output"
        print(f"run={run - args.warmup} {what}_tokens={out_tokens} elapsed_seconds={dt:.4f} "
              f"{what}_tokens_per_second={out_tokens / dt:.2f}")
    if rates:
        what = "prompt" if args.prefill_only else "output"
        print(f"aggregate_runs={args.repeats} {what}_tokens={total_tokens} elapsed_seconds={total_time:.4f} "
              f"{what}_tokens_per_second={total_tokens / total_time:.2f} "
              f"median_{what}_tokens_per_second={statistics.median(rates):.2f}")
    st = engine.stats()
    print(f"engine_steps={st['steps']} preemptions={st['preemptions']} "
          f"pages_free={min(st['pages_free'])}/{st['pages']} prefix_pages_reused={st['prefix_pages_reused']} "
          f"product_shapes_own_kernel={st['product_shapes_own_kernel']}/{st['product_shapes_measured']}",
          file=sys.stderr)
    return 0


REPLAY_HELP = """Trace replay: feed given token ids through a model step by step and write
the logits at the wanted places.  Nothing is sampled.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
    trace_run --config FILE --random-weights [--seed S] --dtype ... (weights drawn, no folder)

Steps are read from standard input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, OUT/<step>.f32 holds the logits at the
wanted places as little-endian float32 [wanted, vocab]; OUT/index.jsonl names, step by
step, the request and position of every row and the block tables the step ran with.
After every step a line "done <step>" is printed."""


def run_replay(argv: List[str], prog: str = "model_main --replay") -> int:
    """``bin/trace_run`` and ``model_main --replay``: the model, step function, cache and
    kernels that generation uses, driven by a trace instead of a scheduler."""
    ap = argparse.ArgumentParser(prog=prog, description=REPLAY_HELP,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--config", help="a config.json, with --random-weights, instead of --model")
    ap.add_argument("--random-weights", action="store_true",
                    help="draw the weights from --seed (the same ones a model folder written with that seed holds)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-live", type=int, default=4, help="most requests live at a time")
    ap.add_argument("--max-step-tokens", type=int, default=8192, help="most tokens in one step")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--kernels", default="own-products", choices=["own-products", "library-products", "measured", "plain"],
                    help="which kernel multiplies more than 128 rows: this library's (the default: the same "
                         "trace then gives the same bytes in every run), the BLAS library's, or 'measured': the "
                         "faster one for the shape, timed when the shape first comes up; "
                         "plain: the simple twins of all tuned kernels (bfloat16 too)")
    args = ap.parse_args(argv)
    if 64 % args.page_size:
        ap.error("--page-size must divide 64")
    if bool(args.model) == bool(args.random_weights):
        ap.error("give --model DIR, or --config FILE with --random-weights")
    print("[trace_run] loading the kernel library (compiled at the first call)", file=sys.stderr, flush=True)
    from .engine.replay import Replayer
    from .engine.runner import ModelRunner
    args.quantization = "none"
    model = _load(args, None)
    cfg = model.spec.architecture
    pages = max(1, (args.max_tokens + args.page_size - 1) // args.page_size)
    runner = ModelRunner(model, model.env, page_size=args.page_size, num_pages=pages,
                         max_requests=args.max_live, max_batch_tokens=args.max_step_tokens)
    print(f"[trace_run] ready: {cfg}, {args.dtype}, {pages} pages of {args.page_size}, "
          f"kernels: {args.kernels}", file=sys.stderr, flush=True)
    Replayer(runner, args.out).run_stream(sys.stdin, ack=sys.stdout)
    return 0


def _ops(device: str, which: str):
    """The kernel library set up as --kernels says, before any weight is loaded (which form of a
    matrix is kept depends on who multiplies with it).  plain: every product, attention and norm
    through the plain kernels; own-products / library-products / measured: products of more than
    128 rows through gemm_rows / the BLAS library / whichever was timed faster for the shape."""
    from .kernels.ops import HipOps
    ops = HipOps(device)
    if which == "plain":
        ops.many_rows = "library"            # the plain kernels read the row-major form
        ops.use_plain_kernels()
    elif which == "library-products":
        ops.many_rows = "library"
    elif which == "measured":
        ops.many_rows = "measure"
    else:                                    # "tuned", "own-products"
        ops.many_rows = "own"
    return ops


USAGE = """usage: model_main --infer [options] | --bench [options] | --replay [options]
  --infer   generate for --prompt-ids (repeatable) and print completion token ids
  --bench   measure output tokens a second over synthetic requests
  --replay  feed a trace of token ids from standard input, write logits (as bin/trace_run)
  add --help after the mode for its options"""


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    try:
        if "--infer" in argv:
            argv.remove("--infer")
            return run_inference(argv)
        if "--bench" in argv:
            argv.remove("--bench")
            return run_benchmark(argv)
        if "--replay" in argv:
            argv.remove("--replay")
            return run_replay(argv)
        print(USAGE, file=sys.stderr)
        return 2
    except SystemExit2 as exc:
        print(f"error: {exc}", file=sys.stderr)
        return 2
    except SystemExit as exc:            # argparse: --help is 0, bad usage is 2
        return int(exc.code or 0)
    except Exception as exc:             # a failure while running
        print(f"error: {exc}", file=sys.stderr)
        return 1
