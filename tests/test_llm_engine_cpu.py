"""The engine end to end on the CPU stand-in kernels: greedy generation equals
the plain implementation token for token, also when the pool is so small that
requests are preempted and computed again; temperature sampling does not
depend on the batch."""
import pytest

import plain_qwen3
from cpu_ops import CpuOps
from helpers import TINY, random_prompt
from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
from tiny_llm_infer_amd.sampling.params import SamplingParams


def _engine(folder, name, **kw):
    args = dict(dtype="float32", device="cpu", max_model_len=128, page_size=TINY[name]["page_size"],
                num_kv_blocks=64, max_num_seqs=4, max_num_batched_tokens=24, ops=CpuOps())
    args.update(kw)
    return LLMEngine.from_folder(folder, **args)


def test_greedy_generation_matches_plain(model_folders):
    """Small serving workload of configuration A: prompts of 5/17/33 tokens, 16
    greedy tokens each, page 8, budget 24."""
    folder = model_folders["A"]
    cfg, w = plain_qwen3.read_model(folder)
    prompts = [random_prompt(256, n, 40 + n) for n in (5, 17, 33)]
    want = [plain_qwen3.greedy(cfg, w, p, 16) for p in prompts]
    eng = _engine(folder, "A")
    got = eng.generate(prompts, SamplingParams(max_tokens=16, ignore_eos=True))
    assert [r.token_ids for r in got] == want
    assert eng.total_generated_tokens == 48
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == [64]
    # a pool too small for all three at once: preemption, same tokens
    small = _engine(folder, "A", num_kv_blocks=9)
    got = small.generate(prompts, SamplingParams(max_tokens=16, ignore_eos=True))
    assert [r.token_ids for r in got] == want
    assert small.scheduler.num_preemptions > 0 and sum(r.preemptions for r in got) > 0
    small.runner.cache.check()


def test_admission_checks(model_folders):
    eng = _engine(model_folders["A"], "A", max_model_len=32)
    with pytest.raises(ValueError, match="prompt is empty"):
        eng.add_request([], SamplingParams())
    with pytest.raises(ValueError, match="holds at most"):
        eng.add_request([1] * 33, SamplingParams(max_tokens=1))
    with pytest.raises(ValueError, match="do not fit max_model_len"):
        eng.add_request([1] * 30, SamplingParams(max_tokens=4))
    with pytest.raises(ValueError, match="at least one new token"):
        eng.add_request([1], SamplingParams(max_tokens=0))
    with pytest.raises(ValueError, match="top_p"):
        eng.add_request([1], SamplingParams(top_p=0.0))
    with pytest.raises(ValueError, match="vocabulary"):
        eng.add_request([256], SamplingParams(max_tokens=4))
    eng.add_request([1] * 30, SamplingParams(max_tokens=3))     # exactly fits: 30 + 3 - 1 = 32


def test_a_request_that_the_cache_can_never_hold_is_refused_when_it_is_added(model_folders):
    """4 pages of 8 tokens: a prompt of 27 tokens with 14 new ones would reach 40 tokens in the
    cache, be preempted for ever and take every other request down with it.  It is refused at
    once; what was added before it finishes as if nothing had happened."""
    folder = model_folders["A"]
    cfg, w = plain_qwen3.read_model(folder)
    eng = _engine(folder, "A", num_kv_blocks=4)
    first = random_prompt(256, 6, 3)
    eng.add_request(first, SamplingParams(max_tokens=14, ignore_eos=True))
    with pytest.raises(ValueError, match="need 5 cache pages of 8 tokens, the cache has 4"):
        eng.add_request(random_prompt(256, 27, 4), SamplingParams(max_tokens=14, ignore_eos=True))
    eng.add_request(random_prompt(256, 27, 4), SamplingParams(max_tokens=6, ignore_eos=True))      # 32 tokens: fits
    done = []
    while not eng.is_finished():
        done += eng.step()
    assert sorted(len(r.token_ids) for r in done) == [6, 14]
    assert [r.token_ids for r in done if len(r.token_ids) == 14] == [plain_qwen3.greedy(cfg, w, first, 14)]
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == [4]
    with pytest.raises(ValueError, match="cache pages"):
        eng.generate([first, random_prompt(256, 27, 4)], SamplingParams(max_tokens=14))            # checked before any is added
    assert eng.is_finished()


def test_eos_stops_a_request(model_folders):
    folder = model_folders["A"]
    cfg, w = plain_qwen3.read_model(folder)
    prompt = random_prompt(256, 12, 5)
    free_run = plain_qwen3.greedy(cfg, w, prompt, 8)
    eng = _engine(folder, "A")
    eng.eos_token_ids = {free_run[3]}
    cut = free_run.index(free_run[3]) + 1
    assert eng.generate([prompt], SamplingParams(max_tokens=8))[0].token_ids == free_run[:cut]
    assert eng.generate([prompt], SamplingParams(max_tokens=8, ignore_eos=True))[0].token_ids == free_run


def test_temperature_tokens_do_not_depend_on_the_batch(model_folders):
    """Configuration B's workload: temperature 0.7 with fixed seeds; a request
    gives the same tokens alone and among others (and under top_p)."""
    folder = model_folders["B"]
    prompts = [random_prompt(384, n, 70 + n) for n in (1, 9, 40, 23, 14)]
    params = [SamplingParams(max_tokens=12, temperature=0.7, ignore_eos=True, seed=100 + i,
                             top_p=1.0 if i % 2 else 0.9) for i in range(5)]
    eng = _engine(folder, "B", max_num_batched_tokens=32)
    together = eng.generate(prompts, params)
    alone = [_engine(folder, "B", max_num_batched_tokens=32).generate([p], [s])[0]
             for p, s in zip(prompts, params)]
    assert [r.token_ids for r in together] == [r.token_ids for r in alone]
    greedy = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    assert [r.token_ids for r in greedy] != [r.token_ids for r in together]


def test_counters(model_folders):
    eng = _engine(model_folders["A"], "A", num_kv_blocks=40, enable_prefix_caching=True)
    prompt = random_prompt(256, 20, 3)
    eng.generate([prompt, prompt[:17] + [1, 2]], SamplingParams(max_tokens=5))
    st = eng.stats()
    assert st["generated_tokens"] == 10 and st["steps"] >= 5
    assert st["waiting"] == 0 and st["running"] == 0 and st["preemptions"] == 0
    assert st["pages"] == 40 and st["pages_taken_total"] > 0
    eng.generate([prompt], SamplingParams(max_tokens=2))
    assert eng.stats()["prefix_pages_reused"] >= 2          # whole pages of the same prompt


def test_prefix_caching_gives_the_same_tokens_and_skips_work(model_folders):
    folder = model_folders["A"]
    shared = random_prompt(256, 40, 9)
    prompts = [shared + random_prompt(256, n, 20 + n) for n in (3, 9, 1)] + [shared[:33]]
    params = SamplingParams(max_tokens=6, ignore_eos=True)
    plain = _engine(folder, "A").generate(prompts, params)
    eng = _engine(folder, "A", enable_prefix_caching=True, max_num_seqs=1)    # one after the other
    got = eng.generate(prompts, params)
    assert [r.token_ids for r in got] == [r.token_ids for r in plain]
    assert eng.runner.cache.prefix_hits == 2 * 5 + 4      # 40 shared tokens = 5 pages of 8; the first request finds none
    eng.runner.cache.check()
    # and together, under preemption
    small = _engine(folder, "A", enable_prefix_caching=True, num_kv_blocks=14)
    got = small.generate(prompts, params)
    assert [r.token_ids for r in got] == [r.token_ids for r in plain]
    small.runner.cache.check()
    assert small.runner.cache.free_pages() == [14]


@pytest.mark.parametrize("budget", [64, 7])
def test_steps_put_on_the_device_ahead_change_nothing(model_folders, budget):
    """The next step is launched before this step's tokens are read; requests that
    stop on an end-of-sequence token or at max_tokens meanwhile, and sampling with a
    temperature, give exactly what the step-by-step engine gives.  With the small
    budget the steps ahead carry portions of prompts beside the decoding requests."""
    folder = model_folders["B"]
    prompts = [random_prompt(384, n, 50 + n) for n in (4, 30, 17, 9)]
    params = [SamplingParams(max_tokens=m, temperature=t, seed=7 + i)
              for i, (m, t) in enumerate([(9, 0.0), (14, 0.8), (3, 0.0), (11, 0.5)])]
    outs = []
    for ahead in (False, True):
        eng = _engine(folder, "B", max_num_batched_tokens=budget)
        eng.lookahead = ahead
        free = _engine(folder, "B", max_num_batched_tokens=budget).generate([prompts[0]], [SamplingParams(max_tokens=9)])
        eng.eos_token_ids = {free[0].token_ids[4]}            # request 0 stops early on this token
        mixed_ahead = 0
        for p, sp in zip(prompts, params):
            eng.add_request(p, sp)
        results = []
        while not eng.is_finished():
            results.extend(eng.step())
            nxt = eng._inflight
            if nxt is not None and any(i.prompt_portion for i in nxt.plan.items) \
                    and any(not i.prompt_portion for i in nxt.plan.items):
                mixed_ahead += 1
        results.sort(key=lambda r: r.request_id)
        outs.append(results)
        assert (eng.num_steps_ahead > 5) == ahead
        assert (mixed_ahead > 2) == (ahead and budget == 7)
        eng.runner.cache.check()
        assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group() and eng.is_finished()
    assert [r.token_ids for r in outs[0]] == [r.token_ids for r in outs[1]]
    assert len(outs[1][0].token_ids) <= 5 and len(outs[1][2].token_ids) <= 3


def test_requests_that_arrive_while_others_are_served(model_folders):
    """Continuous batching as the benchmark mode drives it: a request joins every
    few steps; each one's greedy tokens are those it gets alone."""
    from tiny_llm_infer_amd.cli import _generate_arriving
    folder = model_folders["B"]
    cfg, w = plain_qwen3.read_model(folder)
    prompts = [random_prompt(384, n, 70 + n) for n in (3, 21, 9, 30, 14)]
    want = [plain_qwen3.greedy(cfg, w, p, 10) for p in prompts]
    eng = _engine(folder, "B", max_num_seqs=3)
    params = SamplingParams(max_tokens=10, ignore_eos=True)
    for interval in (1, 4, 40):              # 40: the engine runs dry between arrivals
        got = _generate_arriving(eng, [(p, params) for p in prompts], interval)
        assert [r.token_ids for r in got] == want
        assert [r.prompt_token_ids for r in got] == prompts
        eng.runner.cache.check()


def test_step_ahead_counts_the_pages_of_the_whole_batch(model_folders):
    """Equal-length prompts cross a page border in the same step.  With a pool two pages
    short, the step planned ahead must see that its requests compete for the same free
    pages, take none, and leave the decision to the ordinary path (which preempts):
    the tokens are those of the engine without steps ahead, and no page is lost."""
    folder = model_folders["A"]
    cfg, w = plain_qwen3.read_model(folder)
    prompts = [random_prompt(256, 8, 90 + i) for i in range(3)]
    want = [plain_qwen3.greedy(cfg, w, p, 6) for p in prompts]
    outs = []
    for ahead in (False, True):
        eng = _engine(folder, "A", num_kv_blocks=5)
        eng.lookahead = ahead
        got = eng.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
        outs.append([r.token_ids for r in got])
        assert eng.scheduler.num_preemptions > 0
        eng.runner.cache.check()
        assert eng.runner.cache.free_pages() == [5] and eng.is_finished()
    assert outs[0] == outs[1] == want


def test_a_window_group_has_the_smaller_pool(model_folders):
    """Configuration B with room for 4 requests of 640 tokens: the windowed layers (window 40,
    pages of 16) get 4 * (3 + 2) + 2 pages, not 160, and long prompts pass through them
    portion by portion; the tokens are the plain greedy ones and nothing is preempted."""
    folder = model_folders["B"]
    eng = _engine(folder, "B", num_kv_blocks=160, max_model_len=640)
    cache = eng.runner.cache
    assert cache.pages_per_group() == [160, 22]
    assert [t["k"].shape[:2] for t in eng.runner.group_tensors] == [(1, 161), (2, 23)]
    prompts = [random_prompt(384, n, 11 * n) for n in (150, 3, 77, 240)]
    got = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    cfg, w = plain_qwen3.read_model(folder)
    assert [r.token_ids for r in got] == [plain_qwen3.greedy(cfg, w, p, 12) for p in prompts]
    assert eng.scheduler.num_preemptions == 0
    cache.check()
    assert cache.free_pages() == [160, 22]


def test_a_step_is_told_how_unequal_its_sequences_are(model_folders):
    """``StepView.skew``: the largest power of two (at most 16) that the longest sequence of a step
    has times the average length; rows that only fill a decode step up count as sequences of one
    token.  Launch rules may split the long sequences' work by it."""
    from tiny_llm_infer_amd.engine.runner import StepEntry
    eng = _engine(model_folders["A"], "A", max_model_len=128, num_kv_blocks=64, max_num_seqs=8, max_num_batched_tokens=128)
    runner = eng.runner
    lengths = {"long": 100, "a": 5, "b": 5, "c": 6}
    for key in lengths:
        runner.admit(key)
    view = runner._pack([StepEntry(k, [1] * n, []) for k, n in lengths.items()])
    assert view.max_seq_len == 100 and view.skew == 2                 # 100 against an average of 29
    for k, n in lengths.items():
        runner.cache.reserve(k, n)
        runner.cache.advance(k, n)
    view = runner._pack([StepEntry(k, [1], [0]) for k in lengths], pad_to=8)
    assert view.num_seqs == 8 and view.skew == 4                      # 101 against (101 + 6 + 6 + 7 + 4) / 8
    view = runner._pack([StepEntry(k, [1], [0]) for k in ("a", "b", "c")])
    assert view.skew == 1


@pytest.mark.parametrize("seed", range(10))
def test_random_serving_scenarios_give_plain_greedy_tokens(model_folders, seed):
    """A scenario drawn from the seed: one of the tiny configurations, a page size, up to eight requests of
    1 to 69 prompt tokens and 1 to 13 new ones, a pool between barely enough for the longest request and
    enough for all, a token budget from 2 to 256, a limit of live requests, steps planned ahead or not,
    prefix caching (with a shared prefix) where no layer has a window, requests that arrive while others
    are served, an end-of-sequence token that stops some of them early.  Every request gets the tokens of
    plain greedy generation, whatever was preempted and computed again on the way, and the cache is whole
    at the end."""
    import random
    rng = random.Random(1000 + seed)
    name = rng.choice(sorted(TINY))
    cfg, w = plain_qwen3.read_model(model_folders[name])
    vocab = TINY[name]["vocab_size"]
    page = rng.choice([4, 8, 16, 32]) if rng.random() < 0.5 else TINY[name]["page_size"]
    nreq = rng.randrange(1, 9)
    prompts = [random_prompt(vocab, rng.randrange(1, 70), rng.randrange(10 ** 6)) for _ in range(nreq)]
    outs = [rng.randrange(1, 14) for _ in range(nreq)]
    prefix = not TINY[name].get("use_sliding_window", False) and rng.random() < 0.5
    if prefix:
        head = random_prompt(vocab, rng.randrange(1, 40), 7)
        prompts = [head + p for p in prompts]
    need = (max(len(p) + o for p, o in zip(prompts, outs)) + page - 1) // page + 2
    pool = rng.choice([need, need + 1, need * 2, need * nreq + 4]) + rng.randrange(0, 4)
    eng = _engine(model_folders[name], name, max_model_len=256, page_size=page, num_kv_blocks=pool,
                  max_num_seqs=rng.randrange(1, nreq + 2), max_num_batched_tokens=rng.choice([2, 3, 8, 17, 64, 256]),
                  enable_prefix_caching=prefix)
    eng.lookahead = rng.random() < 0.6
    arrive = rng.choice([0, 0, 1, 3])
    want = [list(plain_qwen3.greedy(cfg, w, prompts[i], outs[i])) for i in range(nreq)]
    # in half of the scenarios a token that some request meets in the middle of its run ends a request:
    # requests then stop at times that no plan made ahead can know
    stops = rng.random() < 0.5 and max(outs) >= 3
    if stops:
        eos = rng.choice([run for run in want if len(run) >= 3])[rng.randrange(1, 3)]
        eng.eos_token_ids = {eos}
        want = [run[:run.index(eos) + 1] if eos in run else run for run in want]
    results, index_of, admitted, steps = {}, {}, 0, 0
    while admitted < nreq or not eng.is_finished():
        while admitted < nreq and (steps >= arrive * admitted or eng.is_finished()):
            index_of[eng.add_request(prompts[admitted], SamplingParams(max_tokens=outs[admitted], ignore_eos=not stops))] = admitted
            admitted += 1
        for r in eng.step():
            results[index_of[r.request_id]] = list(r.token_ids)
        steps += 1
        assert steps < 5000, "no progress"
    for i in range(nreq):
        assert results[i] == want[i], (name, i)
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()
