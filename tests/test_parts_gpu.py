"""Each part alone on the GPU against the plain implementation's function for
it, and a toy mixer with state of its own that is registered, built and
stepped from this test file without a change to the framework."""
import math

import pytest
import torch

import plain_qwen3 as P
from test_kernels_gpu import DEV, close, make_step, rnd

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def envs():
    from tiny_llm_infer_amd.engine.loading import make_env
    return {dt: make_env(dt, DEV, max_model_len=256) for dt in DTYPES}


def _weights(decls, dtype, seed=0):
    from tiny_llm_infer_amd.weights import random_tensors
    return {n: t.to(DEV) for n, t in random_tensors(decls, seed, dtype)}


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(envs, dtype):
    from tiny_llm_infer_amd.config import PartSpec
    from tiny_llm_infer_amd.parts import build_part
    part = build_part("norm", PartSpec("rmsnorm", {"size": 72, "eps": 2e-5}, {"weight": "n.w"}))
    w = _weights(part.tensors(), dtype)
    part.load(w, envs[dtype])
    resid = rnd((6, 72), torch.float32, 1, 2.0)
    delta = rnd((6, 72), dtype, 2)
    r = resid.to(DEV)
    out = part.forward(r, delta.to(DEV))
    total = resid.double() + delta.double()
    close(out, P.rmsnorm(total, w["n.w"].cpu().double(), 2e-5), dtype, "rmsnorm part")
    assert torch.allclose(r.cpu().double(), total, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_part_tables(envs, dtype):
    from tiny_llm_infer_amd.config import PartSpec
    from tiny_llm_infer_amd.parts import build_part
    part = build_part("position", PartSpec("rope_neox", {"head_dim": 48, "theta": 50000.0,
                                                          "max_positions": 200}))
    part.load({}, envs[dtype])
    cos, sin, rd, pairing = part.rotary()
    assert rd == 48 and cos.shape == (200, 24) and pairing == "half"
    ang = P.rope_angles(48, 50000.0, list(range(200)))
    assert torch.allclose(cos.cpu().double(), torch.cos(torch.from_numpy(ang).double()), atol=1e-7)
    assert torch.allclose(sin.cpu().double(), torch.sin(torch.from_numpy(ang).double()), atol=1e-7)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tied", [True, False])
def test_embedding_and_head_parts(envs, dtype, tied):
    """Rows of the table become the float32 residual; the head gives float32 logits
    from its own matrix, or from the embedding's when the model ties them."""
    from tiny_llm_infer_amd.config import PartSpec
    from tiny_llm_infer_amd.parts import build_part
    vocab, hidden = 301, 80
    emb = build_part("embedding", PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": hidden},
                                           {"weight": "emb"}))
    head = build_part("head", PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": hidden, "tied": tied},
                                       {"weight": "emb" if tied else "head"}))
    decls = emb.tensors() + ([] if tied else head.tensors())
    w = _weights(decls, dtype, seed=8)
    emb.load(w, envs[dtype])
    head.load(w, envs[dtype], share_with=emb if tied else None)
    ids = torch.tensor([300, 0, 17, 17, 42], dtype=torch.int32)
    resid = emb.forward(ids.to(DEV), 5)
    assert resid.dtype == torch.float32
    assert torch.equal(resid.cpu(), w["emb"].cpu().float()[ids.long()])
    x = rnd((3, hidden), dtype, 9)
    logits = head.forward(x.to(DEV))
    assert logits.dtype == torch.float32 and tuple(logits.shape) == (3, vocab)
    matrix = w["emb" if tied else "head"].cpu().double()
    close(logits, P.linear(x.double(), matrix), torch.float32 if dtype == torch.float32 else dtype, "head")
    if tied and dtype == torch.float32:
        assert head.weight.w.data_ptr() == emb.table.data_ptr()       # one copy of the matrix
    elif tied:                      # the row-major matrix once (rows are gathered from it), its decode layout once
        assert head.weight._w is None and head.weight.tiled is not None and torch.equal(head.weight.w, emb.table)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part(envs, dtype):
    from tiny_llm_infer_amd.config import PartSpec
    from tiny_llm_infer_amd.parts import build_part
    part = build_part("ffn", PartSpec("swiglu", {"hidden_size": 80, "intermediate_size": 112},
                                      {"gate": "g", "up": "u", "down": "d"}))
    w = _weights(part.tensors(), dtype)
    part.load(w, envs[dtype])
    x = rnd((9, 80), dtype, 3)
    f = {k: v.cpu().double() for k, v in w.items()}
    want = P.linear(P.swiglu(P.linear(x.double(), f["g"]), P.linear(x.double(), f["u"])), f["d"])
    close(envs[dtype].ops.resolve(part.forward(x.to(DEV), None)), want, dtype, "swiglu part")


def _attention_spec(heads, kv, hd, hidden, window, theta=1e4, eps=1e-6):
    from tiny_llm_infer_amd.config import PartSpec
    norm = lambda n: PartSpec("rmsnorm", {"size": hd, "eps": eps}, {"weight": n})
    return PartSpec("paged_attention",
                    {"hidden_size": hidden, "num_heads": heads, "num_kv_heads": kv, "head_dim": hd,
                     "scale": hd ** -0.5, "window": window},
                    {"q": "q", "k": "k", "v": "v", "o": "o"},
                    {"position": PartSpec("rope_neox", {"head_dim": hd, "theta": theta, "max_positions": 256}),
                     "q_norm": norm("qn"), "k_norm": norm("kn")})


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 7])
def test_attention_part_whole_sequence(envs, dtype, window):
    """One whole sequence through the attention part in one step equals the
    plain attention block."""
    from tiny_llm_infer_amd.parts import build_part
    heads, kv, hd, hidden, T = 6, 2, 32, 80, 45
    part = build_part("mixer", _attention_spec(heads, kv, hd, hidden, window))
    w = _weights(part.tensors(), dtype, seed=4)
    part.load(w, envs[dtype])
    assert part.cache_need().window == window
    step, tables, pos, seq = make_step([T], [T], 16, 5, 0, kv, hd, dtype, window)
    x = rnd((T, hidden), dtype, 5)
    out = envs[dtype].ops.resolve(part.forward(x.to(DEV), step))     # (it may come as unadded partial sums)
    f = {("self." + k + ("_proj.weight" if k in "qkvo" else "")): v.cpu().double() for k, v in w.items()}
    f["self.q_norm.weight"], f["self.k_norm.weight"] = f.pop("self.qn"), f.pop("self.kn")
    cfg = dict(num_attention_heads=heads, num_key_value_heads=kv, head_dim=hd, hidden_size=hidden,
               rms_norm_eps=1e-6, rope_theta=1e4)
    want = P.attention_block(x.double(), f, "self.", cfg, list(range(T)), window)
    close(out, want, dtype, "attention part")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd,rd", [(32, 32), (64, 64), (64, 24), (128, 128)])
def test_attention_part_with_a_rotation_of_neighbours(envs, dtype, hd, rd):
    """A position encoding defined here that turns the pairs (2i, 2i + 1), over the whole head
    or the first ``rd`` elements: a whole sequence and then single tokens through the stock
    attention part (heads of 64 and 128: the kernels that take the raw projections) against
    float64 mathematics written out here."""
    from tiny_llm_infer_amd.config import PartSpec
    from tiny_llm_infer_amd.parts import PositionEncoding, build_part, register_part
    from tiny_llm_infer_amd.parts.base import RotaryTables
    heads, kv, hidden, T, more, theta = 4, 2, 80, 37, 5, 300.0
    half = rd // 2
    angles = torch.arange(256, dtype=torch.float64)[:, None] * theta ** (-2.0 * torch.arange(half, dtype=torch.float64) / rd)[None, :]

    class Neighbours(PositionEncoding):
        def load(self, weights, env):
            super().load(weights, env)
            self.cos, self.sin = torch.cos(angles).float().to(env.device), torch.sin(angles).float().to(env.device)

        def rotary(self):
            return RotaryTables(self.cos, self.sin, rd, "interleaved")

    register_part("position", "toy_neighbours", Neighbours, replace=True)
    base = _attention_spec(heads, kv, hd, hidden, None)
    spec = PartSpec(base.kind, base.params, base.names, dict(base.parts, position=PartSpec("toy_neighbours")))
    part = build_part("mixer", spec)
    w = _weights(part.tensors(), dtype, seed=14)
    part.load(w, envs[dtype])
    total = T + more
    step, tables, pos, seq = make_step([T], [T], 8, 8, 0, kv, hd, dtype)
    x = rnd((total, hidden), dtype, 15)
    ops = envs[dtype].ops
    outs = [ops.resolve(part.forward(x[:T].to(DEV), step))]
    for t in range(T, total):                      # the same pages, one token more at a time
        step2, tables2, _, _ = make_step([t + 1], [1], 8, 8, 0, kv, hd, dtype)
        step2.cache.group.tensors["k"].copy_(step.cache.group.tensors["k"])
        step2.cache.group.tensors["v"].copy_(step.cache.group.tensors["v"])
        assert (tables2[0, :(t + 7) // 8] == tables[0, :(t + 7) // 8]).all()       # (the same pages in the same order)
        outs.append(ops.resolve(part.forward(x[t:t + 1].to(DEV), step2)))
        step = step2
        tables = tables2
    got = torch.cat(outs)
    # float64
    f = {k: v.cpu().double() for k, v in w.items()}
    xd = x.double()
    q = (xd @ f["q"].t()).reshape(total, heads, hd)
    k = (xd @ f["k"].t()).reshape(total, kv, hd)
    v = (xd @ f["v"].t()).reshape(total, kv, hd)
    q, k = P.rmsnorm(q, f["qn"], 1e-6), P.rmsnorm(k, f["kn"], 1e-6)
    c, s_ = torch.cos(angles[:total])[:, None, :], torch.sin(angles[:total])[:, None, :]

    def turn(t):
        out = t.clone()
        a, b = t[..., 0:rd:2], t[..., 1:rd:2]
        out[..., 0:rd:2] = a * c - b * s_
        out[..., 1:rd:2] = a * s_ + b * c
        return out
    o = P.causal_attention(turn(q), turn(k), v, hd ** -0.5)
    want = o.reshape(total, heads * hd) @ f["o"].t()
    close(got, want, dtype, f"attention with neighbours paired, head {hd}, rotary {rd}")


def test_attention_part_refuses_what_its_kernels_do_not_do(envs):
    """An inner norm of another kind than the RMS norm, and a pairing of rotated elements that
    is not known, are refused when the part takes its weights, with a message; they are never
    computed as something else."""
    from tiny_llm_infer_amd.config import PartSpec
    from tiny_llm_infer_amd.parts import Norm, PositionEncoding, build_part, register_part
    from tiny_llm_infer_amd.parts.base import RotaryTables
    from tiny_llm_infer_amd.weights import TensorDecl

    class MeanFree(Norm):
        def tensors(self):
            return [TensorDecl(self.spec.names["weight"], (self.spec.params["size"],), "ones_normal")]

        def load(self, weights, env):
            super().load(weights, env)
            self.weight, self.eps = weights[self.spec.names["weight"]].float(), 1e-6     # (what an RMS norm holds too)

        def forward(self, resid, delta, rows=None, num_rows=None):
            raise AssertionError("not run here")

    class Crossed(PositionEncoding):
        def rotary(self):
            z = torch.zeros(256, 16, device=DEV)
            return RotaryTables(z, z, 32, "crossed")

    register_part("norm", "toy_mean_free", MeanFree, replace=True)
    register_part("position", "toy_crossed", Crossed, replace=True)
    base = _attention_spec(4, 2, 32, 80, None)
    env = envs[torch.bfloat16]
    bad_norm = PartSpec(base.kind, base.params, base.names,
                        dict(base.parts, k_norm=PartSpec("toy_mean_free", {"size": 32}, {"weight": "kn"})))
    part = build_part("mixer", bad_norm)
    with pytest.raises(ValueError, match="k norm of an attention layer is 'toy_mean_free'"):
        part.load(_weights(part.tensors(), torch.bfloat16), env)
    part = build_part("mixer", PartSpec(base.kind, base.params, base.names, dict(base.parts, position=PartSpec("toy_crossed"))))
    with pytest.raises(ValueError, match="pairing 'crossed' is not known"):
        part.load(_weights(part.tensors(), torch.bfloat16), env)
    # and the kernel library itself turns halves only
    from tiny_llm_infer_amd.kernels.ops import KernelError
    step, *_ = make_step([5], [5], 8, 2, 0, 2, 32, torch.bfloat16)
    z = torch.zeros(256, 16, device=DEV)
    with pytest.raises(KernelError, match="not the pairing 'interleaved'"):
        env.ops.qkv_attention(rnd((5, 8 * 32), torch.bfloat16, 1).to(DEV), step, step.cache, 4, 2, 32, None, None,
                              (z, z, 32, "interleaved"), 1.0, None)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prenorm_block(envs, dtype):
    from tiny_llm_infer_amd.config import PartSpec
    from tiny_llm_infer_amd.parts import build_part
    heads, kv, hd, hidden, inter, T = 4, 4, 16, 48, 64, 20
    mixer = build_part("mixer", _attention_spec(heads, kv, hd, hidden, None))
    ffn = build_part("ffn", PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter},
                                     {"gate": "g", "up": "u", "down": "d"}))
    norms = {"mixer": build_part("norm", PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6}, {"weight": "n1"})),
             "ffn": build_part("norm", PartSpec("rmsnorm", {"size": hidden, "eps": 1e-6}, {"weight": "n2"}))}
    block = build_part("block", PartSpec("prenorm"), mixer, ffn, norms)
    w = _weights(block.tensors(), dtype, seed=6)
    block.load(w, envs[dtype])
    step, *_ = make_step([T], [T], 8, 4, 0, kv, hd, dtype)
    h0 = rnd((T, hidden), torch.float32, 7)
    resid = h0.to(DEV)
    pending = block.forward(resid, None, step)
    f = {k: v.cpu().double() for k, v in w.items()}
    att = {"s.q_proj.weight": f["q"], "s.k_proj.weight": f["k"], "s.v_proj.weight": f["v"],
           "s.o_proj.weight": f["o"], "s.q_norm.weight": f["qn"], "s.k_norm.weight": f["kn"]}
    cfg = dict(num_attention_heads=heads, num_key_value_heads=kv, head_dim=hd, hidden_size=hidden,
               rms_norm_eps=1e-6, rope_theta=1e4)
    h = h0.double()
    r = h + P.attention_block(P.rmsnorm(h, f["n1"], 1e-6), att, "s.", cfg, list(range(T)), None)
    m = P.rmsnorm(r, f["n2"], 1e-6)
    d = P.linear(P.swiglu(P.linear(m, f["g"]), P.linear(m, f["u"])), f["d"])
    close(resid, r, dtype, "residual after the mixer")     # the second sum is still owed
    close(envs[dtype].ops.resolve(pending), d, dtype, "what the block owes the residual")


# ------------------------------------------------------------------ toy mixer --
def test_toy_mixer_with_state_of_its_own(tmp_path):
    """A mixer defined here, keeping a running sum per request in a state slot:
    y_t = W . mean(x_0..x_t).  It is registered, built into a model of a toy
    architecture and stepped in several cuts through the framework's runner,
    cache manager and replay, none of which is changed for it.  The last block of the toy
    has no feed-forward: norm, mixer, sum."""
    import json

    import numpy as np

    from helpers import collect, trace_mixed, trace_portions, trace_whole
    from tiny_llm_infer_amd import register_architecture
    from tiny_llm_infer_amd.cache import StateNeed
    from tiny_llm_infer_amd.config import BlockSpec, JsonReader, LayerCall, ModelSpec, PartSpec
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.replay import Replayer
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    from tiny_llm_infer_amd.parts import Mixer, register_part
    from tiny_llm_infer_amd.weights import TensorDecl

    class RunningMean(Mixer):
        def __init__(self, spec):
            super().__init__(spec)
            self.n = spec.params["size"]

        def tensors(self):
            return [TensorDecl(self.spec.names["w"], (self.n, self.n))]

        def load(self, weights, env):
            super().load(weights, env)
            self.w = weights[self.spec.names["w"]].float()

        def state_need(self):
            return StateNeed((self.n,), torch.float32)

        def forward(self, x, step):
            out = torch.empty_like(x)
            for i in range(step.num_seqs):
                r0, r1 = step.h_row_start[i], step.h_row_start[i + 1]
                slot, start = step.h_slots[i], step.h_seq_start[i]
                if start == 0:
                    step.state[slot].zero_()          # a slot may have served another request
                cum = step.state[slot] + torch.cumsum(x[r0:r1].float(), 0)
                step.state[slot] = cum[-1]
                count = torch.arange(start + 1, start + 1 + (r1 - r0), device=x.device)[:, None]
                out[r0:r1] = ((cum / count) @ self.w.t()).to(x.dtype)
            return out

    register_part("mixer", "running_mean", RunningMean, replace=True)

    class ToyConfig:
        def __init__(self, d):
            r = JsonReader(d)
            self.size, self.inter = r.integer("size"), r.integer("inter")
            self.layers, self.vocab = r.integer("layers"), r.integer("vocab")
            self.d = d

        def to_dict(self):
            return self.d

    def toy_spec(c):
        rms = lambda n: PartSpec("rmsnorm", {"size": c.size, "eps": 1e-6}, {"weight": n})
        blocks = tuple(BlockSpec(
            "prenorm", PartSpec("running_mean", {"size": c.size}, {"w": f"l{i}.mix"}),
            PartSpec("swiglu", {"hidden_size": c.size, "intermediate_size": c.inter},
                     {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
            {"mixer": rms(f"l{i}.n1"), "ffn": rms(f"l{i}.n2")}) for i in range(c.layers - 1))
        last = c.layers - 1
        blocks += (BlockSpec("prenorm", PartSpec("running_mean", {"size": c.size}, {"w": f"l{last}.mix"}), None,
                             {"mixer": rms(f"l{last}.n1")}),)
        return ModelSpec("ToyStateLM", c.size, c.vocab, 4096,
                         PartSpec("token_embedding", {"vocab_size": c.vocab, "hidden_size": c.size}, {"weight": "emb"}),
                         blocks, tuple(LayerCall(i) for i in range(c.layers)), rms("norm"),
                         PartSpec("linear_head", {"vocab_size": c.vocab, "hidden_size": c.size, "tied": True},
                                  {"weight": "emb"}))

    register_architecture("ToyStateLM", lambda d, origin: ToyConfig(d), toy_spec, replace=True)
    cfg = {"architectures": ["ToyStateLM"], "size": 40, "inter": 56, "layers": 3, "vocab": 97}
    folder = write_random_model(str(tmp_path / "toy"), "ToyStateLM", ToyConfig(cfg), seed=3)

    # the plain version of the toy, whole sequences
    w = {k: v for k, v in P.read_safetensors(str(tmp_path / "toy" / "model.safetensors")).items()}

    def plain(ids):
        h = w["emb"][torch.tensor(ids)]
        for i in range(3):
            n = P.rmsnorm(h, w[f"l{i}.n1"], 1e-6)
            mean = torch.cumsum(n, 0) / torch.arange(1, len(ids) + 1, dtype=torch.float64)[:, None]
            r = h + mean @ w[f"l{i}.mix"].t()
            if i == 2:
                h = r                  # the block without a feed-forward
                break
            m = P.rmsnorm(r, w[f"l{i}.n2"], 1e-6)
            h = r + P.linear(P.swiglu(P.linear(m, w[f"l{i}.g"]), P.linear(m, w[f"l{i}.u"])), w[f"l{i}.d"])
        return P.linear(P.rmsnorm(h, w["norm"], 1e-6), w["emb"]).numpy()

    rng = np.random.default_rng(0)
    reqs = {f"t{i}": rng.integers(0, 97, n).tolist() for i, n in enumerate([30, 51, 9, 44, 27])}
    want = {k: plain(v) for k, v in reqs.items()}
    model, _ = load_model(folder, "float32", DEV)
    assert model.cache_needs() == [] and all(s is not None for s in model.state_needs())
    for steps in (trace_whole(reqs), trace_portions(reqs, 2), trace_mixed(reqs, 256, seed=5)):
        runner = ModelRunner(model, model.env, page_size=16, num_pages=16, max_requests=4,
                             max_batch_tokens=256)
        rp = Replayer(runner)
        got = collect(steps, {s["step"]: rp.run_step(s) for s in steps})
        for k in reqs:
            assert np.abs(got[k] - want[k]).max() <= 2e-5 * max(1.0, np.abs(want[k]).max())
        assert runner.cache.free_slots() == 4


# ------------------------------------------------- toy routing, toy rotation ---
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_another_rotation(tmp_path, dtype):
    """Defined here and registered without a change to the framework: a feed-forward
    that routes every row to experts, and a rotary encoding with its own angles
    (positions scaled, only a part of the head rotated).  The toy architecture puts them
    beside the framework's attention and SwiGLU, chooses parts layer by layer, runs block
    0 twice (each run with a cache layer of its own) and lets the second run of block 1
    read the keys and values that its first run wrote.  All cuts against a plain version
    written here."""
    import numpy as np

    from helpers import collect, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
    from tiny_llm_infer_amd import register_architecture
    from tiny_llm_infer_amd.config import BlockSpec, JsonReader, LayerCall, ModelSpec, PartSpec
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.replay import Replayer
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    from tiny_llm_infer_amd.parts import FeedForward, PositionEncoding, register_part
    from tiny_llm_infer_amd.weights import TensorDecl

    def toy_angles(rd, base, scale, n):
        i = np.arange(rd // 2, dtype=np.float64)
        return (np.arange(n, dtype=np.float64) * scale)[:, None] * (base ** (-i / (rd // 2)))[None, :]

    class ScaledRotation(PositionEncoding):
        """angle[p, i] = scale * p * base^(-i / (rd/2)); pairs (i, i + rd/2) of the first rd dims."""
        def load(self, weights, env):
            super().load(weights, env)
            p = self.spec.params
            a = toy_angles(p["rotary_dim"], p["base"], p["scale"], min(p["max_positions"], env.max_model_len))
            self.cos = torch.from_numpy(np.cos(a).astype(np.float32)).to(env.device)
            self.sin = torch.from_numpy(np.sin(a).astype(np.float32)).to(env.device)

        def rotary(self):
            return self.cos, self.sin, self.spec.params["rotary_dim"]

    class RoutedExperts(FeedForward):
        """Router logits x Wr^T and their softmax in float32; the top_k experts of a row, each
        W2_e silu(W1_e x), weighted by their probabilities (not renormalised)."""
        def __init__(self, spec):
            super().__init__(spec)
            p = spec.params
            self.n, self.inter, self.experts, self.top_k = p["size"], p["inter"], p["experts"], p["top_k"]

        def tensors(self):
            nm = self.spec.names
            out = [TensorDecl(nm["router"], (self.experts, self.n))]
            for e in range(self.experts):
                out += [TensorDecl(f"{nm['experts']}.{e}.w1", (self.inter, self.n)),
                        TensorDecl(f"{nm['experts']}.{e}.w2", (self.n, self.inter))]
            return out

        def load(self, weights, env):
            super().load(weights, env)
            nm = self.spec.names
            self.router = weights[nm["router"]].float()
            self.w1 = [weights[f"{nm['experts']}.{e}.w1"].to(env.dtype).contiguous() for e in range(self.experts)]
            self.w2 = [weights[f"{nm['experts']}.{e}.w2"].to(env.dtype).contiguous() for e in range(self.experts)]

        def forward(self, x, step):
            ops = self.env.ops
            prob = torch.softmax(x.float() @ self.router.t(), dim=-1)
            top = torch.topk(prob, self.top_k, dim=-1).indices
            out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
            for e in range(self.experts):
                rows = (top == e).any(dim=-1).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                h = ops.linear(x[rows].contiguous(), self.w1[e]).float()           # the framework's products
                y = ops.linear((h * torch.sigmoid(h)).to(x.dtype), self.w2[e]).float()
                out[rows] += prob[rows, e:e + 1] * y
            return out.to(x.dtype)

    register_part("position", "toy_scaled_rotation", ScaledRotation, replace=True)
    register_part("ffn", "toy_routed_experts", RoutedExperts, replace=True)

    size, heads, kv, hd, inter, vocab, experts = 128, 4, 2, 64, 96, 211, 3
    top_k = 1 if dtype == "float32" else experts          # in bfloat16 a near tie of the router could go either way
    rot = [dict(rotary_dim=64, base=500.0, scale=0.5), dict(rotary_dim=32, base=10000.0, scale=1.0)]
    windows = [None, 21]

    class ToyConfig:
        def __init__(self, d):
            JsonReader(d).integer("top_k")
            self.d = d

        def to_dict(self):
            return self.d

    def toy_spec(c):
        rms = lambda n, name: PartSpec("rmsnorm", {"size": n, "eps": 1e-5}, {"weight": name})

        def attention(i):
            return PartSpec("paged_attention",
                            {"hidden_size": size, "num_heads": heads, "num_kv_heads": kv, "head_dim": hd,
                             "scale": hd ** -0.5, "window": windows[i]},
                            {k: f"l{i}.{k}" for k in "qkvo"},
                            {"position": PartSpec("toy_scaled_rotation", dict(rot[i], max_positions=512)),
                             "q_norm": rms(hd, f"l{i}.qn"), "k_norm": rms(hd, f"l{i}.kn")})
        ffn0 = PartSpec("toy_routed_experts", {"size": size, "inter": inter, "experts": experts,
                                               "top_k": c.d["top_k"]}, {"router": "l0.router", "experts": "l0.expert"})
        ffn1 = PartSpec("swiglu", {"hidden_size": size, "intermediate_size": inter},
                        {"gate": "l1.g", "up": "l1.u", "down": "l1.d"})
        blocks = tuple(BlockSpec("prenorm", attention(i), ffn, {"mixer": rms(size, f"l{i}.n1"), "ffn": rms(size, f"l{i}.n2")})
                       for i, ffn in enumerate((ffn0, ffn1)))
        # block 0 with cache layer 0, block 1 with cache layer 1, block 0 again with cache layer 2,
        # block 1 again reading cache layer 1
        schedule = (LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(1, 1, False))
        return ModelSpec("ToyMixLM", size, vocab, 512,
                         PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": size}, {"weight": "emb"}),
                         blocks, schedule, rms(size, "norm"),
                         PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": size, "tied": False},
                                  {"weight": "head"}))

    register_architecture("ToyMixLM", lambda d, origin: ToyConfig(d), toy_spec, replace=True)
    cfg = {"architectures": ["ToyMixLM"], "top_k": top_k}
    folder = write_random_model(str(tmp_path / "toymix"), "ToyMixLM", ToyConfig(cfg), seed=9)
    w = {k: v for k, v in P.read_safetensors(str(tmp_path / "toymix" / "model.safetensors")).items()}

    # ---- the plain version, whole sequences, float64
    def rotate(x, i, T):
        rd = rot[i]["rotary_dim"]
        a = torch.from_numpy(toy_angles(rd, rot[i]["base"], rot[i]["scale"], T))
        cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
        first, second, rest = x[..., :rd // 2], x[..., rd // 2:rd], x[..., rd:]
        return torch.cat([first * cos - second * sin, first * sin + second * cos, rest], -1)

    def plain(ids):
        T = len(ids)
        h = w["emb"][torch.tensor(ids)]
        kept = {}
        for call, (i, reads_old) in enumerate(((0, False), (1, False), (0, False), (1, True))):
            n = P.rmsnorm(h, w[f"l{i}.n1"], 1e-5)
            q = P.rmsnorm(P.linear(n, w[f"l{i}.q"]).reshape(T, heads, hd), w[f"l{i}.qn"], 1e-5)
            q = rotate(q, i, T)
            if reads_old:
                k, v = kept[i]
            else:
                k = rotate(P.rmsnorm(P.linear(n, w[f"l{i}.k"]).reshape(T, kv, hd), w[f"l{i}.kn"], 1e-5), i, T)
                v = P.linear(n, w[f"l{i}.v"]).reshape(T, kv, hd)
                kept[i] = (k, v)
            o = P.causal_attention(q, k, v, hd ** -0.5, windows[i])
            r = h + P.linear(o.reshape(T, heads * hd), w[f"l{i}.o"])
            m = P.rmsnorm(r, w[f"l{i}.n2"], 1e-5)
            if i == 0:
                prob = torch.softmax(m @ w["l0.router"].t(), -1)
                top = torch.topk(prob, top_k, -1).indices
                y = torch.zeros_like(m)
                for e in range(experts):
                    a = P.linear(m, w[f"l0.expert.{e}.w1"])
                    ye = P.linear(a / (1 + torch.exp(-a)), w[f"l0.expert.{e}.w2"])
                    y += torch.where((top == e).any(-1, keepdim=True), prob[:, e:e + 1] * ye, torch.zeros_like(ye))
                h = r + y
            else:
                h = r + P.linear(P.swiglu(P.linear(m, w["l1.g"]), P.linear(m, w["l1.u"])), w["l1.d"])
        return P.linear(P.rmsnorm(h, w["norm"], 1e-5), w["head"]).numpy()

    rng = np.random.default_rng(4)
    reqs = {f"m{i}": rng.integers(0, vocab, n).tolist() for i, n in enumerate([37, 58, 12, 45])}
    want = {k: plain(v) for k, v in reqs.items()}
    model, _ = load_model(folder, dtype, DEV)
    assert len(model.cache_needs()) == 3                      # three cache layers for four runs of two blocks
    bound = 2e-5 if dtype == "float32" else 4e-2
    for steps in (trace_whole(reqs), trace_prefill_then_decode(reqs), trace_portions(reqs, 7),
                  trace_mixed(reqs, 192, seed=8)):
        runner = ModelRunner(model, model.env, page_size=8, num_pages=24, max_requests=4, max_batch_tokens=256)
        rp = Replayer(runner)
        got = collect(steps, {s["step"]: rp.run_step(s) for s in steps})
        for k in reqs:
            assert np.abs(got[k] - want[k]).max() <= bound * max(1.0, np.abs(want[k]).max()), (dtype, k)
        runner.cache.check()


# ------------------------------- a toy norm, and a toy mixer with a cache record of its own ---
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_and_a_mixer_that_caches_one_vector_per_token(tmp_path, dtype):
    """Defined here and registered without a change to the framework: a LayerNorm (weight and
    bias, the plain four-argument interface) that stands before the framework's attention and
    SwiGLU, also in bfloat16 where the stock norm hands those parts rows with a factor still
    owed; and a mixer that keeps one float32 vector per token in pages of its own (a record it
    declares itself, with a window, so that its pages are given back as the window passes) and
    answers with the mean of the vectors its window holds.  All cuts against a plain version
    written here, with so few pages that they are used again."""
    import numpy as np

    from helpers import collect, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
    from tiny_llm_infer_amd import register_architecture
    from tiny_llm_infer_amd.cache import PAGE, CacheNeed, CacheRecord
    from tiny_llm_infer_amd.config import BlockSpec, LayerCall, ModelSpec, PartSpec
    from tiny_llm_infer_amd.engine.loading import load_model, write_random_model
    from tiny_llm_infer_amd.engine.replay import Replayer
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    from tiny_llm_infer_amd.engine.sizing import page_bytes, workspace_bytes
    from tiny_llm_infer_amd.parts import Mixer, Norm, register_part
    from tiny_llm_infer_amd.weights import TensorDecl

    size, latent, window, heads, kv, hd, inter, vocab, eps = 128, 24, 13, 4, 2, 64, 96, 157, 1e-5

    class ToyLayerNorm(Norm):
        def tensors(self):
            n = self.spec.params["size"]
            return [TensorDecl(self.spec.names["weight"], (n,), "ones_normal"), TensorDecl(self.spec.names["bias"], (n,))]

        def load(self, weights, env):
            super().load(weights, env)
            self.w, self.b = weights[self.spec.names["weight"]].float(), weights[self.spec.names["bias"]].float()

        def forward(self, resid, delta, rows=None, num_rows=None):
            assert delta is None or isinstance(delta, torch.Tensor)       # never an unfinished product
            if rows is None:
                if delta is not None:
                    resid += delta.float()
                h = resid
            else:
                pick = rows[:num_rows].long()
                h = resid[pick] if delta is None else resid[pick] + delta[pick].float()
            mu = h.mean(-1, keepdim=True)
            var = ((h - mu) ** 2).mean(-1, keepdim=True)
            return ((h - mu) / torch.sqrt(var + eps) * self.w + self.b).to(self.env.dtype)

    class LatentMean(Mixer):
        """c_t = Wc x_t is kept for every token; y_t = Wo mean(c_s, s in the last `window` tokens)."""
        def tensors(self):
            return [TensorDecl(self.spec.names["c"], (latent, size)), TensorDecl(self.spec.names["o"], (size, latent))]

        def load(self, weights, env):
            super().load(weights, env)
            self.wc, self.wo = weights[self.spec.names["c"]].float(), weights[self.spec.names["o"]].float()

        def cache_need(self):
            return CacheNeed((CacheRecord("latent", (PAGE, latent), torch.float32),), window)

        def workspace_elems(self, rows):
            return rows * latent

        def forward(self, x, step):
            cache, g = step.cache.record("latent"), step.cache.group      # [pages, page, latent]
            assert cache.dtype == torch.float32 and tuple(cache.shape[1:]) == (g.page_size, latent)
            c = x.float() @ self.wc.t()
            pos = step.positions[:step.num_rows].long()
            table = g.tables[step.seq_of_row[:step.num_rows].long()]      # [rows, width]
            cache[table.gather(1, (pos // g.page_size)[:, None])[:, 0], pos % g.page_size] = c
            out = torch.empty((step.num_rows, latent), dtype=torch.float32, device=x.device)
            for r in range(step.num_rows):
                p = int(pos[r])
                seen = torch.arange(max(0, p - window + 1), p + 1, device=x.device)
                pages = table[r, seen // g.page_size].long()
                assert int(pages.min()) >= 0                             # every page the window reaches is held
                out[r] = cache[pages, seen % g.page_size].mean(0)
            return (out @ self.wo.t()).to(x.dtype)

    register_part("norm", "toy_layernorm", ToyLayerNorm, replace=True)
    register_part("mixer", "toy_latent_mean", LatentMean, replace=True)

    class ToyConfig:
        def __init__(self, d):
            self.d = d

        def to_dict(self):
            return self.d

    def toy_spec(c):
        ln = lambda name: PartSpec("toy_layernorm", {"size": size}, {"weight": name + ".w", "bias": name + ".b"})
        rms = lambda n, name: PartSpec("rmsnorm", {"size": n, "eps": eps}, {"weight": name})
        mixers = (PartSpec("toy_latent_mean", {}, {"c": "l0.c", "o": "l0.o"}),
                  PartSpec("paged_attention", {"hidden_size": size, "num_heads": heads, "num_kv_heads": kv, "head_dim": hd,
                                               "scale": hd ** -0.5, "window": None}, {k: f"l1.{k}" for k in "qkvo"},
                           {"position": PartSpec("rope_neox", {"head_dim": hd, "theta": 1e4, "max_positions": 512}),
                            "q_norm": rms(hd, "l1.qn"), "k_norm": rms(hd, "l1.kn")}))
        blocks = tuple(BlockSpec("prenorm", mixers[i],
                                 PartSpec("swiglu", {"hidden_size": size, "intermediate_size": inter},
                                          {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                                 {"mixer": ln(f"l{i}.n1"), "ffn": ln(f"l{i}.n2")}) for i in range(2))
        return ModelSpec("ToyLatentLM", size, vocab, 512,
                         PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": size}, {"weight": "emb"}),
                         blocks, (LayerCall(0, 0), LayerCall(1, 1)), ln("norm"),
                         PartSpec("linear_head", {"vocab_size": vocab, "hidden_size": size, "tied": False}, {"weight": "head"}))

    register_architecture("ToyLatentLM", lambda d, origin: ToyConfig(d), toy_spec, replace=True)
    folder = write_random_model(str(tmp_path / "toylatent"), "ToyLatentLM", ToyConfig({"architectures": ["ToyLatentLM"]}), seed=13)
    w = {k: v for k, v in P.read_safetensors(str(tmp_path / "toylatent" / "model.safetensors")).items()}

    def layernorm(h, name):
        mu = h.mean(-1, keepdim=True)
        return (h - mu) / torch.sqrt(((h - mu) ** 2).mean(-1, keepdim=True) + eps) * w[name + ".w"] + w[name + ".b"]

    def plain(ids):
        T = len(ids)
        h = w["emb"][torch.tensor(ids)]
        for i in range(2):
            n = layernorm(h, f"l{i}.n1")
            if i == 0:
                c = n @ w["l0.c"].t()
                mean = torch.stack([c[max(0, t - window + 1):t + 1].mean(0) for t in range(T)])
                r = h + mean @ w["l0.o"].t()
            else:
                cfg = dict(num_attention_heads=heads, num_key_value_heads=kv, head_dim=hd, rms_norm_eps=eps, rope_theta=1e4)
                att = {f"s.{k}_proj.weight": w[f"l1.{k}"] for k in "qkvo"}
                att.update({"s.q_norm.weight": w["l1.qn"], "s.k_norm.weight": w["l1.kn"]})
                r = h + P.attention_block(n, att, "s.", cfg, list(range(T)), None)
            m = layernorm(r, f"l{i}.n2")
            h = r + P.linear(P.swiglu(P.linear(m, w[f"l{i}.g"]), P.linear(m, w[f"l{i}.u"])), w[f"l{i}.d"])
        return P.linear(layernorm(h, "norm"), w["head"]).numpy()

    rng = np.random.default_rng(6)
    reqs = {f"c{i}": rng.integers(0, vocab, n).tolist() for i, n in enumerate([41, 60, 10, 35])}
    want = {k: plain(v) for k, v in reqs.items()}
    model, _ = load_model(folder, dtype, DEV)
    needs = model.cache_needs()
    assert [tuple(r.name for r in n.records) for n in needs] == [("latent",), ("k", "v")]
    # what a page costs and what a step needs aside come from what the parts declare
    elem = 4 if dtype == "float32" else 2
    assert page_bytes(model, 8) == 8 * (latent * 4 + 2 * kv * hd * elem)
    assert workspace_bytes(model, 100) >= 4 * 100 * (latent + 3 * inter)
    bound = 2e-5 if dtype == "float32" else 4e-2
    for steps in (trace_whole(reqs), trace_prefill_then_decode(reqs), trace_portions(reqs, 3),
                  trace_mixed(reqs, 192, seed=4)):
        runner = ModelRunner(model, model.env, page_size=8, num_pages=24, max_requests=4, max_batch_tokens=256)
        assert sorted(runner.group_tensors[0]) == ["latent"] and runner.group_tensors[0]["latent"].dtype == torch.float32
        rp = Replayer(runner)
        got = collect(steps, {s["step"]: rp.run_step(s) for s in steps})
        for k in reqs:
            assert np.abs(got[k] - want[k]).max() <= bound * max(1.0, np.abs(want[k]).max()), (dtype, k)
        runner.cache.check()
        assert runner.cache.pages_returned_total > 0 and runner.cache.free_pages() == [24, 24]
