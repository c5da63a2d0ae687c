"""The plain implementation is pinned by what fixes it beside the reference's
text: library routines it must reduce to, and invariants a plausible mistake
(a wrong sign or pairing, a norm in the wrong place) would break.  The
reference ships no test vectors (its test folders are not in its tree)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as P

torch.manual_seed(0)
D = torch.float64


def test_rmsnorm_is_the_library_routine_and_scale_free():
    x, w = torch.randn(5, 24, dtype=D), torch.randn(24, dtype=D)
    assert torch.allclose(P.rmsnorm(x, w, 1e-6), F.rms_norm(x, (24,), w, 1e-6), atol=1e-12)
    unit = P.rmsnorm(x, torch.ones(24, dtype=D), 0.0)
    assert torch.allclose((unit * unit).mean(-1), torch.ones(5, dtype=D))
    assert torch.allclose(P.rmsnorm(3.0 * x, w, 0.0), P.rmsnorm(x, w, 0.0))
    assert float(P.rmsnorm(x, torch.zeros(24, dtype=D), 1e-6).abs().max()) == 0.0   # w, not 1 + w


def test_rope_is_a_rotation_by_position_of_half_split_pairs():
    x = torch.randn(6, 3, 8, dtype=D)
    pos = [0, 1, 2, 5, 9, 40]
    y = P.rope_neox(x, pos, 10000.0)
    assert torch.allclose(y[0], x[0])                                   # position 0: identity
    n = lambda t: t[..., :4] ** 2 + t[..., 4:] ** 2
    assert torch.allclose(n(y), n(x))                                   # each pair keeps its norm
    # head_dim 2: the plane rotation by `position` radians (theta^0 = 1)
    v = torch.tensor([[[1.0, 0.0]]], dtype=D)
    r = P.rope_neox(v, [3], 10000.0)[0, 0]
    assert torch.allclose(r, torch.tensor([math.cos(3.0), math.sin(3.0)], dtype=D), atol=1e-6)
    # only element i set: it moves towards i + d/2, not i + 1
    e = torch.zeros(1, 1, 8, dtype=D)
    e[0, 0, 1] = 1.0
    r = P.rope_neox(e, [7], 10000.0)[0, 0]
    assert r[5] != 0 and r[2] == 0 and r[0] == 0
    # frequencies: theta^(-2i/d)
    ang = P.rope_angles(8, 10000.0, [1])[0]
    assert np.allclose(ang, [10000.0 ** (-2 * i / 8) for i in range(4)], rtol=1e-6)


def test_rope_scores_depend_on_distance_only():
    q, k = torch.randn(1, 1, 16, dtype=D), torch.randn(1, 1, 16, dtype=D)
    def score(m, n):
        return float((P.rope_neox(q, [m], 1e4)[0, 0] * P.rope_neox(k, [n], 1e4)[0, 0]).sum())
    assert abs(score(9, 4) - score(25, 20)) < 1e-4
    assert abs(score(9, 4) - score(4, 9)) > 1e-3                        # the sign of the angle matters


def test_attention_is_the_library_routine_with_grouped_heads():
    T, H, G, d = 9, 6, 3, 8
    q, k, v = torch.randn(T, H, d, dtype=D), torch.randn(T, G, d, dtype=D), torch.randn(T, G, d, dtype=D)
    got = P.causal_attention(q, k, v, 1 / math.sqrt(d))
    kk = k.repeat_interleave(H // G, dim=1)          # consecutive q heads share a kv head
    vv = v.repeat_interleave(H // G, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                          is_causal=True).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-10)
    assert torch.allclose(got[0], vv[0])             # one key: the output is its value
    # one head, no mask needed for the last row: plain softmax(QK^T/sqrt d)V
    last = torch.softmax((k[:, 0] @ q[-1, 0]) / math.sqrt(d), 0) @ v[:, 0]
    assert torch.allclose(got[-1, 0], last)


def test_window_limits_the_keys_and_equals_all_keys_when_wide():
    T, d = 12, 4
    q, k, v = torch.randn(T, 2, d, dtype=D), torch.randn(T, 1, d, dtype=D), torch.randn(T, 1, d, dtype=D)
    assert torch.allclose(P.causal_attention(q, k, v, 0.5, window=T), P.causal_attention(q, k, v, 0.5))
    w3 = P.causal_attention(q, k, v, 0.5, window=3)
    want = torch.softmax((k[7:10, 0] @ q[9, 1]) * 0.5, 0) @ v[7:10, 0]
    assert torch.allclose(w3[9, 1], want)
    assert torch.allclose(P.causal_attention(q, k, v, 0.5, window=1)[5, 0], v[5, 0])


def test_swiglu_and_linear_are_the_library_routines():
    g, u = torch.randn(4, 10, dtype=D), torch.randn(4, 10, dtype=D)
    assert torch.allclose(P.swiglu(g, u), F.silu(g) * u, atol=1e-12)
    x, w = torch.randn(3, 5, dtype=D), torch.randn(7, 5, dtype=D)
    assert torch.allclose(P.linear(x, w), F.linear(x, w))


def _tiny(tied):
    cfg = dict(hidden_size=16, intermediate_size=24, num_hidden_layers=2, num_attention_heads=4,
               num_key_value_heads=2, head_dim=8, vocab_size=32, rms_norm_eps=1e-6, rope_theta=1e4,
               tie_word_embeddings=tied)
    g = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=g, dtype=D) * 0.3
    w = {"model.embed_tokens.weight": r(32, 16), "model.norm.weight": 1 + r(16), "lm_head.weight": r(32, 16)}
    for i in range(2):
        p = f"model.layers.{i}."
        w.update({p + "input_layernorm.weight": 1 + r(16), p + "post_attention_layernorm.weight": 1 + r(16),
                  p + "self_attn.q_proj.weight": r(32, 16), p + "self_attn.k_proj.weight": r(16, 16),
                  p + "self_attn.v_proj.weight": r(16, 16), p + "self_attn.o_proj.weight": r(16, 32),
                  p + "self_attn.q_norm.weight": 1 + r(8), p + "self_attn.k_norm.weight": 1 + r(8),
                  p + "mlp.gate_proj.weight": r(24, 16), p + "mlp.up_proj.weight": r(24, 16),
                  p + "mlp.down_proj.weight": r(16, 24)})
    return cfg, w


def test_model_is_causal_and_position_shift_changes_nothing_but_rounding():
    cfg, w = _tiny(False)
    ids = [3, 9, 1, 30, 7, 7, 12]
    full = P.forward(cfg, w, ids)
    changed = P.forward(cfg, w, ids[:4] + [0, 1, 2])
    assert torch.allclose(full[:4], changed[:4], atol=1e-12)            # later tokens never reach back
    assert not torch.allclose(full[4:], changed[4:], atol=1e-3)
    # only distances count: all positions shifted by 11 give the same logits
    shifted = P.forward(cfg, w, ids, first_position=11)
    assert torch.allclose(full, shifted, atol=1e-5)


def test_head_is_tied_or_its_own_matrix():
    cfg, w = _tiny(True)
    ids = [1, 2, 3]
    tied = P.forward(cfg, w, ids)
    w2 = dict(w)
    w2["lm_head.weight"] = w["lm_head.weight"] + 1.0
    assert torch.equal(P.forward(cfg, w2, ids), tied)                   # tied: lm_head is not read
    cfg["tie_word_embeddings"] = False
    assert not torch.allclose(P.forward(cfg, w, ids), tied)
    w3 = dict(w)
    w3["model.embed_tokens.weight"] = w["model.embed_tokens.weight"].clone()
    w3["model.embed_tokens.weight"][20] += 5.0                          # a row no token uses
    assert torch.equal(P.forward(cfg, w3, ids), P.forward(cfg, w, ids))


def test_q_and_k_norms_act_per_head_before_the_rotation():
    cfg, w = _tiny(False)
    ids = [4, 8, 15, 16, 23]
    base = P.forward(cfg, w, ids)
    # scaling q_proj changes nothing when q is normalised per head afterwards (eps aside) ...
    w2 = dict(w)
    w2["model.layers.0.self_attn.q_proj.weight"] = w["model.layers.0.self_attn.q_proj.weight"] * 7.0
    assert torch.allclose(P.forward(cfg, w2, ids), base, atol=1e-6)
    # ... while scaling v_proj does: v is not normalised
    w3 = dict(w)
    w3["model.layers.0.self_attn.v_proj.weight"] = w["model.layers.0.self_attn.v_proj.weight"] * 7.0
    assert not torch.allclose(P.forward(cfg, w3, ids), base, atol=1e-3)


# ---- the wiring of a layer around the residual stream ---------------------------------
# (model/src/qwen3_paged_batch.cpp:146-148, 273-279, 297-307: n = norm(h); r = h + attn(n);
# m = norm(r); h' = r + mlp(m); after the last layer norm(h) and the head)
def _library_attention(n, w, p, cfg, T):
    """The attention branch of one layer from library routines; positions 0..T-1."""
    H, G, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = F.rms_norm(F.linear(n, w[p + "q_proj.weight"]).view(T, H, d), (d,), w[p + "q_norm.weight"], cfg["rms_norm_eps"])
    k = F.rms_norm(F.linear(n, w[p + "k_proj.weight"]).view(T, G, d), (d,), w[p + "k_norm.weight"], cfg["rms_norm_eps"])
    v = F.linear(n, w[p + "v_proj.weight"]).view(T, G, d)
    q, k = P.rope_neox(q, list(range(T)), cfg["rope_theta"]), P.rope_neox(k, list(range(T)), cfg["rope_theta"])
    o = F.scaled_dot_product_attention(q.transpose(0, 1), k.repeat_interleave(H // G, dim=1).transpose(0, 1),
                                       v.repeat_interleave(H // G, dim=1).transpose(0, 1), is_causal=True)
    return F.linear(o.transpose(0, 1).reshape(T, H * d), w[p + "o_proj.weight"])


def test_branches_add_to_a_stream_that_is_never_normalised_itself():
    cfg, w = _tiny(False)
    ids = [5, 11, 2, 29, 17, 8]
    eps = cfg["rms_norm_eps"]
    emb = w["model.embed_tokens.weight"][ids]
    bare = F.linear(F.rms_norm(emb, (16,), w["model.norm.weight"], eps), w["lm_head.weight"])
    # both branches of both layers silenced: what is left is embedding -> final norm -> head, so
    # no layer norm touches the stream itself (a post-norm arrangement would)
    w0 = dict(w)
    for i in range(2):
        for name in (f"model.layers.{i}.self_attn.o_proj.weight", f"model.layers.{i}.mlp.down_proj.weight"):
            w0[name] = torch.zeros_like(w[name])
    assert torch.allclose(P.forward(cfg, w0, ids), bare, atol=1e-12)
    assert not torch.allclose(P.forward(cfg, w, ids), bare, atol=1e-3)
    # a stream a million times larger drowns the branches (their inputs are normed, so they stay as
    # they are) and the final norm takes the factor out again
    big = dict(w)
    big["model.embed_tokens.weight"] = w["model.embed_tokens.weight"] * 1e6
    assert torch.allclose(P.forward(cfg, big, ids), bare, atol=1e-3)


def test_one_layer_equals_its_formula_in_library_routines():
    cfg, w = _tiny(False)
    cfg["num_hidden_layers"] = 1
    ids = [5, 11, 2, 29, 17, 8, 8, 3]
    T, eps, p = len(ids), cfg["rms_norm_eps"], "model.layers.0."
    h = w["model.embed_tokens.weight"][ids]
    r = h + _library_attention(F.rms_norm(h, (16,), w[p + "input_layernorm.weight"], eps), w, p + "self_attn.", cfg, T)
    m = F.rms_norm(r, (16,), w[p + "post_attention_layernorm.weight"], eps)          # of r, not of h
    out = r + F.linear(F.silu(F.linear(m, w[p + "mlp.gate_proj.weight"])) * F.linear(m, w[p + "mlp.up_proj.weight"]),
                       w[p + "mlp.down_proj.weight"])                              # onto r, not onto h
    want = F.linear(F.rms_norm(out, (16,), w["model.norm.weight"], eps), w["lm_head.weight"])
    got = P.forward(cfg, w, ids)
    assert torch.allclose(got, want, atol=1e-10)
    # the two plausible mistakes differ by far more than that: a feed-forward that reads the stream
    # before the attention was added, and one that is added onto it
    m_wrong = F.rms_norm(h, (16,), w[p + "post_attention_layernorm.weight"], eps)
    mlp = lambda t: F.linear(F.silu(F.linear(t, w[p + "mlp.gate_proj.weight"])) * F.linear(t, w[p + "mlp.up_proj.weight"]),
                             w[p + "mlp.down_proj.weight"])
    for wrong in (r + mlp(m_wrong), h + mlp(m)):
        logits = F.linear(F.rms_norm(wrong, (16,), w["model.norm.weight"], eps), w["lm_head.weight"])
        assert float((logits - got).abs().max()) > 1e-2
    # silencing the feed-forward leaves stream + attention: the attention branch reaches the logits
    w1 = dict(w)
    w1[p + "mlp.down_proj.weight"] = torch.zeros_like(w[p + "mlp.down_proj.weight"])
    assert torch.allclose(P.forward(cfg, w1, ids),
                          F.linear(F.rms_norm(r, (16,), w["model.norm.weight"], eps), w["lm_head.weight"]), atol=1e-10)
