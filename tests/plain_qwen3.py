"""A plain, slow implementation of the Qwen3 dense decoder, written from the
reference's formulas.  Whole sequences, no cache, one function for each part,
float64 arithmetic (rotation angles in float32, as the reference computes
them).  It shares no code with the engine: it reads config.json as a plain
dict and the weights as a name -> tensor dict.

Paths cited are relative to the reference's root.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np
import torch

F64 = torch.float64


# ---------------------------------------------------------------- weights ----
def read_safetensors(path):
    """Minimal reader (8-byte header length, JSON header, raw data:
    model/src/qwen3_checkpoint.cpp:114-149).  Returns name -> float64 tensor."""
    kinds = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32}
    with open(path, "rb") as fh:
        raw = fh.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        data = bytearray(raw[8 + hlen + b:8 + hlen + e])
        t = torch.frombuffer(data, dtype=kinds[info["dtype"]]).reshape(info["shape"])
        out[name] = t.to(F64)
    return out


def read_model(folder):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ------------------------------------------------------------------ parts ----
def embedding(table, token_ids):
    """x_t = E[token_t]; no scaling (kernels/src/embed_kernel_cpu.cpp:24-44)."""
    return table[torch.as_tensor(token_ids, dtype=torch.long)]


def linear(x, weight):
    """y = x W^T, W stored [out, in] (kernels/src/matmul_kernel_cpu.cpp:27-35)."""
    return x @ weight.t()


def rmsnorm(x, weight, eps):
    """y_j = w_j * x_j * 1/sqrt(sum(x^2)/n + eps) over the last axis
    (kernels/src/rmsnorm_kernel_cpu.cpp:27-43)."""
    n = x.shape[-1]
    scale = 1.0 / torch.sqrt((x * x).sum(dim=-1, keepdim=True) / n + eps)
    return weight * x * scale


def rope_angles(head_dim, theta, positions):
    """angle[p, i] = float32(p) * theta^(-2i/head_dim), i < head_dim/2, with the
    exponent, the power and the product in float32
    (kernels/src/rope_kernel_cpu.cpp:130-138)."""
    half = head_dim // 2
    out = np.zeros((len(positions), half), dtype=np.float32)
    for r, p in enumerate(positions):
        for i in range(half):
            exponent = np.float32(-2.0) * np.float32(i) / np.float32(head_dim)
            freq = np.float32(np.power(np.float32(theta), exponent))
            out[r, i] = np.float32(p) * freq
    return out


def rope_neox(x, positions, theta):
    """x: [T, heads, head_dim].  Pairs are (i, i + head_dim/2):
    first' = first*cos - second*sin, second' = first*sin + second*cos
    (kernels/src/rope_kernel_cpu.cpp:156-166)."""
    T, H, D = x.shape
    half = D // 2
    ang = torch.from_numpy(rope_angles(D, theta, positions).astype(np.float64))
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    first, second = x[..., :half], x[..., half:]
    return torch.cat([first * cos - second * sin, first * sin + second * cos], dim=-1)


def causal_attention(q, k, v, scale, window=None):
    """q: [T, heads, d]; k, v: [T, kv_heads, d].  Head h uses kv head
    h // (heads / kv_heads); the row at position p sees keys 0..p, scores are
    (q.k)*scale, softmax is exp(s - max)/sum, output is the weighted sum of
    values (kernels/src/paged_attention_cpu.cpp:16-69).  With ``window`` w the
    row at p sees keys p-w+1..p (this engine's definition; the reference has no
    window)."""
    T, H, D = q.shape
    kv_mul = H // k.shape[1]
    out = torch.zeros(T, H, D, dtype=F64)
    for h in range(H):
        g = h // kv_mul
        for p in range(T):
            lo = 0 if window is None else max(0, p - window + 1)
            s = (k[lo:p + 1, g] @ q[p, h]) * scale
            w = torch.exp(s - s.max())
            w = w / w.sum()
            out[p, h] = w @ v[lo:p + 1, g]
    return out


def swiglu(gate, up):
    """(g / (1 + exp(-g))) * u (kernels/src/swiglu_kernel_cpu.cpp:20-24)."""
    return gate / (1.0 + torch.exp(-gate)) * up


# ------------------------------------------------------------------ model ----
def layer_windows(cfg):
    """Window per layer from the config.json keys; None = all keys."""
    n = cfg["num_hidden_layers"]
    if not cfg.get("use_sliding_window", False) or cfg.get("sliding_window") is None:
        return [None] * n
    types = cfg.get("layer_types")
    if types is not None:
        return [cfg["sliding_window"] if t == "sliding_attention" else None for t in types]
    first = cfg.get("max_window_layers", n)
    return [cfg["sliding_window"] if i >= first else None for i in range(n)]


def attention_block(x, w, prefix, cfg, positions, window):
    """model/src/qwen3_paged_batch.cpp:150-271: projections, per-head norm of q
    and k (before the rotation, v untouched), rotation, attention, o_proj."""
    heads, kv_heads = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or cfg["hidden_size"] // heads
    eps = cfg.get("rms_norm_eps", 1e-6)
    theta = cfg.get("rope_theta", 1e6)
    T = x.shape[0]
    q = linear(x, w[prefix + "q_proj.weight"]).reshape(T, heads, d)
    k = linear(x, w[prefix + "k_proj.weight"]).reshape(T, kv_heads, d)
    v = linear(x, w[prefix + "v_proj.weight"]).reshape(T, kv_heads, d)
    q = rmsnorm(q, w[prefix + "q_norm.weight"], eps)
    k = rmsnorm(k, w[prefix + "k_norm.weight"], eps)
    q = rope_neox(q, positions, theta)
    k = rope_neox(k, positions, theta)
    o = causal_attention(q, k, v, 1.0 / math.sqrt(d), window)
    return linear(o.reshape(T, heads * d), w[prefix + "o_proj.weight"])


def mlp_block(x, w, prefix):
    """model/src/qwen3_paged_batch.cpp:281-295."""
    g = linear(x, w[prefix + "gate_proj.weight"])
    u = linear(x, w[prefix + "up_proj.weight"])
    return linear(swiglu(g, u), w[prefix + "down_proj.weight"])


def forward(cfg, w, token_ids, first_position=0):
    """Logits [T, vocab] in float64 for one whole sequence.  Pre-norm wiring:
    model/src/qwen3_paged_batch.cpp:146-148, 273-279, 297-307.  The head is
    lm_head.weight unless tie_word_embeddings, then the embedding matrix (the
    reference always ties, model/src/qwen3_layers.cpp:246-265)."""
    eps = cfg.get("rms_norm_eps", 1e-6)
    positions = list(range(first_position, first_position + len(token_ids)))
    h = embedding(w["model.embed_tokens.weight"], token_ids)
    windows = layer_windows(cfg)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        n = rmsnorm(h, w[p + "input_layernorm.weight"], eps)
        r = h + attention_block(n, w, p + "self_attn.", cfg, positions, windows[i])
        m = rmsnorm(r, w[p + "post_attention_layernorm.weight"], eps)
        h = r + mlp_block(m, w, p + "mlp.")
    z = rmsnorm(h, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) \
        else w["lm_head.weight"]
    return linear(z, head)


def greedy(cfg, w, prompt, new_tokens):
    """Arg-max generation, lowest index on ties (engine/src/llm_engine.cpp:81-85)."""
    ids = list(prompt)
    out = []
    for _ in range(new_tokens):
        logits = forward(cfg, w, ids)[-1]
        tok = int(torch.argmax(logits))   # torch.argmax returns the first maximum
        out.append(tok)
        ids.append(tok)
    return out
