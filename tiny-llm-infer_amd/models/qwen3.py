"""Qwen3 dense: from its typed configuration to a ``ModelSpec``.

Tensor names and shapes are those the reference loads
(model/src/qwen3_layers.cpp:207-243); the order of operations inside a block is
that of model/src/qwen3_paged_batch.cpp:146-301: input norm, q/k/v projections,
per-head RMSNorm of q and k, neox rotation, keys and values into the cache,
attention, output projection, residual, post-attention norm, gate/up, SwiGLU,
down, residual; then the final norm and the head (:304-346).
"""
from __future__ import annotations

from ..config.base import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..config.qwen3 import ARCHITECTURE, Qwen3Config
from ..registry import register_architecture


def qwen3_spec(cfg: Qwen3Config) -> ModelSpec:
    def rms(name: str, size: int) -> PartSpec:
        return PartSpec("rmsnorm", {"size": size, "eps": cfg.rms_norm_eps}, {"weight": name})

    blocks = []
    windows = cfg.layer_windows()
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        rope = PartSpec("rope_neox", {"head_dim": cfg.head_dim, "rotary_dim": cfg.head_dim,
                                      "theta": cfg.rope_theta,
                                      "max_positions": cfg.max_position_embeddings})
        mixer = PartSpec(
            "paged_attention",
            {"hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
             "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
             "scale": cfg.head_dim ** -0.5, "window": windows[i]},
            {"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
             "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight"},
            {"position": rope,
             "q_norm": rms(p + "self_attn.q_norm.weight", cfg.head_dim),
             "k_norm": rms(p + "self_attn.k_norm.weight", cfg.head_dim)})
        ffn = PartSpec(
            "swiglu",
            {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size},
            {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
             "down": p + "mlp.down_proj.weight"})
        blocks.append(BlockSpec(
            "prenorm", mixer, ffn,
            {"mixer": rms(p + "input_layernorm.weight", cfg.hidden_size),
             "ffn": rms(p + "post_attention_layernorm.weight", cfg.hidden_size)}))
    head_names = ({"weight": "model.embed_tokens.weight"} if cfg.tie_word_embeddings
                  else {"weight": "lm_head.weight"})
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding",
                           {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size},
                           {"weight": "model.embed_tokens.weight"}),
        blocks=tuple(blocks),
        schedule=tuple(LayerCall(block=i, cache=i, writes_cache=True)
                       for i in range(cfg.num_hidden_layers)),
        final_norm=rms("model.norm.weight", cfg.hidden_size),
        head=PartSpec("linear_head",
                      {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                       "tied": cfg.tie_word_embeddings}, head_names),
        eos_token_ids=cfg.eos_token_ids)


register_architecture(ARCHITECTURE, Qwen3Config.from_dict, qwen3_spec)
