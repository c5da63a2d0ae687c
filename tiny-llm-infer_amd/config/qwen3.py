"""Typed configuration of the Qwen3 dense decoder, read from its config.json keys.

The reference reads hidden_size, intermediate_size, num_hidden_layers,
num_attention_heads, num_key_value_heads, vocab_size, max_position_embeddings
(required) and head_dim, rms_norm_eps, rope_theta (optional, defaults
hidden/heads, 1e-6, 1e6): model/src/qwen3_checkpoint.cpp:30-46.  Its validity
rules are at model/src/qwen3_checkpoint.cpp:177-181.  It never reads
tie_word_embeddings (it always ties, model/src/qwen3_layers.cpp:246-265); this
reader does, so that untied checkpoints get their own lm_head.  The
sliding-window keys of the same config.json (use_sliding_window,
sliding_window, max_window_layers, layer_types) are read here as well; the
reference ignores them, so their meaning is this engine's own and is stated at
``Qwen3Config.layer_windows``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, JsonReader

ARCHITECTURE = "Qwen3ForCausalLM"


@dataclass(frozen=True)
class Qwen3Config:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    use_sliding_window: bool
    sliding_window: Optional[int]
    max_window_layers: int
    layer_types: Optional[Tuple[str, ...]]
    eos_token_ids: Tuple[int, ...]

    # ---- derived sizes (model/src/qwen3_checkpoint.cpp:185-188) ----
    @property
    def query_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def layer_windows(self) -> Tuple[Optional[int], ...]:
        """Window of each layer's attention, None for all keys.

        A layer is windowed when ``use_sliding_window`` is true and either
        ``layer_types[i] == "sliding_attention"`` or, without ``layer_types``,
        ``i >= max_window_layers``.  A query at position p of a windowed layer
        sees the keys at positions p-window+1 .. p."""
        if not self.use_sliding_window or self.sliding_window is None:
            return tuple(None for _ in range(self.num_hidden_layers))
        if self.layer_types is not None:
            return tuple(self.sliding_window if t == "sliding_attention" else None
                         for t in self.layer_types)
        return tuple(self.sliding_window if i >= self.max_window_layers else None
                     for i in range(self.num_hidden_layers))

    # ---- reading -------------------------------------------------------
    @staticmethod
    def from_dict(data: Dict[str, Any], origin: str = "config.json") -> "Qwen3Config":
        r = JsonReader(data, origin)
        model_type = r.string("model_type", None)
        if model_type is not None and model_type != "qwen3":
            raise ConfigError(f"{origin}: model_type '{model_type}' is not 'qwen3'")
        r.raw("architectures")
        hidden = r.integer("hidden_size", minimum=1)
        inter = r.integer("intermediate_size", minimum=1)
        layers = r.integer("num_hidden_layers", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        kv_heads = r.integer("num_key_value_heads", heads, minimum=1)
        vocab = r.integer("vocab_size", minimum=1)
        max_pos = r.integer("max_position_embeddings", minimum=1)
        head_dim = r.integer("head_dim", 0, minimum=0)
        if head_dim == 0:
            if hidden % heads != 0:
                raise ConfigError(f"{origin}: no head_dim given and hidden_size {hidden} "
                                  f"is not a multiple of num_attention_heads {heads}")
            head_dim = hidden // heads
        eps = r.number("rms_norm_eps", 1e-6)
        theta = r.number("rope_theta", 1e6)
        tied = r.boolean("tie_word_embeddings", False)
        if r.boolean("attention_bias", False):
            raise ConfigError(f"{origin}: attention_bias=true is not supported (Qwen3 has no QKV bias)")
        act = r.string("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"{origin}: hidden_act '{act}' is not supported, only 'silu'")
        if r.raw("rope_scaling") is not None:
            raise ConfigError(f"{origin}: rope_scaling is not supported")
        use_window = r.boolean("use_sliding_window", False)
        window = r.integer("sliding_window", None, minimum=1)
        max_window_layers = r.integer("max_window_layers", layers, minimum=0)
        layer_types = r.raw("layer_types")
        if layer_types is not None:
            if (not isinstance(layer_types, list) or len(layer_types) != layers or any(
                    t not in ("full_attention", "sliding_attention") for t in layer_types)):
                raise ConfigError(f"{origin}: layer_types must list 'full_attention' or "
                                  f"'sliding_attention' for each of the {layers} layers")
            layer_types = tuple(layer_types)
        if use_window and window is None:
            raise ConfigError(f"{origin}: use_sliding_window=true needs sliding_window")
        eos = tuple(r.int_list("eos_token_id", []))

        if eps <= 0.0:
            raise ConfigError(f"{origin}: rms_norm_eps must be positive")
        if theta <= 0.0:
            raise ConfigError(f"{origin}: rope_theta must be positive")
        if kv_heads > heads or heads % kv_heads != 0:
            raise ConfigError(f"{origin}: num_attention_heads {heads} must be a multiple of "
                              f"num_key_value_heads {kv_heads}")
        if head_dim % 2 != 0:
            raise ConfigError(f"{origin}: head_dim {head_dim} must be even")
        return Qwen3Config(
            hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers,
            num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
            vocab_size=vocab, max_position_embeddings=max_pos, rms_norm_eps=eps,
            rope_theta=theta, tie_word_embeddings=tied, use_sliding_window=use_window,
            sliding_window=window, max_window_layers=max_window_layers,
            layer_types=layer_types, eos_token_ids=eos)

    def to_dict(self) -> Dict[str, Any]:
        """The config.json this configuration is read back from."""
        out: Dict[str, Any] = {
            "architectures": [ARCHITECTURE],
            "model_type": "qwen3",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": False,
            "hidden_act": "silu",
            "rope_scaling": None,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
            "torch_dtype": "bfloat16",
        }
        if self.layer_types is not None:
            out["layer_types"] = list(self.layer_types)
        if self.eos_token_ids:
            out["eos_token_id"] = (self.eos_token_ids[0] if len(self.eos_token_ids) == 1
                                   else list(self.eos_token_ids))
        return out
