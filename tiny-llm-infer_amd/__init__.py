"""tiny-llm-infer for one AMD MI355X: a small, whole inference engine.

Everything between a request's tokens and its next token for the Qwen3 dense
decoder, built from parts (mixer, feed-forward, norm, position encoding, block)
so that another architecture is another entry of the registry."""
from . import models  # noqa: F401  (registers the architectures)
from .registry import architecture_names, load_config, lookup_architecture, register_architecture

__all__ = ["architecture_names", "load_config", "lookup_architecture", "register_architecture"]
__version__ = "0.1.0"
