from .base import (BlockSpec, ConfigError, JsonReader, LayerCall, ModelSpec, PartSpec,
                   read_config_json)
from .qwen3 import Qwen3Config

__all__ = ["BlockSpec", "ConfigError", "JsonReader", "LayerCall", "ModelSpec", "PartSpec",
           "read_config_json", "Qwen3Config"]
