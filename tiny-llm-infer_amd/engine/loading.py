"""From a model folder to a loaded model: config.json picks the architecture
from the registry, the architecture turns its typed configuration into a
``ModelSpec``, the parts are built and take their weights."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import models  # noqa: F401  (registers the architectures)
from ..parts.base import BuildEnv
from ..registry import load_config, lookup_architecture
from ..weights.loader import write_model_folder
from .model import Model

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"run dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"run dtype must be bfloat16 or float32, got {name!r}") from None


def make_env(dtype, device="cuda:0", max_model_len: int = 1 << 30, ops=None) -> BuildEnv:
    device = torch.device(device)
    if ops is None:
        from ..kernels.ops import HipOps
        ops = HipOps(device)
    return BuildEnv(dtype=parse_dtype(dtype), device=device, ops=ops, max_model_len=max_model_len)


def load_model(model_dir: str, dtype, device="cuda:0", max_model_len: Optional[int] = None,
               ops=None) -> Tuple[Model, object]:
    """Returns (model with weights on the device, typed configuration)."""
    arch, cfg = load_config(model_dir)
    spec = arch.make_spec(cfg)
    limit = spec.max_positions if max_model_len is None else min(max_model_len, spec.max_positions)
    env = make_env(dtype, device, limit, ops)
    model = Model(spec)
    model.load_from(model_dir, env)
    return model, cfg


def random_model(architecture: str, cfg, seed: int, dtype, device="cuda:0",
                 max_model_len: Optional[int] = None, ops=None) -> Model:
    """A model of ``architecture`` with seeded random weights drawn on the device."""
    spec = lookup_architecture(architecture).make_spec(cfg)
    limit = spec.max_positions if max_model_len is None else min(max_model_len, spec.max_positions)
    env = make_env(dtype, device, limit, ops)
    model = Model(spec)
    model.load_random(seed, env)
    return model


def write_random_model(folder: str, architecture: str, cfg, seed: int,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Random-weights mode: write config.json and model.safetensors for ``cfg``."""
    spec = lookup_architecture(architecture).make_spec(cfg)
    return write_model_folder(folder, cfg.to_dict(), Model(spec).tensors(), seed, dtype)
